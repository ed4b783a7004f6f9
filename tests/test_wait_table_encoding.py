"""wait_younger_n (csrc/norm_panel_common.hpp) jumps into a table of 48 `s_waitcnt vmcnt(k)` entries with an address
it computes itself: the table must start 20 bytes behind the instruction after `s_getpc_b64` and every entry must
be 8 bytes long.  That is a property of the instruction encodings the assembler picks, which no run on the GPU
would report if it changed (a wrong entry only waits for another count).  This test cross-compiles a kernel that
calls the function (no GPU needed) and checks the addresses in the disassembly of that code object."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LLVM = "/opt/rocm/llvm/bin"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

SOURCE = r'''
#include <hip/hip_runtime.h>
#include "norm_panel_common.hpp"
extern "C" __global__ void probe(float const *p, float *q, int n) {
  float a = p[threadIdx.x], b = p[threadIdx.x + 64];
  dlmi::wait_younger_n(n);
  q[threadIdx.x] = a + b;
}
'''


@pytest.mark.skipif(not (os.path.exists(HIPCC) and os.path.exists(os.path.join(LLVM, "llvm-objdump"))),
                    reason="no ROCm toolchain here")
def test_every_table_entry_sits_where_the_jump_lands():
    d = tempfile.mkdtemp()
    try:
        src, obj, elf = (os.path.join(d, n) for n in ("probe.hip", "probe.o", "probe.elf"))
        with open(src, "w") as f:
            f.write(SOURCE)
        subprocess.run([HIPCC, "-O3", "--offload-arch=gfx950", "-std=c++17", "--cuda-device-only", "-c", src, "-o", obj,
                        "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "deep-learning_amd", "csrc")],
                       check=True, capture_output=True)
        subprocess.run([os.path.join(LLVM, "clang-offload-bundler"), "--unbundle", "--type=o", "--input=" + obj,
                        "--targets=hip-amdgcn-amd-amdhsa--gfx950", "--output=" + elf], check=True, capture_output=True)
        text = subprocess.run([os.path.join(LLVM, "llvm-objdump"), "-d", elf], check=True, capture_output=True, text=True).stdout
    finally:
        shutil.rmtree(d, ignore_errors=True)
    lines = [(m.group(1).strip(), int(m.group(2), 16)) for m in
             (re.match(r"\s*(.*?)\s*//\s*([0-9A-Fa-f]+):", l) for l in text.splitlines()) if m]
    starts = [i for i, (ins, _) in enumerate(lines) if ins.startswith("s_getpc_b64 vcc")]
    assert len(starts) == 1, "one call, one table"
    i = starts[0]
    base = lines[i + 1][1]  # what s_getpc_b64 returns: the address of the next instruction
    assert lines[i][1] + 4 == base
    assert [ins.split()[0] for ins, _ in lines[i + 1:i + 6]] == ["s_lshl_b32", "s_add_u32", "s_add_u32", "s_addc_u32", "s_setpc_b64"]
    assert " 3" in lines[i + 1][0] and lines[i + 2][0].rstrip().endswith(" 20"), lines[i + 1:i + 3]
    table = lines[i + 6:i + 6 + 96]
    for k in range(48):
        wait, at = table[2 * k]
        assert wait == f"s_waitcnt vmcnt({k})", (k, wait)
        assert at == base + 20 + 8 * k, (k, hex(at), hex(base))
        assert table[2 * k + 1][0].startswith("s_branch"), table[2 * k + 1]
        assert table[2 * k + 1][1] == at + 4
