"""CPU-side checks of the product library: it loads, and it exports every symbol
include/dlmi.h declares (no compute calls here: those need a GPU)."""
import ctypes
import os
import re

from conftest import ROOT, load_package


def declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dlmi_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    pkg = load_package()
    assert os.path.exists(pkg.LIB_PATH), "build it first: python deep-learning_amd/build.py"
    lib = ctypes.CDLL(pkg.LIB_PATH)
    names = declared_symbols("dlmi.h")
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), "missing export " + n
    assert sorted(pkg.C_ABI_SYMBOLS) == names
    if os.path.exists(os.path.join(ROOT, "include", "dlmi_model.h")):
        for n in declared_symbols("dlmi_model.h"):
            assert hasattr(lib, n), "missing export " + n


def test_no_gpu_means_error_not_fallback():
    """Without a device the context cannot be created: there is no CPU path."""
    import torch
    if torch.cuda.is_available():
        return
    pkg = load_package()
    lib = ctypes.CDLL(pkg.LIB_PATH)
    ctx = ctypes.c_void_p()
    assert lib.dlmi_ctx_create(ctypes.byref(ctx), 0, None) != 0
    assert not ctx.value
    try:
        pkg.Dlmi(0)
    except pkg.DlmiError:
        pass
    else:
        raise AssertionError("Dlmi() must raise without a GPU")


def test_product_never_imports_the_oracle():
    """The oracle is a checker: nothing under deep-learning_amd/ may name it."""
    for base, _, files in os.walk(os.path.join(ROOT, "deep-learning_amd")):
        if os.sep + "build" in base or os.sep + "lib" in base:
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(base, f), errors="ignore").read()
                assert "dloracle" not in text and "oracle." not in text and "dlref" not in text, f
