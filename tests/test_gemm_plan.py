"""Which kernel variant a product takes is host arithmetic (dlmi_gemm_plan: no device needed).  The choices for
the products of the five benchmark configurations on 256 compute units are pinned here, with the measurements
they come from in the comments; and a few properties every plan must have."""
import ctypes
import os

import pytest

from conftest import load_package

c_sz = ctypes.c_size_t


@pytest.fixture(scope="module")
def plan():
    for k in ("DLMI_GEMM_TILE", "DLMI_GEMM_SPLIT"):
        assert k not in os.environ, k + " forces a shape: unset it for this test"
    lib = ctypes.CDLL(load_package().LIB_PATH)

    def f(M, N, K, cus=256):
        tm, tn, st = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        sl = ctypes.c_uint()
        rc = lib.dlmi_gemm_plan(ctypes.c_int(cus), c_sz(M), c_sz(N), c_sz(K), ctypes.byref(tm), ctypes.byref(tn),
                                ctypes.byref(sl), ctypes.byref(st))
        assert rc == 0
        return tm.value, tn.value, sl.value, st.value

    return f


def products(B, K, H):
    """forward, dX, dW of a layer [B, K] -> [B, H] as (M, N, K)."""
    return (B, H, K), (B, K, H), (H, K, B)


def test_plans_of_the_benchmark_configurations(plan):
    # c3, 8192 x 4096 x 4096: two rounds of 256 x 256 tiles, one workgroup per CU (93 % of the matrix peak)
    for p in products(8192, 4096, 4096):
        assert plan(*p) == (256, 256, 1, 1)
    # c4, 1024 x 2048 x 2048: forward and dX have 128 tiles of 128 x 128 for 256 CUs, so 64 x 64 (two per CU) with
    # two register stages (K = 2048: 128 K tiles); dW's 2048 x 2048 output is exactly 256 tiles of 128 x 128
    fwd, dx, dw = products(1024, 2048, 2048)
    assert plan(*fwd) == (64, 64, 1, 2)
    assert plan(*dx) == (64, 64, 1, 2)
    assert plan(*dw) == (128, 128, 1, 2)
    # c5, 65536 x 256 x 256: one round of 256 x 256 tiles would store 256 KiB per CU all at once (7.4 of 73 us);
    # 128-wide tiles share a CU and overlap their stores (70 us); 16 K tiles: one register stage.  dW's 256 x 256
    # output behind K = 65536 runs 128 x 128 tiles over 64 K slices
    fwd, dx, dw = products(65536, 256, 256)
    assert plan(*fwd) == (128, 128, 1, 1)
    assert plan(*dx) == (128, 128, 1, 1)
    assert plan(*dw) == (128, 128, 64, 2)
    # c1, the hidden layers of 784-512-512-10 on 128 rows: small outputs, 64 x 64 tiles split over K
    for p in products(128, 784, 512) + products(128, 512, 512):
        tm, tn, slices, stages = plan(*p)
        assert (tm, tn) == (64, 64) and slices >= 1


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (7, 13, 5), (300, 224, 96), (4096, 4096, 8192), (100000, 8, 16), (256, 256, 1 << 20)])
@pytest.mark.parametrize("cus", [256, 304, 64])
def test_every_plan_is_launchable(plan, M, N, K, cus):
    tm, tn, slices, stages = plan(M, N, K, cus)
    assert (tm, tn) in ((64, 64), (128, 128), (256, 128), (256, 256))
    assert stages in (1, 2) and (stages == 1 or tm * tn <= 128 * 128)
    ktiles = -(-K // 16)
    assert 1 <= slices <= max(1, ktiles)
    if slices > 1:
        assert -(-ktiles // slices) >= 1  # no empty slice


def test_plan_refuses_empty_products(plan):
    lib = ctypes.CDLL(load_package().LIB_PATH)
    assert lib.dlmi_gemm_plan(ctypes.c_int(256), c_sz(0), c_sz(4), c_sz(4), None, None, None, None) != 0
    assert lib.dlmi_gemm_plan(ctypes.c_int(0), c_sz(4), c_sz(4), c_sz(4), None, None, None, None) != 0
