"""Comparison helpers shared by the CPU and GPU tests."""
import numpy as np

# Tolerances of the hot path (fp32): 1e-5 relative for element-wise results,
# 1e-4 after reductions and GEMMs.  "Relative" is taken against the larger of
# |expected| and the tensor's RMS: an element that is the small difference of
# two large terms (x - mean, a dot product that cancels) cannot be reproduced
# to 1e-5 of ITSELF by any implementation that sums in another order, only to
# 1e-5 of the terms it was formed from.
RTOL_ELEMENTWISE = 1e-5
RTOL_REDUCED = 1e-4
# oracle (our C restatement) against the reference: same operation order, so
# only last-place differences from FMA contraction / vectorization remain
RTOL_RESTATEMENT = 4e-6


def rms(a):
    a = np.asarray(a, np.float64)
    return float(np.sqrt(np.mean(a * a))) if a.size else 0.0


def max_rel_err(got, exp, floor=0.0):
    """max |got-exp| / max(|exp|, rms(exp), floor) (0 for empty tensors).
    `floor` names the natural scale of a quantity whose expected value may be
    identically zero (a shift in units of sigma, a gradient that cancels)."""
    got = np.asarray(got, np.float64)
    exp = np.asarray(exp, np.float64)
    if exp.size == 0:
        return 0.0
    den = np.maximum(np.abs(exp), max(rms(exp), floor, 1e-30))
    return float(np.max(np.abs(got - exp) / den))


def max_rel_err_strict(got, exp):
    """The element-wise metric of the measurement contract: max |got-exp| / max(|exp|, 1e-6 * max|exp|).
    Every element is judged against ITSELF; only elements a million times below the largest one share a
    floor.  Holds at 1e-5 for element-wise leaves outside their cancellation zones (exp(x)-1 and
    2/(1+exp(-2x))-1 near x = 0, where the reference's own float evaluation is no better); it cannot hold
    at 1e-4 for every element of a reduction or a GEMM output (an element that happens to cancel to
    1e-3 of the typical magnitude carries the absolute error of its terms), which is why the assertions
    behind reductions use max_rel_err above and this one is reported beside it."""
    got = np.asarray(got, np.float64)
    exp = np.asarray(exp, np.float64)
    if exp.size == 0:
        return 0.0
    den = np.maximum(np.abs(exp), max(1e-6 * float(np.max(np.abs(exp))), 1e-300))
    return float(np.max(np.abs(got - exp) / den))


def assert_close(got, exp, rtol, what="", floor=0.0):
    got = np.asarray(got)
    exp = np.asarray(exp)
    assert got.shape == exp.shape, f"{what}: shape {got.shape} != {exp.shape}"
    assert np.all(np.isfinite(got) == np.isfinite(exp)), f"{what}: non-finite pattern differs"
    fin = np.isfinite(exp)
    # infinities / NaNs must match in kind
    assert np.array_equal(got[~fin].astype(str), exp[~fin].astype(str)), f"{what}: inf/nan differ"
    err = max_rel_err(got[fin], exp[fin], floor)
    assert err <= rtol, f"{what}: max rel err {err:.3e} > {rtol:.1e}"
    return err
