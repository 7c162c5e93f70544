"""Tolerances of the parity tests (GPU result vs CPU oracle).

fp32 ops and the attention core: every element must satisfy
    |gpu - ref| <= 1e-4 * |ref| + 1e-4 * rms(ref)
i.e. a maximum relative error of 1e-4 with an absolute floor of 1e-4 of the tensor's typical
magnitude, so that elements that happen to be near zero are judged against the scale of the tensor
rather than against themselves.  Where a result is a difference of nearly equal terms (attention
gradients: dS = P * (dP - D) vanishes identically for a row with one visible key), rms(ref) can be
arbitrarily small or zero; such tests pass `scale`, the magnitude of the terms being combined, and the
floor becomes 1e-4 * max(rms(ref), scale).  (The reference's own GPU-vs-CPU tests use absolute
tolerances: 1e-3 for attention, tests/backend/cuda/ops_tests.cu:342-363.)
bf16 projections and their gradients use 2e-2 in the same formula.
Integer / index / copy work (embedding gather, argmax, concat) must be bit-exact.
"""
import numpy as np

FP32_TOL = 1e-4
BF16_TOL = 2e-2


# largest |gpu - ref| / max|ref| seen by assert_close since the last take_worst(), per first word of `what`
_worst = {}


def take_worst():
    """The measured errors collected since the last call ({first word of `what`: max |gpu-ref| / max|ref|}), and a reset."""
    out = dict(_worst)
    _worst.clear()
    return out


def assert_close(actual, expected, tol=FP32_TOL, what="", scale=0.0):
    """|gpu - ref| <= tol * |ref| + tol * max(rms(ref), scale) for every element: a relative bound with an ABSOLUTE floor of
    tol times the tensor's rms (or `scale`, for tensors that are differences of nearly equal terms).  With the default
    tol = 1e-4 a `scale` of 0.05 * max|ref| is an absolute floor of 5e-6 of the largest element."""
    actual = np.asarray(actual, np.float64)
    expected = np.asarray(expected, np.float64)
    assert actual.shape == expected.shape, f"{what}: shape {actual.shape} != {expected.shape}"
    if expected.size == 0:
        return
    assert np.isfinite(actual).all(), f"{what}: non-finite values in the GPU result"
    rms = float(np.sqrt(np.mean(expected ** 2)))
    bound = tol * np.abs(expected) + tol * max(rms, float(scale)) + 1e-30
    err = np.abs(actual - expected)
    worst = int(np.argmax(err - bound))
    _worst[what.split(" ")[0] if what else ""] = max(_worst.get(what.split(" ")[0] if what else "", 0.0),
                                                     float(err.max() / (np.abs(expected).max() + 1e-30)))
    assert (err <= bound).all(), (
        f"{what}: |gpu-ref|={err.flat[worst]:.3e} > bound {bound.flat[worst]:.3e} at flat index {worst} "
        f"(ref={expected.flat[worst]:.6e}, gpu={actual.flat[worst]:.6e}, rms={rms:.3e}); "
        f"max rel err over tensor max = {err.max() / (np.abs(expected).max() + 1e-30):.3e}")


def assert_bits_equal(actual, expected, what=""):
    a = np.ascontiguousarray(actual, np.float32).view(np.uint32)
    e = np.ascontiguousarray(expected, np.float32).view(np.uint32)
    assert a.shape == e.shape, f"{what}: shape"
    np.testing.assert_array_equal(a, e, err_msg=what)
