"""GPU test of bf_hip_bias_grad_static, the column sum that takes no device memory from the driver or the pool
(its partial sums live in an array inside the library's code object).  It shares its kernels with
bf_hip_bias_grad, so the two must agree bit for bit; the oracle's column sum bounds both."""
import ctypes

import numpy as np
import pytest

from parity import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu
f32 = np.float32


def pool_stats(hip):
    stats = hip.capi.PoolStats()
    hip.capi.call("bf_hip_pool_stats", ctypes.byref(stats))
    return stats.driver_allocations, stats.acquires


def column_sums(hip, entry, g, out):
    rows, features = g.shape
    hip.capi.call(entry, g.ptr, out.ptr, rows, features, None)
    return out.toHost()


def test_static_workspace_bias_grad_matches_the_pooled_one(hip, oracle):
    """Two calls in a row, the second smaller: what the first left in the shared array must not leak into it."""
    D = hip.DeviceTensor
    rng = np.random.default_rng(77)
    for rows, features in ((5000, 3072), (700, 768), (33, 50), (1, 8192), (4096, 8192)):
        host = (rng.standard_normal((rows, features)) * 2).astype(f32)
        g = D.fromHost(host)
        pooled, static = D.zeros((features,)), D.zeros((features,))
        expected = column_sums(hip, "bf_hip_bias_grad", g, pooled)
        before = pool_stats(hip)
        got = column_sums(hip, "bf_hip_bias_grad_static", g, static)
        assert pool_stats(hip) == before, "the static entry point took memory from the pool"
        assert_bits_equal(got, expected, f"bias_grad_static {rows}x{features}")
        assert_close(got, oracle.addBiasBackward(host)[1], what=f"bias_grad_static vs oracle {rows}x{features}",
                     scale=float(np.sqrt(rows)) * 2)


def test_static_workspace_limit_is_an_error_not_a_fault(hip):
    D = hip.DeviceTensor
    rows, features = 4096, 8200   # 256 partial rows of 8200 columns: beyond 2^21 floats
    g, out = D.zeros((rows, features)), D.zeros((features,))
    with pytest.raises(ValueError, match="static workspace"):
        hip.capi.call("bf_hip_bias_grad_static", g.ptr, out.ptr, rows, features, None)
    # a short matrix of the same width needs few partial rows and is accepted
    hip.capi.call("bf_hip_bias_grad_static", g.ptr, out.ptr, 64, features, None)
    assert not out.toHost().any()
    # empty inputs: zero rows give zero sums, zero features launch nothing
    hip.capi.call("bf_hip_bias_grad_static", None, out.ptr, 0, features, None)
    hip.capi.call("bf_hip_bias_grad_static", None, None, 5, 0, None)
