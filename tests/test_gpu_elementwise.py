"""GPU parity: elementwise family, row-wise ops, bias gradients -- through the C ABI, against the oracle."""
import ctypes

import numpy as np
import pytest

import refvectors as rv
from parity import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu
f32 = np.float32

SIZES = [1, 3, 4, 255, 1024, 4099, 1 << 20]


def r(rng, *s, scale=1.0):
    return (rng.standard_normal(s) * scale).astype(f32)


@pytest.mark.parametrize("n", SIZES)
def test_flat_ops(hip, oracle, rng, n):
    D, ops = hip.DeviceTensor, hip.ops
    x, g = r(rng, n, scale=3), r(rng, n)
    dx, dg = D.fromHost(x), D.fromHost(g)
    assert_bits_equal(ops.add(dx, dg).toHost(), oracle.add(x, g), "add")
    assert_bits_equal(ops.scale(dx, 0.37).toHost(), oracle.scale(x, 0.37), "scale")
    assert_bits_equal(ops.relu(dx).toHost(), oracle.relu(x), "relu")
    assert_bits_equal(ops.reluBackward(dx, dg).toHost(), oracle.reluBackward(x, g), "reluBackward")
    # The reference's gelu, 0.5 x (1 + tanh u), adds nearly opposite numbers once x < -4 (tanh u -> -1): there its value,
    # of the order of 1e-6, carries an absolute error of about 1e-7 |x|.  The GPU evaluates the same function as
    # x / (1 + exp(-2u)), which has no such subtraction, so the two agree to that absolute error, not to 1e-4 of a value that
    # small: `scale` (the magnitude of the terms the reference combines) sets the floor for tensors that hold nothing else.
    for name in ("silu", "gelu"):
        scale = float(np.abs(x).max()) if name == "gelu" else 0.0
        assert_close(getattr(ops, name)(dx).toHost(), getattr(oracle, name)(x), what=name, scale=scale)
        assert_close(getattr(ops, name + "Backward")(dx, dg).toHost(), getattr(oracle, name + "Backward")(x, g), what=name + "Backward",
                     scale=scale * float(np.abs(g).max()))
    t = D.fromHost(x)
    ops.accumulate(t, dg)
    assert_bits_equal(t.toHost(), x + g, "accumulate")


def test_unaligned_pointers_take_the_scalar_path(hip, oracle, rng):
    """Sub-buffers that start 4 bytes into an allocation are not 16-byte aligned."""
    n = 1003
    x, y = r(rng, n + 1), r(rng, n + 1)
    dx, dy, out = hip.DeviceTensor.fromHost(x), hip.DeviceTensor.fromHost(y), hip.DeviceTensor.zeros((n + 1,))
    off = lambda t: ctypes.c_void_p(t.ptr.value + 4)
    hip.capi.call("bf_hip_add", off(dx), off(dy), off(out), n, None)
    assert_bits_equal(out.toHost()[1:], x[1:] + y[1:])
    hip.capi.call("bf_hip_act_forward", off(dx), off(out), n, hip.capi.ACT_SILU, None)
    assert_close(out.toHost()[1:], oracle.silu(x[1:]))


def test_shape_errors_raise_before_launch(hip):
    D, ops = hip.DeviceTensor, hip.ops
    a, b = D.zeros((2,)), D.zeros((3,))
    for fn in (ops.add, ops.siluBackward, ops.rmsnormBackward):
        with pytest.raises(ValueError):
            fn(a, b)
    with pytest.raises(ValueError):
        ops.rmsnorm(D.zeros((4,)))
    with pytest.raises(ValueError):
        ops.softmax(D.zeros((4,)))
    with pytest.raises(ValueError):
        ops.addBias(D.zeros((2, 3)), D.zeros((4,)))
    with pytest.raises(ValueError):
        hip.capi.call("bf_hip_act_forward", a.ptr, a.ptr, 2, 99, None)


def test_zero_sized_tensors_launch_nothing(hip):
    D, ops = hip.DeviceTensor, hip.ops
    e = D((0, 4))
    assert ops.add(e, D((0, 4))).toHost().shape == (0, 4)
    assert ops.rmsnorm(e).toHost().shape == (0, 4)
    assert ops.silu(D((0,))).toHost().size == 0


@pytest.mark.parametrize("rows,features", [(1, 1), (2, 2), (5, 7), (512, 128), (33, 768), (64, 3072), (3, 50257), (7, 1000)])
def test_bias_family(hip, oracle, rng, rows, features):
    D, ops, capi = hip.DeviceTensor, hip.ops, hip.capi
    x, res, dh = r(rng, rows, features), r(rng, rows, features), r(rng, rows, features)
    bias = r(rng, features)
    dx, db, dres, ddh = D.fromHost(x), D.fromHost(bias), D.fromHost(res), D.fromHost(dh)
    assert_bits_equal(ops.addBias(dx, db).toHost(), oracle.addBias(x, bias), "addBias")
    assert_bits_equal(ops.addBiasResidual(dx, db, dres).toHost(), oracle.add(oracle.addBias(x, bias), res), "addBiasResidual")
    for act, name in ((capi.ACT_SILU, "silu"), (capi.ACT_GELU, "gelu"), (capi.ACT_RELU, "relu")):
        pre = oracle.addBias(x, bias)
        assert_close(ops.addBiasAct(dx, db, act).toHost(), getattr(oracle, name)(pre), what="addBias+" + name)
        dgemm, dbias = ops.addBiasActBackward(dx, db, ddh, act)
        exp = getattr(oracle, name + "Backward")(pre, dh)
        assert_close(dgemm.toHost(), exp, what="addBiasActBackward.dGemm " + name)
        assert_close(dbias.toHost(), oracle.addBiasBackward(exp)[1], what="addBiasActBackward.dBias " + name)
    assert_close(ops.biasGradientOnly(dx).toHost(), oracle.addBiasBackward(x)[1], what="biasGradientOnly")
    di, dbias = ops.addBiasBackward(dx)
    assert_bits_equal(di.toHost(), x)


@pytest.mark.parametrize("rows,features", [(2, 4), (1, 1), (3, 2), (512, 128), (9, 768), (5, 1000), (4, 1024), (3, 2048), (2, 8192),
                                           (2, 10007), (2, 50257), (1, 70001)])
def test_row_ops(hip, oracle, rng, rows, features):
    D, ops = hip.DeviceTensor, hip.ops
    x, g = r(rng, rows, features, scale=2), r(rng, rows, features)
    dx, dg = D.fromHost(x), D.fromHost(g)
    assert_close(ops.rmsnorm(dx).toHost(), oracle.rmsnorm(x), what="rmsnorm")
    assert_close(ops.rmsnormBackward(dx, dg).toHost(), oracle.rmsnormBackward(x, g), what="rmsnormBackward")
    # the residual connection's gradient joined in the same pass: the separate add's result, bit for bit
    res = r(rng, rows, features)
    assert_bits_equal(ops.rmsnormBackwardAdd(dx, dg, D.fromHost(res)).toHost(), ops.add(D.fromHost(res), ops.rmsnormBackward(dx, dg)).toHost(),
                      "rmsnormBackwardAdd")
    assert_close(ops.softmax(dx).toHost(), oracle.softmax(x), what="softmax")
    assert_close(ops.softmaxBackward(dx, dg).toHost(), oracle.softmaxBackward(x, g), what="softmaxBackward")


def test_row_ops_rank3_and_reference_literals(hip, oracle):
    """The literal cases of the reference's CUDA tests (tests/backend/cuda/ops_tests.cu:149-208)."""
    D, ops = hip.DeviceTensor, hip.ops
    x = np.array([1, 2, 3, 4, -1, -1, -1, -1], f32).reshape(1, 2, 4)
    out = ops.rmsnorm(D.fromHost(x)).toHost()
    assert out.shape == (1, 2, 4)
    assert_close(out, oracle.rmsnorm(x))
    np.testing.assert_allclose(ops.softmax(D.fromHost(np.full((1, 3), 1000, f32))).toHost(), 1 / 3, atol=1e-6)
    np.testing.assert_allclose(ops.softmax(D.fromHost(np.array([[1, 2, 3], [-1, 0, 1]], f32))).toHost().sum(1), 1.0, atol=1e-6)


def test_golden_rows_and_activations(hip):
    """Replays the fixtures written by the real reference build."""
    import os
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz"))
    D, ops = hip.DeviceTensor, hip.ops
    x, g = D.fromHost(gold["rows_x"]), D.fromHost(gold["rows_g"])
    assert_close(ops.rmsnorm(x).toHost(), gold["rows_rmsnorm"])
    assert_close(ops.rmsnormBackward(x, g).toHost(), gold["rows_rmsnorm_bwd"])
    assert_close(ops.softmax(x).toHost(), gold["rows_softmax"])
    assert_close(ops.softmaxBackward(x, g).toHost(), gold["rows_softmax_bwd"])
    for name in ("silu", "gelu", "relu"):
        assert_close(getattr(ops, name)(x).toHost(), gold["act_" + name])
        assert_close(getattr(ops, name + "Backward")(x, g).toHost(), gold["act_" + name + "_bwd"])


def test_zero_fused(hip, rng):
    D, ops = hip.DeviceTensor, hip.ops
    tensors = [D.fromHost(r(rng, n)) for n in (1, 5, 8192, 8193, 100000)]
    guard = D.fromHost(np.ones(16, f32))
    ops.zeroFused(tensors)
    for t in tensors:
        assert not t.toHost().any()
    assert (guard.toHost() == 1).all()
    ops.zeroFused(tensors)  # unchanged descriptor table: cached path


def test_pool_reuses_blocks(hip):
    D = hip.DeviceTensor
    stats = hip.capi.PoolStats()
    a = D((1000,))
    p = a.ptr.value
    del a
    b = D((1001,))  # same size class
    assert b.ptr.value == p
    hip.capi.call("bf_hip_pool_stats", ctypes.byref(stats))
    assert stats.driver_allocations >= 1 and stats.acquires >= 2
