"""GPU parity of the kernel variants that stream past the last-level cache.

A launch that moves more than 256 MB uses loads and stores with the non-temporal hint; smaller launches (every other
test) use the plain accesses.  These cases are just large enough to take the streaming variants of every
bandwidth-bound kernel, and are checked against the oracle like their small counterparts (bit-exact where the op is)."""
import ctypes

import numpy as np
import pytest

from parity import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu
f32 = np.float32
N = 41_000_000   # 164 MB per fp32 tensor: every op below moves more than 256 MB


def r(rng, *s, scale=1.0):
    return rng.standard_normal(s, dtype=f32) * f32(scale)


def test_flat_ops_streaming(hip, oracle):
    rng = np.random.default_rng(1)
    D, ops = hip.DeviceTensor, hip.ops
    x, g = r(rng, N, scale=3), r(rng, N)
    dx, dg = D.fromHost(x), D.fromHost(g)
    assert_bits_equal(ops.add(dx, dg).toHost(), oracle.add(x, g), "add")
    assert_bits_equal(ops.scale(dx, 0.37).toHost(), oracle.scale(x, 0.37), "scale")
    assert_bits_equal(ops.relu(dx).toHost(), oracle.relu(x), "relu")
    for name in ("silu", "gelu"):
        assert_close(getattr(ops, name)(dx).toHost(), getattr(oracle, name)(x), what=name)
        assert_close(getattr(ops, name + "Backward")(dx, dg).toHost(), getattr(oracle, name + "Backward")(x, g), what=name + "Backward")
    t = D.fromHost(x)
    ops.accumulate(t, dg)
    assert_bits_equal(t.toHost(), x + g, "accumulate")
    # mean squared error: 12 bytes per element
    res = ops.meanSquaredError(dx, dg)
    ev, eg = oracle.meanSquaredError(x, g)
    assert abs(res.value - ev) <= 1e-4 * ev
    assert_close(res.grad.toHost(), eg, what="mse grad")
    # fp32 -> bf16 image: 6 bytes per element; 45M elements
    big = r(rng, 45_000_000 - N)
    both = np.concatenate([x, big])
    out = D((both.size,), itemsize=2)
    hip.capi.call("bf_hip_cvt_f32_bf16", D.fromHost(both).ptr, out.ptr, both.size, None)
    assert_bits_equal((out.toHost().astype(np.uint32) << 16).view(f32), oracle.roundToBf16(both), "bf16 image")


def test_bias_family_streaming(hip, oracle):
    rng = np.random.default_rng(2)
    D, ops, capi = hip.DeviceTensor, hip.ops, hip.capi
    rows, features = 10000, 4100
    x, res, dh, bias = r(rng, rows, features), r(rng, rows, features), r(rng, rows, features), r(rng, features)
    dx, db, dres, ddh = D.fromHost(x), D.fromHost(bias), D.fromHost(res), D.fromHost(dh)
    pre = oracle.addBias(x, bias)
    assert_bits_equal(ops.addBias(dx, db).toHost(), pre, "addBias")
    assert_bits_equal(ops.addBiasResidual(dx, db, dres).toHost(), oracle.add(pre, res), "addBiasResidual")
    assert_close(ops.addBiasAct(dx, db, capi.ACT_GELU).toHost(), oracle.gelu(pre), what="addBias+gelu")
    dgemm, dbias = ops.addBiasActBackward(dx, db, ddh, capi.ACT_SILU)
    exp = oracle.siluBackward(pre, dh)
    assert_close(dgemm.toHost(), exp, what="addBiasActBackward.dGemm")
    assert_close(dbias.toHost(), exp.astype(np.float64).sum(0).astype(f32), what="addBiasActBackward.dBias", scale=float(np.sqrt(rows)))
    # plain column sums read 4 bytes per element: a taller matrix
    tall = r(rng, 16400, features)
    assert_close(ops.biasGradientOnly(D.fromHost(tall)).toHost(), tall.astype(np.float64).sum(0).astype(f32), what="biasGradientOnly",
                 scale=float(np.sqrt(16400)))


def test_row_ops_streaming(hip, oracle):
    rng = np.random.default_rng(3)
    D, ops = hip.DeviceTensor, hip.ops
    rows, features = 20000, 2052
    x, g, res = r(rng, rows, features, scale=2), r(rng, rows, features), r(rng, rows, features)
    dx, dg = D.fromHost(x), D.fromHost(g)
    assert_close(ops.rmsnorm(dx).toHost(), oracle.rmsnorm(x), what="rmsnorm")
    bwd = ops.rmsnormBackward(dx, dg).toHost()
    assert_close(bwd, oracle.rmsnormBackward(x, g), what="rmsnormBackward")
    assert_bits_equal(ops.rmsnormBackwardAdd(dx, dg, D.fromHost(res)).toHost(), res + bwd, "rmsnormBackwardAdd")
    assert_close(ops.softmax(dx).toHost(), oracle.softmax(x), what="softmax")
    assert_close(ops.softmaxBackward(dx, dg).toHost(), oracle.softmaxBackward(x, g), what="softmaxBackward")


@pytest.mark.parametrize("rows,classes", [(1300, 32000), (830, 50257)])
def test_cross_entropy_streaming(hip, oracle, rows, classes):
    """Aligned rows (32000) and rows of odd length reached through shifted 16-byte accesses (50257)."""
    rng = np.random.default_rng(rows)
    D, ops = hip.DeviceTensor, hip.ops
    logits = r(rng, rows, classes, scale=3)
    idx = rng.integers(0, classes, rows).astype(f32)
    res = ops.softmaxCrossEntropySparse(D.fromHost(logits), D.fromHost(idx))
    ev, eg = oracle.softmaxCrossEntropySparse(logits, idx)
    assert abs(res.value - ev) <= 1e-4 * abs(ev)
    assert_close(res.grad.toHost(), eg, what="sparse CE grad")
    masked = np.where(rng.random(rows) < 0.5, idx, -1).astype(f32)
    res = ops.softmaxCrossEntropyMasked(D.fromHost(logits), D.fromHost(masked))
    ev, eg = oracle.softmaxCrossEntropyMasked(logits, masked)
    assert abs(res.value - ev) <= 1e-4 * abs(ev)
    assert_close(res.grad.toHost(), eg, what="masked CE grad")


def test_optimizers_and_zero_streaming(hip, oracle):
    rng = np.random.default_rng(4)
    D, ops = hip.DeviceTensor, hip.ops
    sizes = [5, 70_000_001, 8195, 3_000_000]   # 73M parameters: 292 MB for zero, 0.9 GB for SGD, 2 GB for AdamW
    host_p = [r(rng, n) for n in sizes]
    grads = [r(rng, n) for n in sizes]
    params = [ops.Parameter(f"t{i}", D.fromHost(a), D.fromHost(g)) for i, (a, g) in enumerate(zip(host_p, grads))]
    opt = ops.AdamW(1e-2)
    m = [np.zeros(n, f32) for n in sizes]
    v = [np.zeros(n, f32) for n in sizes]
    for step in (1, 2):
        opt.step(params)
        for i, g in enumerate(grads):
            host_p[i], m[i], v[i] = oracle.adamwStep(host_p[i], g, m[i], v[i], step, 1e-2)
    for prm, e in zip(params, host_p):
        assert_close(prm.value.toHost(), e, what="AdamW after 2 steps")
    ops.SGD(0.05).step(params)
    for prm, e, g in zip(params, host_p, grads):
        assert_bits_equal(prm.value.toHost(), oracle.sgdStep(e, g, 0.05), "SGD")
    guard = D.fromHost(np.ones(16, f32))
    ops.zeroFused([p.grad for p in params])
    for p in params:
        assert not p.grad.toHost().any()
    assert (guard.toHost() == 1).all()
