"""Pins the CPU oracle against the known-answer vectors held in the reference's own tests.

Every case cites the reference test whose literals it reuses.  The same cases also run against
oracle/_ref (the real reference build) where present, which checks the C wrapper around it.
"""
import math

import numpy as np
import pytest

import refvectors as rv

f32 = np.float32


@pytest.fixture(params=["oracle", "ref"])
def impl(request):
    return request.getfixturevalue(request.param)


def arr(*v, shape=None):
    a = np.array(v, f32)
    return a.reshape(shape) if shape else a


# tests/backend/cpu/ops_tests.cpp:10-23
def test_add(impl):
    np.testing.assert_array_equal(impl.add(arr(1, 2), arr(10, 20)), arr(11, 22))
    with pytest.raises(ValueError):
        impl.add(arr(1, 2), arr(1, 2, 3))


# ops_tests.cpp:25-34
def test_add_bias_broadcasts_rows(impl):
    out = impl.addBias(arr(1, 2, 3, 4, shape=(2, 2)), arr(10, 20))
    np.testing.assert_array_equal(out.ravel(), arr(11, 22, 13, 24))


# ops_tests.cpp:36-52
def test_matmul_2x2(impl):
    out = impl.matmul(arr(1, 2, 3, 4, shape=(2, 2)), arr(5, 6, 7, 8, shape=(2, 2)))
    np.testing.assert_array_equal(out.ravel(), arr(19, 22, 43, 50))
    with pytest.raises(ValueError):
        impl.matmul(np.ones((2, 3), f32), np.ones((2, 2), f32))


# ops_tests.cpp:54-63
def test_linear_identity(impl):
    out = impl.linear(arr(3, 4, shape=(1, 2)), arr(1, 0, 0, 1, shape=(2, 2)), arr(10, 20))
    np.testing.assert_array_equal(out.ravel(), arr(13, 24))


# ops_tests.cpp:173-184
def test_linear_rank3(impl):
    x = arr(1, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6, 6, shape=(2, 3, 2))
    out = impl.linear(x, arr(1, 1, shape=(2, 1)), arr(0))
    assert out.shape == (2, 3, 1)
    np.testing.assert_array_equal(out.ravel(), x[..., 0].ravel() + x[..., 1].ravel())


# ops_tests.cpp:65-90
def test_activations_literals(impl):
    np.testing.assert_array_equal(impl.relu(arr(-2, 0, 3)), arr(0, 0, 3))
    s = impl.silu(arr(0, 20, -20))
    assert s[0] == 0 and abs(s[1] - 20) < 0.01 and abs(s[2]) < 0.01
    g = impl.gelu(arr(0, 20, -20))
    assert g[0] == 0 and abs(g[1] - 20) < 0.01 and abs(g[2]) < 0.01


# ops_tests.cpp:92-124
def test_rmsnorm_unit_rms_and_ratio(impl):
    out = impl.rmsnorm(arr(1, 2, 3, 4, -1, -1, -1, -1, shape=(2, 4)))
    rms = np.sqrt((out.astype(np.float64) ** 2).mean(axis=1))
    np.testing.assert_allclose(rms, 1.0, atol=1e-3)
    out = impl.rmsnorm(arr(2, -4, shape=(1, 2)))
    assert out[0, 0] > 0 > out[0, 1] and abs(out[0, 1] / out[0, 0] + 2) < 1e-4
    with pytest.raises(ValueError):
        impl.rmsnorm(arr(1, 2, 3, 4))


# ops_tests.cpp:126-170
def test_softmax_literals(impl):
    out = impl.softmax(arr(1, 2, 3, -1, 0, 1, shape=(2, 3)))
    np.testing.assert_allclose(out.sum(axis=1), 1.0, atol=1e-5)
    assert (impl.softmax(arr(-10, 0, 5, 3, shape=(1, 4))) > 0).all()
    np.testing.assert_allclose(impl.softmax(arr(2, 2, 2, 2, shape=(1, 4))), 0.25, atol=1e-5)
    np.testing.assert_allclose(impl.softmax(arr(1000, 1000, 1000, shape=(1, 3))), 1 / 3, atol=1e-4)
    with pytest.raises(ValueError):
        impl.softmax(arr(1, 2, 3, 4))


# ops_tests.cpp:201-236
def test_matmul_transpose_b(impl):
    out = impl.matmulTransposeB(arr(1, 2, 3, 4, 5, 6, shape=(2, 3)), arr(1, 0, 0, 0, 1, 0, shape=(2, 3)))
    np.testing.assert_array_equal(out.ravel(), arr(1, 2, 4, 5))
    a = arr(0.5, -1.0, 2.0, 0.3, -0.7, 1.2, shape=(3, 2))
    b = arr(1.0, 2.0, -1.0, 0.5, 0.3, -0.2, 2.0, 1.0, shape=(4, 2))
    np.testing.assert_allclose(impl.matmulTransposeB(a, b), impl.matmul(a, np.ascontiguousarray(b.T)), atol=1e-5)


# ops_tests.cpp:238-262
def test_embedding_lookup(impl):
    table = arr(10, 11, 20, 21, 30, 31, shape=(3, 2))
    out = impl.embeddingLookup(arr(0, 2, 1, shape=(1, 3)), table)
    np.testing.assert_array_equal(out.ravel(), arr(10, 11, 30, 31, 20, 21))
    for bad in (3.0, -1.0):
        with pytest.raises(ValueError):
            impl.embeddingLookup(arr(bad, shape=(1, 1)), table)


# ops_tests.cpp:264-286, 435-461
def test_positional_embedding(impl):
    x = arr(0, 0, 0, 0, 100, 100, 100, 100, shape=(2, 2, 2))
    out = impl.addPositionalEmbedding(x, arr(1, 2, 3, 4, shape=(2, 2)))
    np.testing.assert_array_equal(out.ravel()[:6], arr(1, 2, 3, 4, 101, 102))
    with pytest.raises(ValueError):
        impl.addPositionalEmbedding(np.zeros((1, 3, 2), f32), arr(1, 2, 3, 4, shape=(2, 2)))
    table = arr(1, 2, 3, 4, 5, 6, 7, 8, shape=(4, 2))
    x = arr(0.1, -0.2, 0.3, 0.4, shape=(1, 2, 2))
    np.testing.assert_array_equal(impl.addPositionalEmbeddingAt(x, table, 0), impl.addPositionalEmbedding(x, table))
    np.testing.assert_array_equal(impl.addPositionalEmbeddingAt(np.zeros((1, 1, 2), f32), table, 2).ravel(), arr(5, 6))
    with pytest.raises(ValueError):
        impl.addPositionalEmbeddingAt(np.zeros((1, 2, 2), f32), arr(1, 2, 3, 4, 5, 6, shape=(3, 2)), 2)


# ops_tests.cpp:290-322
def test_zero_weights_give_residual_identity(impl):
    x = arr(0.1, -0.2, 0.3, 0.4, -0.5, 0.6, shape=(1, 2, 3))
    out = impl.feedForward(x, np.zeros((3, 4), f32), np.zeros(4, f32), np.zeros((4, 3), f32), np.zeros(3, f32))
    np.testing.assert_array_equal(out, x)
    z = np.zeros((4, 4), f32)
    np.testing.assert_array_equal(impl.selfAttention(rv.ATTN_INPUT, z, z, z, z, 2), rv.ATTN_INPUT)


# ops_tests.cpp:324-351 and :359-391
def test_causal_mask_independence_from_future(impl):
    a = rv.ATTN_INPUT
    b = a.copy()
    b[0, 2, 0] = 99.0
    w = (rv.ATTN_WQ, rv.ATTN_WK, rv.ATTN_WV, rv.ATTN_WOUT)
    ra, rb = impl.selfAttention(a, *w, 2), impl.selfAttention(b, *w, 2)
    np.testing.assert_array_equal(ra.ravel()[:8], rb.ravel()[:8])
    na, nb = impl.selfAttention(a, *w, 2, causal=False), impl.selfAttention(b, *w, 2, causal=False)
    assert np.abs(na.ravel()[:8] - nb.ravel()[:8]).max() > 1e-4
    with pytest.raises(ValueError):
        impl.selfAttention(np.zeros((1, 2, 3), f32), *(np.zeros((3, 3), f32),) * 4, 2)


# ops_tests.cpp:393-425
def test_incremental_attention_matches_full(impl):
    w = (rv.ATTN_WQ, rv.ATTN_WK, rv.ATTN_WV, rv.ATTN_WOUT)
    full = impl.selfAttention(rv.ATTN_INPUT, *w, 2)
    kc = vc = None
    for s in range(3):
        out, kc, vc = impl.selfAttentionIncremental(rv.ATTN_INPUT[:, s:s + 1, :], *w, 2, kc, vc)
        np.testing.assert_allclose(out[0, 0], full[0, s], atol=1e-4)
    assert kc.shape[1] == 3


# tests/backend/cpu/autodiff_tests.cpp:180-199
def test_embedding_backward_accumulates_repeated_ids(impl):
    dt = impl.embeddingLookupBackward(arr(0, 1, 0, shape=(1, 3)), arr(1, 2, 10, 20, 3, 4, shape=(1, 3, 2)), 3)
    np.testing.assert_array_equal(dt.ravel(), arr(4, 6, 10, 20, 0, 0))


# tests/backend/cpu/loss_tests.cpp:10-29
def test_mse(impl):
    v, _ = impl.meanSquaredError(arr(1, 2), arr(0, 0))
    assert v == f32(2.5)
    p = arr(0.1, -0.2, 0.3)
    assert impl.meanSquaredError(p, p)[0] == 0.0
    with pytest.raises(ValueError):
        impl.meanSquaredError(arr(1, 2), arr(1, 2, 3))


# loss_tests.cpp:51-76
def test_cross_entropy_uniform(impl):
    v, g = impl.softmaxCrossEntropy(arr(0, 0, shape=(1, 2)), arr(1, 0, shape=(1, 2)))
    assert abs(v - math.log(2)) < 1e-5
    np.testing.assert_allclose(g.ravel(), [-0.5, 0.5], atol=1e-5)
    v, _ = impl.softmaxCrossEntropy(arr(20, -20, shape=(1, 2)), arr(1, 0, shape=(1, 2)))
    assert abs(v) < 1e-4


# loss_tests.cpp:115-140
def test_sparse_ce_equals_dense(impl):
    logits = arr(0.5, -1.2, 0.3, 2.0, 0.1, -0.5, shape=(2, 3))
    dv, dg = impl.softmaxCrossEntropy(logits, arr(0, 1, 0, 1, 0, 0, shape=(2, 3)))
    sv, sg = impl.softmaxCrossEntropySparse(logits, arr(1, 0))
    assert abs(dv - sv) < 1e-6
    np.testing.assert_allclose(sg, dg, atol=1e-6)
    with pytest.raises(ValueError):
        impl.softmaxCrossEntropySparse(arr(0.1, 0.2, 0.3, shape=(1, 3)), arr(5))
    with pytest.raises(ValueError):
        impl.softmaxCrossEntropySparse(arr(0.1, 0.2, 0.3, 0.4, 0.5, 0.6, shape=(2, 3)), arr(0, 1, 2))


# tests/backend/cpu/optimizer_tests.cpp:10-59
def test_sgd_and_adamw_first_step(impl):
    p = impl.sgdStep(arr(1, -2), arr(0.5, 0.5), 0.1)
    np.testing.assert_array_equal(p, arr(1, -2) - f32(0.1) * f32(0.5))
    p, _, _ = impl.adamwStep(arr(1), arr(0.2), arr(0), arr(0), 1, lr=0.1, wd=0.0)
    expected = 1.0 - 0.1 * (0.2 / (math.sqrt(0.04) + 1e-8))
    assert abs(p[0] - expected) < 1e-5
    # decoupled weight decay acts at zero gradient: 1 - 0.1*0.1*1
    p, _, _ = impl.adamwStep(arr(1), arr(0), arr(0), arr(0), 1, lr=0.1, wd=0.1)
    assert p[0] == f32(1.0) - f32(0.1) * f32(0.1) * f32(1.0)


# tests/backend/cpu/quantize_tests.cpp:35-59
def test_round_to_bf16(impl):
    x = arr(1 / 3, 12345.6789, np.inf, -np.inf, np.nan, 1.0, 0.0)
    q = impl.roundToBf16(x)
    assert q[0] != x[0] and abs(q[0] - x[0]) < 0.01
    np.testing.assert_array_equal(impl.roundToBf16(q), q)  # idempotent
    assert q[2] == np.inf and q[3] == -np.inf and np.isnan(q[4]) and q[5] == 1.0 and q[6] == 0.0
    # low 16 bits cleared
    assert (q[np.isfinite(q)].view(np.uint32) & 0xFFFF).max() == 0


# src/main.cpp:504-518: strict '>' keeps the first maximum
def test_argmax_first_max_wins(impl):
    logits = arr(0, 5, 1, 9, 9, 2, 9, 3, shape=(2, 4))
    assert impl.argmaxLastPosition(logits) == 0
    logits[1] = [1, 7, 7, 3]
    assert impl.argmaxLastPosition(logits) == 1
