"""Pins the oracle against what the mathematics fixes, independent of any reference run.

float64 numpy restatements of the textbook formulas (masked softmax(QK^T*scale)V, tanh-GELU, SiLU,
RMSNorm, softmax-CE, AdamW), closed-form special cases and central-difference gradient checks.  A
dropped term, a wrong sign, a transposed operand or an off-by-one in the causal mask fails here.
"""
import numpy as np
import pytest

from oracle import bfo

f64 = np.float64
f32 = np.float32


def sdpa64(q, k, v, heads, scale, old_len):
    """Textbook causal attention in float64: query i sees keys j <= old_len + i."""
    b, nl, dim = q.shape
    tot, hd = k.shape[1], dim // heads
    qh = q.astype(f64).reshape(b, nl, heads, hd).transpose(0, 2, 1, 3)
    kh = k.astype(f64).reshape(b, tot, heads, hd).transpose(0, 2, 1, 3)
    vh = v.astype(f64).reshape(b, tot, heads, hd).transpose(0, 2, 1, 3)
    s = np.einsum("bhid,bhjd->bhij", qh, kh) * scale
    mask = np.arange(tot)[None, :] > (old_len + np.arange(nl))[:, None]
    s = np.where(mask, -np.inf, s)
    m = s.max(-1, keepdims=True)
    p = np.exp(s - m)
    l = p.sum(-1, keepdims=True)
    p = p / l
    o = np.einsum("bhij,bhjd->bhid", p, vh).transpose(0, 2, 1, 3).reshape(b, nl, dim)
    return o, m[..., 0], l[..., 0], p, (qh, kh, vh)


def sdpa64_backward(go, q, k, v, heads, scale, old_len):
    b, nl, dim = q.shape
    tot, hd = k.shape[1], dim // heads
    _, _, _, p, (qh, kh, vh) = sdpa64(q, k, v, heads, scale, old_len)
    goh = go.astype(f64).reshape(b, nl, heads, hd).transpose(0, 2, 1, 3)
    dv = np.einsum("bhij,bhid->bhjd", p, goh)
    dp = np.einsum("bhid,bhjd->bhij", goh, vh)
    ds = p * (dp - (dp * p).sum(-1, keepdims=True)) * scale
    dq = np.einsum("bhij,bhjd->bhid", ds, kh)
    dk = np.einsum("bhij,bhid->bhjd", ds, qh)
    back = lambda t, n: t.transpose(0, 2, 1, 3).reshape(b, n, dim)
    return back(dq, nl), back(dk, tot), back(dv, tot), ds


def r(rng, *s, scale=1.0):
    return (rng.standard_normal(s) * scale).astype(f32)


@pytest.mark.parametrize("b,h,nl,ol,hd", [(1, 1, 1, 0, 4), (2, 3, 19, 0, 8), (1, 2, 7, 11, 16), (1, 1, 64, 0, 32)])
def test_attention_core_is_textbook_sdpa(oracle, rng, b, h, nl, ol, hd):
    dim, tot = h * hd, nl + ol
    q, k, v, go = r(rng, b, nl, dim), r(rng, b, tot, dim), r(rng, b, tot, dim), r(rng, b, nl, dim)
    scale = 1.0 / np.sqrt(hd)
    o, m, l = oracle.attentionCoreForward(q, k, v, h, scale, ol)
    o64, m64, l64, _, _ = sdpa64(q, k, v, h, scale, ol)
    np.testing.assert_allclose(o, o64, rtol=0, atol=2e-6 * np.abs(o64).max() + 1e-6)
    np.testing.assert_allclose(m, m64, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(l, l64, rtol=1e-6)
    dq, dk, dv = oracle.attentionCoreBackward(go, q, k, v, h, scale, ol)
    dq64, dk64, dv64, ds = sdpa64_backward(go, q, k, v, h, scale, ol)
    for a, e in ((dq, dq64), (dk, dk64), (dv, dv64)):
        np.testing.assert_allclose(a, e, rtol=0, atol=1e-5 * np.abs(e).max() + 1e-6)
    assert np.abs(ds.sum(-1)).max() < 1e-12  # rows of dS sum to zero


def test_attention_special_cases(oracle, rng):
    # one position: O = V
    q, k, v = r(rng, 2, 1, 8), r(rng, 2, 1, 8), r(rng, 2, 1, 8)
    o, m, l = oracle.attentionCoreForward(q, k, v, 2, 0.5)
    np.testing.assert_allclose(o, v, rtol=1e-6)
    np.testing.assert_allclose(l, 1.0)
    # identical keys: uniform weights, so O is the running mean of V
    k1 = np.repeat(r(rng, 1, 1, 4), 6, axis=1)
    q, v = r(rng, 1, 6, 4), r(rng, 1, 6, 4)
    o, _, l = oracle.attentionCoreForward(q, k1, v, 1, 0.7)
    running = np.cumsum(v.astype(f64), axis=1) / np.arange(1, 7)[None, :, None]
    np.testing.assert_allclose(o, running, atol=1e-6)
    np.testing.assert_allclose(l[0, 0], np.arange(1, 7), rtol=1e-6)
    # causal: changing a future key/value leaves earlier rows untouched, bit for bit
    q, k, v = r(rng, 1, 5, 4), r(rng, 1, 5, 4), r(rng, 1, 5, 4)
    o1, _, _ = oracle.attentionCoreForward(q, k, v, 1, 0.5)
    k[0, 4], v[0, 4] = 50.0, -7.0
    o2, _, _ = oracle.attentionCoreForward(q, k, v, 1, 0.5)
    np.testing.assert_array_equal(o1[0, :4], o2[0, :4])
    assert np.abs(o1[0, 4] - o2[0, 4]).max() > 1e-3


def central_difference(fn, x, eps=1e-3):
    g = np.zeros(x.size, f64)
    flat = x.reshape(-1)
    for i in range(x.size):
        old = flat[i]
        flat[i] = old + eps
        hi = fn()
        flat[i] = old - eps
        lo = fn()
        flat[i] = old
        g[i] = (hi - lo) / (2 * eps)
    return g.reshape(x.shape)


def test_block_gradients_by_central_differences(oracle, rng):
    """Same procedure as the reference's autodiff tests (eps 1e-3, tol 1e-2 / 3e-2 for attention)."""
    x, g = r(rng, 1, 3, 4, scale=.5), r(rng, 1, 3, 4)
    w = [r(rng, 4, 4, scale=.3) for _ in range(4)]
    grads = oracle.selfAttentionBackward(x, *w, 2, g)
    loss = lambda: float((oracle.selfAttention(x, *w, 2).astype(f64) * g).sum())
    for t, a in zip([x] + w, grads):
        np.testing.assert_allclose(a, central_difference(loss, t), atol=3e-2)
    for act in (0, 1):
        p = [r(rng, 4, 6, scale=.3), r(rng, 6, scale=.1), r(rng, 6, 4, scale=.3), r(rng, 4, scale=.1)]
        grads = oracle.feedForwardBackward(x, *p, g, act)
        loss = lambda: float((oracle.feedForward(x, *p, act).astype(f64) * g).sum())
        for t, a in zip([x] + p, grads):
            np.testing.assert_allclose(a, central_difference(loss, t), atol=1e-2)


def test_elementwise_closed_forms(oracle, rng):
    x = r(rng, 500, scale=3)
    x64 = x.astype(f64)
    sig = 1 / (1 + np.exp(-x64))
    np.testing.assert_allclose(oracle.silu(x), x64 * sig, rtol=2e-6, atol=1e-7)
    inner = np.sqrt(2 / np.pi) * (x64 + 0.044715 * x64 ** 3)
    np.testing.assert_allclose(oracle.gelu(x), 0.5 * x64 * (1 + np.tanh(inner)), rtol=1e-5, atol=1e-6)
    g = r(rng, 500)
    np.testing.assert_allclose(oracle.siluBackward(x, g), g * sig * (1 + x64 * (1 - sig)), rtol=1e-5, atol=1e-6)
    dinner = np.sqrt(2 / np.pi) * (1 + 3 * 0.044715 * x64 ** 2)
    dgelu = 0.5 * (1 + np.tanh(inner)) + 0.5 * x64 * (1 - np.tanh(inner) ** 2) * dinner
    np.testing.assert_allclose(oracle.geluBackward(x, g), g * dgelu, rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(oracle.reluBackward(x, g), np.where(x > 0, g, 0))


def test_rows_closed_forms(oracle, rng):
    x, g = r(rng, 5, 40, scale=2), r(rng, 5, 40)
    x64, g64 = x.astype(f64), g.astype(f64)
    rr = np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6)
    np.testing.assert_allclose(oracle.rmsnorm(x), x64 / rr, rtol=1e-6)
    dx = g64 / rr - x64 * (g64 * x64).sum(-1, keepdims=True) / (40 * rr ** 3)
    np.testing.assert_allclose(oracle.rmsnormBackward(x, g), dx, rtol=1e-5, atol=1e-6)
    e = np.exp(x64 - x64.max(-1, keepdims=True))
    y = e / e.sum(-1, keepdims=True)
    np.testing.assert_allclose(oracle.softmax(x), y, rtol=1e-6)
    np.testing.assert_allclose(oracle.softmaxBackward(x, g), y * (g64 - (g64 * y).sum(-1, keepdims=True)), rtol=1e-5, atol=1e-7)
    idx = rng.integers(0, 40, 5)
    v, gr = oracle.softmaxCrossEntropySparse(x, idx.astype(f32))
    assert abs(v - (-np.log(y[np.arange(5), idx]).mean())) < 1e-6
    onehot = np.eye(40)[idx]
    np.testing.assert_allclose(gr, (y - onehot) / 5, rtol=1e-5, atol=1e-8)


def test_matmul_family_against_float64(oracle, rng):
    a, b, g = r(rng, 9, 31), r(rng, 31, 13), r(rng, 9, 13)
    np.testing.assert_allclose(oracle.matmul(a, b), a.astype(f64) @ b, rtol=1e-5, atol=1e-5)
    da, db = oracle.matmulBackward(a, b, g)
    np.testing.assert_allclose(da, g.astype(f64) @ b.T, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(db, a.T.astype(f64) @ g, rtol=1e-5, atol=1e-5)
    bt = np.ascontiguousarray(b.T)
    np.testing.assert_allclose(oracle.matmulTransposeB(a, bt), a.astype(f64) @ b, rtol=1e-5, atol=1e-5)
    da, dbt = oracle.matmulTransposeBBackward(a, bt, g)
    np.testing.assert_allclose(da, g.astype(f64) @ bt, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dbt, g.T.astype(f64) @ a, rtol=1e-5, atol=1e-5)


def test_adamw_many_steps_against_float64(oracle, rng):
    p, m, v = r(rng, 64), np.zeros(64, f32), np.zeros(64, f32)
    p64, m64, v64 = p.astype(f64), np.zeros(64), np.zeros(64)
    lr, b1, b2, eps, wd = 1e-2, 0.9, 0.999, 1e-8, 0.01
    for t in range(1, 21):
        g = r(rng, 64)
        p, m, v = oracle.adamwStep(p, g, m, v, t, lr, b1, b2, eps, wd)
        m64 = b1 * m64 + (1 - b1) * g
        v64 = b2 * v64 + (1 - b2) * g.astype(f64) ** 2
        p64 = p64 - lr * ((m64 / (1 - b1 ** t)) / (np.sqrt(v64 / (1 - b2 ** t)) + eps) + wd * p64)
    np.testing.assert_allclose(p, p64, rtol=2e-5, atol=1e-6)


def test_bf16_rounding_is_nearest_even(oracle):
    # 1 + 2^-8 is exactly halfway between bf16 neighbours 1 and 1+2^-7: ties go to even (1.0);
    # 1 + 3*2^-8 is halfway between 1+2^-7 (odd) and 1+2^-6 (even): goes up.
    x = np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, 1 + 2.0 ** -8 + 2.0 ** -20, -(1 + 2.0 ** -8)], f32)
    np.testing.assert_array_equal(oracle.roundToBf16(x), np.array([1.0, 1 + 2.0 ** -6, 1 + 2.0 ** -7, -1.0], f32))


def test_masked_cross_entropy_reduces_to_the_sparse_loss_on_the_kept_rows(oracle, rng):
    """The cases of tests/backend/cpu/loss_tests.cpp:142-196 and their general form: with no -1 the masked loss IS the sparse
    loss; otherwise it is the sparse loss of the kept rows alone, ignored rows get a zero gradient, and with every row
    ignored loss and gradient are zero."""
    f32 = np.float32
    logits = np.array([[0.5, -1.2, 0.3], [2.0, 0.1, -0.5]], f32)
    v, g = oracle.softmaxCrossEntropyMasked(logits, np.array([1, 0], f32))
    sv, sg = oracle.softmaxCrossEntropySparse(logits, np.array([1, 0], f32))
    assert abs(v - sv) <= 1e-6 and np.abs(g - sg).max() <= 1e-6
    logits = np.array([[1, 2, 3], [0.5, -1.0, 0.2], [-0.3, 0.1, 0.4]], f32)
    v, g = oracle.softmaxCrossEntropyMasked(logits, np.array([-1, 2, -1], f32))
    sv, sg = oracle.softmaxCrossEntropySparse(logits[1:2], np.array([2], f32))
    assert not g[0].any() and not g[2].any()
    assert abs(v - sv) <= 1e-5 and np.abs(g[1] - sg[0]).max() <= 1e-6
    v, g = oracle.softmaxCrossEntropyMasked(logits[:2], np.array([-1, -1], f32))
    assert v == 0.0 and not g.any()
    with pytest.raises(Exception):
        oracle.softmaxCrossEntropyMasked(np.array([[0.1, 0.2, 0.3]], f32), np.array([7], f32))
    # general form on random data, against float64
    rows, classes = 50, 11
    x = rng.standard_normal((rows, classes)).astype(f32) * 2
    idx = np.where(rng.random(rows) < 0.3, rng.integers(0, classes, rows), -1)
    v, g = oracle.softmaxCrossEntropyMasked(x, idx.astype(f32))
    keep = idx >= 0
    z = x.astype(np.float64) - x.max(-1, keepdims=True)
    p = np.exp(z) / np.exp(z).sum(-1, keepdims=True)
    onehot = np.zeros_like(p)
    onehot[keep, idx[keep]] = 1
    expect = np.where(keep[:, None], (p - onehot) / keep.sum(), 0.0)
    assert abs(v - (-np.log(p[keep, idx[keep]])).mean()) <= 1e-6
    assert np.abs(g - expect).max() <= 1e-7


def test_bidirectional_attention_sees_later_positions(oracle):
    """tests/backend/cpu/ops_tests.cpp:359-391: changing token 2 changes the outputs at positions 0 and 1, which it must
    not do under the causal mask."""
    f32 = np.float32
    wq = np.array([0.3, -0.1, 0.2, 0.05, 0.1, 0.4, -0.2, 0.15, -0.3, 0.2, 0.1, -0.05, 0.2, -0.1, 0.3, 0.1], f32).reshape(4, 4)
    wk = np.array([0.1, 0.2, -0.1, 0.3, -0.2, 0.1, 0.4, -0.1, 0.3, -0.3, 0.1, 0.2, -0.1, 0.2, -0.2, 0.1], f32).reshape(4, 4)
    wv = np.array([0.2, 0.1, -0.1, 0.3, 0.1, -0.2, 0.3, 0.1, -0.1, 0.3, 0.2, -0.1, 0.3, 0.1, -0.2, 0.2], f32).reshape(4, 4)
    wo = np.array([0.1, -0.1, 0.2, 0.1, 0.2, 0.1, -0.1, 0.2, -0.1, 0.2, 0.1, -0.1, 0.1, 0.2, -0.1, 0.2], f32).reshape(4, 4)
    a = np.array([0.1, -0.2, 0.3, 0.4, -0.5, 0.6, 0.2, -0.1, 0.3, 0.2, -0.4, 0.5], f32).reshape(1, 3, 4)
    b = a.copy()
    b[0, 2, 0] = 99.0
    ya, yb = (oracle.selfAttention(x, wq, wk, wv, wo, 2, causal=False) for x in (a, b))
    assert np.abs(ya[0, :2] - yb[0, :2]).max() > 1e-4
    ca, cb = (oracle.selfAttention(x, wq, wk, wv, wo, 2, causal=True) for x in (a, b))
    assert np.abs(ca[0, :2] - cb[0, :2]).max() == 0.0


def test_textbook_attention_slice_helper_agrees_with_the_oracle(oracle, rng):
    """tests/textbook.attention_slice is the float64 reference of the GPU tests at sizes the C oracle is too slow for;
    here it is held against the oracle (itself pinned above and against the reference build) on a small slice."""
    from textbook import attention_slice
    for nl, ol, hd in ((37, 0, 16), (20, 9, 128)):
        q, k, v, go = r(rng, 1, nl, hd), r(rng, 1, nl + ol, hd), r(rng, 1, nl + ol, hd), r(rng, 1, nl, hd)
        scale = 1.0 / np.sqrt(hd)
        o, m, l = oracle.attentionCoreForward(q, k, v, 1, scale, ol)
        dq, dk, dv = oracle.attentionCoreBackward(go, q, k, v, 1, scale, ol)
        got = attention_slice(q[0], k[0], v[0], go[0], scale, ol)
        for a, e in zip(got, (o[0], m[0, 0], l[0, 0], dq[0], dk[0], dv[0])):
            np.testing.assert_allclose(a, e, rtol=0, atol=1e-5 * np.abs(e).max() + 1e-6)
