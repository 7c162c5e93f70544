"""Seeded random shapes through the C ABI against float64 numpy: the products, the attention core, the row kernels and
the embedding scatter at sizes no hand-picked case names (odd extents, single rows, contractions just past a tile edge,
one id repeated thousands of times).  Every case prints its shape before it runs, so a failure names it."""
import numpy as np
import pytest

from parity import assert_close
from textbook import attention_slice

pytestmark = pytest.mark.gpu
f32 = np.float32


def _rnd(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(f32)


def _bf16(x):
    """Round to nearest even to bf16, returned as float32 (quantize.cpp:16-31 of the reference)."""
    u = np.ascontiguousarray(x, f32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32).view(f32).reshape(x.shape)


def _extent(rng):
    r = rng.random()
    if r < 0.3:
        return int(rng.integers(1, 130))
    if r < 0.7:
        return int(rng.integers(100, 700))
    return int(rng.choice([256, 512, 768, 1024, 1536, 2048])) + int(rng.choice([0, 0, 1, -1, 8, -8]))


@pytest.mark.parametrize("seed", range(12))
def test_bf16_projection_random_shape(hip, seed):
    rng = np.random.default_rng(1000 + seed)
    m, n, k = _extent(rng), _extent(rng), _extent(rng)
    if seed % 4 == 0:
        m = int(rng.choice([2048, 4096, 8192]))   # enough rows for the large-tile forms
    print(f"bf16 projection m={m} n={n} k={k}", flush=True)
    D, ops = hip.DeviceTensor, hip.ops
    a, w, g, bias, res = _rnd(rng, m, k), _rnd(rng, k, n, scale=0.1), _rnd(rng, m, n), _rnd(rng, n), _rnd(rng, m, n)
    ar, wr, gr = (_bf16(t).astype(np.float64) for t in (a, w, g))
    da, dw, dg = D.fromHost(a), D.fromHost(w), D.fromHost(g)
    # the oracle's definition: an fp32-accumulated product of bf16-rounded operands; 2e-4 leaves room for the order of the sums
    assert_close(ops.matmulBf16(da, dw).toHost(), ar @ wr, tol=2e-4, what="matmulBf16", scale=0.1 * np.sqrt(k))
    dA, dB = ops.matmulBf16Backward(da, dw, dg)
    assert_close(dA.toHost(), gr @ wr.T, tol=2e-4, what="dA", scale=0.1 * np.sqrt(n))
    assert_close(dB.toHost(), ar.T @ gr, tol=2e-4, what="dB", scale=np.sqrt(m))
    y = ops.linearBf16Fused(da, dw, D.fromHost(bias), D.fromHost(res)).toHost()
    assert_close(y, ar @ wr + bias + res, tol=2e-4, what="linear + bias + residual", scale=0.1 * np.sqrt(k))


@pytest.mark.parametrize("seed", range(12))
def test_fp32_gemm_random_shape(hip, seed):
    rng = np.random.default_rng(2000 + seed)
    m, n, k = _extent(rng), _extent(rng), _extent(rng)
    if seed % 2 == 0:
        m, n = 4 * int(rng.integers(1, 70)), 4 * int(rng.integers(1, 70))   # a few tiles: the 32 x 32 form
    if seed % 5 == 0:
        k = int(rng.integers(2000, 6000))                                    # long enough for K slices
    print(f"fp32 gemm m={m} n={n} k={k}", flush=True)
    D, ops = hip.DeviceTensor, hip.ops
    a, b, bt, g = _rnd(rng, m, k), _rnd(rng, k, n), _rnd(rng, n, k), _rnd(rng, m, n)
    da, db, dbt, dg = map(D.fromHost, (a, b, bt, g))
    A, B, BT, G = (t.astype(np.float64) for t in (a, b, bt, g))
    assert_close(ops.matmul(da, db).toHost(), A @ B, what="matmul", scale=np.sqrt(k))
    assert_close(ops.matmulTransposeB(da, dbt).toHost(), A @ BT.T, what="matmulTransposeB", scale=np.sqrt(k))
    dA, dB = ops.matmulBackward(da, db, dg)
    assert_close(dA.toHost(), G @ B.T, what="matmulBackward.dA", scale=np.sqrt(n))
    assert_close(dB.toHost(), A.T @ G, what="matmulBackward.dB", scale=np.sqrt(m))
    dA, dB = ops.matmulTransposeBBackward(da, dbt, dg)
    assert_close(dA.toHost(), G @ BT, what="matmulTransposeBBackward.dA", scale=np.sqrt(n))
    assert_close(dB.toHost(), G.T @ A, what="matmulTransposeBBackward.dB", scale=np.sqrt(m))


@pytest.mark.parametrize("seed", range(16))
def test_attention_random_shape(hip, seed):
    rng = np.random.default_rng(3000 + seed)
    b, h = int(rng.integers(1, 3)), int(rng.integers(1, 4))
    hd = int(rng.choice([4, 8, 16, 32, 40, 64, 96, 128, 256]))
    new = int(rng.integers(1, 330))
    old = int(rng.integers(0, 200)) if seed % 2 else 0
    if seed % 7 == 0:
        new, old = 1, int(rng.integers(0, 700))   # one decoded token against a long cache
    print(f"attention batch={b} heads={h} head_dim={hd} newLen={new} oldLen={old}", flush=True)
    D, ops = hip.DeviceTensor, hip.ops
    dim, scale = h * hd, 1.0 / np.sqrt(hd)
    q, go = _rnd(rng, b, new, dim), _rnd(rng, b, new, dim)
    k, v = _rnd(rng, b, new + old, dim), _rnd(rng, b, new + old, dim)
    dq_, dk_, dv_, dgo = map(D.fromHost, (q, k, v, go))
    fwd = ops.fusedAttentionForward(dq_, dk_, dv_, h, float(scale), old)
    grad = ops.fusedAttentionBackward(dgo, dq_, dk_, dv_, fwd.output, fwd.m, fwd.l, h, float(scale), old)
    O, dQ, dK, dV = fwd.output.toHost(), grad.dQ.toHost(), grad.dK.toHost(), grad.dV.toHost()
    for bi in range(b):
        for hi in range(h):
            sl = slice(hi * hd, (hi + 1) * hd)
            o, _, _, dq, dk, dv = attention_slice(q[bi, :, sl], k[bi, :, sl], v[bi, :, sl], go[bi, :, sl], scale, old)
            assert_close(O[bi, :, sl], o, what="O")
            # gradients are differences of nearly equal terms (dS vanishes for a row with one visible key): floor at the terms' size
            assert_close(dQ[bi, :, sl], dq, what="dQ", scale=0.05)
            assert_close(dK[bi, :, sl], dk, what="dK", scale=0.05)
            assert_close(dV[bi, :, sl], dv, what="dV", scale=0.05)


@pytest.mark.parametrize("seed", range(16))
def test_decoding_step_kernels_random_shape(hip, seed):
    """The kernels of an incremental decoding step at random extents: products of one to eight rows in both precisions
    (walks over the weights) with bias and residual, and attention of one to eight queries over a cache whose buffers are
    longer than the cached positions (the walk over the cache), against float64."""
    import ctypes
    rng = np.random.default_rng(5000 + seed)
    m, n, k = int(rng.integers(1, 9)), _extent(rng), _extent(rng)
    if seed % 3 == 0:
        k = 8 * int(rng.integers(1, 600))          # the bf16 walk asks for a multiple of eight; other lengths stay on the tiles
    if seed % 4 == 0:
        n = int(rng.integers(8000, 40000))         # wide enough for four columns a wavefront
    print(f"few-row products m={m} n={n} k={k}", flush=True)
    D, ops, call = hip.DeviceTensor, hip.ops, hip.capi.call
    a, w, bias, res = _rnd(rng, m, k), _rnd(rng, k, n, scale=0.1), _rnd(rng, n), _rnd(rng, m, n)
    da, dw, dbias, dres = map(D.fromHost, (a, w, bias, res))
    y = ops.linearBf16Fused(da, dw, dbias, dres).toHost()
    assert_close(y, _bf16(a).astype(np.float64) @ _bf16(w).astype(np.float64) + bias + res, tol=2e-4, what="bf16 few-row product", scale=0.1 * np.sqrt(k))
    out = D((m, n))
    call("bf_hip_gemm_f32_adds", 0, 0, da.ptr, dw.ptr, dbias.ptr, dres.ptr, out.ptr, m, n, k, None)
    assert_close(out.toHost(), a.astype(np.float64) @ w.astype(np.float64) + bias + res, what="fp32 few-row product", scale=0.1 * np.sqrt(k))

    b, h, new = int(rng.integers(1, 4)), int(rng.integers(1, 5)), int(rng.integers(1, 9))
    hd = int(rng.choice([4, 8, 16, 32, 40, 64, 96, 128, 192, 256]))
    old = int(rng.integers(0, 3000))
    rows = old + new + int(rng.integers(0, 300))
    print(f"few-query attention batch={b} heads={h} head_dim={hd} newLen={new} oldLen={old} rows={rows}", flush=True)
    dim, scale = h * hd, 1.0 / np.sqrt(hd)
    q = _rnd(rng, b, new, dim)
    kc, vc = (np.full((b, rows, dim), np.nan, f32) for _ in range(2))
    kc[:, :old + new], vc[:, :old + new] = _rnd(rng, b, old + new, dim), _rnd(rng, b, old + new, dim)
    dq_, dk_, dv_ = map(D.fromHost, (q, kc, vc))
    o, mm, ll = D((b, new, dim)), D((b, h, new)), D((b, h, new))
    call("bf_hip_attention_forward_rows", dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, None, 0, mm.ptr, ll.ptr, b, h, new, old + new, rows, dim,
         ctypes.c_float(scale), old, None)
    O, M, L = o.toHost(), mm.toHost(), ll.toHost()
    zero = np.zeros((new, hd))
    for bi in range(b):
        for hi in range(h):
            sl = slice(hi * hd, (hi + 1) * hd)
            eo, em, el, _, _, _ = attention_slice(q[bi, :, sl], kc[bi, :old + new, sl], vc[bi, :old + new, sl], zero, scale, old)
            assert_close(O[bi, :, sl], eo, what="O")
            assert_close(M[bi, hi], em, what="m", scale=1.0)
            assert_close(L[bi, hi], el, what="l")


@pytest.mark.parametrize("seed", range(12))
def test_row_kernels_random_shape(hip, seed):
    rng = np.random.default_rng(4000 + seed)
    feat = int(rng.choice([1, 3, 7, 64, 100, 128, 257, 768, 1000, 2048, 4097, 9000, 32000, 50257]))
    rows = int(rng.integers(1, 9)) if feat > 9000 else int(rng.integers(1, 400))
    print(f"rows={rows} features={feat}", flush=True)
    D, ops = hip.DeviceTensor, hip.ops
    x, g = _rnd(rng, rows, feat), _rnd(rng, rows, feat)
    X, G = x.astype(np.float64), g.astype(np.float64)
    r = np.sqrt((X ** 2).mean(-1, keepdims=True) + 1e-6)
    assert_close(ops.rmsnorm(D.fromHost(x)).toHost(), X / r, what="rmsnorm")
    dx = G / r - X * (G * X).sum(-1, keepdims=True) / (feat * r ** 3)
    assert_close(ops.rmsnormBackward(D.fromHost(x), D.fromHost(g)).toHost(), dx, what="rmsnormBackward", scale=float(np.sqrt(np.mean(G ** 2))))
    e = np.exp(X - X.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    assert_close(ops.softmax(D.fromHost(x)).toHost(), p, what="softmax")
    tgt = rng.integers(0, feat, rows)
    res = ops.softmaxCrossEntropySparse(D.fromHost(x), D.fromHost(tgt.astype(f32)))
    loss = -np.log(np.maximum(p[np.arange(rows), tgt], 1e-12)).mean()
    grad = p.copy()
    grad[np.arange(rows), tgt] -= 1
    assert abs(res.value - loss) <= 1e-4 * abs(loss) + 1e-6
    assert_close(res.grad.toHost(), grad / rows, what="cross-entropy gradient")
    assert_close(ops.biasGradientOnly(D.fromHost(g)).toHost(), G.sum(0), what="bias gradient", scale=np.sqrt(rows))


@pytest.mark.parametrize("seed", range(12))
def test_embedding_random_shape(hip, seed):
    """Gather and scatter-add stay bit-exact (sums in token order, like the CPU loop) for one id repeated by every token,
    a handful of ids, and ids spread over the table."""
    rng = np.random.default_rng(5000 + seed)
    vocab, dim = int(rng.integers(1, 3000)), int(rng.choice([1, 4, 6, 32, 128, 130, 768]))
    tokens = int(rng.integers(1, 3000))
    ids = (np.full(tokens, int(rng.integers(0, vocab))), rng.integers(0, min(vocab, 4), tokens), rng.integers(0, vocab, tokens))[seed % 3]
    print(f"embedding vocab={vocab} dim={dim} tokens={tokens} distinct ids={len(np.unique(ids))}", flush=True)
    D, ops = hip.DeviceTensor, hip.ops
    table, g = _rnd(rng, vocab, dim), _rnd(rng, tokens, dim)
    di = D.fromHost(ids.astype(f32).reshape(1, tokens))
    out = ops.embeddingLookup(di, D.fromHost(table)).toHost().reshape(tokens, dim)
    np.testing.assert_array_equal(out, table[ids])
    got = ops.embeddingLookupBackward(di, D.fromHost(g.reshape(1, tokens, dim)), vocab).toHost()
    want = np.zeros((vocab, dim), f32)
    for t in range(tokens):
        want[ids[t]] += g[t]
    np.testing.assert_array_equal(got, want)
