"""The C restatement against the REAL reference CPU backend (oracle/_ref), bit for bit.

Runs only where oracle/_ref/libbf_ref.so has been built (it is compiled from the reference's own
sources by oracle/Makefile).  Every function of the oracle is called with the same seeded random
inputs through both libraries and the outputs must be identical as bit patterns, because the
restatement keeps the reference's loop order and float/double choices.
"""
import numpy as np
import pytest

from oracle import bfo

f32 = np.float32


def same(a, b):
    a, b = np.asarray(a), np.asarray(b)
    assert a.shape == b.shape
    np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))


def r(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(f32)


@pytest.mark.parametrize("n", [1, 7, 1000])
def test_elementwise(oracle, ref, rng, n):
    x, g = r(rng, n, scale=3), r(rng, n)
    for name in ("silu", "relu", "gelu", "roundToBf16"):
        same(getattr(oracle, name)(x), getattr(ref, name)(x))
    for name in ("siluBackward", "reluBackward", "geluBackward"):
        same(getattr(oracle, name)(x, g), getattr(ref, name)(x, g))
    same(oracle.add(x, g), ref.add(x, g))
    same(oracle.scale(x, 0.37), ref.scale(x, 0.37))


@pytest.mark.parametrize("m,k,n", [(1, 1, 1), (5, 7, 3), (33, 65, 17)])
def test_matmuls(oracle, ref, rng, m, k, n):
    a, b, bt, g = r(rng, m, k), r(rng, k, n), r(rng, n, k), r(rng, m, n)
    same(oracle.matmul(a, b), ref.matmul(a, b))
    same(oracle.matmulTransposeB(a, bt), ref.matmulTransposeB(a, bt))
    for x, y in zip(oracle.matmulBackward(a, b, g), ref.matmulBackward(a, b, g)):
        same(x, y)
    for x, y in zip(oracle.matmulTransposeBBackward(a, bt, g), ref.matmulTransposeBBackward(a, bt, g)):
        same(x, y)
    bias = r(rng, n)
    same(oracle.linear(a, b, bias), ref.linear(a, b, bias))
    same(oracle.addBias(g, bias), ref.addBias(g, bias))
    same(oracle.addBiasBackward(g)[1], ref.addBiasBackward(g)[1])


@pytest.mark.parametrize("rows,f", [(1, 1), (4, 33), (9, 300)])
def test_row_ops(oracle, ref, rng, rows, f):
    x, g = r(rng, rows, f, scale=2), r(rng, rows, f)
    same(oracle.rmsnorm(x), ref.rmsnorm(x))
    same(oracle.softmax(x), ref.softmax(x))
    same(oracle.rmsnormBackward(x, g), ref.rmsnormBackward(x, g))
    same(oracle.softmaxBackward(x, g), ref.softmaxBackward(x, g))


def test_embedding_and_positional(oracle, ref, rng):
    vocab, dim, batch, seq = 11, 6, 3, 5
    ids = rng.integers(0, vocab, (batch, seq)).astype(f32)
    table, g = r(rng, vocab, dim), r(rng, batch, seq, dim)
    same(oracle.embeddingLookup(ids, table), ref.embeddingLookup(ids, table))
    same(oracle.embeddingLookupBackward(ids, g, vocab), ref.embeddingLookupBackward(ids, g, vocab))
    pos = r(rng, 9, dim)
    for off in (0, 2, 4):
        same(oracle.addPositionalEmbeddingAt(g, pos, off), ref.addPositionalEmbeddingAt(g, pos, off))
    same(oracle.addPositionalEmbeddingBackward(g, 9)[1], ref.addPositionalEmbeddingBackward(g, 9)[1])


@pytest.mark.parametrize("act", [0, 1])
def test_feed_forward(oracle, ref, rng, act):
    rows, dim, hidden = 6, 8, 20
    x, g = r(rng, 2, 3, dim), r(rng, 2, 3, dim)
    w1, b1, w2, b2 = r(rng, dim, hidden, scale=.3), r(rng, hidden, scale=.1), r(rng, hidden, dim, scale=.3), r(rng, dim, scale=.1)
    same(oracle.feedForward(x, w1, b1, w2, b2, act), ref.feedForward(x, w1, b1, w2, b2, act))
    for a, b in zip(oracle.feedForwardBackward(x, w1, b1, w2, b2, g, act), ref.feedForwardBackward(x, w1, b1, w2, b2, g, act)):
        same(a, b)


@pytest.mark.parametrize("batch,seq,dim,heads", [(1, 3, 4, 2), (2, 9, 12, 3), (1, 17, 32, 1)])
@pytest.mark.parametrize("causal", [True, False])
def test_self_attention(oracle, ref, rng, batch, seq, dim, heads, causal):
    x, g = r(rng, batch, seq, dim), r(rng, batch, seq, dim)
    w = [r(rng, dim, dim, scale=.3) for _ in range(4)]
    same(oracle.selfAttention(x, *w, heads, causal), ref.selfAttention(x, *w, heads, causal))
    for a, b in zip(oracle.selfAttentionBackward(x, *w, heads, g, causal), ref.selfAttentionBackward(x, *w, heads, g, causal)):
        same(a, b)


def test_self_attention_incremental(oracle, ref, rng):
    batch, dim, heads = 2, 8, 2
    w = [r(rng, dim, dim, scale=.3) for _ in range(4)]
    ko = vo = kr = vr = None
    for new_len in (3, 1, 2):
        x = r(rng, batch, new_len, dim)
        oo, ko, vo = oracle.selfAttentionIncremental(x, *w, heads, ko, vo)
        rr, kr, vr = ref.selfAttentionIncremental(x, *w, heads, kr, vr)
        same(oo, rr), same(ko, kr), same(vo, vr)


@pytest.mark.parametrize("batch,heads,new_len,old_len,hd", [(1, 1, 1, 0, 2), (2, 2, 5, 0, 4), (1, 3, 4, 6, 8), (2, 1, 33, 0, 16)])
def test_attention_core(oracle, ref, rng, batch, heads, new_len, old_len, hd):
    dim, total = heads * hd, old_len + new_len
    q, k, v, g = r(rng, batch, new_len, dim), r(rng, batch, total, dim), r(rng, batch, total, dim), r(rng, batch, new_len, dim)
    scale = 1.0 / np.sqrt(f32(hd))
    for a, b in zip(oracle.attentionCoreForward(q, k, v, heads, scale, old_len), ref.attentionCoreForward(q, k, v, heads, scale, old_len)):
        same(a, b)
    for a, b in zip(oracle.attentionCoreBackward(g, q, k, v, heads, scale, old_len), ref.attentionCoreBackward(g, q, k, v, heads, scale, old_len)):
        same(a, b)


def test_losses(oracle, ref, rng):
    rows, classes = 7, 13
    logits = r(rng, rows, classes, scale=3)
    dense = np.zeros((rows, classes), f32)
    idx = rng.integers(0, classes, rows)
    dense[np.arange(rows), idx] = 1
    for name, tgt in (("softmaxCrossEntropy", dense), ("softmaxCrossEntropySparse", idx.astype(f32)), ("meanSquaredError", r(rng, rows, classes))):
        (va, ga), (vb, gb) = getattr(oracle, name)(logits, tgt), getattr(ref, name)(logits, tgt)
        assert f32(va).view(np.uint32) == f32(vb).view(np.uint32)
        same(ga, gb)


@pytest.mark.parametrize("rows,classes,keep", [(7, 13, 0.5), (40, 5, 0.15), (6, 9, 1.0), (5, 4, 0.0)])
def test_masked_cross_entropy(oracle, ref, rng, rows, classes, keep):
    logits = r(rng, rows, classes, scale=3)
    idx = np.where(rng.random(rows) < keep, rng.integers(0, classes, rows), -1).astype(f32)
    (va, ga), (vb, gb) = oracle.softmaxCrossEntropyMasked(logits, idx), ref.softmaxCrossEntropyMasked(logits, idx)
    assert f32(va).view(np.uint32) == f32(vb).view(np.uint32)
    same(ga, gb)
    bad = idx.copy()
    bad[0] = classes
    for impl in (oracle, ref):
        with pytest.raises(bfo.OracleInvalidArgument):
            impl.softmaxCrossEntropyMasked(logits, bad)


def test_optimizers(oracle, ref, rng):
    p, g = r(rng, 50), r(rng, 50)
    same(oracle.sgdStep(p, g, 0.05), ref.sgdStep(p, g, 0.05))
    z = np.zeros(50, f32)
    for a, b in zip(oracle.adamwStep(p, g, z, z, 1), ref.adamwStep(p, g, z, z, 1)):
        same(a, b)


TINY_LM = [(bfo.EMBEDDING, 17, 8), (bfo.POSITIONAL, 6), (bfo.ATTENTION, 2), (bfo.FEEDFORWARD, 16, 0), (bfo.LINEAR, 17)]
MLP = [(bfo.LINEAR, 12), (bfo.SILU,), (bfo.LINEAR, 5), (bfo.RMSNORM,), (bfo.GELU,), (bfo.RELU,), (bfo.SOFTMAX,)]
TINY_MLM = [(bfo.EMBEDDING, 17, 8), (bfo.POSITIONAL, 6), (bfo.BIDIRECTIONAL_ATTENTION, 2), (bfo.FEEDFORWARD, 16, 0), (bfo.LINEAR, 17)]


@pytest.mark.parametrize("layers,in_features,kind", [(TINY_LM, 0, "lm"), (MLP, 9, "mlp"), (TINY_MLM, 0, "mlm")])
def test_model_training_steps(oracle, ref, rng, layers, in_features, kind):
    """Three full steps (zeroGrad, forward, loss, backward, AdamW) through cpu::Model and the restatement."""
    mo, mr = oracle.model(layers, in_features), ref.model(layers, in_features)
    assert mo.names == mr.names and mo.counts == mr.counts
    for i, c in enumerate(mo.counts):
        w = r(rng, c, scale=0.1)
        mo.value(i)[:] = w
        mr.value(i)[:] = w
    for step in range(3):
        if kind == "lm":
            x = rng.integers(0, 17, (2, 5)).astype(f32)
            target = rng.integers(0, 17, 10).astype(f32)
        elif kind == "mlm":
            x = rng.integers(0, 17, (2, 5)).astype(f32)
            target = np.where(rng.random(10) < 0.4, x.ravel(), -1).astype(f32)
            target[3] = x.ravel()[3]   # at least one row counts
        else:
            x = r(rng, 4, 9)
            target = rng.integers(0, 5, 4).astype(f32)
        outs = []
        for o, m in ((oracle, mo), (ref, mr)):
            m.zeroGrad()
            y = m.forward(x)
            classes = 5 if kind == "mlp" else 17
            loss_fn = o.softmaxCrossEntropyMasked if kind == "mlm" else o.softmaxCrossEntropySparse
            loss, grad = loss_fn(y.reshape(-1, classes), target)
            m.backward(grad)
            grads = [m.grad(i).copy() for i in range(len(m.counts))]
            m.adamwStep(lr=1e-2)
            outs.append((y, f32(loss), grads, [m.value(i).copy() for i in range(len(m.counts))]))
        (yo, lo, go, po), (yr, lr_, gr, pr) = outs
        same(yo, yr)
        assert lo.view(np.uint32) == lr_.view(np.uint32)
        for a, b in zip(go, gr):
            same(a, b)
        for a, b in zip(po, pr):
            same(a, b)
