"""The C restatement replayed on the committed fixtures written by the real reference build.

tests/golden/reference_vectors.npz (made by tests/golden/make_golden.py) holds seeded inputs and the
reference's outputs for the composite blocks, the attention core and a tiny LM trained for three
AdamW steps.  This runs everywhere (no reference tree needed) and requires identical bits.
"""
import os

import numpy as np
import pytest

import refvectors as rv

f32 = np.float32
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLDEN)


def same(a, b):
    a, b = np.asarray(a, f32), np.asarray(b, f32)
    assert a.shape == b.shape
    np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))


def test_attention_block_fixture(oracle, gold):
    w = (rv.ATTN_WQ, rv.ATTN_WK, rv.ATTN_WV, rv.ATTN_WOUT)
    same(oracle.selfAttention(rv.ATTN_INPUT, *w, rv.ATTN_HEADS), gold["attnfix_out"])
    got = oracle.selfAttentionBackward(rv.ATTN_INPUT, *w, rv.ATTN_HEADS, gold["attnfix_grad"])
    for n, a in zip(("dx", "dwq", "dwk", "dwv", "dwout"), got):
        same(a, gold["attnfix_" + n])


def test_feed_forward_fixture(oracle, gold):
    ff = (rv.FF_W1, rv.FF_B1, rv.FF_W2, rv.FF_B2)
    same(oracle.feedForward(rv.FF_INPUT, *ff), gold["fffix_out"])
    for n, a in zip(("dx", "dw1", "db1", "dw2", "db2"), oracle.feedForwardBackward(rv.FF_INPUT, *ff, rv.FF_GRAD)):
        same(a, gold["fffix_" + n])


def test_attention_core_cases(oracle, gold):
    for i, (b, h, nl, ol, hd) in enumerate(gold["core_cases"]):
        g = {n: gold[f"core{i}_{n}"] for n in "q k v go o m l dq dk dv".split()}
        scale = f32(1.0) / np.sqrt(f32(hd))
        o, m, l = oracle.attentionCoreForward(g["q"], g["k"], g["v"], int(h), scale, int(ol))
        same(o, g["o"]), same(m, g["m"]), same(l, g["l"])
        dq, dk, dv = oracle.attentionCoreBackward(g["go"], g["q"], g["k"], g["v"], int(h), scale, int(ol))
        same(dq, g["dq"]), same(dk, g["dk"]), same(dv, g["dv"])


def test_rows_activations_losses(oracle, gold):
    x, g = gold["rows_x"], gold["rows_g"]
    same(oracle.rmsnorm(x), gold["rows_rmsnorm"])
    same(oracle.rmsnormBackward(x, g), gold["rows_rmsnorm_bwd"])
    same(oracle.softmax(x), gold["rows_softmax"])
    same(oracle.softmaxBackward(x, g), gold["rows_softmax_bwd"])
    for name in ("silu", "gelu", "relu"):
        same(getattr(oracle, name)(x), gold["act_" + name])
        same(getattr(oracle, name + "Backward")(x, g), gold["act_" + name + "_bwd"])
    v, gr = oracle.softmaxCrossEntropySparse(x, gold["ce_idx"])
    same(f32(v), gold["ce_value"]), same(gr, gold["ce_grad"])
    v, gr = oracle.meanSquaredError(x, g)
    same(f32(v), gold["mse_value"]), same(gr, gold["mse_grad"])


def test_tiny_lm_three_steps(oracle, gold):
    layers = [tuple(int(v) for v in row) for row in gold["lm_layers"]]
    model = oracle.model(layers)
    for i in range(len(model.counts)):
        model.value(i)[:] = gold[f"lm_init{i}"]
    for step in range(3):
        model.zeroGrad()
        logits = model.forward(gold[f"lm_step{step}_ids"])
        same(logits, gold[f"lm_step{step}_logits"])
        loss, grad = oracle.softmaxCrossEntropySparse(logits.reshape(16, 32), gold[f"lm_step{step}_tgt"])
        same(f32(loss), gold[f"lm_step{step}_loss"])
        model.backward(grad)
        for i in range(len(model.counts)):
            same(model.grad(i), gold[f"lm_step{step}_grad{i}"])
        model.adamwStep(lr=1e-2)
        for i in range(len(model.counts)):
            same(model.value(i), gold[f"lm_step{step}_param{i}"])
