"""Writes tests/golden/reference_vectors.npz from the REAL reference CPU backend.

Run in a container that has the reference tree (oracle/_ref/libbf_ref.so is built from it by
oracle/Makefile):  python tests/golden/make_golden.py
The file holds data only: seeded inputs and the outputs the reference produced for them, for the
functions whose expected numbers the reference's own tests do not spell out (composite blocks, the
attention core, a tiny LM trained for three steps).  tests/test_oracle_golden.py replays the inputs
through the C restatement and requires identical bits.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import bfo  # noqa: E402
import refvectors as rv  # noqa: E402

f32 = np.float32
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")

TINY_LM = [(bfo.EMBEDDING, 32, 16), (bfo.POSITIONAL, 8), (bfo.ATTENTION, 4), (bfo.FEEDFORWARD, 32, 0), (bfo.LINEAR, 32)]


def main():
    ref = bfo.reference()
    if ref is None:
        raise SystemExit("oracle/_ref/libbf_ref.so is not built; run `make -C oracle ref` where the reference exists")
    rng = np.random.default_rng(20240607)
    r = lambda *s, scale=1.0: (rng.standard_normal(s) * scale).astype(f32)
    d = {}

    # the reference's shared attention fixture (inputs from its tests; outputs from the real build)
    w = (rv.ATTN_WQ, rv.ATTN_WK, rv.ATTN_WV, rv.ATTN_WOUT)
    g = r(1, 3, 4)
    d["attnfix_grad"] = g
    d["attnfix_out"] = ref.selfAttention(rv.ATTN_INPUT, *w, rv.ATTN_HEADS)
    for n, a in zip(("dx", "dwq", "dwk", "dwv", "dwout"), ref.selfAttentionBackward(rv.ATTN_INPUT, *w, rv.ATTN_HEADS, g)):
        d["attnfix_" + n] = a
    # the reference's feed-forward fixture
    ff = (rv.FF_W1, rv.FF_B1, rv.FF_W2, rv.FF_B2)
    d["fffix_out"] = ref.feedForward(rv.FF_INPUT, *ff)
    for n, a in zip(("dx", "dw1", "db1", "dw2", "db2"), ref.feedForwardBackward(rv.FF_INPUT, *ff, rv.FF_GRAD)):
        d["fffix_" + n] = a

    # attention core: (batch, heads, newLen, oldLen, headDim)
    cases = [(2, 2, 5, 0, 2), (2, 2, 33, 0, 32), (1, 2, 70, 0, 64), (1, 1, 40, 0, 128), (2, 2, 3, 9, 16), (1, 2, 1, 37, 32)]
    d["core_cases"] = np.array(cases, np.int64)
    for i, (b, h, nl, ol, hd) in enumerate(cases):
        dim, tot = h * hd, ol + nl
        q, k, v, go = r(b, nl, dim), r(b, tot, dim), r(b, tot, dim), r(b, nl, dim)
        scale = f32(1.0) / np.sqrt(f32(hd))
        o, m, l = ref.attentionCoreForward(q, k, v, h, scale, ol)
        dq, dk, dv = ref.attentionCoreBackward(go, q, k, v, h, scale, ol)
        for n, a in zip("q k v go o m l dq dk dv".split(), (q, k, v, go, o, m, l, dq, dk, dv)):
            d[f"core{i}_{n}"] = a

    # rows / losses / activations on seeded inputs
    x, gx = r(6, 70, scale=2), r(6, 70)
    d["rows_x"], d["rows_g"] = x, gx
    d["rows_rmsnorm"], d["rows_rmsnorm_bwd"] = ref.rmsnorm(x), ref.rmsnormBackward(x, gx)
    d["rows_softmax"], d["rows_softmax_bwd"] = ref.softmax(x), ref.softmaxBackward(x, gx)
    for name in ("silu", "gelu", "relu"):
        d["act_" + name] = getattr(ref, name)(x)
        d["act_" + name + "_bwd"] = getattr(ref, name + "Backward")(x, gx)
    idx = rng.integers(0, 70, 6).astype(f32)
    d["ce_idx"] = idx
    v_, g_ = ref.softmaxCrossEntropySparse(x, idx)
    d["ce_value"], d["ce_grad"] = f32(v_), g_
    v_, g_ = ref.meanSquaredError(x, gx)
    d["mse_value"], d["mse_grad"] = f32(v_), g_

    # tiny LM, three AdamW steps through the reference's cpu::Model
    model = ref.model(TINY_LM)
    d["lm_layers"] = np.array([(l + (0, 0))[:3] for l in TINY_LM], np.int64)
    init = [r(c, scale=0.08) for c in model.counts]
    for i, a in enumerate(init):
        model.value(i)[:] = a
        d[f"lm_init{i}"] = a
    for step in range(3):
        ids = rng.integers(0, 32, (2, 8)).astype(f32)
        tgt = rng.integers(0, 32, 16).astype(f32)
        model.zeroGrad()
        logits = model.forward(ids)
        loss, grad = ref.softmaxCrossEntropySparse(logits.reshape(16, 32), tgt)
        model.backward(grad)
        d[f"lm_step{step}_ids"], d[f"lm_step{step}_tgt"] = ids, tgt
        d[f"lm_step{step}_logits"], d[f"lm_step{step}_loss"] = logits, f32(loss)
        for i in range(len(model.counts)):
            d[f"lm_step{step}_grad{i}"] = model.grad(i).copy()
        model.adamwStep(lr=1e-2)
        for i in range(len(model.counts)):
            d[f"lm_step{step}_param{i}"] = model.value(i).copy()

    np.savez_compressed(OUT, **d)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(d), "arrays")


if __name__ == "__main__":
    main()
