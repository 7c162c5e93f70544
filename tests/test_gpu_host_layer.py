"""GPU parity of the C++ operator layer (include/blackforge/backend/hip/): the C++ API test program, the
composite blocks, and whole training steps of hip::Model against the CPU oracle and the golden fixtures."""
import os
import subprocess

import numpy as np
import pytest

import refvectors as rv
from parity import BF16_TOL, assert_bits_equal, assert_close, take_worst

pytestmark = pytest.mark.gpu
f32 = np.float32
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden", "reference_vectors.npz")


def r(rng, *s, scale=1.0):
    return (rng.standard_normal(s) * scale).astype(f32)


def test_cpp_api_program(hip):
    """tests/cpp/host_api_test.cpp: the reference's literal test vectors through namespace blackforge::backend::hip."""
    exe = os.path.join(ROOT, "blackforge_amd", "host", "bin", "host_api_test")
    assert os.path.exists(exe), "run `make -C blackforge_amd/host` (the driver's build() does)"
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(proc.stdout[-3000:])
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-1000:]


def test_attention_block_fixture_and_golden(hip, oracle):
    """The reference's shared 4x4 attention fixture: forward and every gradient against the real reference's numbers."""
    gold = np.load(GOLDEN)
    D, ops = hip.DeviceTensor, hip.ops
    w = [D.fromHost(a) for a in (rv.ATTN_WQ, rv.ATTN_WK, rv.ATTN_WV, rv.ATTN_WOUT)]
    x, g = D.fromHost(rv.ATTN_INPUT), D.fromHost(gold["attnfix_grad"])
    assert_close(ops.selfAttention(x, *w, rv.ATTN_HEADS).toHost(), gold["attnfix_out"], what="selfAttention fixture")
    grad = ops.selfAttentionBackward(x, *w, rv.ATTN_HEADS, g)
    for name, got in zip(("dx", "dwq", "dwk", "dwv", "dwout"), (grad.dInput, grad.dWq, grad.dWk, grad.dWv, grad.dWout)):
        assert_close(got.toHost(), gold["attnfix_" + name], what="selfAttentionBackward fixture " + name, scale=1e-2)
    ff = [D.fromHost(a) for a in (rv.FF_W1, rv.FF_B1, rv.FF_W2, rv.FF_B2)]
    assert_close(ops.feedForward(D.fromHost(rv.FF_INPUT), *ff).toHost(), gold["fffix_out"], what="feedForward fixture")
    fg = ops.feedForwardBackward(D.fromHost(rv.FF_INPUT), *ff, D.fromHost(rv.FF_GRAD))
    for name, got in zip(("dx", "dw1", "db1", "dw2", "db2"), (fg.dInput, fg.dW1, fg.dB1, fg.dW2, fg.dB2)):
        assert_close(got.toHost(), gold["fffix_" + name], what="feedForwardBackward fixture " + name, scale=1e-2)


@pytest.mark.parametrize("batch,seq,dim,heads,hidden", [(2, 9, 12, 3, 20), (8, 64, 128, 4, 512), (1, 130, 64, 2, 96), (2, 40, 256, 2, 264)])
@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("cached", [False, True])
def test_blocks_against_oracle(hip, oracle, rng, batch, seq, dim, heads, hidden, act, cached):
    """The composite blocks of the C++ operator layer (hip::selfAttention[Backward], hip::feedForward[Backward], and with
    `cached` the *ForwardCached / *BackwardCached pair that hip::Model calls) against the CPU backend's blocks: fp32 at
    the fp32 bound, the bf16 variants (stateless, and cached with the fused feed-forward and shared-input routes) at 2e-2."""
    D, ops = hip.DeviceTensor, hip.ops
    x, g = r(rng, batch, seq, dim), r(rng, batch, seq, dim)
    w = [r(rng, dim, dim, scale=dim ** -0.5) for _ in range(4)]
    dw = [D.fromHost(a) for a in w]
    dx, dg = D.fromHost(x), D.fromHost(g)
    names = ("dInput", "dWq", "dWk", "dWv", "dWout")
    if act == 0:
        eo, eg = oracle.selfAttention(x, *w, heads), oracle.selfAttentionBackward(x, *w, heads, g)
        assert_close(ops.selfAttention(dx, *dw, heads, cached=cached).toHost(), eo, what="selfAttention")
        grad = ops.selfAttentionBackward(dx, *dw, heads, dg, cached=cached)
        for got, e, n in zip((grad.dInput, grad.dWq, grad.dWk, grad.dWv, grad.dWout), eg, names):
            assert_close(got.toHost(), e, what="selfAttentionBackward." + n, scale=float(np.abs(e).max()) * 0.1)
        assert_close(ops.selfAttention(dx, *dw, heads, useBf16=True, cached=cached).toHost(), eo, tol=BF16_TOL, what="selfAttentionBf16")
        grad = ops.selfAttentionBackward(dx, *dw, heads, dg, useBf16=True, cached=cached)
        for got, e, n in zip((grad.dInput, grad.dWq, grad.dWk, grad.dWv, grad.dWout), eg, names):
            assert_close(got.toHost(), e, tol=BF16_TOL, what="selfAttentionBf16Backward." + n, scale=float(np.abs(e).max()))
    p = [r(rng, dim, hidden, scale=dim ** -0.5), r(rng, hidden, scale=.1), r(rng, hidden, dim, scale=hidden ** -0.5), r(rng, dim, scale=.1)]
    dp = [D.fromHost(a) for a in p]
    eo, eg = oracle.feedForward(x, *p, act), oracle.feedForwardBackward(x, *p, g, act)
    names = ("dInput", "dW1", "dB1", "dW2", "dB2")
    assert_close(ops.feedForward(dx, *dp, act, cached=cached).toHost(), eo, what="feedForward")
    fg = ops.feedForwardBackward(dx, *dp, dg, act, cached=cached)
    for got, e, n in zip((fg.dInput, fg.dW1, fg.dB1, fg.dW2, fg.dB2), eg, names):
        assert_close(got.toHost(), e, what="feedForwardBackward." + n, scale=float(np.abs(e).max()) * 0.1)
    assert_close(ops.feedForward(dx, *dp, act, useBf16=True, cached=cached).toHost(), eo, tol=BF16_TOL, what="feedForwardBf16")
    fg = ops.feedForwardBackward(dx, *dp, dg, act, useBf16=True, cached=cached)
    for got, e, n in zip((fg.dInput, fg.dW1, fg.dB1, fg.dW2, fg.dB2), eg, names):
        assert_close(got.toHost(), e, tol=BF16_TOL, what="feedForwardBf16Backward." + n, scale=float(np.abs(e).max()))


@pytest.mark.parametrize("batch,seq,dim,heads", [(2, 9, 12, 3), (4, 64, 128, 4), (1, 130, 64, 2), (1, 200, 256, 2)])
def test_bidirectional_attention_block(hip, oracle, rng, batch, seq, dim, heads):
    """bidirectionalSelfAttention and its backward (cpu ops.cpp:504-507, autodiff.cpp:492-496): the block with every key
    visible to every query."""
    D, ops = hip.DeviceTensor, hip.ops
    x, g = r(rng, batch, seq, dim), r(rng, batch, seq, dim)
    w = [r(rng, dim, dim, scale=dim ** -0.5) for _ in range(4)]
    dw = [D.fromHost(a) for a in w]
    dx, dg = D.fromHost(x), D.fromHost(g)
    exp = oracle.selfAttention(x, *w, heads, causal=False)
    assert_close(ops.bidirectionalSelfAttention(dx, *dw, heads).toHost(), exp, what="bidirectionalSelfAttention")
    assert np.abs(exp - oracle.selfAttention(x, *w, heads, causal=True)).max() > 1e-3, "the case must tell the two masks apart"
    grad = ops.bidirectionalSelfAttentionBackward(dx, *dw, heads, dg)
    for got, e, n in zip((grad.dInput, grad.dWq, grad.dWk, grad.dWv, grad.dWout), oracle.selfAttentionBackward(x, *w, heads, g, causal=False),
                         ("dInput", "dWq", "dWk", "dWv", "dWout")):
        assert_close(got.toHost(), e, what="bidirectionalSelfAttentionBackward." + n, scale=float(np.abs(e).max()) * 0.1)
    # bf16 projections: the documented bf16 tolerance
    got = ops.bidirectionalSelfAttention(dx, *dw, heads, useBf16=True).toHost()
    assert_close(got, exp, tol=2e-2, what="bidirectionalSelfAttention bf16")


def test_bidirectional_attention_reference_case(hip):
    """tests/backend/cpu/ops_tests.cpp:359-391: a change at position 2 reaches the outputs at positions 0 and 1."""
    D, ops = hip.DeviceTensor, hip.ops
    wq = np.array([0.3, -0.1, 0.2, 0.05, 0.1, 0.4, -0.2, 0.15, -0.3, 0.2, 0.1, -0.05, 0.2, -0.1, 0.3, 0.1], f32).reshape(4, 4)
    wk = np.array([0.1, 0.2, -0.1, 0.3, -0.2, 0.1, 0.4, -0.1, 0.3, -0.3, 0.1, 0.2, -0.1, 0.2, -0.2, 0.1], f32).reshape(4, 4)
    wv = np.array([0.2, 0.1, -0.1, 0.3, 0.1, -0.2, 0.3, 0.1, -0.1, 0.3, 0.2, -0.1, 0.3, 0.1, -0.2, 0.2], f32).reshape(4, 4)
    wo = np.array([0.1, -0.1, 0.2, 0.1, 0.2, 0.1, -0.1, 0.2, -0.1, 0.2, 0.1, -0.1, 0.1, 0.2, -0.1, 0.2], f32).reshape(4, 4)
    a = np.array([0.1, -0.2, 0.3, 0.4, -0.5, 0.6, 0.2, -0.1, 0.3, 0.2, -0.4, 0.5], f32).reshape(1, 3, 4)
    b = a.copy()
    b[0, 2, 0] = 99.0
    dw = [D.fromHost(t) for t in (wq, wk, wv, wo)]
    ya, yb = (ops.bidirectionalSelfAttention(D.fromHost(t), *dw, 2).toHost() for t in (a, b))
    assert np.abs(ya[0, :2] - yb[0, :2]).max() > 1e-4
    ca, cb = (ops.selfAttention(D.fromHost(t), *dw, 2).toHost() for t in (a, b))
    assert np.abs(ca[0, :2] - cb[0, :2]).max() == 0.0


def test_mlm_model_steps_against_oracle(hip, oracle, rng):
    """A masked-language-model pipeline (embedding, positions, bidirectional attention, feed-forward, linear) through the
    C++ host layer's Model for three steps with the masked loss and AdamW, against the CPU restatement."""
    from blackforge_amd import hostlayer as hl
    from oracle import bfo
    vocab, dim, seq, heads, hidden, batch = 37, 32, 12, 4, 48, 3
    mk = lambda m: [(m.EMBEDDING, vocab, dim), (m.POSITIONAL, seq), (m.BIDIRECTIONAL_ATTENTION, heads), (m.FEEDFORWARD, hidden, 0),
                    (m.LINEAR, vocab)]
    gpu, cpu = hl.HostModel(mk(hl)), oracle.model(mk(bfo))
    assert gpu.names == cpu.names and any(n.startswith("bidirectional_attention3.") for n in gpu.names)
    for i, c in enumerate(gpu.counts):
        w = r(rng, c, scale=0.1)
        gpu.set_value(i, w)
        cpu.value(i)[:] = w
    D = hip.DeviceTensor
    for step in range(3):
        ids = rng.integers(0, vocab, (batch, seq)).astype(f32)
        target = np.where(rng.random(batch * seq) < 0.3, ids.ravel(), -1).astype(f32)
        target[1] = ids.ravel()[1]
        cpu.zeroGrad()
        logits = cpu.forward(ids)
        loss, grad = oracle.softmaxCrossEntropyMasked(logits.reshape(-1, vocab), target)
        cpu.backward(grad)
        gpu.trainStep(D.fromHost(ids), D.fromHost(target), hl.LOSS_MASKED_CE, optimizer=0)
        assert abs(gpu.readLossSum() - loss) <= 1e-4 * abs(loss) + 1e-6
        for i in range(len(gpu.counts)):
            e = cpu.grad(i)
            assert_close(gpu.grad(i), e, what=f"step {step} grad {gpu.names[i]}", scale=float(np.abs(e).max()) * 0.05)
        cpu.adamwStep(lr=1e-2)
        gpu.adamwStep(lr=1e-2)
        for i in range(len(gpu.counts)):
            assert_close(gpu.value(i), cpu.value(i), what=f"step {step} param {gpu.names[i]}", scale=0.02 * 1e-2 / 1e-4)
        print(f"step {step}: measured max |gpu - cpu| / max |cpu| over all gradients and parameters: {max(take_worst().values()):.2e}")


@pytest.mark.parametrize("use_bf16", [False, True])
def test_incremental_decode_block(hip, oracle, rng, use_bf16):
    """hip::selfAttentionIncremental[Bf16] with a growing hip::KVCache against the CPU backend's incremental block
    (ops.cpp:509-566): prefill, single tokens, a longer continuation."""
    D, ops = hip.DeviceTensor, hip.ops
    batch, dim, heads = 2, 32, 4
    w = [r(rng, dim, dim, scale=dim ** -0.5) for _ in range(4)]
    dw = [D.fromHost(a) for a in w]
    cache, kc, vc = ops.KVCache(), None, None
    tol = BF16_TOL if use_bf16 else 1e-4
    for new_len in (5, 1, 1, 3):
        x = r(rng, batch, new_len, dim)
        got = ops.selfAttentionIncremental(D.fromHost(x), *dw, heads, cache, useBf16=use_bf16).toHost()
        exp, kc, vc = oracle.selfAttentionIncremental(x, *w, heads, kc, vc)
        assert_close(got, exp, tol=tol, what=f"incremental newLen={new_len}")
    assert cache.length == 10
    assert_close(cache.keys(batch, dim), kc, tol=tol, what="KV cache K")
    assert_close(cache.values(batch, dim), vc, tol=tol, what="KV cache V")
    # the cache has room to grow and is re-made only when that runs out: continuations across two such moments
    seen = {cache.capacity}
    for new_len in (120, 1, 1, 130, 1, 2):
        x = r(rng, batch, new_len, dim)
        got = ops.selfAttentionIncremental(D.fromHost(x), *dw, heads, cache, useBf16=use_bf16).toHost()
        exp, kc, vc = oracle.selfAttentionIncremental(x, *w, heads, kc, vc)
        assert_close(got, exp, tol=tol, what=f"incremental newLen={new_len} at length {cache.length}")
        assert cache.capacity >= cache.length
        seen.add(cache.capacity)
    assert cache.length == 265 and len(seen) == 3, seen
    assert_close(cache.keys(batch, dim), kc, tol=tol, what="KV cache K after growing")
    assert_close(cache.values(batch, dim), vc, tol=tol, what="KV cache V after growing")


def _lm_layers(hl, vocab, dim, seq, heads, hidden, act, blocks=1):
    layers = [(hl.EMBEDDING, vocab, dim), (hl.POSITIONAL, seq)]
    for _ in range(blocks):
        layers += [(hl.ATTENTION, heads), (hl.FEEDFORWARD, hidden, act)]
    return layers + [(hl.LINEAR, vocab)]


def test_tiny_lm_three_steps_match_the_reference_fixture(hip):
    """hip::Model against numbers produced by the reference's cpu::Model: logits, loss, every gradient and every
    parameter after each of three AdamW steps (fixture: tests/golden/make_golden.py)."""
    from blackforge_amd import hostlayer as hl
    gold = np.load(GOLDEN)
    layers = [tuple(int(v) for v in row) for row in gold["lm_layers"]]
    model = hl.HostModel(layers)
    for i in range(len(model.counts)):
        model.set_value(i, gold[f"lm_init{i}"])
    D = hip.DeviceTensor
    for step in range(3):
        model.zeroGrad()
        logits = model.forward(D.fromHost(gold[f"lm_step{step}_ids"]))
        assert_close(logits, gold[f"lm_step{step}_logits"], what=f"step {step} logits")
        model.loss(D.fromHost(gold[f"lm_step{step}_tgt"]))
        loss = model.readLossSum() / 16
        assert abs(loss - float(gold[f"lm_step{step}_loss"])) <= 1e-4 * float(gold[f"lm_step{step}_loss"])
        model.backward()
        for i in range(len(model.counts)):
            e = gold[f"lm_step{step}_grad{i}"]
            assert_close(model.grad(i), e, what=f"step {step} grad {model.names[i]}", scale=float(np.abs(e).max()) * 0.05)
        model.adamwStep(lr=1e-2)
        for i in range(len(model.counts)):
            # floor: 2 % of the AdamW step bound lr = 1e-2 (the update is lr * m / (sqrt(v) + eps), ill-conditioned
            # where the gradient is comparable to eps)
            assert_close(model.value(i), gold[f"lm_step{step}_param{i}"], what=f"step {step} param {model.names[i]}", scale=0.02 * 1e-2 / 1e-4)
        print(f"step {step}: measured max |gpu - reference| / max |reference| over all gradients and parameters: {max(take_worst().values()):.2e}")


@pytest.mark.parametrize("use_bf16", [False, True])
def test_model_forward_incremental_matches_full_forward(hip, oracle, rng, use_bf16):
    """hip::Model::forwardIncremental (model.cu:385-424; the reference's own check is token-by-token == full forward,
    tests/backend/cuda/model_tests.cu:536-611): prefill five tokens, then single tokens; each call's logits against
    Model::forward over the whole prefix at the same positions and against the CPU model; greedy argmax of the last
    position; resetGenerationState() starts over at position 0."""
    from blackforge_amd import hostlayer as hl
    from oracle import bfo
    vocab, dim, seq, heads, hidden, blocks = 61, 64, 16, 4, 96, 2
    gpu = hl.HostModel(_lm_layers(hl, vocab, dim, seq, heads, hidden, 0, blocks), use_bf16=use_bf16)
    cpu = oracle.model(_lm_layers(bfo, vocab, dim, seq, heads, hidden, 0, blocks))
    for i, c in enumerate(gpu.counts):
        w = r(rng, c, scale=0.2)
        gpu.set_value(i, w)
        cpu.value(i)[:] = w
    D = hip.DeviceTensor
    ids = rng.integers(0, vocab, (1, 9)).astype(f32)
    tol = BF16_TOL if use_bf16 else 1e-4

    def decode():
        done, outs = 0, []
        for new_len in (5, 1, 1, 2):
            logits = gpu.forwardIncremental(D.fromHost(ids[:, done:done + new_len])).reshape(new_len, vocab)
            choice = gpu.argmaxLast(vocab)
            done += new_len
            full = gpu.forward(D.fromHost(ids[:, :done])).reshape(done, vocab)
            # same kernels on the same rows: only the attention tiling (one call over the prefix against new rows over a
            # cache) and, in bf16 mode, the cached weight images differ
            assert_close(logits, full[done - new_len:], tol=1e-4 if not use_bf16 else 5e-3, what=f"incremental vs full forward at {done}")
            expected = cpu.forward(ids[:, :done]).reshape(done, vocab)
            assert_close(logits, expected[done - new_len:], tol=tol, what=f"incremental vs CPU model at {done}",
                         scale=float(np.abs(expected).max()) if use_bf16 else 0.0)
            assert choice == int(np.argmax(logits[-1])), "argmaxLastPosition over the incremental logits"
            if not use_bf16:
                assert choice == oracle.argmaxLastPosition(expected[None])
            outs.append(logits)
        return outs

    first = decode()
    gpu.resetGenerationState()
    second = decode()
    for a, b in zip(first, second):
        assert_bits_equal(a, b, "decode after resetGenerationState")
    # without a reset the positions continue: the positional table has 16 rows, so 9 + 9 > 16 must be refused
    with pytest.raises(ValueError):
        gpu.forwardIncremental(D.fromHost(ids))


@pytest.mark.parametrize("use_bf16,heads,dim", [(False, 4, 32), (True, 4, 32), (True, 2, 264)])
def test_greedy_generation_without_reading_back(hip, rng, use_bf16, heads, dim):
    """hip::Model::generateGreedy: the loop of the reference's `generate` command (main.cpp:594-617: forwardIncremental, argmax
    of the last logits, feed it back) with token and position kept on the device, so that no step waits for a read-back.
    Checked against the loop over forwardIncremental fed with the same tokens: every token is the argmax of that loop's logits
    at its step (up to a near tie: the attention splits the cache into chunks differently), across the 128-key chunk
    boundary of the attention walk, and the model is left where the eager loop would be."""
    from blackforge_amd import hostlayer as hl
    vocab, seq, hidden, blocks = 96, 400, 64, 2
    D = hip.DeviceTensor
    model = hl.HostModel(_lm_layers(hl, vocab, dim, seq, heads, hidden, 1, blocks), use_bf16=use_bf16)
    for i, c in enumerate(model.counts):
        model.set_value(i, r(rng, c, scale=0.3))
    prompt = rng.integers(0, vocab, (1, 7)).astype(f32)
    count = 200
    tokens = model.generateGreedy(D.fromHost(prompt), count)
    assert len(tokens) == count and all(0 <= t < vocab for t in tokens)
    after = model.forwardIncremental(D.fromHost(np.array([[tokens[-1]]], f32))).reshape(vocab)   # the generation continues eagerly
    assert model.generateGreedy(D.fromHost(prompt), count) == tokens, "the same generation twice"
    assert model.generateGreedy(D.fromHost(prompt), 1) == tokens[:1] and model.generateGreedy(D.fromHost(prompt), 0) == []

    model.resetGenerationState()
    logits = model.forwardIncremental(D.fromHost(prompt)).reshape(-1, vocab)[-1]
    near_ties = 0
    for step, t in enumerate(tokens):
        best = int(np.argmax(logits))
        if t != best:   # generateGreedy's logits differ from these in the last bits
            near_ties += 1
            assert logits[best] - logits[t] <= (5e-3 if use_bf16 else 1e-4) * np.abs(logits).max(), f"token {step}: {t} is not the eager argmax {best}"
        logits = model.forwardIncremental(D.fromHost(np.array([[t]], f32))).reshape(vocab)
    assert near_ties <= 2
    assert_close(after, logits, tol=5e-3 if use_bf16 else 1e-4, what="logits after the generation vs the eager loop's")
    with pytest.raises(ValueError):
        model.generateGreedy(D.fromHost(prompt), seq)   # positions past the positional table


@pytest.mark.parametrize("use_bf16", [False, True])
def test_decoding_at_the_gpt_small_shape(hip, rng, use_bf16):
    """The decoding path at the widths BASELINE.json's configs[3] names (d_model 768, 12 heads of 64, ffn 3072, vocab 32000,
    12 blocks), where the small cases above do not reach: the walks over 768- and 3072-wide weights, the 32000-wide head
    with four columns a wavefront, the cache of a 150-token prompt.  Size-independent properties: the logits of
    forwardIncremental at each new position equal those of Model::forward over the whole prefix (model.cu:385-424 against
    :174-239; the reference's own check, model_tests.cu:536-611), and generateGreedy returns the argmax tokens of that
    loop."""
    from blackforge_amd import hostlayer as hl
    vocab, dim, seq, heads, hidden, blocks = 32000, 768, 256, 12, 3072, 12
    D = hip.DeviceTensor
    model = hl.HostModel(_lm_layers(hl, vocab, dim, seq, heads, hidden, 1, blocks), use_bf16=use_bf16)
    for i, c in enumerate(model.counts):
        model.set_value(i, rng.standard_normal(c, dtype=f32) * f32(0.02))   # N(0, 0.02), the configuration's initialisation
    prompt = rng.integers(0, vocab, (1, 150)).astype(f32)
    tokens = model.generateGreedy(D.fromHost(prompt), 4)
    model.resetGenerationState()
    ids = prompt
    logits = model.forwardIncremental(D.fromHost(prompt)).reshape(-1, vocab)[-1]
    # bf16 mode: the new position's products add in another order than the full pass's tiles, and one last-bit difference
    # that flips the bf16 rounding of an operand moves the logits by a per cent of their size (measured with the SAME
    # kernels on both sides: scaling one input row by 1 + 3e-7 changes the logits of a model like this one by 1.5e-2 of
    # their rms); with the tile kernels forced on both sides the two agree bit for bit
    tol = BF16_TOL if use_bf16 else 1e-4
    for step, t in enumerate(tokens):
        full = model.forward(D.fromHost(ids)).reshape(-1, vocab)[-1]
        assert_close(logits, full, tol=tol, what=f"incremental logits at position {ids.shape[1] - 1} vs the full forward",
                     scale=float(np.abs(full).max()) if use_bf16 else 0.0)
        best = int(np.argmax(logits))
        assert t == best or logits[best] - logits[t] <= tol * np.abs(logits).max(), f"token {step}: {t} against the loop's argmax {best}"
        ids = np.concatenate([ids, np.array([[t]], f32)], axis=1)
        logits = model.forwardIncremental(D.fromHost(np.array([[t]], f32))).reshape(vocab)
    if use_bf16:   # the same comparison with every product and the attention on the tile kernels: the same additions in the same order
        hip.capi.call("bf_hip_gemm_bf16_set_route", 1)
        hip.capi.call("bf_hip_attention_set_route", 7 | 8)
        try:
            model.resetGenerationState()
            model.forwardIncremental(D.fromHost(ids[:, :-1]))
            last = model.forwardIncremental(D.fromHost(ids[:, -1:])).reshape(vocab)
            assert_bits_equal(last, model.forward(D.fromHost(ids)).reshape(-1, vocab)[-1], "incremental vs full forward on one kernel family")
        finally:
            hip.capi.call("bf_hip_gemm_bf16_set_route", 0)
            hip.capi.call("bf_hip_attention_set_route", 7)


@pytest.mark.parametrize("act", [0, 1])
def test_config1_tiny_lm_full_step_against_oracle(hip, oracle, rng, act):
    """BASELINE config 1 shape: vocab 256, d_model 128, 4 heads, 1 attention + 1 feedforward(512) block, seq 64,
    batch 8; forward, sparse CE, backward, one AdamW step (lr 1e-3, wd 0.01).  act=1 is the GELU variant."""
    from blackforge_amd import hostlayer as hl
    from oracle import bfo
    vocab, dim, seq, batch, heads, hidden = 256, 128, 64, 8, 4, 512
    gpu = hl.HostModel(_lm_layers(hl, vocab, dim, seq, heads, hidden, act))
    cpu = oracle.model(_lm_layers(bfo, vocab, dim, seq, heads, hidden, act))
    assert gpu.names == cpu.names
    for i, c in enumerate(gpu.counts):
        w = r(rng, c, scale=0.02)
        gpu.set_value(i, w)
        cpu.value(i)[:] = w
    D = hip.DeviceTensor
    ids = rng.integers(0, vocab, (batch, seq)).astype(f32)
    tgt = rng.integers(0, vocab, batch * seq).astype(f32)
    cpu.zeroGrad()
    logits = cpu.forward(ids)
    loss, grad = oracle.softmaxCrossEntropySparse(logits.reshape(-1, vocab), tgt)
    cpu.backward(grad)
    gpu.zeroGrad()
    assert_close(gpu.forward(D.fromHost(ids), trusted=True), logits, what="logits")
    gpu.loss(D.fromHost(tgt))
    assert abs(gpu.readLossSum() / (batch * seq) - loss) <= 1e-4 * loss
    gpu.backward(trusted=True)
    for i in range(len(gpu.counts)):
        e = cpu.grad(i)
        assert_close(gpu.grad(i), e, what="grad " + gpu.names[i], scale=float(np.abs(e).max()) * 0.05)
    cpu.adamwStep()
    gpu.adamwStep()
    for i in range(len(gpu.counts)):
        # AdamW's first step is lr * g / (|g| + eps): where |g| is comparable to eps = 1e-8 the step depends on
        # the gradient's last bits, but it never exceeds lr, so the floor is a small fraction (2 %) of lr = 1e-3
        assert_close(gpu.value(i), cpu.value(i), what="param " + gpu.names[i], scale=0.02 * 1e-3 / 1e-4)
    print(f"config 1 step: measured max |gpu - cpu| / max |cpu| over all gradients and parameters: {max(take_worst().values()):.2e}")


@pytest.mark.parametrize("use_bf16", [False, True])
def test_gradients_accumulate_over_backward_passes(hip, rng, use_bf16):
    """cuda::Model::backward adds into the parameters' gradients (model.cu:40-46, 332-383).  The first pass after
    zeroGrad() writes them in place of adding to zeros; a second pass without zeroGrad() must double them, and
    zeroGrad() must bring back the single-pass values."""
    from blackforge_amd import hostlayer as hl
    vocab, dim, seq, batch, heads, hidden = 96, 64, 32, 4, 2, 128
    gpu = hl.HostModel(_lm_layers(hl, vocab, dim, seq, heads, hidden, 0), use_bf16=use_bf16)
    for i, c in enumerate(gpu.counts):
        gpu.set_value(i, r(rng, c, scale=0.05))
    D = hip.DeviceTensor
    x = D.fromHost(rng.integers(0, vocab, (batch, seq)).astype(f32))
    t = D.fromHost(rng.integers(0, vocab, batch * seq).astype(f32))

    def one_pass():
        gpu.forward(x, trusted=True)
        gpu.loss(t)
        gpu.backward(trusted=True)

    gpu.zeroGrad()
    one_pass()
    single = [gpu.grad(i).copy() for i in range(len(gpu.counts))]
    assert any(np.abs(g).max() > 0 for g in single)
    one_pass()
    for i, g in enumerate(single):
        assert_close(gpu.grad(i), 2 * g, tol=1e-6, what="accumulated grad " + gpu.names[i])
    gpu.zeroGrad()
    for i in range(len(gpu.counts)):
        assert not gpu.grad(i).any(), "zeroGrad " + gpu.names[i]
    one_pass()
    for i, g in enumerate(single):
        assert_bits_equal(gpu.grad(i), g, "grad after zeroGrad " + gpu.names[i])


@pytest.mark.parametrize("vocab", [96, 4096, 4099])
def test_bf16_model_step_stays_within_bf16_tolerance(hip, oracle, rng, vocab):
    """bf16 projections (precision.compute = bf16): logits and gradients within 2e-2 of the fp32 CPU reference.  With a
    vocabulary of 4096 the step takes the loss of the language-model head in its fused form (gradient as a bf16 image
    plus the head's bias gradient, no fp32 gradient); with an odd vocabulary of 4099 the form whose image rows are
    padded to a multiple of 8 and whose bias gradient is the image's column sums."""
    from blackforge_amd import hostlayer as hl
    from oracle import bfo
    dim, seq, batch, heads, hidden = 64, 32, 4, 2, 128
    gpu = hl.HostModel(_lm_layers(hl, vocab, dim, seq, heads, hidden, 0), use_bf16=True)
    cpu = oracle.model(_lm_layers(bfo, vocab, dim, seq, heads, hidden, 0))
    for i, c in enumerate(gpu.counts):
        w = r(rng, c, scale=0.05)
        gpu.set_value(i, w)
        cpu.value(i)[:] = w
    D = hip.DeviceTensor
    ids = rng.integers(0, vocab, (batch, seq)).astype(f32)
    tgt = rng.integers(0, vocab, batch * seq).astype(f32)
    logits = cpu.forward(ids)
    loss, grad = oracle.softmaxCrossEntropySparse(logits.reshape(-1, vocab), tgt)
    cpu.zeroGrad()
    cpu.backward(grad)
    x, t = D.fromHost(ids), D.fromHost(tgt)
    gpu.trainStep(x, t, optimizer=0)
    assert abs(gpu.readLossSum() / (batch * seq) - loss) <= BF16_TOL * loss
    for i in range(len(gpu.counts)):
        e = cpu.grad(i)
        assert_close(gpu.grad(i), e, tol=BF16_TOL, what="bf16 grad " + gpu.names[i], scale=float(np.abs(e).max()))


def test_mlp_config2_shape_small(hip, oracle, rng):
    """BASELINE config 2 pipeline (linear -> silu -> linear, MSE) at a reduced width, bf16 projections."""
    from blackforge_amd import hostlayer as hl
    from oracle import bfo
    tokens, width = 256, 192
    layers = lambda m: [(m.LINEAR, width), (m.SILU,), (m.LINEAR, width)]
    gpu = hl.HostModel(layers(hl), input_features=width, use_bf16=True)
    cpu = oracle.model(layers(bfo), input_features=width)
    for i, c in enumerate(gpu.counts):
        w = r(rng, c, scale=width ** -0.5) if gpu.names[i].endswith("weight") else np.zeros(c, f32)
        gpu.set_value(i, w)
        cpu.value(i)[:] = w
    x, y = r(rng, tokens, width), r(rng, tokens, width)
    out = cpu.forward(x)
    loss, grad = oracle.meanSquaredError(out.reshape(tokens, width), y)
    cpu.zeroGrad()
    cpu.backward(grad)
    dx, dy = hip.DeviceTensor.fromHost(x), hip.DeviceTensor.fromHost(y)
    gpu.trainStep(dx, dy, loss_kind=hl.LOSS_MSE, optimizer=0)
    assert abs(gpu.readLossSum() / (tokens * width) - loss) <= BF16_TOL * loss
    for i in range(len(gpu.counts)):
        e = cpu.grad(i)
        assert_close(gpu.grad(i), e, tol=BF16_TOL, what="mlp grad " + gpu.names[i], scale=float(np.abs(e).max()))


@pytest.mark.parametrize("use_bf16", [False, True])
def test_train_steps_do_not_carry_gradients_over(hip, rng, use_bf16):
    """A training step zeroes the gradients by having its backward pass WRITE them (no zeroing pass): the gradients after
    steps on batch A and then batch B must be the bits of a twin model that only ever saw batch B, for every layer kind
    (embedding, positional table, attention, feed-forward, linear head, and a linear-gelu-linear triple on its own model),
    and zeroGrad() on its own must still leave zeros behind."""
    from blackforge_amd import hostlayer as hl
    D = hip.DeviceTensor
    vocab, dim, seq, batch, heads, hidden = 64, 32, 16, 4, 2, 64
    models = []
    for layers, kw in ((_lm_layers(hl, vocab, dim, seq, heads, hidden, 0), {}),
                       ([(hl.LINEAR, 48), (hl.GELU,), (hl.LINEAR, 40), (hl.SILU,), (hl.LINEAR, 24)], {"input_features": 40})):
        a, b = hl.HostModel(layers, use_bf16=use_bf16, **kw), hl.HostModel(layers, use_bf16=use_bf16, **kw)
        for i, c in enumerate(a.counts):
            w = r(rng, c, scale=0.1)
            a.set_value(i, w)
            b.set_value(i, w)
        models.append((a, b, not kw))
    for a, b, is_lm in models:
        def make():
            if is_lm:
                return D.fromHost(rng.integers(0, vocab, (batch, seq)).astype(f32)), D.fromHost(rng.integers(0, vocab, batch * seq).astype(f32)), hl.LOSS_SPARSE_CE
            return D.fromHost(r(rng, 12, 40)), D.fromHost(r(rng, 12, 24)), hl.LOSS_MSE
        xa, ta, kind = make()
        xb, tb, _ = make()
        a.trainStep(xa, ta, kind, optimizer=0)
        a.trainStep(xb, tb, kind, optimizer=0)
        b.trainStep(xb, tb, kind, optimizer=0)
        for i in range(len(a.counts)):
            assert_bits_equal(a.grad(i), b.grad(i), "gradient of " + a.names[i] + " after two steps against one")
        a.zeroGrad()
        for i in range(len(a.counts)):
            assert not a.grad(i).any(), "zeroGrad() leaves zeros: " + a.names[i]
