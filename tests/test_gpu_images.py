"""GPU parity of the bf16 operand images that producers write in place of a separate conversion pass, and of the
projection entry points that consume them.

An image must hold exactly the round-to-nearest-even bf16 of the fp32 values the same kernel writes (checked against the
oracle's roundToBf16 of the fp32 output), and a projection fed an image must give the bits of the same projection fed
the fp32 tensor (which the other GEMM tests hold against the oracle)."""
import ctypes

import numpy as np
import pytest

from parity import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu
f32 = np.float32


def r(rng, *s, scale=1.0):
    return rng.standard_normal(s, dtype=f32) * f32(scale)


def image_of(hip, shape):
    """Raw bf16 storage for a [rows, cols] image."""
    return hip.DeviceTensor(shape, itemsize=2)


def as_f32(image_host):
    return (image_host.astype(np.uint32) << 16).view(f32)


def to_image(hip, host):
    """Device bf16 image of a host fp32 matrix (through the library's own conversion entry point)."""
    t = hip.DeviceTensor.fromHost(host)
    img = image_of(hip, host.shape)
    hip.capi.call("bf_hip_cvt_f32_bf16", t.ptr, img.ptr, host.size, None)
    return img


@pytest.mark.parametrize("rows,features", [(3, 8), (37, 64), (512, 128), (9, 768), (4, 1024), (5, 2048), (3, 8192), (2, 16384), (2, 70000)])
def test_rmsnorm_images(hip, oracle, rng, rows, features):
    D, call = hip.DeviceTensor, hip.capi.call
    x, g, res = r(rng, rows, features, scale=2), r(rng, rows, features), r(rng, rows, features)
    dx, dg, dres = D.fromHost(x), D.fromHost(g), D.fromHost(res)
    out, img = D((rows, features)), image_of(hip, (rows, features))
    call("bf_hip_rmsnorm_img", dx.ptr, out.ptr, img.ptr, rows, features, None)
    plain = hip.ops.rmsnorm(dx).toHost()
    assert_bits_equal(out.toHost(), plain, "rmsnorm fp32 output with an image beside it")
    assert_bits_equal(as_f32(img.toHost()), oracle.roundToBf16(plain), "rmsnorm image")
    only = image_of(hip, (rows, features))
    call("bf_hip_rmsnorm_img", dx.ptr, None, only.ptr, rows, features, None)
    np.testing.assert_array_equal(only.toHost(), img.toHost())
    # backward with the residual gradient joined and the image of the sum
    out2, img2 = D((rows, features)), image_of(hip, (rows, features))
    call("bf_hip_rmsnorm_backward_add_img", dx.ptr, dg.ptr, dres.ptr, out2.ptr, img2.ptr, rows, features, None)
    plain2 = hip.ops.rmsnormBackwardAdd(dx, dg, dres).toHost()
    assert_bits_equal(out2.toHost(), plain2, "rmsnormBackwardAdd with an image beside it")
    assert_bits_equal(as_f32(img2.toHost()), oracle.roundToBf16(plain2), "rmsnormBackwardAdd image")


def test_image_shape_requirements(hip):
    D, call = hip.DeviceTensor, hip.capi.call
    x, out, img = D.zeros((4, 12)), D((4, 12)), image_of(hip, (4, 12))
    with pytest.raises(ValueError, match="multiple of 8"):
        call("bf_hip_rmsnorm_img", x.ptr, out.ptr, img.ptr, 4, 12, None)
    with pytest.raises(ValueError, match="multiple of 8"):
        call("bf_hip_rmsnorm_backward_add_img", x.ptr, x.ptr, None, out.ptr, img.ptr, 4, 12, None)
    call("bf_hip_rmsnorm_img", x.ptr, out.ptr, None, 4, 12, None)   # no image: any width


@pytest.mark.parametrize("batch,heads,seq,hd,old_len", [(2, 2, 70, 32, 0), (1, 3, 129, 64, 0), (2, 2, 40, 128, 0), (1, 2, 200, 24, 0),
                                                        (1, 4, 33, 16, 33), (1, 1, 300, 256, 0)])
@pytest.mark.parametrize("route", ["hand-over", "recompute"])
def test_attention_images(hip, oracle, rng, batch, heads, seq, hd, old_len, route):
    """O with its image; dQ, dK, dV as column slices of one [rows, 3 dim] image with no fp32 gradient written at all."""
    D, call = hip.DeviceTensor, hip.capi.call
    dim, scale = heads * hd, float(f32(1.0) / np.sqrt(f32(hd)))
    q, k, v, go = (r(rng, batch, seq, dim) for _ in range(4))
    dq_, dk_, dv_, dgo = map(D.fromHost, (q, k, v, go))
    fwd = hip.ops.fusedAttentionForward(dq_, dk_, dv_, heads, scale, old_len)
    out, m, l = D((batch, seq, dim)), D((batch, heads, seq)), D((batch, heads, seq))
    out_img = image_of(hip, (batch * seq, dim))
    call("bf_hip_attention_forward_img", dq_.ptr, dk_.ptr, dv_.ptr, out.ptr, out_img.ptr, dim, m.ptr, l.ptr, batch, heads, seq, seq, dim,
         ctypes.c_float(scale), old_len, None)
    assert_bits_equal(out.toHost(), fwd.output.toHost(), "O with an image beside it")
    assert_bits_equal(as_f32(out_img.toHost()).reshape(batch, seq, dim), oracle.roundToBf16(fwd.output.toHost()), "O image")
    hip.capi.call("bf_hip_attention_set_workspace_limit", 0 if route == "recompute" else 2 ** 64 - 1)
    try:
        grad = hip.ops.fusedAttentionBackward(dgo, dq_, dk_, dv_, fwd.output, fwd.m, fwd.l, heads, scale, old_len)
        img = image_of(hip, (batch * seq, 3 * dim))
        base = img.ptr.value
        call("bf_hip_attention_backward_img", dgo.ptr, dq_.ptr, dk_.ptr, dv_.ptr, fwd.output.ptr, fwd.m.ptr, fwd.l.ptr, None, None, None,
             ctypes.c_void_p(base), ctypes.c_void_p(base + 2 * dim), ctypes.c_void_p(base + 4 * dim), 3 * dim, batch, heads, seq, seq, dim,
             ctypes.c_float(scale), old_len, None)
    finally:
        hip.capi.call("bf_hip_attention_set_workspace_limit", 2 ** 64 - 1)
    got = as_f32(img.toHost()).reshape(batch, seq, 3, dim)
    for i, (name, t) in enumerate((("dQ", grad.dQ), ("dK", grad.dK), ("dV", grad.dV))):
        assert_bits_equal(got[:, :, i], oracle.roundToBf16(t.toHost()), name + " image")


@pytest.mark.parametrize("batch,heads,new_len,old_len,hd,kv_rows", [(1, 12, 1, 1023, 64, 1088), (2, 3, 1, 4000, 64, 4001), (3, 2, 8, 300, 128, 1024),
                                                                    (1, 2, 5, 0, 32, 64), (2, 2, 1, 77, 192, 128), (1, 1, 2, 5000, 256, 8192),
                                                                    (1, 3, 4, 130, 48, 200), (70, 4, 1, 200, 16, 256), (1, 2, 1, 0, 8, 1)])
def test_few_queries_over_a_cache_with_room_to_grow(hip, oracle, rng, batch, heads, new_len, old_len, hd, kv_rows):
    """bf_hip_attention_forward_rows: the forward pass of fusedAttentionForward (fused_attention.cu:297) over K and V that
    lie in buffers of kv_rows rows per sequence (hip::KVCache).  At most eight queries are served by a walk over the
    cache instead of the tile kernels: compared with the oracle, with the tile kernels on the same operands, and with
    rows past totalLen holding NaN, which no kernel may read; the output image is the rounded output."""
    D, call = hip.DeviceTensor, hip.capi.call
    dim, total, scale = heads * hd, old_len + new_len, float(f32(1.0) / np.sqrt(f32(hd)))
    q, k, v = r(rng, batch, new_len, dim), r(rng, batch, total, dim), r(rng, batch, total, dim)
    wide_k, wide_v = (np.full((batch, kv_rows, dim), np.nan, f32) for _ in range(2))
    wide_k[:, :total], wide_v[:, :total] = k, v
    dq_, dk_, dv_ = map(D.fromHost, (q, wide_k, wide_v))

    def run(with_image):
        out, m, l = D((batch, new_len, dim)), D((batch, heads, new_len)), D((batch, heads, new_len))
        img = image_of(hip, (batch * new_len, dim)) if with_image else None
        call("bf_hip_attention_forward_rows", dq_.ptr, dk_.ptr, dv_.ptr, out.ptr, img.ptr if img else None, dim if img else 0, m.ptr, l.ptr, batch,
             heads, new_len, total, kv_rows, dim, ctypes.c_float(scale), old_len, None)
        return out.toHost(), m.toHost(), l.toHost(), (as_f32(img.toHost()).reshape(batch, new_len, dim) if img else None)

    o, m, l, img = run(True)
    eo, em, el = oracle.attentionCoreForward(q, k, v, heads, scale, old_len)
    for got, exp, name in ((o, eo, "O"), (m, em, "m"), (l, el, "l")):
        assert_close(got, exp, what=f"{name} from the walk over the cache")
    assert_bits_equal(img, oracle.roundToBf16(o), "O image")
    o2, m2, l2, _ = run(False)
    for got, exp, name in ((o2, o, "O"), (m2, m, "m"), (l2, l, "l")):
        assert_bits_equal(got, exp, f"{name} of the same call again, without the image")
    call("bf_hip_attention_set_route", 7 | 8)   # the default products, tile kernels only
    try:
        to, tm, tl, timg = run(True)
    finally:
        call("bf_hip_attention_set_route", 7)
    for got, exp, name in ((to, o, "O"), (tm, m, "m"), (tl, l, "l")):
        assert_close(got, exp, tol=2e-5, what=f"{name}: tile kernels against the walk")
    assert_bits_equal(timg, oracle.roundToBf16(to), "O image of the tile kernels")


@pytest.mark.parametrize("m,d,hidden,act", [(1, 768, 3072, 1), (3, 72, 264, 0), (8, 1032, 520, 2), (1, 8, 8, 1), (2, 256, 256, 0), (9, 64, 128, 1), (2, 40000, 64, 2),
                                            (8, 8200, 64, 0), (40, 128, 512, 1)])
def test_blocks_of_a_decoding_step_normalise_inside_the_product(hip, oracle, rng, m, d, hidden, act):
    """bf_hip_rmsnorm_matmul_bf16_shared_input and bf_hip_rmsnorm_feedforward_bf16 (the projections and the feed-forward
    block of selfAttentionIncremental / forwardIncremental, ops_transformer.cu:133-215) against the separate operators
    (rmsnorm, then the bf16 products): one or two rows normalise inside the product's kernel, more rows (and rows too long
    for that kernel's LDS) run the row kernel first.  Same arithmetic either way; the sum of squares is taken in another
    order, so the agreement is to the last bits, not bit for bit."""
    D, ops, call = hip.DeviceTensor, hip.ops, hip.capi.call
    x = r(rng, m, d, scale=2.0)
    normed = ops.rmsnorm(D.fromHost(x))
    assert_close(normed.toHost(), oracle.rmsnorm(x), tol=1e-5, what="rmsnorm")
    for count, n in ((3, 256), (3, hidden), (1, hidden), (2, 512)):
        ws = [r(rng, d, n, scale=0.1) for _ in range(count)]
        dws = [D.fromHost(w) for w in ws]
        outs = [D((m, n)) for _ in range(count)]
        barr = (ctypes.c_void_p * count)(*[w.ptr for w in dws])
        carr = (ctypes.c_void_p * count)(*[o.ptr for o in outs])
        dx = D.fromHost(x)
        call("bf_hip_rmsnorm_matmul_bf16_shared_input", dx.ptr, barr, carr, count, m, d, n, 0, None)
        for i in range(count):
            assert_close(outs[i].toHost(), ops.matmulBf16(normed, dws[i]).toHost(), tol=2e-5, what=f"projection {i} of {count} of the normalised rows")
    w1, b1, w2, b2 = r(rng, d, hidden, scale=0.1), r(rng, hidden, scale=0.5), r(rng, hidden, d, scale=0.1), r(rng, d)
    dw1, db1, dw2, db2, dx = map(D.fromHost, (w1, b1, w2, b2, x))
    out = D((m, d))
    call("bf_hip_rmsnorm_feedforward_bf16", dx.ptr, dw1.ptr, db1.ptr, dw2.ptr, db2.ptr, act, out.ptr, m, d, hidden, 0, None)
    expected, _, _, _ = ops.feedForwardBf16Fused(normed, dw1, db1, dw2, db2, dx, act)
    assert_close(out.toHost(), expected.toHost(), tol=2e-5, what="feed-forward block of a decoding step")
    again = D((m, d))
    call("bf_hip_rmsnorm_feedforward_bf16", dx.ptr, dw1.ptr, db1.ptr, dw2.ptr, db2.ptr, act, again.ptr, m, d, hidden, 0, None)
    assert_bits_equal(again.toHost(), out.toHost(), "the same block twice")
    # the fp32 forms of the two blocks (bf_hip_rmsnorm_matmul_f32_shared_input, bf_hip_rmsnorm_feedforward_f32)
    for count, n in ((3, hidden), (1, 41)):
        ws = [r(rng, d, n, scale=0.1) for _ in range(count)]
        dws = [D.fromHost(w) for w in ws]
        outs = [D((m, n)) for _ in range(count)]
        barr = (ctypes.c_void_p * count)(*[w.ptr for w in dws])
        carr = (ctypes.c_void_p * count)(*[o.ptr for o in outs])
        call("bf_hip_rmsnorm_matmul_f32_shared_input", dx.ptr, barr, carr, count, m, d, n, None)
        for i in range(count):
            assert_close(outs[i].toHost(), ops.matmul(normed, dws[i]).toHost(), tol=2e-5, what=f"fp32 projection {i} of {count} of the normalised rows")
    out32 = D((m, d))
    call("bf_hip_rmsnorm_feedforward_f32", dx.ptr, dw1.ptr, db1.ptr, dw2.ptr, db2.ptr, act, out32.ptr, m, d, hidden, None)
    hidden32 = ops.addBiasAct(ops.matmul(normed, dw1), db1, act)
    expected32 = ops.addBiasResidual(ops.matmul(hidden32, dw2), db2, dx)
    assert_close(out32.toHost(), expected32.toHost(), tol=2e-5, what="fp32 feed-forward block of a decoding step")
    if act != 2:   # the CPU backend's block knows silu and gelu
        assert_close(out32.toHost(), oracle.feedForward(x, w1, b1, w2, b2, act), what="fp32 feed-forward block vs the CPU backend's")


@pytest.mark.parametrize("batch,new_len,dim", [(1, 1, 768), (1, 2, 256), (1, 1, 72), (2, 1, 256), (1, 3, 512), (3, 2, 40)])
def test_projections_of_a_decoding_step_at_a_position_on_the_device(hip, oracle, rng, batch, new_len, dim):
    """bf_hip_decode_projections_{bf16,f32}: q, k and v of selfAttentionIncremental (ops_transformer.cu:133-160: rmsnorm,
    three projections, the new keys and values joined to the cache) with the cache's length read from device memory.  One
    sequence of one or two rows takes the single launch that stores keys and values in place, the other cases the scratch
    rows and the append; both against the separate operators, the rest of the caches untouched, rows that would not fit
    not written."""
    D, ops, call = hip.DeviceTensor, hip.ops, hip.capi.call
    capacity, at = 9, 4
    x = r(rng, batch * new_len, dim, scale=2.0)
    ws = [r(rng, dim, dim, scale=0.1) for _ in range(3)]
    dx, dws = D.fromHost(x), [D.fromHost(w) for w in ws]
    normed = ops.rmsnorm(dx)
    position = D.fromHost(np.array([at], np.int32).view(f32))
    for mode in ("bf16", "f32"):
        kc, vc = r(rng, batch, capacity, dim), r(rng, batch, capacity, dim)
        dk, dv, q = D.fromHost(kc), D.fromHost(vc), D((batch * new_len, dim))
        args = [dx.ptr, dws[0].ptr, dws[1].ptr, dws[2].ptr, q.ptr, dk.ptr, dv.ptr, batch, new_len, dim, capacity, position.ptr]
        call("bf_hip_decode_projections_" + mode, *(args + ([0] if mode == "bf16" else []) + [None]))
        product = ops.matmulBf16 if mode == "bf16" else ops.matmul
        eq, ek, ev = (product(normed, w).toHost() for w in dws)
        assert_close(q.toHost(), eq, tol=2e-5, what=f"{mode} q")
        gk, gv = dk.toHost(), dv.toHost()
        assert_close(gk[:, at:at + new_len].reshape(-1, dim), ek, tol=2e-5, what=f"{mode} keys at the device-side position")
        assert_close(gv[:, at:at + new_len].reshape(-1, dim), ev, tol=2e-5, what=f"{mode} values at the device-side position")
        keep = np.ones(capacity, bool)
        keep[at:at + new_len] = False
        assert_bits_equal(gk[:, keep], kc[:, keep], f"{mode}: the other rows of the key cache")
        assert_bits_equal(gv[:, keep], vc[:, keep], f"{mode}: the other rows of the value cache")
        full = D.fromHost(np.array([capacity - new_len + 1], np.int32).view(f32))   # the last new row would not fit
        before = dk.toHost()
        args[-1] = full.ptr
        call("bf_hip_decode_projections_" + mode, *(args + ([0] if mode == "bf16" else []) + [None]))
        after = dk.toHost()
        assert_bits_equal(after[:, :capacity - new_len + 1], before[:, :capacity - new_len + 1], f"{mode}: rows below a position that does not fit")


@pytest.mark.parametrize("rows,classes", [(5, 16), (7, 1000), (300, 256), (3, 32000), (2, 40000)])
def test_cross_entropy_gradient_image(hip, oracle, rng, rows, classes):
    D, call = hip.DeviceTensor, hip.capi.call
    logits = r(rng, rows, classes, scale=3)
    idx = rng.integers(0, classes, rows).astype(f32)
    dl, di = D.fromHost(logits), D.fromHost(idx)
    plain = hip.ops.softmaxCrossEntropySparse(dl, di)
    grad, img, loss = D((rows, classes)), image_of(hip, (rows, classes)), D.zeros((1,))
    call("bf_hip_cross_entropy_sparse_img", dl.ptr, di.ptr, grad.ptr, img.ptr, loss.ptr, rows, classes, 0, None)
    assert_bits_equal(grad.toHost(), plain.grad.toHost(), "CE gradient with an image beside it")
    assert_bits_equal(as_f32(img.toHost()), oracle.roundToBf16(plain.grad.toHost()), "CE gradient image")
    assert abs(loss.toHost()[0] / rows - plain.value) <= 1e-6 * abs(plain.value)
    with pytest.raises(ValueError, match="multiple of 8"):
        call("bf_hip_cross_entropy_sparse_img", dl.ptr, di.ptr, grad.ptr, img.ptr, loss.ptr, rows, classes - 4, 0, None)


@pytest.mark.parametrize("rows,classes", [(3, 4096), (700, 4104), (5, 16384), (1100, 16392), (9, 32000), (600, 32768), (1, 8192)])
def test_cross_entropy_of_a_language_model_head(hip, oracle, rng, rows, classes):
    """bf_hip_cross_entropy_sparse_head: the loss and the gradient image of bf_hip_cross_entropy_sparse_img (bit for bit
    where that kernel holds a row the same way) without the fp32 gradient, and the gradient's column sums (the head's bias gradient) against float64 sums of the
    oracle's gradient.  Row counts below and above the number of workgroups that walk the rows (one partial row of
    column sums per workgroup), class counts at both register plans, their upper ends, and just past a multiple of 4096."""
    D, call = hip.DeviceTensor, hip.capi.call
    logits = r(rng, rows, classes, scale=3)
    idx = rng.integers(0, classes, rows).astype(f32)
    idx[0], idx[-1] = 0, classes - 1
    dl, di = D.fromHost(logits), D.fromHost(idx)
    grad, img, loss = D((rows, classes)), image_of(hip, (rows, classes)), D.zeros((1,))
    call("bf_hip_cross_entropy_sparse_img", dl.ptr, di.ptr, grad.ptr, img.ptr, loss.ptr, rows, classes, 0, None)
    img2, bias, loss2 = image_of(hip, (rows, classes)), D.fromHost(np.full(classes, 7.0, f32)), D.fromHost(np.array([2.5], f32))
    call("bf_hip_cross_entropy_sparse_head", dl.ptr, di.ptr, img2.ptr, bias.ptr, loss2.ptr, rows, classes, 1, None)
    if classes > 8192:   # the separate kernel holds such rows the same way (1024 threads a row): the same bits
        np.testing.assert_array_equal(img2.toHost(), img.toHost(), err_msg="gradient image")
        assert loss2.toHost()[0] == np.float32(2.5) + loss.toHost()[0], "the loss is added to the accumulator"
    else:                # shorter rows are summed in another order there: the same values to an fp32 rounding
        a, b = as_f32(img2.toHost()).astype(np.float64), as_f32(img.toHost()).astype(np.float64)
        assert (np.abs(a - b) <= 2.0 ** -7 * np.abs(b)).all(), "gradient image: more than one bf16 step apart"
        assert (a != b).mean() < 1e-3, "gradient image: too many values on the other side of a rounding boundary"
        assert abs(loss2.toHost()[0] - 2.5 - loss.toHost()[0]) <= 1e-6 * abs(loss.toHost()[0]) + 1e-6
    expected_loss, expected_grad = oracle.softmaxCrossEntropySparse(logits, idx)
    assert abs(loss.toHost()[0] / rows - expected_loss) <= 1e-5 * abs(expected_loss)
    sums = expected_grad.astype(np.float64).sum(axis=0)
    assert_close(bias.toHost(), sums.astype(f32), tol=1e-4, what="column sums of the gradient", scale=float(np.abs(expected_grad).max()))


@pytest.mark.parametrize("rows,classes,offset", [(3, 50257, 0), (300, 50257, 0), (5, 40000, 0), (64, 4099, 0), (130, 53248, 0), (7, 4100, 0),
                                                 (33, 8192, 1), (2, 53241, 3),
                                                 # rows longer than a block's registers: walked twice
                                                 (3, 53249, 0), (40, 128256, 0), (2, 151937, 1), (1, 256000, 0)])
def test_cross_entropy_of_a_head_with_an_odd_or_large_vocabulary(hip, oracle, rng, rows, classes, offset):
    """bf_hip_cross_entropy_sparse_head beyond its one-pass form (class counts that are not multiples of 8, more than
    32768 classes up to vocabularies of 256000 words, logits that do not start on a 16-byte boundary): the loss, the gradient image in rows of classes
    rounded up to 8 (the padding zero), within one bf16 step of the rounded fp32 gradient of bf_hip_cross_entropy_sparse,
    and as bias gradient the column sums of that image."""
    D, call = hip.DeviceTensor, hip.capi.call
    logits = r(rng, rows, classes, scale=3)
    idx = rng.integers(0, classes, rows).astype(f32)
    idx[0], idx[-1] = 0, classes - 1
    flat = np.concatenate([np.zeros(offset, f32), logits.ravel()])
    dflat, di = D.fromHost(flat), D.fromHost(idx)
    at = ctypes.c_void_p(dflat.ptr.value + 4 * offset)   # the logits start `offset` floats into the allocation
    grad, loss = D((rows, classes)), D.zeros((1,))
    call("bf_hip_cross_entropy_sparse", at, di.ptr, grad.ptr, loss.ptr, rows, classes, 0, None)
    pitch = (classes + 7) // 8 * 8
    img = D.fromHost(np.full((rows, pitch // 2), 7.0, f32))   # raw storage of the image, filled with something else
    bias, loss2 = D.fromHost(np.full(classes, 7.0, f32)), D.fromHost(np.array([2.5], f32))
    call("bf_hip_cross_entropy_sparse_head", at, di.ptr, img.ptr, bias.ptr, loss2.ptr, rows, classes, 1, None)
    image = as_f32(img.toHost().view(np.uint16).reshape(rows, pitch)).astype(np.float64)
    assert (image[:, classes:] == 0).all(), "the columns past the row are zero"
    g = grad.toHost().astype(np.float64)
    assert (np.abs(image[:, :classes] - g) <= 2.0 ** -8 * np.abs(g) + 1e-30).all(), "gradient image: more than half a bf16 step from the fp32 gradient"
    assert abs(loss2.toHost()[0] - 2.5 - loss.toHost()[0]) <= 1e-6 * abs(loss.toHost()[0]) + 1e-6
    expected_loss, expected_grad = oracle.softmaxCrossEntropySparse(logits, idx)
    assert abs(loss.toHost()[0] / rows - expected_loss) <= 1e-5 * abs(expected_loss)
    sums = image[:, :classes].sum(axis=0)
    assert_close(bias.toHost(), sums.astype(f32), tol=1e-5, what="column sums of the image", scale=float(np.abs(image).max()))
    exact = expected_grad.astype(np.float64).sum(axis=0)   # the bias gradient proper: within the rounding of its terms
    room = 2.0 ** -8 * np.abs(expected_grad).astype(np.float64).sum(axis=0) + 1e-12
    assert (np.abs(bias.toHost() - exact) <= room).all(), "bias gradient: further from the fp32 sums than the rounding of the terms allows"


def test_cross_entropy_head_refuses_what_it_does_not_serve(hip, rng):
    D, call = hip.DeviceTensor, hip.capi.call
    for rows, classes in ((4, 1000), (4, 4095), (1, (1 << 20) + 8)):
        dl, di = D.fromHost(r(rng, rows, classes)), D.fromHost(np.zeros(rows, f32))
        img, bias, loss = image_of(hip, (rows, classes + 8)), D((classes,)), D.zeros((1,))
        with pytest.raises(Exception, match="not served"):
            call("bf_hip_cross_entropy_sparse_head", dl.ptr, di.ptr, img.ptr, bias.ptr, loss.ptr, rows, classes, 0, None)
    dl, di = D.fromHost(r(rng, 4, 8192)), D.fromHost(np.zeros(4, f32))
    img, bias, loss = image_of(hip, (4, 8200)), D((8192,)), D.zeros((1,))
    with pytest.raises(Exception, match="not served"):   # an image that does not start on a 16-byte boundary
        call("bf_hip_cross_entropy_sparse_head", dl.ptr, di.ptr, ctypes.c_void_p(img.ptr.value + 2), bias.ptr, loss.ptr, 4, 8192, 0, None)


# (m, k, n): the small-tile route with transposed images, a ragged one, and the large-tile routes (fragments transposed in LDS)
GEMM_SHAPES = [(64, 40, 24), (300, 72, 520), (4100, 136, 264), (8192, 256, 768), (6001, 520, 1032)]


@pytest.mark.parametrize("m,k,n", GEMM_SHAPES)
def test_projections_fed_with_images(hip, rng, m, k, n):
    """linear, its two gradients: fp32 operands against the same operands as bf16 images, bit for bit."""
    D, call = hip.DeviceTensor, hip.capi.call
    a, w, g, bias, res = r(rng, m, k), r(rng, k, n, scale=0.1), r(rng, m, n), r(rng, n), r(rng, m, n)
    da, dw, dg, db, dres = map(D.fromHost, (a, w, g, bias, res))
    a_img, g_img = to_image(hip, a), to_image(hip, g)
    out0, out1 = D((m, n)), D((m, n))
    call("bf_hip_linear_bf16", da.ptr, dw.ptr, db.ptr, dres.ptr, out0.ptr, m, k, n, 0, None)
    call("bf_hip_linear_bf16_img", None, a_img.ptr, dw.ptr, db.ptr, dres.ptr, out1.ptr, m, k, n, 0, None)
    assert_bits_equal(out1.toHost(), out0.toHost(), "linear from an image")
    dA0, dB0, dA1, dB1 = D((m, k)), D((k, n)), D((m, k)), D((k, n))
    call("bf_hip_matmul_bf16_backward", da.ptr, dw.ptr, dg.ptr, dA0.ptr, dB0.ptr, m, k, n, 0, None)
    call("bf_hip_matmul_bf16_backward_img", None, a_img.ptr, dw.ptr, None, g_img.ptr, dA1.ptr, dB1.ptr, m, k, n, 0, None)
    assert_bits_equal(dA1.toHost(), dA0.toHost(), "dA from images")
    assert_bits_equal(dB1.toHost(), dB0.toHost(), "dB from images")
    # mixed: one operand as an image, the other in fp32; and a single gradient requested
    call("bf_hip_matmul_bf16_backward_img", da.ptr, None, dw.ptr, dg.ptr, g_img.ptr, dA1.ptr, dB1.ptr, m, k, n, 0, None)
    assert_bits_equal(dB1.toHost(), dB0.toHost(), "dB from the gradient's image and the fp32 input")
    only = D((k, n))
    call("bf_hip_matmul_bf16_backward_img", None, a_img.ptr, dw.ptr, None, g_img.ptr, None, only.ptr, m, k, n, 0, None)
    assert_bits_equal(only.toHost(), dB0.toHost(), "dB alone from images")


@pytest.mark.parametrize("m,k,n,count", [(50, 40, 24, 3), (300, 136, 256, 3), (4100, 256, 256, 3), (8192, 520, 256, 3), (260, 72, 512, 2),
                                         (64, 32, 48, 1)])
def test_shared_input_projections_fed_with_images(hip, rng, m, k, n, count):
    D, call = hip.DeviceTensor, hip.capi.call
    a = r(rng, m, k)
    ws = [r(rng, k, n, scale=0.1) for _ in range(count)]
    gs = [r(rng, m, n) for _ in range(count)]
    da, dws, dgs = D.fromHost(a), [D.fromHost(w) for w in ws], [D.fromHost(g) for g in gs]
    arr = lambda ts: (ctypes.c_void_p * count)(*[t.ptr for t in ts])
    a_img = to_image(hip, a)
    g_img = to_image(hip, np.concatenate(gs, axis=1))   # side by side: [m, count * n]
    c0, c1 = [D((m, n)) for _ in range(count)], [D((m, n)) for _ in range(count)]
    call("bf_hip_matmul_bf16_shared_input", da.ptr, arr(dws), arr(c0), count, m, k, n, 0, None)
    call("bf_hip_matmul_bf16_shared_input_img", None, a_img.ptr, arr(dws), arr(c1), count, m, k, n, 0, None)
    for x, y in zip(c0, c1):
        assert_bits_equal(y.toHost(), x.toHost(), "shared-input product from an image")
    dA0, dA1 = D((m, k)), D((m, k))
    dB0, dB1 = [D((k, n)) for _ in range(count)], [D((k, n)) for _ in range(count)]
    call("bf_hip_matmul_bf16_shared_input_backward", da.ptr, arr(dws), arr(dgs), dA0.ptr, arr(dB0), count, m, k, n, 0, None)
    call("bf_hip_matmul_bf16_shared_input_backward_img", None, a_img.ptr, arr(dws), None, g_img.ptr, dA1.ptr, arr(dB1), count, m, k, n, 0, None)
    assert_bits_equal(dA1.toHost(), dA0.toHost(), "dA from images")
    for x, y in zip(dB0, dB1):
        assert_bits_equal(y.toHost(), x.toHost(), "dB from images")


@pytest.mark.parametrize("m,d,hidden,act", [(64, 32, 128, 0), (300, 72, 264, 1), (4096, 256, 1024, 0), (8192, 768, 3072, 1)])
def test_feed_forward_fed_with_images(hip, rng, m, d, hidden, act):
    D, ops, call = hip.DeviceTensor, hip.ops, hip.capi.call
    x, w1, b1 = r(rng, m, d), r(rng, d, hidden, scale=0.1), r(rng, hidden, scale=0.5)
    w2, b2, res, g = r(rng, hidden, d, scale=0.1), r(rng, d), r(rng, m, d), r(rng, m, d)
    dx, dw1, db1, dw2, db2, dres, dg = map(D.fromHost, (x, w1, b1, w2, b2, res, g))
    out0, z0, h0, xi0 = ops.feedForwardBf16Fused(dx, dw1, db1, dw2, db2, dres, act)
    x_img, g_img = to_image(hip, x), to_image(hip, g)
    z1, h1, out1 = D((m, hidden)), D((m, hidden // 2)), D((m, d))
    call("bf_hip_feedforward_bf16", None, dw1.ptr, db1.ptr, dw2.ptr, db2.ptr, dres.ptr, act, z1.ptr, h1.ptr, x_img.ptr, out1.ptr, m, d, hidden, 0, None)
    assert_bits_equal(out1.toHost(), out0.toHost(), "feed-forward from the input's image")
    assert_bits_equal(z1.toHost(), z0.toHost(), "pre-activation from the input's image")
    ref = ops.feedForwardBf16FusedBackward(dx, None, dw1, dw2, z0, h0, dg, act)
    outs = [D((m, d)), D(w1.shape), D((hidden,)), D(w2.shape), D((d,))]
    call("bf_hip_feedforward_bf16_backward_img", None, x_img.ptr, dw1.ptr, dw2.ptr, z0.ptr, h0.ptr, dg.ptr, g_img.ptr, act,
         *[t.ptr for t in outs], m, d, hidden, 0, None)
    for got, exp, name in zip(outs, ref, ("dX", "dW1", "dB1", "dW2", "dB2")):
        assert_bits_equal(got.toHost(), exp.toHost(), name + " from images")
    # without the fp32 gradient only the bias gradient of the second projection is unavailable
    outs2 = [D((m, d)), D(w1.shape), D((hidden,)), D(w2.shape)]
    call("bf_hip_feedforward_bf16_backward_img", None, x_img.ptr, dw1.ptr, dw2.ptr, z0.ptr, h0.ptr, None, g_img.ptr, act,
         *[t.ptr for t in outs2], None, m, d, hidden, 0, None)
    for got, exp, name in zip(outs2, ref, ("dX", "dW1", "dB1", "dW2")):
        assert_bits_equal(got.toHost(), exp.toHost(), name + " from the gradient image alone")
    with pytest.raises(ValueError, match="dB2"):
        call("bf_hip_feedforward_bf16_backward_img", None, x_img.ptr, dw1.ptr, dw2.ptr, z0.ptr, h0.ptr, None, g_img.ptr, act,
             *[t.ptr for t in outs], m, d, hidden, 0, None)


def in_use(hip):
    stats = hip.capi.PoolStats()
    hip.capi.call("bf_hip_pool_stats", ctypes.byref(stats))
    return stats.bytes_in_use


def test_weight_image_cache_fills_pairs_and_lets_go_of_idle_weights(hip, rng):
    """The cached forward image of a weight comes with the plain image its input-gradient product reads (same bits as
    the uncached route); images of weights that sat out a whole generation go back to the pool."""
    D, call = hip.DeviceTensor, hip.capi.call
    m, k, n = 300, 136, 264
    a, w, g = r(rng, m, k), r(rng, k, n, scale=0.1), r(rng, m, n)
    da, dw, dg = map(D.fromHost, (a, w, g))
    call("bf_hip_invalidate_bf16_weight_cache")
    call("bf_hip_invalidate_bf16_weight_cache")   # two in a row: nothing of earlier tests is left in the cache
    out0, out1, dA0, dA1 = D((m, n)), D((m, n)), D((m, k)), D((m, k))
    base = in_use(hip)   # the pool counts whole size classes, so compare levels rather than sums of tensor sizes
    call("bf_hip_linear_bf16", da.ptr, dw.ptr, None, None, out0.ptr, m, k, n, 0, None)
    assert in_use(hip) == base, "the uncached route returns its images"
    call("bf_hip_linear_bf16", da.ptr, dw.ptr, None, None, out1.ptr, m, k, n, 1, None)
    assert_bits_equal(out1.toHost(), out0.toHost(), "linear with a cached weight image")
    assert in_use(hip) - base >= 2 * (k * n * 2), "the transposed image and its plain counterpart are both held"
    call("bf_hip_matmul_bf16_backward", da.ptr, dw.ptr, dg.ptr, dA0.ptr, None, m, k, n, 0, None)
    before = in_use(hip)
    call("bf_hip_matmul_bf16_backward", da.ptr, dw.ptr, dg.ptr, dA1.ptr, None, m, k, n, 1, None)
    assert in_use(hip) == before, "the plain image was there already"
    assert_bits_equal(dA1.toHost(), dA0.toHost(), "dA from the plain image that the forward pass left")
    # the weights change (an optimizer step): the next forward must not be served the old image
    w2 = r(rng, k, n, scale=0.1)
    hip.capi.call("bf_hip_memcpy_h2d", dw.ptr, w2.ctypes.data_as(ctypes.c_void_p), w2.nbytes)
    call("bf_hip_invalidate_bf16_weight_cache")
    call("bf_hip_linear_bf16", da.ptr, dw.ptr, None, None, out0.ptr, m, k, n, 0, None)
    call("bf_hip_linear_bf16", da.ptr, dw.ptr, None, None, out1.ptr, m, k, n, 1, None)
    assert_bits_equal(out1.toHost(), out0.toHost(), "linear after the weights changed")
    call("bf_hip_matmul_bf16_backward", da.ptr, dw.ptr, dg.ptr, dA0.ptr, None, m, k, n, 0, None)
    call("bf_hip_matmul_bf16_backward", da.ptr, dw.ptr, dg.ptr, dA1.ptr, None, m, k, n, 1, None)
    assert_bits_equal(dA1.toHost(), dA0.toHost(), "dA after the weights changed")
    # a generation in which nobody asks for them, and the images are returned
    call("bf_hip_invalidate_bf16_weight_cache")
    call("bf_hip_invalidate_bf16_weight_cache")
    assert in_use(hip) == base, "only this test's own tensors are still checked out"


def test_weight_images_refreshed_in_one_launch_after_an_update(hip, rng):
    """bf_hip_bf16_weight_cache_refresh after weights changed in place: the images of the listed weights (single weights
    of aligned and odd shapes, and a group of three that share an input) are made again at the call, bit for bit what a
    fresh conversion gives; a weight left out of the list is only invalidated."""
    D, call = hip.DeviceTensor, hip.capi.call
    m = 200
    shapes = [(136, 264), (77, 50), (64, 512), (130, 8)]
    a = {k: D.fromHost(r(rng, m, k)) for k in {s[0] for s in shapes} | {128}}
    singles = [D.fromHost(r(rng, k, n, scale=0.1)) for k, n in shapes]
    group = [D.fromHost(r(rng, 128, 96, scale=0.1)) for _ in range(3)]
    wide_group = [D.fromHost(r(rng, 128, 256, scale=0.1)) for _ in range(3)]   # stacked images: one product for the three
    left_out = D.fromHost(r(rng, 136, 264, scale=0.1))
    arr = lambda ts: (ctypes.c_void_p * len(ts))(*[t.ptr for t in ts])

    def run(cached):
        outs = []
        for (k, n), w in zip(shapes, singles):
            out, dA = D((m, n)), D((m, k))
            call("bf_hip_linear_bf16", a[k].ptr, w.ptr, None, None, out.ptr, m, k, n, cached, None)
            call("bf_hip_matmul_bf16_backward", a[k].ptr, w.ptr, out.ptr, dA.ptr, None, m, k, n, cached, None)
            outs += [out.toHost(), dA.toHost()]
        cs = [D((m, 96)) for _ in range(3)]
        call("bf_hip_matmul_bf16_shared_input", a[128].ptr, arr(group), arr(cs), 3, m, 128, 96, cached, None)
        dA, dBs = D((m, 128)), [D((128, 96)) for _ in range(3)]
        call("bf_hip_matmul_bf16_shared_input_backward", a[128].ptr, arr(group), arr(cs), dA.ptr, arr(dBs), 3, m, 128, 96, cached, None)
        outs += [c.toHost() for c in cs] + [dA.toHost()]
        cs = [D((m, 256)) for _ in range(3)]
        call("bf_hip_matmul_bf16_shared_input", a[128].ptr, arr(wide_group), arr(cs), 3, m, 128, 256, cached, None)
        dA, dBs = D((m, 128)), [D((128, 256)) for _ in range(3)]
        call("bf_hip_matmul_bf16_shared_input_backward", a[128].ptr, arr(wide_group), arr(cs), dA.ptr, arr(dBs), 3, m, 128, 256, cached, None)
        outs += [c.toHost() for c in cs] + [dA.toHost()]
        out = D((m, 264))
        call("bf_hip_linear_bf16", a[136].ptr, left_out.ptr, None, None, out.ptr, m, 136, 264, cached, None)
        return outs + [out.toHost()]

    def rewrite(tensors):
        for t in tensors:
            fresh = r(rng, *t.shape, scale=0.1)
            call("bf_hip_memcpy_h2d", t.ptr, fresh.ctypes.data_as(ctypes.c_void_p), fresh.nbytes)

    call("bf_hip_invalidate_bf16_weight_cache")
    for got, exp in zip(run(1), run(0)):
        assert_bits_equal(got, exp, "cached images before the update")
    everything = singles + group + wide_group + [left_out]
    rewrite(everything)   # "an optimizer step"
    listed = singles + group + wide_group + [a[128]]   # a tensor that has no image may be in the list; left_out is not
    call("bf_hip_bf16_weight_cache_refresh", arr(listed), len(listed), None)
    expected = run(0)
    # the images were made AT the call: weights rewritten behind the cache's back afterwards do not show in the cached
    # route until the next invalidation (left_out, only invalidated, converts at its next use and does show them)
    rewrite(singles + group + wide_group)
    got = run(1)
    for i, (g, e) in enumerate(zip(got[:-1], expected[:-1])):
        assert_bits_equal(g, e, f"result {i} from the images made by the refresh")
    assert_bits_equal(got[-1], expected[-1], "a weight that was not listed is converted again at its next use")
    call("bf_hip_invalidate_bf16_weight_cache")
    for g, e in zip(run(1), run(0)):
        assert_bits_equal(g, e, "after the next invalidation the cache follows the weights again")
    call("bf_hip_bf16_weight_cache_refresh", None, 0, None)   # an empty list only invalidates
    call("bf_hip_invalidate_bf16_weight_cache")


@pytest.mark.parametrize("m,d,hidden,act", [(2048, 256, 3072, 1), (2000, 264, 3080, 0), (4096, 1024, 4096, 0), (3000, 128, 2304, 2),
                                            (8192, 768, 3072, 1)])
def test_feed_forward_activation_fused_into_the_products(hip, rng, m, d, hidden, act):
    """Products large enough for the one-tile-per-workgroup kernels write the activation's image (forward) and
    bf16(dH . act'(z)) with its column sums (backward) from their own store.  A kernel named by the caller keeps the
    separate passes: z, the image of act(z) and the weight gradients (dW1 is made from the image of dz) must have the
    same bits either way; the bias gradient dB1 adds its rows in another order."""
    D, call = hip.DeviceTensor, hip.capi.call
    x, w1, b1 = r(rng, m, d), r(rng, d, hidden, scale=0.1), r(rng, hidden, scale=0.5)
    w2, b2, res, g = r(rng, hidden, d, scale=0.1), r(rng, d), r(rng, m, d), r(rng, m, d)
    dx, dw1, db1, dw2, db2, dres, dg = map(D.fromHost, (x, w1, b1, w2, b2, res, g))

    def run(route):
        call("bf_hip_gemm_bf16_set_route", route)
        try:
            z, h, xi, out = D((m, hidden)), D((m, hidden // 2)), D((m, d // 2)), D((m, d))
            call("bf_hip_feedforward_bf16", dx.ptr, dw1.ptr, db1.ptr, dw2.ptr, db2.ptr, dres.ptr, act, z.ptr, h.ptr, xi.ptr, out.ptr, m, d,
                 hidden, 0, None)
            outs = [D((m, d)), D(w1.shape), D((hidden,)), D(w2.shape), D((d,))]
            call("bf_hip_feedforward_bf16_backward", dx.ptr, xi.ptr, dw1.ptr, dw2.ptr, z.ptr, h.ptr, dg.ptr, act, *[t.ptr for t in outs],
                 m, d, hidden, 0, None)
            return [t.toHost() for t in (z, h, out, *outs)]
        finally:
            call("bf_hip_gemm_bf16_set_route", 0)

    names = ("z", "image of act(z)", "out", "dX", "dW1", "dB1", "dW2", "dB2")
    fused, separate = run(0), run(1)
    for name, a, b in zip(names, fused, separate):
        if name == "dB1":
            scale = float(np.abs(b).max())
            assert float(np.abs(a - b).max()) <= 2e-6 * scale * np.sqrt(m), "dB1 from the products' partial column sums"
        elif name not in ("z", "image of act(z)") and m * d < 8192 * 768:
            # narrow products (d columns) of a long contraction: the named kernel adds all of K in one workgroup, the
            # library's own choice may cut K into slices, so the order of the fp32 additions differs; the largest case
            # has no such products and must agree bit for bit (dW1 is made from the image of dz)
            assert float(np.abs(a - b).max()) <= 1e-5 * float(np.abs(b).max()), name
        else:
            assert_bits_equal(a, b, name + " with the activation fused into the product's store")
    # and dB1 against float64 of the same terms (the fp32 products are summed, not their bf16 roundings)
    def rounded(a):   # round-to-nearest-even bf16 of finite fp32 values
        bits = np.ascontiguousarray(a, dtype=f32).view(np.uint32).astype(np.uint64)
        bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
        return bits.astype(np.uint32).view(f32).astype(np.float64)

    zf = fused[0].astype(np.float64)
    dH = rounded(g) @ rounded(w2).T
    if act == 0:
        sg = 1.0 / (1.0 + np.exp(-zf))
        dact = sg * (1.0 + zf * (1.0 - sg))
    elif act == 1:
        t = np.tanh(0.7978845608 * (zf + 0.044715 * zf ** 3))
        dact = 0.5 * (1.0 + t) + 0.5 * zf * (1.0 - t * t) * 0.7978845608 * (1.0 + 3.0 * 0.044715 * zf * zf)
    else:
        dact = (zf > 0).astype(np.float64)
    expect = (dH * dact).sum(axis=0)
    assert float(np.abs(fused[5] - expect).max()) <= 1e-4 * float(np.abs(expect).max()), "dB1 against float64"
