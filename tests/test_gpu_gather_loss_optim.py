"""GPU parity: embedding / positional / concat / argmax (bit-exact), losses, optimizers."""
import numpy as np
import pytest

from parity import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu
f32 = np.float32


def r(rng, *s, scale=1.0):
    return (rng.standard_normal(s) * scale).astype(f32)


@pytest.mark.parametrize("batch,seq,vocab,dim", [(1, 3, 3, 2), (2, 5, 11, 6), (8, 64, 256, 128), (3, 33, 1000, 770), (2, 17, 50257, 8)])
def test_embedding_gather_and_scatter_are_bit_exact(hip, oracle, rng, batch, seq, vocab, dim):
    D, ops = hip.DeviceTensor, hip.ops
    ids = rng.integers(0, vocab, (batch, seq)).astype(f32)
    ids[0, 0] = vocab - 1
    ids.flat[-1] = ids.flat[0]  # a repeated id
    table, g = r(rng, vocab, dim), r(rng, batch, seq, dim)
    assert_bits_equal(ops.embeddingLookup(D.fromHost(ids), D.fromHost(table)).toHost(), oracle.embeddingLookup(ids, table))
    # gradient rows are summed in token order, like the CPU loop: identical bits
    assert_bits_equal(ops.embeddingLookupBackward(D.fromHost(ids), D.fromHost(g), vocab).toHost(),
                      oracle.embeddingLookupBackward(ids, g, vocab))


@pytest.mark.parametrize("tokens,vocab,dim,hot", [(8192, 32000, 64, 0), (8192, 300, 32, 3000), (16384, 50257, 16, 5000), (70000, 1000, 8, 100),
                                                  (500, 200001, 4, 50), (65535, 76800, 4, 0), (16384, 8192, 1028, 0), (777, 5000, 770, 30), (300, 4000, 7, 4)])
def test_embedding_scatter_routes(hip, oracle, tokens, vocab, dim, hot):
    """The route without a sort (up to 16384 tokens against a table at least half as large: one wavefront per token, the
    first token of an id sums its row) and the counting-sort route (more tokens, or a small table), with an id that `hot`
    tokens share: every route sums in token order, so the result is the CPU loop's bit for bit."""
    rng = np.random.default_rng(tokens + vocab)
    D, ops = hip.DeviceTensor, hip.ops
    ids = rng.integers(0, vocab, (1, tokens)).astype(f32)
    if hot:
        ids[0, rng.choice(tokens, hot, replace=False)] = 7 % vocab
    ids[0, -1] = vocab - 1
    g = r(rng, 1, tokens, dim)
    assert_bits_equal(ops.embeddingLookupBackwardPreValidated(D.fromHost(ids), D.fromHost(g), vocab).toHost(),
                      oracle.embeddingLookupBackward(ids, g, vocab))


def test_embedding_ids_outside_the_table_touch_nothing(hip, oracle, rng):
    """The pre-validated entry points trust their caller; an id outside [0, vocab) must still not read or write outside
    the tensors: the lookup gives zeros for it and the gradient ignores it (both routes of the sort)."""
    D, ops = hip.DeviceTensor, hip.ops
    vocab, dim = 50, 12
    for tokens in (40, 70000):
        ids = rng.integers(0, vocab, (1, tokens)).astype(f32)
        bad = np.array([3, 11, tokens - 1])
        ids[0, bad] = [-1.0, float(vocab), 1e9]
        table, g = r(rng, vocab, dim), r(rng, 1, tokens, dim)
        out = ops.embeddingLookupPreValidated(D.fromHost(ids), D.fromHost(table)).toHost()
        good = np.ones(tokens, bool)
        good[bad] = False
        clipped = np.where(good, ids[0], 0).astype(f32)[None]
        expected = oracle.embeddingLookup(clipped, table)
        expected[0, bad] = 0
        assert_bits_equal(out, expected)
        gz = g.copy()
        gz[0, bad] = 0   # the ignored tokens contribute nothing; their stand-in id 0 then only adds zeros
        assert_bits_equal(ops.embeddingLookupBackwardPreValidated(D.fromHost(ids), D.fromHost(g), vocab).toHost(),
                          oracle.embeddingLookupBackward(clipped, gz, vocab))


def test_embedding_reference_literals_and_range_errors(hip):
    """tests/backend/cpu/ops_tests.cpp:238-262, autodiff_tests.cpp:180-199, cuda/ops_tests.cu:300-306."""
    D, ops = hip.DeviceTensor, hip.ops
    table = D.fromHost(np.array([10, 11, 20, 21, 30, 31], f32).reshape(3, 2))
    out = ops.embeddingLookup(D.fromHost(np.array([[0, 2, 1]], f32)), table).toHost()
    np.testing.assert_array_equal(out.ravel(), [10, 11, 30, 31, 20, 21])
    for bad in (3.0, -1.0):
        with pytest.raises(ValueError):
            ops.embeddingLookup(D.fromHost(np.array([[bad]], f32)), table)
        with pytest.raises(ValueError):
            ops.embeddingLookupBackward(D.fromHost(np.array([[bad]], f32)), D.zeros((1, 1, 2)), 3)
    dt = ops.embeddingLookupBackward(D.fromHost(np.array([[0, 1, 0]], f32)),
                                     D.fromHost(np.array([1, 2, 10, 20, 3, 4], f32).reshape(1, 3, 2)), 3).toHost()
    np.testing.assert_array_equal(dt.ravel(), [4, 6, 10, 20, 0, 0])
    # rounding of float ids: 1.4 -> 1, 1.6 -> 2 (lround)
    out = ops.embeddingLookup(D.fromHost(np.array([[1.4, 1.6]], f32)), table).toHost()
    np.testing.assert_array_equal(out.ravel(), [20, 21, 30, 31])


@pytest.mark.parametrize("batch,seq,dim,max_seq", [(2, 2, 2, 2), (3, 5, 7, 9), (8, 64, 128, 64), (2, 100, 772, 128)])
def test_positional_embedding(hip, oracle, rng, batch, seq, dim, max_seq):
    D, ops = hip.DeviceTensor, hip.ops
    x, table = r(rng, batch, seq, dim), r(rng, max_seq, dim)
    for off in {0, max_seq - seq}:
        assert_bits_equal(ops.addPositionalEmbeddingAt(D.fromHost(x), D.fromHost(table), off).toHost(),
                          oracle.addPositionalEmbeddingAt(x, table, off))
    di, dt = ops.addPositionalEmbeddingBackward(D.fromHost(x), max_seq)
    assert_bits_equal(di.toHost(), x)
    assert_bits_equal(dt.toHost(), oracle.addPositionalEmbeddingBackward(x, max_seq)[1])
    with pytest.raises(ValueError):
        ops.addPositionalEmbeddingAt(D.fromHost(x), D.fromHost(table), max_seq - seq + 1)
    with pytest.raises(ValueError):
        ops.addPositionalEmbeddingBackward(D.fromHost(x), seq - 1)


def test_concat_seq_and_argmax(hip, oracle, rng):
    D, ops = hip.DeviceTensor, hip.ops
    a, b = r(rng, 3, 4, 10), r(rng, 3, 2, 10)
    assert_bits_equal(ops.concatSeq(D.fromHost(a), D.fromHost(b)).toHost(), np.concatenate([a, b], axis=1))
    for vocab in (1, 5, 1000, 50257):
        logits = r(rng, 1, 3, vocab)
        logits[0, 2, vocab // 2] = logits[0, 2].max()  # a tie: the lower index must win
        assert ops.argmaxLastPosition(D.fromHost(logits)) == oracle.argmaxLastPosition(logits[0])
    logits = np.zeros((2, 9), f32)
    assert ops.argmaxLastPosition(D.fromHost(logits)) == 0


def test_position_on_the_device_entry_points(hip, oracle, rng):
    """The entry points of a decoding step that read the position from device memory (bf_hip_positional_forward_indirect,
    bf_hip_kv_append_indirect, bf_hip_argmax_last_position_device, bf_hip_counter_add) and the strided copy of the growing
    cache (bf_hip_copy_pitched), each against the host-position operator it mirrors (addPositionalEmbeddingAt ops.hpp:391,
    concatSeq ops_transformer.cu:22-58, argmaxLastPosition main.cpp:504-518) or numpy, bit for bit; a position that does
    not fit writes nothing."""
    import ctypes
    D, ops, call = hip.DeviceTensor, hip.ops, hip.capi.call
    counter = D.fromHost(np.array([5], np.int32).view(f32))
    as_int = lambda: int(counter.toHost().view(np.int32)[0])
    call("bf_hip_counter_add", counter.ptr, 3, None)
    call("bf_hip_counter_add", counter.ptr, -1, None)
    assert as_int() == 7
    for dim in (12, 7):   # 16-byte rows and rows that are not
        batch, seq, max_seq = 3, 2, 11
        x, table = r(rng, batch, seq, dim), r(rng, max_seq, dim)
        out, dx, dtable = D.fromHost(np.zeros_like(x)), D.fromHost(x), D.fromHost(table)   # named: a temporary's buffer goes back to the pool at once
        call("bf_hip_positional_forward_indirect", dx.ptr, dtable.ptr, out.ptr, batch, seq, dim, max_seq, counter.ptr, None)
        assert_bits_equal(out.toHost(), ops.addPositionalEmbeddingAt(D.fromHost(x), D.fromHost(table), 7).toHost(), "positions from the device")
        too_far = D.fromHost(np.array([max_seq - 1], np.int32).view(f32))
        untouched = D.fromHost(np.full_like(x, 3.0))
        call("bf_hip_positional_forward_indirect", dx.ptr, dtable.ptr, untouched.ptr, batch, seq, dim, max_seq, too_far.ptr, None)
        assert_bits_equal(untouched.toHost(), np.full_like(x, 3.0), "a position past the table writes nothing")
        # append at row 7 of caches with 10 rows a sequence
        capacity = 10
        kc, vc = r(rng, batch, capacity, dim), r(rng, batch, capacity, dim)
        kn, vn = r(rng, batch, seq, dim), r(rng, batch, seq, dim)
        dk, dv, dkn, dvn = D.fromHost(kc), D.fromHost(vc), D.fromHost(kn), D.fromHost(vn)
        call("bf_hip_kv_append_indirect", dk.ptr, dv.ptr, dkn.ptr, dvn.ptr, batch, seq, dim, capacity, counter.ptr, None)
        ek, ev = kc.copy(), vc.copy()
        ek[:, 7:9], ev[:, 7:9] = kn, vn
        assert_bits_equal(dk.toHost(), ek, "keys appended at the device-side position")
        assert_bits_equal(dv.toHost(), ev, "values appended at the device-side position")
        dk2, dv2 = D.fromHost(kc), D.fromHost(vc)
        call("bf_hip_kv_append", dk2.ptr, dv2.ptr, dkn.ptr, dvn.ptr, batch, seq, dim, capacity, 7, None)   # the position from the host
        assert_bits_equal(dk2.toHost(), ek, "keys appended at the caller's position")
        assert_bits_equal(dv2.toHost(), ev, "values appended at the caller's position")
        with pytest.raises(ValueError):
            call("bf_hip_kv_append", dk2.ptr, dv2.ptr, dkn.ptr, dvn.ptr, batch, seq, dim, capacity, 9, None)
        full = D.fromHost(np.array([9], np.int32).view(f32))
        call("bf_hip_kv_append_indirect", dk.ptr, dv.ptr, dkn.ptr, dvn.ptr, batch, seq, dim, capacity, full.ptr, None)
        assert_bits_equal(dk.toHost(), ek, "rows that do not fit are not written")
        # the dense [batch, length, dim] view of a cache and back
        dense = D((batch, 9, dim))
        call("bf_hip_copy_pitched", dense.ptr, 9 * dim, dk.ptr, capacity * dim, 9 * dim, batch, None)
        assert_bits_equal(dense.toHost(), ek[:, :9], "dense view of the cache")
    for vocab in (1, 5, 1000, 50257):
        logits = r(rng, 1, 3, vocab)
        logits[0, 2, vocab // 2] = logits[0, 2].max()   # a tie: the lower index must win
        token, history, dlogits = D.fromHost(np.zeros((1, 1), f32)), D.fromHost(np.full(4, -1.0, f32)), D.fromHost(logits)
        call("bf_hip_argmax_last_position_device", dlogits.ptr, 3, vocab, token.ptr, history.ptr, 4, counter.ptr, 0, ctypes.c_longlong(-5), None)
        expected = oracle.argmaxLastPosition(logits[0])
        assert token.toHost()[0, 0] == expected
        np.testing.assert_array_equal(history.toHost(), [-1, -1, expected, -1])   # slot 7 - 5
        call("bf_hip_argmax_last_position_device", dlogits.ptr, 3, vocab, token.ptr, history.ptr, 4, counter.ptr, 0, ctypes.c_longlong(0), None)
        np.testing.assert_array_equal(history.toHost(), [-1, -1, expected, -1])   # slot 7 lies outside: left alone
        call("bf_hip_argmax_last_position_device", dlogits.ptr, 3, vocab, token.ptr, history.ptr, 4, counter.ptr, 1, ctypes.c_longlong(-5), None)
        np.testing.assert_array_equal(history.toHost(), [-1, -1, expected, expected])   # the counter moves on first: slot 8 - 5
        assert as_int() == 8
        call("bf_hip_counter_add", counter.ptr, -1, None)


@pytest.mark.parametrize("rows,classes", [(1, 2), (2, 3), (7, 13), (512, 256), (5, 1000), (3, 32000), (2, 50257), (1, 70001), (3, 40000),
                                          (2, 50260)])
def test_cross_entropy(hip, oracle, rng, rows, classes):
    D, ops = hip.DeviceTensor, hip.ops
    logits = r(rng, rows, classes, scale=3)
    idx = rng.integers(0, classes, rows)
    res = ops.softmaxCrossEntropySparse(D.fromHost(logits), D.fromHost(idx.astype(f32)))
    ev, eg = oracle.softmaxCrossEntropySparse(logits, idx.astype(f32))
    assert abs(res.value - ev) <= 1e-4 * abs(ev) + 1e-6
    assert_close(res.grad.toHost(), eg, what="sparse CE grad")
    if rows * classes < 10_000_000:
        dense = np.zeros((rows, classes), f32)
        dense[np.arange(rows), idx] = 0.7
        dense[np.arange(rows), (idx + 1) % classes] += 0.3
        res = ops.softmaxCrossEntropy(D.fromHost(logits), D.fromHost(dense))
        ev, eg = oracle.softmaxCrossEntropy(logits, dense)
        assert abs(res.value - ev) <= 1e-4 * abs(ev) + 1e-6
        assert_close(res.grad.toHost(), eg, what="dense CE grad")


@pytest.mark.parametrize("classes", [37, 1000, 4099, 16384, 32000, 32003, 50257])
def test_cross_entropy_target_at_every_kind_of_position(hip, oracle, rng, classes):
    """The target class at the ends of the row and either side of every boundary the kernel's layouts have (16-byte
    groups, wavefronts, 256- and 1024-thread iterations), on rows of every alignment (odd class counts shift each row
    by a different amount): the one element whose gradient is (p - 1) / rows must be exactly that one."""
    D, ops = hip.DeviceTensor, hip.ops
    marks = [0, 1, 3, 4, 5, 63, 64, 255, 256, 257, 1023, 1024, 1027, 4095, 4096, 4097, 16383, 16384, 32767, 32768, 32771,
             classes // 2, classes - 5, classes - 4, classes - 2, classes - 1]
    idx = np.array(sorted({m for m in marks if 0 <= m < classes}))
    rows = len(idx)
    logits = r(rng, rows, classes, scale=3)
    res = ops.softmaxCrossEntropySparse(D.fromHost(logits), D.fromHost(idx.astype(f32)))
    ev, eg = oracle.softmaxCrossEntropySparse(logits, idx.astype(f32))
    got = res.grad.toHost()
    assert abs(res.value - ev) <= 1e-4 * abs(ev) + 1e-6
    assert_close(got, eg, what="sparse CE grad")
    assert (got[np.arange(rows), idx] < 0).all() and (np.delete(got, idx[0], axis=1)[0] >= 0).all()


@pytest.mark.parametrize("rows,classes,keep", [(1, 2, 1.0), (7, 13, 0.5), (512, 256, 0.15), (33, 1000, 0.3), (6, 32000, 0.5), (4, 50257, 0.5),
                                               (2, 70001, 1.0), (9, 40, 0.0)])
def test_masked_cross_entropy(hip, oracle, rng, rows, classes, keep):
    """softmaxCrossEntropyMasked: rows with index -1 are ignored, means over the others (cpu loss.cpp:149-215)."""
    D, ops = hip.DeviceTensor, hip.ops
    logits = r(rng, rows, classes, scale=3)
    idx = np.where(rng.random(rows) < keep, rng.integers(0, classes, rows), -1).astype(f32)
    res = ops.softmaxCrossEntropyMasked(D.fromHost(logits), D.fromHost(idx))
    ev, eg = oracle.softmaxCrossEntropyMasked(logits, idx)
    assert abs(res.value - ev) <= 1e-4 * abs(ev) + 1e-6
    got = res.grad.toHost()
    assert_close(got, eg, what="masked CE grad")
    assert not got[idx == -1].any(), "ignored rows must have an exactly zero gradient"
    if keep == 0.0:
        assert res.value == 0.0 and not got.any()
    # accumulate form: adds the mean of each call
    acc = D.zeros((1,))
    for _ in range(3):
        g = ops.softmaxCrossEntropyMaskedAccumulate(D.fromHost(logits), D.fromHost(idx), acc)
    assert_close(g.toHost(), eg, what="masked CE grad (accumulate)")
    assert abs(acc.toHost()[0] - 3 * ev) <= 1e-4 * 3 * abs(ev) + 1e-6


def test_masked_cross_entropy_reference_cases(hip):
    """tests/backend/cpu/loss_tests.cpp:142-196."""
    D, ops = hip.DeviceTensor, hip.ops
    logits = np.array([[0.5, -1.2, 0.3], [2.0, 0.1, -0.5]], f32)
    masked = ops.softmaxCrossEntropyMasked(D.fromHost(logits), D.fromHost(np.array([1, 0], f32)))
    sparse = ops.softmaxCrossEntropySparse(D.fromHost(logits), D.fromHost(np.array([1, 0], f32)))
    assert abs(masked.value - sparse.value) <= 1e-6
    np.testing.assert_allclose(masked.grad.toHost(), sparse.grad.toHost(), atol=1e-6)
    logits = np.array([[1, 2, 3], [0.5, -1.0, 0.2], [-0.3, 0.1, 0.4]], f32)
    masked = ops.softmaxCrossEntropyMasked(D.fromHost(logits), D.fromHost(np.array([-1, 2, -1], f32)))
    single = ops.softmaxCrossEntropySparse(D.fromHost(logits[1:2]), D.fromHost(np.array([2], f32)))
    g = masked.grad.toHost()
    assert not g[0].any() and not g[2].any()
    assert abs(masked.value - single.value) <= 1e-5
    none = ops.softmaxCrossEntropyMasked(D.fromHost(logits[:2]), D.fromHost(np.array([-1, -1], f32)))
    assert none.value == 0.0 and not none.grad.toHost().any()
    with pytest.raises(ValueError):
        ops.softmaxCrossEntropyMasked(D.fromHost(np.array([[0.1, 0.2, 0.3]], f32)), D.fromHost(np.array([7], f32)))
    with pytest.raises(ValueError):
        ops.softmaxCrossEntropyMasked(D.fromHost(np.array([[0.1, 0.2, 0.3]], f32)), D.fromHost(np.array([-2], f32)))


def test_loss_literals_errors_and_accumulate(hip, oracle, rng):
    """tests/backend/cpu/loss_tests.cpp:10-16,51-69,115-140; cuda/loss_tests.cu:124-130."""
    import math
    D, ops = hip.DeviceTensor, hip.ops
    assert ops.meanSquaredError(D.fromHost(np.array([1, 2], f32)), D.fromHost(np.zeros(2, f32))).value == 2.5
    res = ops.softmaxCrossEntropy(D.fromHost(np.zeros((1, 2), f32)), D.fromHost(np.array([[1, 0]], f32)))
    assert abs(res.value - math.log(2)) < 1e-6
    np.testing.assert_allclose(res.grad.toHost().ravel(), [-0.5, 0.5], atol=1e-6)
    with pytest.raises(ValueError):
        ops.softmaxCrossEntropySparse(D.fromHost(np.array([[0.1, 0.2, 0.3]], f32)), D.fromHost(np.array([5], f32)))
    with pytest.raises(ValueError):
        ops.softmaxCrossEntropySparse(D.zeros((2, 3)), D.zeros((3,)))
    with pytest.raises(ValueError):
        ops.meanSquaredError(D.zeros((2,)), D.zeros((3,)))
    with pytest.raises(ValueError):
        ops.softmaxCrossEntropy(D.zeros((2,)), D.zeros((2,)))
    # *Accumulate: the accumulator receives the SUM of row losses of each call (loss.hpp:39-57)
    p, t = r(rng, 6, 10), r(rng, 6, 10)
    acc = D.zeros((1,))
    for _ in range(3):
        g = ops.meanSquaredErrorAccumulate(D.fromHost(p), D.fromHost(t), acc)
    ev, eg = oracle.meanSquaredError(p, t)
    assert_close(g.toHost(), eg)
    assert abs(acc.toHost()[0] - 3 * ev * p.size) <= 1e-4 * 3 * ev * p.size
    idx = rng.integers(0, 10, 6).astype(f32)
    acc = D.zeros((1,))
    for _ in range(2):
        g = ops.softmaxCrossEntropySparseAccumulate(D.fromHost(p), D.fromHost(idx), acc)
    ev, eg = oracle.softmaxCrossEntropySparse(p, idx)
    assert_close(g.toHost(), eg)
    assert abs(acc.toHost()[0] - 2 * ev * 6) <= 1e-4 * 2 * ev * 6


@pytest.mark.parametrize("n", [1, 1000, 1 << 20])
def test_mse(hip, oracle, rng, n):
    D, ops = hip.DeviceTensor, hip.ops
    p, t = r(rng, n), r(rng, n)
    res = ops.meanSquaredError(D.fromHost(p), D.fromHost(t))
    ev, eg = oracle.meanSquaredError(p, t)
    assert abs(res.value - ev) <= 1e-4 * ev + 1e-12
    assert_close(res.grad.toHost(), eg)


def test_optimizers_multi_tensor(hip, oracle, rng):
    """SGD / AdamW closed forms of tests/backend/cpu/optimizer_tests.cpp:10-59, then 10 steps on ragged tensors."""
    import math
    D, ops = hip.DeviceTensor, hip.ops
    p = ops.Parameter("p", D.fromHost(np.array([1, -2], f32)), D.fromHost(np.array([0.5, 0.5], f32)))
    ops.SGD(0.1).step([p])
    assert_bits_equal(p.value.toHost(), np.array([1, -2], f32) - f32(0.1) * f32(0.5))
    p = ops.Parameter("p", D.fromHost(np.array([1], f32)), D.fromHost(np.array([0.2], f32)))
    ops.AdamW(0.1, 0.9, 0.999, 1e-8, 0.0).step([p])
    assert abs(p.value.toHost()[0] - (1.0 - 0.1 * (0.2 / (math.sqrt(0.04) + 1e-8)))) < 1e-5
    p = ops.Parameter("p", D.fromHost(np.array([1], f32)), D.fromHost(np.array([0], f32)))
    ops.AdamW(0.1, 0.9, 0.999, 1e-8, 0.1).step([p])
    assert p.value.toHost()[0] == f32(1.0) - f32(0.1) * f32(0.1)

    sizes = [1, 7, 8192, 8195, 300001]
    host_p = [r(rng, n) for n in sizes]
    params = [ops.Parameter(f"t{i}", D.fromHost(a), D.zeros((n,))) for i, (a, n) in enumerate(zip(host_p, sizes))]
    opt = ops.AdamW(1e-2)
    m = [np.zeros(n, f32) for n in sizes]
    v = [np.zeros(n, f32) for n in sizes]
    for step in range(1, 11):
        grads = [r(rng, n) for n in sizes]
        for prm, g in zip(params, grads):
            prm.grad = D.fromHost(g)
        opt.step(params)
        for i, g in enumerate(grads):
            host_p[i], m[i], v[i] = oracle.adamwStep(host_p[i], g, m[i], v[i], step, 1e-2)
    for prm, e in zip(params, host_p):
        assert_close(prm.value.toHost(), e, what="AdamW after 10 steps")
    sgd = ops.SGD(0.05)
    sgd.step(params)
    for prm, e, g in zip(params, host_p, grads):
        assert_close(prm.value.toHost(), oracle.sgdStep(e, g, 0.05), what="SGD")
