"""GPU test of the recorded training step (hip::CapturedTrainStep over bf_hip_capture_begin/end): replays against the
eager step, bit for bit.

A graph replay runs the kernels the eager step launches, with the same arguments, so every parameter, the AdamW
moments (through the parameters of later steps) and the accumulated loss must be IDENTICAL, not close.  The replays
are interleaved with eager work and synchronisations of the same process (other models' steps, pool traffic, reads),
and every replay is checked: a recording that only works the first time, or whose buffers somebody else gets hold of,
fails here."""
import ctypes

import numpy as np
import pytest

from parity import assert_bits_equal

pytestmark = pytest.mark.gpu
f32 = np.float32


def lm_layers(hl, vocab, dim, seq, heads, hidden, blocks=1):
    layers = [(hl.EMBEDDING, vocab, dim), (hl.POSITIONAL, seq)]
    for _ in range(blocks):
        layers += [(hl.ATTENTION, heads), (hl.FEEDFORWARD, hidden, 0)]
    return layers + [(hl.LINEAR, vocab)]


def twin_models(hl, rng, layers, use_bf16):
    a, b = hl.HostModel(layers, use_bf16=use_bf16), hl.HostModel(layers, use_bf16=use_bf16)
    for i, c in enumerate(a.counts):
        w = (rng.standard_normal(c) * 0.05).astype(f32)
        a.set_value(i, w)
        b.set_value(i, w)
    return a, b


def in_use(hip):
    stats = hip.capi.PoolStats()
    hip.capi.call("bf_hip_pool_stats", ctypes.byref(stats))
    return stats.bytes_in_use


@pytest.mark.parametrize("use_bf16,optimizer", [(False, 1), (True, 1), (False, 2)])
def test_replays_equal_eager_steps(hip, rng, use_bf16, optimizer):
    from blackforge_amd import hostlayer as hl
    D = hip.DeviceTensor
    vocab, dim, seq, batch, heads, hidden = 256, 128, 64, 8, 4, 512
    eager, recorded = twin_models(hl, rng, lm_layers(hl, vocab, dim, seq, heads, hidden), use_bf16)
    batches = [(rng.integers(0, vocab, (batch, seq)).astype(f32), rng.integers(0, vocab, batch * seq).astype(f32)) for _ in range(5)]
    x, t = D.fromHost(batches[0][0]), D.fromHost(batches[0][1])
    before = [recorded.value(i).copy() for i in range(len(recorded.counts))]
    step = recorded.captureTrainStep(x, t, hl.LOSS_SPARSE_CE, optimizer, 1e-3)
    for i, b in enumerate(before):   # recording executes nothing
        np.testing.assert_array_equal(recorded.value(i), b)
    assert recorded.readLossSum() == 0.0
    bystander = hl.HostModel(lm_layers(hl, 64, 32, 16, 2, 64))   # eager work of another model between the replays
    bx, bt = D.fromHost(rng.integers(0, 64, (2, 16)).astype(f32)), D.fromHost(rng.integers(0, 64, 32).astype(f32))
    for n, (ids, tgt) in enumerate(batches):
        lr = 1e-3 * (1.0 - 0.1 * n)   # a schedule: the rate is read from device memory, not frozen into the graph
        hip.capi.call("bf_hip_memcpy_h2d", x.ptr, ids.ctypes.data_as(ctypes.c_void_p), ids.nbytes)
        hip.capi.call("bf_hip_memcpy_h2d", t.ptr, tgt.ctypes.data_as(ctypes.c_void_p), tgt.nbytes)
        step.run(lr)
        eager.trainStep(D.fromHost(ids), D.fromHost(tgt), hl.LOSS_SPARSE_CE, optimizer if optimizer == 1 else 0, lr)
        if optimizer == 2:
            eager.sgdStep(lr)
        bystander.trainStep(bx, bt, hl.LOSS_SPARSE_CE, 1, 1e-3)
        junk = [D.fromHost(rng.standard_normal(s).astype(f32)) for s in (1000, 70000, 300)]   # pool traffic
        del junk
        for i in range(len(eager.counts)):
            assert_bits_equal(recorded.value(i), eager.value(i), f"step {n + 1}: {eager.names[i]}")
            assert_bits_equal(recorded.grad(i), eager.grad(i), f"step {n + 1}: gradient of {eager.names[i]}")
        assert recorded.readLossSum() == eager.readLossSum(), f"step {n + 1}: accumulated loss"
    # the model still works eagerly beside its recording, and the recording after that
    recorded.trainStep(D.fromHost(batches[0][0]), D.fromHost(batches[0][1]), hl.LOSS_SPARSE_CE, optimizer if optimizer == 1 else 0, 1e-3)
    eager.trainStep(D.fromHost(batches[0][0]), D.fromHost(batches[0][1]), hl.LOSS_SPARSE_CE, optimizer if optimizer == 1 else 0, 1e-3)
    if optimizer == 2:
        recorded.sgdStep(1e-3)
        eager.sgdStep(1e-3)
    hip.capi.call("bf_hip_memcpy_h2d", x.ptr, batches[1][0].ctypes.data_as(ctypes.c_void_p), batches[1][0].nbytes)
    hip.capi.call("bf_hip_memcpy_h2d", t.ptr, batches[1][1].ctypes.data_as(ctypes.c_void_p), batches[1][1].nbytes)
    step.run(1e-3)
    eager.trainStep(D.fromHost(batches[1][0]), D.fromHost(batches[1][1]), hl.LOSS_SPARSE_CE, optimizer if optimizer == 1 else 0, 1e-3)
    if optimizer == 2:
        eager.sgdStep(1e-3)
    for i in range(len(eager.counts)):
        assert_bits_equal(recorded.value(i), eager.value(i), f"after an eager step in between: {eager.names[i]}")
    step.close()


def test_recording_memory_belongs_to_the_graph_until_it_is_destroyed(hip, rng):
    from blackforge_amd import hostlayer as hl
    D = hip.DeviceTensor
    model, _ = twin_models(hl, rng, lm_layers(hl, 64, 32, 16, 2, 64), False)
    x, t = D.fromHost(rng.integers(0, 64, (2, 16)).astype(f32)), D.fromHost(rng.integers(0, 64, 32).astype(f32))
    model.trainStep(x, t, hl.LOSS_SPARSE_CE, 1, 1e-3)   # the optimizer state exists
    hip.capi.call("bf_hip_synchronize")
    level = in_use(hip)
    step = model.captureTrainStep(x, t, hl.LOSS_SPARSE_CE, 1, 1e-3)
    hip.capi.call("bf_hip_pool_trim")   # must not free what the graph addresses
    step.run(1e-3)
    step.run(1e-3)
    hip.capi.call("bf_hip_synchronize")
    assert np.isfinite(model.readLossSum())
    step.close()
    with pytest.raises(ValueError):
        hip.capi.call("bf_hip_capture_end", None)   # nothing in progress: reported, not crashed (NULL = abandon)


def test_capture_rules_are_reported(hip):
    with pytest.raises(ValueError):
        hip.capi.call("bf_hip_capture_begin", None)
    st = hip.Stream()
    hip.capi.call("bf_hip_capture_begin", st.handle)
    with pytest.raises(ValueError):
        hip.capi.call("bf_hip_capture_begin", st.handle)   # one at a time
    hip.capi.call("bf_hip_capture_end", None)               # abandon
    a = hip.DeviceTensor.fromHost(np.ones(8, f32))
    assert (hip.ops.scale(a, 2.0).toHost() == 2).all()      # eager calls run again


def test_eager_backward_after_a_recording_is_refused(hip, rng):
    """Recording walks the layers without running a kernel, so the activation caches it leaves describe nothing: an eager
    backward pass right after it must raise, not differentiate against unwritten buffers; after an eager forward pass it
    works again."""
    from blackforge_amd import hostlayer as hl
    D = hip.DeviceTensor
    model, _ = twin_models(hl, rng, lm_layers(hl, 64, 32, 16, 2, 64), False)
    x, t = D.fromHost(rng.integers(0, 64, (2, 16)).astype(f32)), D.fromHost(rng.integers(0, 64, 32).astype(f32))
    model.forward(x)
    model.loss(t)
    model.backward()          # an ordinary eager pass works
    step = model.captureTrainStep(x, t, hl.LOSS_SPARSE_CE, 1, 1e-3)
    with pytest.raises(ValueError, match="no forward pass to differentiate"):
        model.backward()
    model.forward(x)
    model.loss(t)
    model.backward()
    step.close()


def test_cached_weight_image_follows_a_replay(hip, oracle, rng):
    """A replay steps the optimizer over the weights; a cached-weight projection called afterwards through the C ABI must
    multiply by the NEW weights (the eager weight-image cache is marked stale by every graph launch)."""
    from blackforge_amd import hostlayer as hl
    D, call = hip.DeviceTensor, hip.capi.call
    width, rows = 64, 32
    model = hl.HostModel([(hl.LINEAR, width)], input_features=width, use_bf16=True)
    model.set_value(0, (rng.standard_normal(width * width) * 0.1).astype(f32))
    model.set_value(1, np.zeros(width, f32))
    x, y = D.fromHost(rng.standard_normal((rows, width)).astype(f32)), D.fromHost(rng.standard_normal((rows, width)).astype(f32))
    step = model.captureTrainStep(x, y, hl.LOSS_MSE, 2, 0.5)
    a = rng.standard_normal((rows, width)).astype(f32)
    da, out = D.fromHost(a), D((rows, width))
    w_ptr = model._value_ptrs[0]

    def product():
        call("bf_hip_linear_bf16", da.ptr, w_ptr, None, None, out.ptr, rows, width, width, 1, None)
        return out.toHost()

    def expected():
        w = model.value(0).reshape(width, width)
        return oracle.matmul(oracle.roundToBf16(a), oracle.roundToBf16(w))

    np.testing.assert_allclose(product(), expected(), rtol=1e-4, atol=1e-5)
    before = model.value(0).copy()
    step.run(0.5)
    hip.capi.call("bf_hip_synchronize")
    assert np.abs(model.value(0) - before).max() > 1e-3          # the replay did move the weights
    np.testing.assert_allclose(product(), expected(), rtol=1e-4, atol=1e-5)
    step.close()


@pytest.mark.parametrize("loss_kind,use_bf16,optimizer", [(2, False, 1), (3, False, 1), (1, False, 2), (1, True, 2), (0, True, 2)])
def test_replays_equal_eager_steps_for_every_loss(hip, rng, loss_kind, use_bf16, optimizer):
    """The masked and the dense cross-entropy and the mean squared error recorded into the graph (a device-side count of
    the rows that are not ignored, the partial sums of the squared error), and SGD over bf16 projections: replays against
    eager steps, bit for bit, over three batches."""
    from blackforge_amd import hostlayer as hl
    D = hip.DeviceTensor
    vocab, dim, seq, batch, heads, hidden = 64, 32, 16, 4, 2, 64
    eager, recorded = twin_models(hl, rng, lm_layers(hl, vocab, dim, seq, heads, hidden), use_bf16)

    def targets():
        if loss_kind in (0, 2):
            t = rng.integers(0, vocab, batch * seq).astype(f32)
            if loss_kind == 2:
                t[rng.random(batch * seq) < 0.3] = -1.0
            return t
        if loss_kind == 3:
            p = rng.random((batch, seq, vocab)).astype(f32)
            return (p / p.sum(axis=-1, keepdims=True)).astype(f32)
        return rng.standard_normal((batch, seq, vocab)).astype(f32)

    batches = [(rng.integers(0, vocab, (batch, seq)).astype(f32), targets()) for _ in range(3)]
    x, t = D.fromHost(batches[0][0]), D.fromHost(batches[0][1])
    step = recorded.captureTrainStep(x, t, loss_kind, optimizer, 1e-2)
    for n, (ids, tgt) in enumerate(batches):
        hip.capi.call("bf_hip_memcpy_h2d", x.ptr, ids.ctypes.data_as(ctypes.c_void_p), ids.nbytes)
        hip.capi.call("bf_hip_memcpy_h2d", t.ptr, tgt.ctypes.data_as(ctypes.c_void_p), tgt.nbytes)
        step.run(1e-2)
        eager.trainStep(D.fromHost(ids), D.fromHost(tgt), loss_kind, optimizer if optimizer == 1 else 0, 1e-2)
        if optimizer == 2:
            eager.sgdStep(1e-2)
        for i in range(len(eager.counts)):
            assert_bits_equal(recorded.value(i), eager.value(i), f"step {n + 1}: {eager.names[i]}")
        assert recorded.readLossSum() == eager.readLossSum(), f"step {n + 1}: accumulated loss"
    step.close()
