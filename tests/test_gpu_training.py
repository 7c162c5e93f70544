"""GPU parity of the training run around the hot path: hip::runTraining, hip::saveCheckpoint/loadCheckpoint and the
BFDATA1 reader (include/blackforge/backend/hip/{train_runner,checkpoint,dataset}.hpp) against what the real
reference's cpu::runTraining produced for the same dataset files and starting checkpoints (tests/golden/)."""
import numpy as np
import pytest

import trainfixtures as tf
from parity import assert_close

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.fixture(scope="module")
def expected():
    return np.load(tf.EXPECTED)


def host_model(name, use_bf16=False):
    from blackforge_amd import hostlayer
    layers, features = tf.RUNS[name][:2]
    return hostlayer.HostModel(layers, features, use_bf16=use_bf16)


@pytest.mark.parametrize("name", sorted(tf.RUNS))
def test_training_run_matches_the_reference(hip, expected, tmp_path, name):
    """Same files in, same epoch losses and final weights out as cpu::runTraining (train_runner.cpp:38-211), fp32 path.
    Losses: 1e-4 relative.  Weights after the last step: 1e-4 of the weight scale plus 2 % of the distance the run moved
    them (AdamW divides by sqrt(v): where a gradient is near zero its sign, and so the step, is ill-conditioned)."""
    layers, features, loss, optimizer, epochs, batch, lr, cosine = tf.RUNS[name]
    model = host_model(name)
    out = str(tmp_path / "final.bfckpt")
    losses = model.runTraining(tf.path(name, ".bfdata"), loss, optimizer, epochs, batch, lr=lr, cosine=cosine,
                               from_checkpoint=tf.path(name, "_init.bfckpt"), save_checkpoint=out)
    np.testing.assert_allclose(losses, expected[name + "_epoch_losses"], rtol=1e-4)
    got, want, start = tf.read_checkpoint(out), tf.read_checkpoint(tf.path(name, "_final.bfckpt")), tf.read_checkpoint(tf.path(name, "_init.bfckpt"))
    assert [(n, s) for n, s, _ in got] == [(n, s) for n, s, _ in want], "same parameter names, order and shapes as the reference file"
    for (pname, _, g), (_, _, w), (_, _, s) in zip(got, want, start):
        moved = float(np.abs(w - s).max())
        assert_close(g, w, tol=1e-4, what=f"{name}: {pname} after training", scale=200 * moved + 1e-3)
        np.testing.assert_array_equal(model.value(model.names.index(pname)), g)   # the file holds the device values


def test_checkpoint_round_trip_and_interop(hip, oracle, tmp_path):
    """A checkpoint written by the reference loads into hip::Model (same forward output as the oracle with those
    weights); saving it again reproduces the file byte for byte; loader errors are std::runtime_error."""
    name = "train_lm"
    model = host_model(name)
    model.loadCheckpoint(tf.path(name, "_final.bfckpt"))
    saved = str(tmp_path / "again.bfckpt")
    model.saveCheckpoint(saved)
    assert open(saved, "rb").read() == open(tf.path(name, "_final.bfckpt"), "rb").read()
    layers, features = tf.RUNS[name][:2]
    om = oracle.model(layers, features)
    om.loadCheckpoint(tf.path(name, "_final.bfckpt"))
    ids, _ = tf.read_dataset(tf.path(name, ".bfdata"))
    assert_close(model.forward(hip.DeviceTensor.fromHost(ids[:4])), om.forward(ids[:4]), what="forward from a reference checkpoint")
    raw = open(tf.path(name, "_final.bfckpt"), "rb").read()
    # a file that is refused leaves every parameter as it was, also when the fault lies behind records that are fine:
    # the loader matches the whole table of contents before it copies anything
    fresh = host_model(name)
    before = [fresh.value(i).copy() for i in range(len(fresh.names))]
    for label, data in {"magic": b"XXCKPT1\0" + raw[8:], "truncated": raw[:-3], "unknown": raw.replace(b"attention3.wq", b"attention3.wz"),
                        "huge extent": raw[:8 + 4 + 4 + len(fresh.names[0]) + 4] + b"\xff" * 8 + raw[8 + 4 + 4 + len(fresh.names[0]) + 4 + 8:]}.items():
        p = str(tmp_path / f"bad_{label}.bfckpt")
        open(p, "wb").write(data)
        with pytest.raises(RuntimeError):
            fresh.loadCheckpoint(p)
        for i, b in enumerate(before):
            np.testing.assert_array_equal(fresh.value(i), b)
    with pytest.raises(RuntimeError):
        host_model("train_mlp").loadCheckpoint(tf.path(name, "_final.bfckpt"))   # another model's parameters
    with pytest.raises(RuntimeError):
        model.loadCheckpoint(str(tmp_path / "missing.bfckpt"))


def test_training_run_rejects_what_the_reference_rejects(hip, oracle, tmp_path):
    """batch_size above the dataset size is a runtime_error (train_runner.cu:178-181); a token id outside the
    vocabulary or a class index outside the logits is an invalid_argument raised from the host copy (:60-69)."""
    name = "train_lm"
    model = host_model(name)
    with pytest.raises(RuntimeError):
        model.runTraining(tf.path(name, ".bfdata"), "cross_entropy_sparse", "adamw", 1, 25, from_checkpoint=tf.path(name, "_init.bfckpt"))
    ids, targets = tf.read_dataset(tf.path(name, ".bfdata"))
    bad_ids, bad_targets = ids.copy(), targets.copy()
    bad_ids[3, 2] = 32
    bad_targets[5, 1] = -1
    for label, (i, t) in {"ids": (bad_ids, targets), "targets": (ids, bad_targets)}.items():
        p = str(tmp_path / f"bad_{label}.bfdata")
        oracle.saveDataset(p, i, t)
        with pytest.raises(ValueError):
            model.runTraining(p, "cross_entropy_sparse", "adamw", 1, 4, from_checkpoint=tf.path(name, "_init.bfckpt"))


def test_training_run_with_bf16_projections(hip, expected, tmp_path):
    """The same run with bf16 projections stays within the bf16 bound of the fp32 reference's losses."""
    name = "train_lm"
    layers, features, loss, optimizer, epochs, batch, lr, cosine = tf.RUNS[name]
    losses = host_model(name, use_bf16=True).runTraining(tf.path(name, ".bfdata"), loss, optimizer, epochs, batch, lr=lr, cosine=cosine,
                                                         from_checkpoint=tf.path(name, "_init.bfckpt"))
    np.testing.assert_allclose(losses, expected[name + "_epoch_losses"], rtol=2e-2)
