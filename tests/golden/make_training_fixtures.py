"""Writes the training-run fixtures under tests/golden/ from the REAL reference CPU backend.

Run in a container that has the reference tree (oracle/_ref/libbf_ref.so is built from it by oracle/Makefile):
    python tests/golden/make_training_fixtures.py
Data only: a few small BFDATA1 datasets (seeded random numbers), the BFCKPT1 checkpoint of each model as the reference
initialises it (seed 42), the checkpoint the reference's own cpu::runTraining leaves after training on them, its
epoch losses, and the permutations of data::Dataset::shuffle for a few sizes and seeds.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import bfo  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
f32 = np.float32

# name -> (layers, input features, loss, optimizer, epochs, batch, lr, cosine)
RUNS = {
    "train_lm": ([(bfo.EMBEDDING, 32, 16), (bfo.POSITIONAL, 8), (bfo.ATTENTION, 2), (bfo.FEEDFORWARD, 32, 0), (bfo.LINEAR, 32)], 0,
                 "cross_entropy_sparse", "adamw", 3, 4, 1e-2, True),
    "train_mlp": ([(bfo.LINEAR, 16), (bfo.SILU,), (bfo.LINEAR, 4)], 8, "mse", "sgd", 4, 5, 0.05, False),
    "train_dense": ([(bfo.LINEAR, 12), (bfo.RELU,), (bfo.LINEAR, 6)], 8, "cross_entropy", "adamw", 2, 6, 5e-3, True),
    # masked language model: no causal mask, loss over the masked positions only (targets -1 elsewhere)
    "train_mlm": ([(bfo.EMBEDDING, 32, 16), (bfo.POSITIONAL, 8), (bfo.BIDIRECTIONAL_ATTENTION, 2), (bfo.FEEDFORWARD, 32, 0),
                   (bfo.LINEAR, 32)], 0, "cross_entropy_masked", "adamw", 3, 4, 1e-2, False),
}
SHUFFLES = [(n, seed) for n in (2, 3, 5, 17, 24, 100) for seed in (1, 2, 3)]


def datasets(rng):
    ids, tgt = rng.integers(0, 32, (24, 8)).astype(f32), rng.integers(0, 32, (24, 8)).astype(f32)
    x, y = rng.standard_normal((20, 8)).astype(f32), rng.standard_normal((20, 4)).astype(f32)
    xd = rng.standard_normal((18, 8)).astype(f32)
    yd = rng.random((18, 6)).astype(f32)
    yd /= yd.sum(-1, keepdims=True)
    mlm_ids = rng.integers(0, 32, (24, 8)).astype(f32)
    mlm_tgt = np.where(rng.random((24, 8)) < 0.3, mlm_ids, f32(-1.0)).astype(f32)
    mlm_tgt[5] = -1.0   # an example with nothing masked
    return {"train_lm": (ids, tgt), "train_mlp": (x, y), "train_dense": (xd, yd), "train_mlm": (mlm_ids, mlm_tgt)}


def main():
    ref = bfo.reference()
    if ref is None:
        raise SystemExit("oracle/_ref/libbf_ref.so is not built; run `make -C oracle ref` where the reference exists")
    rng = np.random.default_rng(20240611)
    expected = {}
    for name, (inputs, targets) in datasets(rng).items():
        layers, features, loss, optimizer, epochs, batch, lr, cosine = RUNS[name]
        base = os.path.join(HERE, name)
        ref.saveDataset(base + ".bfdata", inputs, targets)
        model = ref.model(layers, features)
        model.writeInitialCheckpoint(base + "_init.bfckpt")
        losses = model.runTraining(base + ".bfdata", loss, optimizer, epochs, batch, lr=lr, cosine=cosine,
                                   from_checkpoint=base + "_init.bfckpt", save_checkpoint=base + "_final.bfckpt")
        expected[name + "_epoch_losses"] = np.array(losses, np.float64)
    for n, seed in SHUFFLES:
        expected[f"shuffle_{n}_{seed}"] = ref.shuffleOrder(n, seed)
    expected["cosine"] = np.array([[ref.cosineAnnealingLearningRate(e, total, 1e-3) for e in range(1, 8)] for total in (1, 2, 7)], f32)
    np.savez(os.path.join(HERE, "training_expected.npz"), **expected)
    print("wrote", sorted(os.listdir(HERE)))


if __name__ == "__main__":
    main()
