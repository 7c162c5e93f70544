"""The training-run fixtures under tests/golden/ (written by tests/golden/make_training_fixtures.py from the real
reference) and the run descriptions they belong to, for the CPU and GPU training tests."""
import os
import struct

import numpy as np

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
EXPECTED = os.path.join(GOLDEN_DIR, "training_expected.npz")

# layer kinds as the oracle and the host layer number them (bf_oracle.h: BFO_LINEAR = 0 ... BFO_BIDIRECTIONAL_ATTENTION = 10)
LINEAR, SILU, RELU, GELU, RMSNORM, SOFTMAX, EMBEDDING, POSITIONAL, ATTENTION, FEEDFORWARD, BIDIRECTIONAL_ATTENTION = range(11)

# name -> (layers, input features, loss, optimizer, epochs, batch, lr, cosine): the same table the generator uses
RUNS = {
    "train_lm": ([(EMBEDDING, 32, 16), (POSITIONAL, 8), (ATTENTION, 2), (FEEDFORWARD, 32, 0), (LINEAR, 32)], 0,
                 "cross_entropy_sparse", "adamw", 3, 4, 1e-2, True),
    "train_mlp": ([(LINEAR, 16), (SILU,), (LINEAR, 4)], 8, "mse", "sgd", 4, 5, 0.05, False),
    "train_dense": ([(LINEAR, 12), (RELU,), (LINEAR, 6)], 8, "cross_entropy", "adamw", 2, 6, 5e-3, True),
    "train_mlm": ([(EMBEDDING, 32, 16), (POSITIONAL, 8), (BIDIRECTIONAL_ATTENTION, 2), (FEEDFORWARD, 32, 0), (LINEAR, 32)], 0,
                  "cross_entropy_masked", "adamw", 3, 4, 1e-2, False),
}
SHUFFLES = [(n, seed) for n in (2, 3, 5, 17, 24, 100) for seed in (1, 2, 3)]


def path(name, suffix):
    return os.path.join(GOLDEN_DIR, name + suffix)


def read_checkpoint(file_path):
    """BFCKPT1 -> ordered list of (name, shape, float32 array): the layout of cpu/checkpoint.cpp:45-83."""
    raw = open(file_path, "rb").read()
    assert raw[:8] == b"BFCKPT1\0", "not a BFCKPT1 file"
    (count,), pos, out = struct.unpack_from("<I", raw, 8), 12, []
    for _ in range(count):
        (n,) = struct.unpack_from("<I", raw, pos); pos += 4
        name = raw[pos:pos + n].decode(); pos += n
        (rank,) = struct.unpack_from("<I", raw, pos); pos += 4
        shape = struct.unpack_from(f"<{rank}Q", raw, pos); pos += 8 * rank
        size = int(np.prod(shape)) if rank else 1
        out.append((name, tuple(shape), np.frombuffer(raw, np.float32, size, pos).copy())); pos += 4 * size
    assert pos == len(raw), "trailing bytes in checkpoint"
    return out


def read_dataset(file_path):
    """BFDATA1 -> (inputs [examples, *shape], targets [examples, *shape]): the layout of data/dataset.cpp:133-184."""
    raw = open(file_path, "rb").read()
    assert raw[:8] == b"BFDATA1\0"
    (n,), pos, shapes = struct.unpack_from("<I", raw, 8), 12, []
    for _ in range(2):
        (rank,) = struct.unpack_from("<I", raw, pos); pos += 4
        shapes.append(struct.unpack_from(f"<{rank}Q", raw, pos)); pos += 8 * rank
    sizes = [int(np.prod(s)) for s in shapes]
    inputs = np.frombuffer(raw, np.float32, n * sizes[0], pos).reshape((n,) + tuple(shapes[0])); pos += 4 * n * sizes[0]
    targets = np.frombuffer(raw, np.float32, n * sizes[1], pos).reshape((n,) + tuple(shapes[1]))
    return inputs.copy(), targets.copy()
