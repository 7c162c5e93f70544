"""ctypes binding for the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Loads ``oracle/libbf_oracle.so`` (the C restatement of the reference CPU backend) and, when it has
been built, ``oracle/_ref/libbf_ref.so`` (the real reference CPU backend behind the same C
signatures).  Both are exposed as :class:`Oracle` objects with numpy-in / numpy-out methods whose
names follow the reference functions.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this module; the shipped package never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_LIB = os.path.join(_HERE, "libbf_oracle.so")
REF_LIB = os.path.join(_HERE, "_ref", "libbf_ref.so")

_f32p = ctypes.POINTER(ctypes.c_float)
_sz = ctypes.c_size_t

LINEAR, SILU, RELU, GELU, RMSNORM, SOFTMAX, EMBEDDING, POSITIONAL, ATTENTION, FEEDFORWARD, BIDIRECTIONAL_ATTENTION = range(11)


class OracleInvalidArgument(ValueError):
    """Raised where the reference throws std::invalid_argument."""


def build(ref: bool = True) -> None:
    """Compile the oracle libraries (the reference build only where /root/reference exists)."""
    subprocess.check_call(["make", "-C", _HERE, "oracle"] + (["ref"] if ref else []))


def _f(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a: np.ndarray):
    return a.ctypes.data_as(_f32p)


class Oracle:
    def __init__(self, path: str):
        self.path = path
        self.lib = ctypes.CDLL(path)
        self.lib.bfo_model_create.restype = ctypes.c_void_p
        self.lib.bfo_model_param_value.restype = _f32p
        self.lib.bfo_model_param_grad.restype = _f32p
        self.lib.bfo_cosine_learning_rate.restype = ctypes.c_float
        self.is_reference = bool(self.lib.bfo_is_reference())

    # -- plumbing ---------------------------------------------------------------------------
    def _call(self, name, *args):
        fn = getattr(self.lib, name)
        conv = []
        for a in args:
            if isinstance(a, np.ndarray):
                conv.append(_p(a))
            elif isinstance(a, float):
                conv.append(ctypes.c_float(a))
            elif isinstance(a, (int, np.integer)):
                conv.append(_sz(int(a)))
            else:
                conv.append(a)
        status = fn(*conv)
        if status != 0:
            raise OracleInvalidArgument(f"{name} returned {status}")

    # -- forward ----------------------------------------------------------------------------
    def add(self, a, b):
        a, b = _f(a), _f(b)
        if a.shape != b.shape:
            raise OracleInvalidArgument("add: shapes differ")
        out = np.empty_like(a)
        self._call("bfo_add", a, b, out, a.size)
        return out

    def scale(self, x, factor):
        x = _f(x)
        out = np.empty_like(x)
        self._call("bfo_scale", x, float(factor), out, x.size)
        return out

    def addBias(self, x, bias):
        x, bias = _f(x), _f(bias)
        if x.ndim < 2 or bias.ndim != 1 or x.shape[-1] != bias.shape[0]:
            raise OracleInvalidArgument("addBias: shapes")
        out = np.empty_like(x)
        self._call("bfo_add_bias", x, bias, out, x.size // x.shape[-1], x.shape[-1])
        return out

    def matmul(self, a, b):
        a, b = _f(a), _f(b)
        if a.ndim != 2 or b.ndim != 2 or a.shape[1] != b.shape[0]:
            raise OracleInvalidArgument("matmul: shapes")
        c = np.empty((a.shape[0], b.shape[1]), np.float32)
        self._call("bfo_matmul", a, b, c, a.shape[0], a.shape[1], b.shape[1])
        return c

    def matmulTransposeB(self, a, b):
        a, b = _f(a), _f(b)
        if a.ndim != 2 or b.ndim != 2 or a.shape[1] != b.shape[1]:
            raise OracleInvalidArgument("matmulTransposeB: shapes")
        c = np.empty((a.shape[0], b.shape[0]), np.float32)
        self._call("bfo_matmul_transpose_b", a, b, c, a.shape[0], a.shape[1], b.shape[0])
        return c

    def _unary(self, name, x):
        x = _f(x)
        out = np.empty_like(x)
        self._call(name, x, out, x.size)
        return out

    def silu(self, x):
        return self._unary("bfo_silu", x)

    def relu(self, x):
        return self._unary("bfo_relu", x)

    def gelu(self, x):
        return self._unary("bfo_gelu", x)

    def linear(self, x, w, bias):
        x, w, bias = _f(x), _f(w), _f(bias)
        if x.ndim < 2 or x.shape[-1] != w.shape[0] or bias.shape != (w.shape[1],):
            raise OracleInvalidArgument("linear: shapes")
        out = np.empty(x.shape[:-1] + (w.shape[1],), np.float32)
        self._call("bfo_linear", x, w, bias, out, x.size // x.shape[-1], w.shape[0], w.shape[1])
        return out

    def _rows(self, name, x):
        x = _f(x)
        if x.ndim < 2:
            raise OracleInvalidArgument(f"{name}: rank < 2")
        out = np.empty_like(x)
        self._call(name, x, out, x.size // x.shape[-1], x.shape[-1])
        return out

    def rmsnorm(self, x):
        return self._rows("bfo_rmsnorm", x)

    def softmax(self, x):
        return self._rows("bfo_softmax", x)

    def embeddingLookup(self, ids, table):
        ids, table = _f(ids), _f(table)
        if ids.ndim != 2 or table.ndim != 2:
            raise OracleInvalidArgument("embeddingLookup: ranks")
        out = np.empty(ids.shape + (table.shape[1],), np.float32)
        self._call("bfo_embedding_lookup", ids, table, out, ids.shape[0], ids.shape[1], table.shape[0], table.shape[1])
        return out

    def addPositionalEmbeddingAt(self, x, table, offset=0):
        x, table = _f(x), _f(table)
        if x.ndim != 3 or table.ndim != 2 or table.shape[1] != x.shape[2]:
            raise OracleInvalidArgument("addPositionalEmbedding: shapes")
        out = np.empty_like(x)
        self._call("bfo_add_positional_embedding_at", x, table, out, x.shape[0], x.shape[1], x.shape[2],
                   table.shape[0], offset)
        return out

    def addPositionalEmbedding(self, x, table):
        return self.addPositionalEmbeddingAt(x, table, 0)

    def feedForward(self, x, w1, b1, w2, b2, act=0):
        x, w1, b1, w2, b2 = map(_f, (x, w1, b1, w2, b2))
        out = np.empty_like(x)
        self._call("bfo_feed_forward", x, w1, b1, w2, b2, out, x.size // x.shape[-1], x.shape[-1], w1.shape[1],
                   ctypes.c_int(act))
        return out

    def selfAttention(self, x, wq, wk, wv, wout, heads, causal=True):
        x, wq, wk, wv, wout = map(_f, (x, wq, wk, wv, wout))
        if x.ndim != 3:
            raise OracleInvalidArgument("selfAttention: rank")
        out = np.empty_like(x)
        self._call("bfo_self_attention", x, wq, wk, wv, wout, out, x.shape[0], x.shape[1], x.shape[2], heads,
                   ctypes.c_int(1 if causal else 0))
        return out

    def selfAttentionIncremental(self, x_new, wq, wk, wv, wout, heads, k_cache=None, v_cache=None):
        x_new, wq, wk, wv, wout = map(_f, (x_new, wq, wk, wv, wout))
        batch, new_len, dim = x_new.shape
        old_len = 0 if k_cache is None else k_cache.shape[1]
        kc = _f(k_cache) if old_len else np.zeros(1, np.float32)
        vc = _f(v_cache) if old_len else np.zeros(1, np.float32)
        out = np.empty_like(x_new)
        k_out = np.empty((batch, old_len + new_len, dim), np.float32)
        v_out = np.empty_like(k_out)
        self._call("bfo_self_attention_incremental", x_new, wq, wk, wv, wout, out, kc, vc, k_out, v_out, batch,
                   new_len, old_len, dim, heads)
        return out, k_out, v_out

    def attentionCoreForward(self, q, k, v, heads, scale, old_len=0):
        q, k, v = _f(q), _f(k), _f(v)
        batch, new_len, dim = q.shape
        total = k.shape[1]
        out = np.empty_like(q)
        m = np.empty((batch, heads, new_len), np.float32)
        l = np.empty_like(m)
        self._call("bfo_attention_core_forward", q, k, v, out, m, l, batch, heads, new_len, total, dim, float(scale),
                   old_len)
        return out, m, l

    def attentionCoreBackward(self, d_out, q, k, v, heads, scale, old_len=0):
        d_out, q, k, v = _f(d_out), _f(q), _f(k), _f(v)
        batch, new_len, dim = q.shape
        total = k.shape[1]
        dq = np.empty_like(q)
        dk = np.empty_like(k)
        dv = np.empty_like(v)
        self._call("bfo_attention_core_backward", d_out, q, k, v, dq, dk, dv, batch, heads, new_len, total, dim,
                   float(scale), old_len)
        return dq, dk, dv

    # -- backward ---------------------------------------------------------------------------
    def matmulBackward(self, a, b, g):
        a, b, g = _f(a), _f(b), _f(g)
        if a.ndim != 2 or b.ndim != 2 or g.shape != (a.shape[0], b.shape[1]) or a.shape[1] != b.shape[0]:
            raise OracleInvalidArgument("matmulBackward: shapes")
        da, db = np.empty_like(a), np.empty_like(b)
        self._call("bfo_matmul_backward", a, b, g, da, db, a.shape[0], a.shape[1], b.shape[1])
        return da, db

    def matmulTransposeBBackward(self, a, b, g):
        a, b, g = _f(a), _f(b), _f(g)
        da, db = np.empty_like(a), np.empty_like(b)
        self._call("bfo_matmul_transpose_b_backward", a, b, g, da, db, a.shape[0], a.shape[1], b.shape[0])
        return da, db

    def addBiasBackward(self, g):
        g = _f(g)
        if g.ndim < 2:
            raise OracleInvalidArgument("addBiasBackward: rank")
        db = np.empty(g.shape[-1], np.float32)
        self._call("bfo_add_bias_backward", g, db, g.size // g.shape[-1], g.shape[-1])
        return g.copy(), db

    def _binary(self, name, x, g):
        x, g = _f(x), _f(g)
        if x.shape != g.shape:
            raise OracleInvalidArgument(f"{name}: shapes differ")
        out = np.empty_like(x)
        self._call(name, x, g, out, x.size)
        return out

    def siluBackward(self, x, g):
        return self._binary("bfo_silu_backward", x, g)

    def reluBackward(self, x, g):
        return self._binary("bfo_relu_backward", x, g)

    def geluBackward(self, x, g):
        return self._binary("bfo_gelu_backward", x, g)

    def _rows2(self, name, x, g):
        x, g = _f(x), _f(g)
        if x.shape != g.shape or x.ndim < 2:
            raise OracleInvalidArgument(f"{name}: shapes")
        out = np.empty_like(x)
        self._call(name, x, g, out, x.size // x.shape[-1], x.shape[-1])
        return out

    def rmsnormBackward(self, x, g):
        return self._rows2("bfo_rmsnorm_backward", x, g)

    def softmaxBackward(self, x, g):
        return self._rows2("bfo_softmax_backward", x, g)

    def embeddingLookupBackward(self, ids, g, vocab):
        ids, g = _f(ids), _f(g)
        if ids.ndim != 2 or g.ndim != 3 or ids.shape != g.shape[:2]:
            raise OracleInvalidArgument("embeddingLookupBackward: shapes")
        dt = np.empty((vocab, g.shape[2]), np.float32)
        self._call("bfo_embedding_lookup_backward", ids, g, dt, ids.shape[0], ids.shape[1], vocab, g.shape[2])
        return dt

    def addPositionalEmbeddingBackward(self, g, max_seq):
        g = _f(g)
        if g.ndim != 3:
            raise OracleInvalidArgument("addPositionalEmbeddingBackward: rank")
        dt = np.empty((max_seq, g.shape[2]), np.float32)
        self._call("bfo_add_positional_embedding_backward", g, dt, g.shape[0], g.shape[1], g.shape[2], max_seq)
        return g.copy(), dt

    def feedForwardBackward(self, x, w1, b1, w2, b2, g, act=0):
        x, w1, b1, w2, b2, g = map(_f, (x, w1, b1, w2, b2, g))
        dx, dw1, db1, dw2, db2 = (np.empty_like(t) for t in (x, w1, b1, w2, b2))
        self._call("bfo_feed_forward_backward", x, w1, b1, w2, b2, g, dx, dw1, db1, dw2, db2,
                   x.size // x.shape[-1], x.shape[-1], w1.shape[1], ctypes.c_int(act))
        return dx, dw1, db1, dw2, db2

    def selfAttentionBackward(self, x, wq, wk, wv, wout, heads, g, causal=True):
        x, wq, wk, wv, wout, g = map(_f, (x, wq, wk, wv, wout, g))
        dx, dwq, dwk, dwv, dwo = (np.empty_like(t) for t in (x, wq, wk, wv, wout))
        self._call("bfo_self_attention_backward", x, wq, wk, wv, wout, g, dx, dwq, dwk, dwv, dwo, x.shape[0],
                   x.shape[1], x.shape[2], heads, ctypes.c_int(1 if causal else 0))
        return dx, dwq, dwk, dwv, dwo

    # -- losses -----------------------------------------------------------------------------
    def meanSquaredError(self, pred, target):
        pred, target = _f(pred), _f(target)
        if pred.shape != target.shape:
            raise OracleInvalidArgument("meanSquaredError: shapes differ")
        grad = np.empty_like(pred)
        value = ctypes.c_float()
        self._call("bfo_mean_squared_error", pred, target, grad, ctypes.byref(value), pred.size)
        return value.value, grad

    def softmaxCrossEntropy(self, logits, target):
        logits, target = _f(logits), _f(target)
        if logits.shape != target.shape or logits.ndim < 2:
            raise OracleInvalidArgument("softmaxCrossEntropy: shapes")
        grad = np.empty_like(logits)
        value = ctypes.c_float()
        self._call("bfo_softmax_cross_entropy", logits, target, grad, ctypes.byref(value),
                   logits.size // logits.shape[-1], logits.shape[-1])
        return value.value, grad

    def softmaxCrossEntropySparse(self, logits, target_idx):
        logits, target_idx = _f(logits), _f(target_idx)
        if logits.ndim < 2 or target_idx.size != logits.size // logits.shape[-1]:
            raise OracleInvalidArgument("softmaxCrossEntropySparse: shapes")
        grad = np.empty_like(logits)
        value = ctypes.c_float()
        self._call("bfo_softmax_cross_entropy_sparse", logits, target_idx, grad, ctypes.byref(value),
                   logits.size // logits.shape[-1], logits.shape[-1])
        return value.value, grad

    def softmaxCrossEntropyMasked(self, logits, target_idx):
        """loss.cpp:149-215: index -1 = row ignored; means over the other rows."""
        logits, target_idx = _f(logits), _f(target_idx)
        if logits.ndim < 2 or target_idx.size != logits.size // logits.shape[-1]:
            raise OracleInvalidArgument("softmaxCrossEntropyMasked: shapes")
        grad = np.empty_like(logits)
        value = ctypes.c_float()
        self._call("bfo_softmax_cross_entropy_masked", logits, target_idx, grad, ctypes.byref(value),
                   logits.size // logits.shape[-1], logits.shape[-1])
        return value.value, grad

    # -- optimizers / misc --------------------------------------------------------------------
    def sgdStep(self, param, grad, lr):
        param = _f(param).copy()
        self._call("bfo_sgd_step", param, _f(grad), param.size, float(lr))
        return param

    def adamwStep(self, param, grad, m, v, step, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01):
        param, m, v = _f(param).copy(), _f(m).copy(), _f(v).copy()
        self._call("bfo_adamw_step", param, _f(grad), m, v, param.size, ctypes.c_longlong(step), float(lr),
                   float(beta1), float(beta2), float(eps), float(wd))
        return param, m, v

    def roundToBf16(self, x):
        return self._unary("bfo_round_to_bf16", x)

    def argmaxLastPosition(self, logits):
        logits = _f(logits)
        seq, vocab = logits.shape[-2], logits.shape[-1]
        idx = ctypes.c_longlong()
        self._call("bfo_argmax_last_position", logits, seq, vocab, ctypes.byref(idx))
        return idx.value

    def shuffleOrder(self, num_examples: int, seed: int) -> np.ndarray:
        """The permutation data::Dataset::shuffle(seed) applies: result[i] = example that moves to position i."""
        order = (_sz * max(num_examples, 1))()
        if self.lib.bfo_shuffle_order(_sz(num_examples), ctypes.c_uint(seed), order) != 0:
            raise OracleInvalidArgument("shuffle_order")
        return np.array(order[:num_examples], dtype=np.int64)

    def cosineAnnealingLearningRate(self, epoch: int, total_epochs: int, base: float) -> float:
        return float(self.lib.bfo_cosine_learning_rate(ctypes.c_longlong(epoch), ctypes.c_longlong(total_epochs), ctypes.c_float(base)))

    def saveDataset(self, path: str, inputs, targets) -> None:
        """inputs: [examples, *inputShape], targets: [examples, *targetShape] (data::saveDataset, BFDATA1)."""
        inputs, targets = _f(inputs), _f(targets)
        ins, tgs = inputs.shape[1:], targets.shape[1:]
        st = self.lib.bfo_save_dataset(path.encode(), len(ins), (_sz * max(len(ins), 1))(*ins), len(tgs), (_sz * max(len(tgs), 1))(*tgs),
                                       _p(inputs), _p(targets), _sz(inputs.shape[0]))
        if st != 0:
            raise OracleInvalidArgument("save_dataset")

    def model(self, layers, input_features=0):
        return OracleModel(self, layers, input_features)


class OracleModel:
    """A trainable pipeline: ``layers`` is a list of ``(kind, arg0, arg1)`` tuples."""

    def __init__(self, oracle: Oracle, layers, input_features=0):
        self.o = oracle
        n = len(layers)
        kinds = (ctypes.c_int * n)(*[l[0] for l in layers])
        a0 = (ctypes.c_longlong * n)(*[(l[1] if len(l) > 1 else 0) for l in layers])
        a1 = (ctypes.c_longlong * n)(*[(l[2] if len(l) > 2 else 0) for l in layers])
        self.handle = ctypes.c_void_p(oracle.lib.bfo_model_create(n, kinds, a0, a1, _sz(input_features)))
        if not self.handle:
            raise OracleInvalidArgument("model_create failed")
        self.names, self.counts = [], []
        for i in range(oracle.lib.bfo_model_num_params(self.handle)):
            buf = ctypes.create_string_buffer(96)
            cnt = _sz()
            oracle.lib.bfo_model_param_info(self.handle, i, buf, _sz(96), ctypes.byref(cnt))
            self.names.append(buf.value.decode())
            self.counts.append(cnt.value)
        self._out_count = 0

    def __del__(self):
        if getattr(self, "handle", None):
            self.o.lib.bfo_model_destroy(self.handle)
            self.handle = None

    def value(self, i) -> np.ndarray:
        """A writable numpy view of parameter ``i``."""
        ptr = self.o.lib.bfo_model_param_value(self.handle, i)
        return np.ctypeslib.as_array(ptr, shape=(self.counts[i],))

    def grad(self, i) -> np.ndarray:
        ptr = self.o.lib.bfo_model_param_grad(self.handle, i)
        return np.ctypeslib.as_array(ptr, shape=(self.counts[i],))

    def forward(self, x, out_capacity: Optional[int] = None):
        x = _f(x)
        shape = (_sz * x.ndim)(*x.shape)
        cap = out_capacity or max(x.size * 8, 1 << 20)
        while True:
            out = np.empty(cap, np.float32)
            cnt = _sz()
            status = self.o.lib.bfo_model_forward(self.handle, _p(x), x.ndim, shape, _p(out), _sz(cap),
                                                  ctypes.byref(cnt))
            if status != 0 and cnt.value > cap:
                cap = cnt.value
                continue
            if status != 0:
                raise OracleInvalidArgument("model_forward")
            self._out_count = cnt.value
            return out[: cnt.value].copy()

    def backward(self, grad):
        grad = _f(grad)
        if self.o.lib.bfo_model_backward(self.handle, _p(grad), _sz(grad.size)) != 0:
            raise OracleInvalidArgument("model_backward")

    def zeroGrad(self):
        self.o.lib.bfo_model_zero_grad(self.handle)

    def adamwStep(self, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01):
        f = ctypes.c_float
        if self.o.lib.bfo_model_adamw_step(self.handle, f(lr), f(beta1), f(beta2), f(eps), f(wd)) != 0:
            raise OracleInvalidArgument("model_adamw_step")


    def saveCheckpoint(self, path: str) -> None:
        if self.o.lib.bfo_model_save_checkpoint(self.handle, path.encode()) != 0:
            raise OracleInvalidArgument("save_checkpoint")

    def loadCheckpoint(self, path: str) -> None:
        if self.o.lib.bfo_model_load_checkpoint(self.handle, path.encode()) != 0:
            raise OracleInvalidArgument("load_checkpoint")

    def writeInitialCheckpoint(self, path: str) -> None:
        """Reference build only: the checkpoint of this model as cpu::Model(modelIR, seed 42) initialises it."""
        if self.o.lib.bfo_model_write_initial_checkpoint(self.handle, path.encode()) != 0:
            raise OracleInvalidArgument("write_initial_checkpoint")

    def runTraining(self, dataset_path, loss, optimizer, epochs, batch_size, lr=1e-3, cosine=False, from_checkpoint="",
                    save_checkpoint=""):
        """cpu::runTraining.  loss: 'mse' | 'cross_entropy' | 'cross_entropy_sparse'; optimizer: 'sgd' | 'adamw'.
        Returns the list of epoch losses; the trained values are left in this model."""
        losses = (ctypes.c_double * max(epochs, 1))()
        st = self.o.lib.bfo_model_run_training(self.handle, dataset_path.encode(), {"mse": 0, "cross_entropy": 1, "cross_entropy_sparse": 2, "cross_entropy_masked": 3}[loss],
                                               {"sgd": 0, "adamw": 1}[optimizer], ctypes.c_longlong(epochs), _sz(batch_size),
                                               ctypes.c_float(lr), int(bool(cosine)), from_checkpoint.encode(), save_checkpoint.encode(),
                                               losses)
        if st != 0:
            raise OracleInvalidArgument("run_training")
        return list(losses[:epochs])


_cache = {}


def oracle() -> Oracle:
    """The C restatement (built on demand)."""
    if "oracle" not in _cache:
        if not os.path.exists(ORACLE_LIB):
            build(ref=False)
        _cache["oracle"] = Oracle(ORACLE_LIB)
    return _cache["oracle"]


def reference() -> Optional[Oracle]:
    """The real reference build, or None where oracle/_ref has not been built."""
    if "ref" not in _cache:
        _cache["ref"] = Oracle(REF_LIB) if os.path.exists(REF_LIB) else None
    return _cache["ref"]
