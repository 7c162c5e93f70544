"""ctypes binding of blackforge_amd/lib/libbf_hip_host.so: C entry points over the C++ operator layer
(blackforge::backend::hip::Model and friends, include/blackforge/backend/hip/).  Used by the benchmark and
the parity tests to run whole training steps of the C++ host layer."""
from __future__ import annotations

import ctypes
import os
from typing import List, Sequence, Tuple

import numpy as np

from . import capi
from .tensor import DeviceTensor

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libbf_hip_host.so")

LINEAR, SILU, RELU, GELU, RMSNORM, SOFTMAX, EMBEDDING, POSITIONAL, ATTENTION, FEEDFORWARD, BIDIRECTIONAL_ATTENTION = range(11)
LOSS_SPARSE_CE, LOSS_MSE, LOSS_MASKED_CE, LOSS_DENSE_CE = 0, 1, 2, 3

_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        capi.load()
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `make -C blackforge_amd/host` after building libbf_hip.so")
        lib = ctypes.CDLL(LIB_PATH)
        lib.bfh_last_error.restype = ctypes.c_char_p
        lib.bfh_model_create.restype = ctypes.c_void_p
        lib.bfh_model_create.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_longlong),
                                         ctypes.POINTER(ctypes.c_longlong), ctypes.c_size_t, ctypes.c_int]
        lib.bfh_model_destroy.argtypes = [ctypes.c_void_p]
        lib.bfh_model_num_params.argtypes = [ctypes.c_void_p]
        lib.bfh_model_param_info.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t,
                                             ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_void_p),
                                             ctypes.POINTER(ctypes.c_void_p)]
        lib.bfh_model_forward.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_size_t),
                                          ctypes.c_int, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_size_t)]
        lib.bfh_model_loss.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int]
        lib.bfh_model_loss_grad.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_size_t)]
        lib.bfh_model_backward.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.bfh_model_zero_grad.argtypes = [ctypes.c_void_p]
        lib.bfh_model_weights_changed.argtypes = [ctypes.c_void_p]
        lib.bfh_model_adamw_step.argtypes = [ctypes.c_void_p] + [ctypes.c_float] * 5
        lib.bfh_model_sgd_step.argtypes = [ctypes.c_void_p, ctypes.c_float]
        lib.bfh_model_train_step.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_size_t),
                                             ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_float]
        lib.bfh_model_capture_train_step.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_size_t),
                                                     ctypes.c_void_p, ctypes.c_int, ctypes.POINTER(ctypes.c_size_t), ctypes.c_int,
                                                     ctypes.c_int, ctypes.c_float, ctypes.POINTER(ctypes.c_void_p)]
        lib.bfh_captured_step_run.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_int]
        lib.bfh_captured_step_destroy.argtypes = [ctypes.c_void_p]
        lib.bfh_model_read_loss.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_float)]
        lib.bfh_model_run_training.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int, ctypes.c_longlong,
                                               ctypes.c_size_t, ctypes.c_double, ctypes.c_int, ctypes.c_char_p, ctypes.c_char_p,
                                               ctypes.POINTER(ctypes.c_double)]
        lib.bfh_model_save_checkpoint.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        lib.bfh_model_load_checkpoint.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        lib.bfh_shuffle_order.argtypes = [ctypes.c_size_t, ctypes.c_uint, ctypes.POINTER(ctypes.c_size_t)]
        P, Z, I = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
        lib.bfh_self_attention.argtypes = [P] * 5 + [Z] * 4 + [I, I, P]
        lib.bfh_self_attention_backward.argtypes = [P] * 6 + [Z] * 4 + [I, I] + [P] * 5
        lib.bfh_feed_forward.argtypes = [P, I, ctypes.POINTER(Z)] + [P] * 4 + [Z, I, I, P]
        lib.bfh_feed_forward_backward.argtypes = [P, I, ctypes.POINTER(Z)] + [P] * 5 + [Z, I, I] + [P] * 5
        lib.bfh_kv_cache_create.restype = P
        lib.bfh_kv_cache_destroy.argtypes = [P]
        lib.bfh_kv_cache_info.argtypes = [P, ctypes.POINTER(Z), ctypes.POINTER(Z), ctypes.POINTER(P), ctypes.POINTER(P)]
        lib.bfh_self_attention_incremental.argtypes = [P] * 6 + [Z] * 4 + [I, P]
        lib.bfh_model_forward_incremental.argtypes = [P, P, I, ctypes.POINTER(Z), ctypes.POINTER(P), ctypes.POINTER(Z)]
        lib.bfh_model_reset_generation.argtypes = [P]
        lib.bfh_model_generate_greedy.argtypes = [P, P, Z, Z, ctypes.POINTER(ctypes.c_longlong)]
        lib.bfh_model_argmax_last.argtypes = [P, Z, ctypes.POINTER(ctypes.c_longlong)]
        _lib = lib
    return _lib


def _check(status: int):
    if status == 0:
        return
    message = load().bfh_last_error().decode(errors="replace")
    raise ValueError(message) if status == 1 else RuntimeError(message)


class CapturedStep:
    """A recorded training step of a HostModel; keeps the model and the input tensors alive, and goes before them."""

    def __init__(self, model, handle, optimizer, tensors):
        self.model, self.handle, self.optimizer, self.tensors = model, handle, optimizer, tensors

    def run(self, lr: float = 1e-3) -> None:
        _check(load().bfh_captured_step_run(self.model.handle, self.handle, lr, self.optimizer))

    def close(self) -> None:
        if self.handle:
            _check(load().bfh_captured_step_destroy(self.handle))
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class HostModel:
    """A blackforge::backend::hip::Model built from ``(kind, arg0, arg1)`` layer tuples."""

    def __init__(self, layers: Sequence[Tuple[int, ...]], input_features: int = 0, use_bf16: bool = False):
        lib = load()
        n = len(layers)
        kinds = (ctypes.c_int * n)(*[l[0] for l in layers])
        a0 = (ctypes.c_longlong * n)(*[(l[1] if len(l) > 1 else 0) for l in layers])
        a1 = (ctypes.c_longlong * n)(*[(l[2] if len(l) > 2 else 0) for l in layers])
        self.handle = ctypes.c_void_p(lib.bfh_model_create(n, kinds, a0, a1, input_features, int(use_bf16)))
        if not self.handle:
            _check(1)
        self.names: List[str] = []
        self.counts: List[int] = []
        self._value_ptrs, self._grad_ptrs = [], []
        for i in range(lib.bfh_model_num_params(self.handle)):
            name = ctypes.create_string_buffer(96)
            count, vp, gp = ctypes.c_size_t(), ctypes.c_void_p(), ctypes.c_void_p()
            lib.bfh_model_param_info(self.handle, i, name, 96, ctypes.byref(count), ctypes.byref(vp), ctypes.byref(gp))
            self.names.append(name.value.decode())
            self.counts.append(count.value)
            self._value_ptrs.append(vp)
            self._grad_ptrs.append(gp)

    def __del__(self):
        if getattr(self, "handle", None):
            load().bfh_model_destroy(self.handle)
            self.handle = None

    def set_value(self, i: int, host) -> None:
        host = np.ascontiguousarray(host, np.float32).reshape(-1)
        assert host.size == self.counts[i]
        capi.call("bf_hip_memcpy_h2d", self._value_ptrs[i], host.ctypes.data_as(ctypes.c_void_p), host.nbytes)
        _check(load().bfh_model_weights_changed(self.handle))   # the model's cached bf16 weight images are stale now

    def _read(self, ptr, count) -> np.ndarray:
        out = np.empty(count, np.float32)
        capi.call("bf_hip_memcpy_d2h", out.ctypes.data_as(ctypes.c_void_p), ptr, out.nbytes)
        return out

    def value(self, i: int) -> np.ndarray:
        return self._read(self._value_ptrs[i], self.counts[i])

    def grad(self, i: int) -> np.ndarray:
        return self._read(self._grad_ptrs[i], self.counts[i])

    def forward(self, x: DeviceTensor, trusted: bool = False) -> np.ndarray:
        shape = (ctypes.c_size_t * len(x.shape))(*x.shape)
        out, count = ctypes.c_void_p(), ctypes.c_size_t()
        _check(load().bfh_model_forward(self.handle, x.ptr, len(x.shape), shape, int(trusted), ctypes.byref(out), ctypes.byref(count)))
        return self._read(out, count.value)

    def loss(self, target: DeviceTensor, kind: int = LOSS_SPARSE_CE) -> None:
        _check(load().bfh_model_loss(self.handle, target.ptr, kind))

    def backward(self, trusted: bool = False) -> None:
        _check(load().bfh_model_backward(self.handle, int(trusted)))

    def zeroGrad(self) -> None:
        _check(load().bfh_model_zero_grad(self.handle))

    def adamwStep(self, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01) -> None:
        _check(load().bfh_model_adamw_step(self.handle, lr, beta1, beta2, eps, wd))

    def sgdStep(self, lr: float) -> None:
        _check(load().bfh_model_sgd_step(self.handle, lr))

    def trainStep(self, x: DeviceTensor, target: DeviceTensor, loss_kind: int = LOSS_SPARSE_CE, optimizer: int = 1, lr: float = 1e-3):
        shape = (ctypes.c_size_t * len(x.shape))(*x.shape)
        _check(load().bfh_model_train_step(self.handle, x.ptr, len(x.shape), shape, target.ptr, loss_kind, optimizer, lr))

    def captureTrainStep(self, x: DeviceTensor, target: DeviceTensor, loss_kind: int = LOSS_SPARSE_CE, optimizer: int = 1, lr: float = 1e-3):
        """hip::CapturedTrainStep over x and target: the step recorded once (nothing executes), replayed by run()."""
        shape = (ctypes.c_size_t * len(x.shape))(*x.shape)
        tshape = (ctypes.c_size_t * len(target.shape))(*target.shape)
        step = ctypes.c_void_p()
        _check(load().bfh_model_capture_train_step(self.handle, x.ptr, len(x.shape), shape, target.ptr, len(target.shape), tshape, loss_kind,
                                                   optimizer, lr, ctypes.byref(step)))
        return CapturedStep(self, step, optimizer, (x, target))

    def _refresh_params(self) -> None:
        """Re-reads names, counts and device pointers of the parameters (a checkpoint load replaces the buffers)."""
        lib = load()
        self.names, self.counts, self._value_ptrs, self._grad_ptrs = [], [], [], []
        for i in range(lib.bfh_model_num_params(self.handle)):
            buf, cnt = ctypes.create_string_buffer(96), ctypes.c_size_t()
            val, grd = ctypes.c_void_p(), ctypes.c_void_p()
            _check(lib.bfh_model_param_info(self.handle, i, buf, 96, ctypes.byref(cnt), ctypes.byref(val), ctypes.byref(grd)))
            self.names.append(buf.value.decode())
            self.counts.append(cnt.value)
            self._value_ptrs.append(val)
            self._grad_ptrs.append(grd)

    def saveCheckpoint(self, path: str) -> None:
        """hip::saveCheckpoint: BFCKPT1, the format of the CPU and CUDA backends."""
        _check(load().bfh_model_save_checkpoint(self.handle, path.encode()))

    def loadCheckpoint(self, path: str) -> None:
        _check(load().bfh_model_load_checkpoint(self.handle, path.encode()))
        self._refresh_params()

    def runTraining(self, dataset_path: str, loss: str, optimizer: str, epochs: int, batch_size: int, lr: float = 1e-3,
                    cosine: bool = False, from_checkpoint: str = "", save_checkpoint: str = ""):
        """hip::runTraining over a BFDATA1 file; returns the epoch losses."""
        losses = (ctypes.c_double * max(epochs, 1))()
        _check(load().bfh_model_run_training(self.handle, dataset_path.encode(), {"mse": 0, "cross_entropy": 1, "cross_entropy_sparse": 2, "cross_entropy_masked": 3}[loss],
                                             {"sgd": 0, "adamw": 1}[optimizer], epochs, batch_size, lr, int(cosine),
                                             from_checkpoint.encode(), save_checkpoint.encode(), losses))
        self._refresh_params()
        return list(losses[:epochs])

    def forwardIncremental(self, x: DeviceTensor, read: bool = True):
        """hip::Model::forwardIncremental on the new positions only (K/V of earlier ones come from the model's caches).
        read=False leaves the logits on the device (argmaxLast picks the next token there) and returns None."""
        shape = (ctypes.c_size_t * len(x.shape))(*x.shape)
        out, count = ctypes.c_void_p(), ctypes.c_size_t()
        _check(load().bfh_model_forward_incremental(self.handle, x.ptr, len(x.shape), shape, ctypes.byref(out), ctypes.byref(count)))
        return self._read(out, count.value) if read else None

    def generateGreedy(self, prompt: DeviceTensor, count: int) -> list:
        """hip::Model::generateGreedy: `count` greedy tokens after a [1, n] prompt; token and position stay on the device between steps."""
        tokens = (ctypes.c_longlong * max(count, 1))()
        _check(load().bfh_model_generate_greedy(self.handle, prompt.ptr, prompt.shape[1], count, tokens))
        return list(tokens[:count])

    def resetGenerationState(self) -> None:
        _check(load().bfh_model_reset_generation(self.handle))

    def argmaxLast(self, vocab: int) -> int:
        """hip::argmaxLastPosition over the last output of forward / forwardIncremental."""
        index = ctypes.c_longlong()
        _check(load().bfh_model_argmax_last(self.handle, vocab, ctypes.byref(index)))
        return index.value

    def readLossSum(self) -> float:
        v = ctypes.c_float()
        _check(load().bfh_model_read_loss(self.handle, ctypes.byref(v)))
        return v.value


def shuffleOrder(num_examples: int, seed: int) -> np.ndarray:
    """The permutation hip::HostDataset::shuffle(seed) applies: result[i] = example that moves to position i."""
    order = (ctypes.c_size_t * max(num_examples, 1))()
    _check(load().bfh_shuffle_order(num_examples, seed, order))
    return np.array(order[:num_examples], dtype=np.int64)


# ---- composite blocks of the C++ operator layer (hip::selfAttention*, hip::feedForward*) --------------------
# variant: 0 stateless fp32, 1 stateless bf16, 2 the ForwardCached/BackwardCached pair in fp32, 3 that pair in bf16.
def _require_rank3(name: str, x: DeviceTensor):
    if x.rank() != 3:
        raise ValueError(f"{name}: needs an input of rank 3 [batch, seq, dim]")


def selfAttention(x, wq, wk, wv, wout, heads: int, variant: int = 0, causal: bool = True) -> DeviceTensor:
    _require_rank3("selfAttention", x)
    batch, seq, dim = x.shape
    out = DeviceTensor(x.shape)
    _check(load().bfh_self_attention(x.ptr, wq.ptr, wk.ptr, wv.ptr, wout.ptr, batch, seq, dim, heads, variant, int(causal), out.ptr))
    return out


def selfAttentionBackward(x, wq, wk, wv, wout, heads: int, g, variant: int = 0, causal: bool = True):
    """Returns (dInput, dWq, dWk, dWv, dWout)."""
    _require_rank3("selfAttentionBackward", x)
    batch, seq, dim = x.shape
    outs = [DeviceTensor(x.shape)] + [DeviceTensor((dim, dim)) for _ in range(4)]
    _check(load().bfh_self_attention_backward(x.ptr, wq.ptr, wk.ptr, wv.ptr, wout.ptr, g.ptr, batch, seq, dim, heads, variant,
                                              int(causal), *[t.ptr for t in outs]))
    return tuple(outs)


def feedForward(x, w1, b1, w2, b2, act: int = 0, variant: int = 0) -> DeviceTensor:
    shape = (ctypes.c_size_t * len(x.shape))(*x.shape)
    out = DeviceTensor(x.shape)
    _check(load().bfh_feed_forward(x.ptr, len(x.shape), shape, w1.ptr, b1.ptr, w2.ptr, b2.ptr, w1.shape[1], variant, act, out.ptr))
    return out


def feedForwardBackward(x, w1, b1, w2, b2, g, act: int = 0, variant: int = 0):
    """Returns (dInput, dW1, dB1, dW2, dB2)."""
    shape = (ctypes.c_size_t * len(x.shape))(*x.shape)
    outs = [DeviceTensor(x.shape), DeviceTensor(w1.shape), DeviceTensor(b1.shape), DeviceTensor(w2.shape), DeviceTensor(b2.shape)]
    _check(load().bfh_feed_forward_backward(x.ptr, len(x.shape), shape, w1.ptr, b1.ptr, w2.ptr, b2.ptr, g.ptr, w1.shape[1], variant,
                                            act, *[t.ptr for t in outs]))
    return tuple(outs)


class KVCache:
    """hip::KVCache behind a handle."""

    def __init__(self):
        self.handle = ctypes.c_void_p(load().bfh_kv_cache_create())

    def __del__(self):
        if getattr(self, "handle", None):
            load().bfh_kv_cache_destroy(self.handle)
            self.handle = None

    def _info(self, tensors=True):
        length, capacity, k, v = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_void_p(), ctypes.c_void_p()
        st = load().bfh_kv_cache_info(self.handle, ctypes.byref(length), ctypes.byref(capacity), ctypes.byref(k) if tensors else None,
                                      ctypes.byref(v) if tensors else None)
        if st != 0:
            raise RuntimeError("bfh_kv_cache_info failed")
        self._capacity = capacity.value
        return length.value, k, v

    @property
    def length(self) -> int:
        return self._info(False)[0]

    @property
    def capacity(self) -> int:
        self._info(False)
        return self._capacity

    def keys(self, batch: int, dim: int) -> np.ndarray:
        length, k, _ = self._info()
        out = np.empty((batch, length, dim), np.float32)
        capi.call("bf_hip_memcpy_d2h", out.ctypes.data_as(ctypes.c_void_p), k, out.nbytes)
        return out

    def values(self, batch: int, dim: int) -> np.ndarray:
        length, _, v = self._info()
        out = np.empty((batch, length, dim), np.float32)
        capi.call("bf_hip_memcpy_d2h", out.ctypes.data_as(ctypes.c_void_p), v, out.nbytes)
        return out


def selfAttentionIncremental(xNew, wq, wk, wv, wout, heads: int, cache: KVCache, useBf16: bool = False) -> DeviceTensor:
    _require_rank3("selfAttentionIncremental", xNew)
    batch, newLen, dim = xNew.shape
    out = DeviceTensor(xNew.shape)
    _check(load().bfh_self_attention_incremental(cache.handle, xNew.ptr, wq.ptr, wk.ptr, wv.ptr, wout.ptr, batch, newLen, dim, heads,
                                                 int(useBf16), out.ptr))
    return out
