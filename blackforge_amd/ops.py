"""Python mirror of the reference GPU operator interface, on top of the C ABI.

Function names, argument order and error behaviour follow the free functions of
``blackforge::backend::cuda`` (reference ``include/blackforge/backend/cuda/{ops,autodiff,
fused_attention,loss,optimizer}.hpp``): ops take ``DeviceTensor`` and return fresh ``DeviceTensor``
objects, shape errors raise ``ValueError`` (std::invalid_argument in the reference) before anything is
launched.  Every computation is done by ``libbf_hip.so``; this file only validates shapes, allocates
results from the pool and sequences the composite blocks.
"""
from __future__ import annotations

import ctypes
import math

import numpy as np
from dataclasses import dataclass, field
from typing import Dict, List, Optional

from . import capi
from .capi import ACT_GELU, ACT_RELU, ACT_SILU
from .tensor import DeviceTensor

_call = capi.call


def _rows(t: DeviceTensor):
    features = t.shape[-1]
    return (t.elementCount() // features if features else 0), features


def _require(cond: bool, message: str):
    if not cond:
        raise ValueError(message)


# ------------------------------------------------------------------------------------------------
# elementwise (ops.hpp:8-30, 82-84)
# ------------------------------------------------------------------------------------------------
def add(a: DeviceTensor, b: DeviceTensor) -> DeviceTensor:
    _require(a.shape == b.shape, f"add: incompatible shapes {a.shape} and {b.shape}")
    out = DeviceTensor(a.shape)
    _call("bf_hip_add", a.ptr, b.ptr, out.ptr, a.elementCount(), None)
    return out


def scale(x: DeviceTensor, factor: float) -> DeviceTensor:
    out = DeviceTensor(x.shape)
    _call("bf_hip_scale", x.ptr, factor, out.ptr, x.elementCount(), None)
    return out


def _check_bias(name, x, bias):
    _require(x.rank() >= 2 and bias.rank() == 1 and x.shape[-1] == bias.shape[0],
             f"{name}: expected input [..., features] and bias [features], got {x.shape} and {bias.shape}")


def addBias(x: DeviceTensor, bias: DeviceTensor) -> DeviceTensor:
    _check_bias("addBias", x, bias)
    out = DeviceTensor(x.shape)
    _call("bf_hip_add_bias", x.ptr, bias.ptr, out.ptr, *_rows(x), None)
    return out


def addBiasAct(gemm: DeviceTensor, bias: DeviceTensor, act: int) -> DeviceTensor:
    _check_bias("addBiasAct", gemm, bias)
    out = DeviceTensor(gemm.shape)
    _call("bf_hip_add_bias_act", gemm.ptr, bias.ptr, out.ptr, *_rows(gemm), act, None)
    return out


def addBiasSilu(gemm: DeviceTensor, bias: DeviceTensor) -> DeviceTensor:
    return addBiasAct(gemm, bias, ACT_SILU)


def addBiasResidual(gemm: DeviceTensor, bias: DeviceTensor, residual: DeviceTensor) -> DeviceTensor:
    _check_bias("addBiasResidual", gemm, bias)
    _require(gemm.shape == residual.shape, "addBiasResidual: residual shape differs")
    out = DeviceTensor(gemm.shape)
    _call("bf_hip_add_bias_residual", gemm.ptr, bias.ptr, residual.ptr, out.ptr, *_rows(gemm), None)
    return out


def _act(x, act):
    out = DeviceTensor(x.shape)
    _call("bf_hip_act_forward", x.ptr, out.ptr, x.elementCount(), act, None)
    return out


def silu(x): return _act(x, ACT_SILU)
def relu(x): return _act(x, ACT_RELU)
def gelu(x): return _act(x, ACT_GELU)


def _act_bwd(name, x, g, act):
    _require(x.shape == g.shape, f"{name}: incompatible shapes")
    out = DeviceTensor(x.shape)
    _call("bf_hip_act_backward", x.ptr, g.ptr, out.ptr, x.elementCount(), act, None)
    return out


def siluBackward(x, g): return _act_bwd("siluBackward", x, g, ACT_SILU)
def reluBackward(x, g): return _act_bwd("reluBackward", x, g, ACT_RELU)
def geluBackward(x, g): return _act_bwd("geluBackward", x, g, ACT_GELU)


def accumulate(target: DeviceTensor, delta: DeviceTensor) -> None:
    _call("bf_hip_accumulate", target.ptr, delta.ptr, target.elementCount(), None)


def zeroFused(tensors: List[DeviceTensor]) -> None:
    n = len(tensors)
    if n == 0:
        return
    ptrs = (ctypes.c_void_p * n)(*[t.ptr.value if t.ptr else None for t in tensors])
    counts = (ctypes.c_size_t * n)(*[t.elementCount() for t in tensors])
    _call("bf_hip_zero_multi", ptrs, counts, n, None)


# ------------------------------------------------------------------------------------------------
# rows (ops.hpp:92-98, autodiff.hpp:52-84)
# ------------------------------------------------------------------------------------------------
def rmsnorm(x: DeviceTensor) -> DeviceTensor:
    _require(x.rank() >= 2, "rmsnorm: needs a tensor of rank >= 2")
    out = DeviceTensor(x.shape)
    _call("bf_hip_rmsnorm", x.ptr, out.ptr, *_rows(x), None)
    return out


def rmsnormBackward(x: DeviceTensor, g: DeviceTensor) -> DeviceTensor:
    _require(x.shape == g.shape, "rmsnormBackward: incompatible shapes")
    _require(x.rank() >= 2, "rmsnormBackward: needs a tensor of rank >= 2")
    out = DeviceTensor(x.shape)
    _call("bf_hip_rmsnorm_backward", x.ptr, g.ptr, out.ptr, *_rows(x), None)
    return out


def rmsnormBackwardAdd(x: DeviceTensor, g: DeviceTensor, residualGrad: DeviceTensor) -> DeviceTensor:
    """residualGrad + rmsnormBackward(x, g) in one pass."""
    _require(x.shape == g.shape == residualGrad.shape, "rmsnormBackward: incompatible shapes")
    _require(x.rank() >= 2, "rmsnormBackward: needs a tensor of rank >= 2")
    out = DeviceTensor(x.shape)
    _call("bf_hip_rmsnorm_backward_add", x.ptr, g.ptr, residualGrad.ptr, out.ptr, *_rows(x), None)
    return out


def softmax(x: DeviceTensor) -> DeviceTensor:
    _require(x.rank() >= 2, "softmax: needs a tensor of rank >= 2")
    out = DeviceTensor(x.shape)
    _call("bf_hip_softmax", x.ptr, out.ptr, *_rows(x), None)
    return out


def softmaxBackward(x: DeviceTensor, g: DeviceTensor) -> DeviceTensor:
    _require(x.shape == g.shape, "softmaxBackward: incompatible shapes")
    _require(x.rank() >= 2, "softmaxBackward: needs a tensor of rank >= 2")
    out = DeviceTensor(x.shape)
    _call("bf_hip_softmax_backward", x.ptr, g.ptr, out.ptr, *_rows(x), None)
    return out


def biasGradientOnly(g: DeviceTensor) -> DeviceTensor:
    _require(g.rank() >= 2, "biasGradientOnly: needs a gradient of rank >= 2")
    out = DeviceTensor((g.shape[-1],))
    _call("bf_hip_bias_grad", g.ptr, out.ptr, *_rows(g), None)
    return out


def addBiasBackward(g: DeviceTensor):
    """Returns (dInput, dBias); dInput is a copy of g, as in the reference."""
    _require(g.rank() >= 2, "addBiasBackward: needs a gradient of rank >= 2")
    return g.clone(), biasGradientOnly(g)


def addBiasActBackward(gemm: DeviceTensor, bias: DeviceTensor, dHidden: DeviceTensor, act: int):
    _require(gemm.shape == dHidden.shape and bias.rank() == 1 and gemm.shape[-1] == bias.shape[0],
             "addBiasSiluBackward: incompatible shapes")
    dGemm = DeviceTensor(gemm.shape)
    dBias = DeviceTensor(bias.shape)
    _call("bf_hip_add_bias_act_backward", gemm.ptr, bias.ptr, dHidden.ptr, dGemm.ptr, dBias.ptr, *_rows(gemm), act,
          None)
    return dGemm, dBias


def addBiasSiluBackward(gemm, bias, dHidden):
    return addBiasActBackward(gemm, bias, dHidden, ACT_SILU)


# ------------------------------------------------------------------------------------------------
# gather / scatter (ops.hpp:104-122, autodiff.hpp:90-106)
# ------------------------------------------------------------------------------------------------
def _validate_ids(name: str, ids: DeviceTensor, limit: int, what: str):
    bad, first = ctypes.c_size_t(), ctypes.c_longlong()
    _call("bf_hip_count_out_of_range", ids.ptr, ids.elementCount(), limit, ctypes.byref(bad), ctypes.byref(first), None)
    _require(bad.value == 0, f"{name}: {what} {first.value} outside [0, {limit})")


def embeddingLookupPreValidated(ids: DeviceTensor, table: DeviceTensor) -> DeviceTensor:
    _require(ids.rank() == 2, "embeddingLookup: token ids must have rank 2 [batch, seq]")
    _require(table.rank() == 2, "embeddingLookup: table must have rank 2 [vocabSize, dim]")
    out = DeviceTensor(ids.shape + (table.shape[1],))
    _call("bf_hip_embedding_forward", ids.ptr, table.ptr, out.ptr, ids.elementCount(), table.shape[0], table.shape[1],
          None)
    return out


def embeddingLookup(ids: DeviceTensor, table: DeviceTensor) -> DeviceTensor:
    _require(ids.rank() == 2, "embeddingLookup: token ids must have rank 2 [batch, seq]")
    _require(table.rank() == 2, "embeddingLookup: table must have rank 2 [vocabSize, dim]")
    _validate_ids("embeddingLookup", ids, table.shape[0], "token id")
    return embeddingLookupPreValidated(ids, table)


def embeddingLookupBackwardPreValidated(ids: DeviceTensor, g: DeviceTensor, vocabSize: int) -> DeviceTensor:
    _require(ids.rank() == 2 and g.rank() == 3 and ids.shape == g.shape[:2],
             "embeddingLookupBackward: incompatible shapes")
    out = DeviceTensor((vocabSize, g.shape[2]))
    _call("bf_hip_embedding_backward", ids.ptr, g.ptr, out.ptr, ids.elementCount(), vocabSize, g.shape[2], None)
    return out


def embeddingLookupBackward(ids: DeviceTensor, g: DeviceTensor, vocabSize: int) -> DeviceTensor:
    _require(ids.rank() == 2 and g.rank() == 3 and ids.shape == g.shape[:2],
             "embeddingLookupBackward: incompatible shapes")
    _validate_ids("embeddingLookupBackward", ids, vocabSize, "token id")
    return embeddingLookupBackwardPreValidated(ids, g, vocabSize)


def addPositionalEmbeddingAt(x: DeviceTensor, table: DeviceTensor, offset: int) -> DeviceTensor:
    _require(x.rank() == 3, "addPositionalEmbedding: needs an input of rank 3 [batch, seq, dim]")
    _require(table.rank() == 2 and table.shape[1] == x.shape[2], "addPositionalEmbedding: table [maxSeqLen, dim] mismatch")
    out = DeviceTensor(x.shape)
    _call("bf_hip_positional_forward", x.ptr, table.ptr, out.ptr, x.shape[0], x.shape[1], x.shape[2], table.shape[0],
          offset, None)
    return out


def addPositionalEmbedding(x, table):
    return addPositionalEmbeddingAt(x, table, 0)


def addPositionalEmbeddingBackward(g: DeviceTensor, maxSeqLen: int):
    """Returns (dInput, dTable)."""
    _require(g.rank() == 3, "addPositionalEmbeddingBackward: needs a gradient of rank 3")
    dTable = DeviceTensor((maxSeqLen, g.shape[2]))
    _call("bf_hip_positional_backward", g.ptr, dTable.ptr, g.shape[0], g.shape[1], g.shape[2], maxSeqLen, None)
    return g.clone(), dTable


def concatSeq(a: DeviceTensor, b: DeviceTensor) -> DeviceTensor:
    out = DeviceTensor((a.shape[0], a.shape[1] + b.shape[1], a.shape[2]))
    _call("bf_hip_concat_seq", a.ptr, b.ptr, out.ptr, a.shape[0], a.shape[1], b.shape[1], a.shape[2], None)
    return out


def argmaxLastPosition(logits: DeviceTensor) -> int:
    """Greedy next-token choice over [1, seq, vocab] (or [seq, vocab]) logits, computed on the device."""
    seq, vocab = logits.shape[-2], logits.shape[-1]
    idx = ctypes.c_longlong()
    _call("bf_hip_argmax_last_position", logits.ptr, seq, vocab, ctypes.byref(idx), None)
    return idx.value


# ------------------------------------------------------------------------------------------------
# GEMM (ops.hpp:35-80,247-258; autodiff.hpp:23-44)
# ------------------------------------------------------------------------------------------------
def _gemm(ta, tb, a, b, m, n, k):
    out = DeviceTensor((m, n))
    _call("bf_hip_gemm_f32", ta, tb, a.ptr, b.ptr, out.ptr, m, n, k, None)
    return out


def matmul(a: DeviceTensor, b: DeviceTensor) -> DeviceTensor:
    _require(a.rank() == 2 and b.rank() == 2 and a.shape[1] == b.shape[0], f"matmul: incompatible shapes {a.shape} x {b.shape}")
    return _gemm(0, 0, a, b, a.shape[0], b.shape[1], a.shape[1])


def matmulTransposeB(a: DeviceTensor, b: DeviceTensor) -> DeviceTensor:
    _require(a.rank() == 2 and b.rank() == 2 and a.shape[1] == b.shape[1], "matmulTransposeB: incompatible shapes")
    return _gemm(0, 1, a, b, a.shape[0], b.shape[0], a.shape[1])


def _check_mm_bwd(name, a, b, g):
    _require(a.rank() == 2 and b.rank() == 2 and g.rank() == 2 and a.shape[1] == b.shape[0]
             and g.shape == (a.shape[0], b.shape[1]), f"{name}: incompatible shapes")


def matmulBackward(a, b, g):
    """Returns (dA, dB) of c = a @ b."""
    _check_mm_bwd("matmulBackward", a, b, g)
    m, k, n = a.shape[0], a.shape[1], b.shape[1]
    return _gemm(0, 1, g, b, m, k, n), _gemm(1, 0, a, g, k, n, m)


def matmulTransposeBBackward(a, b, g):
    """Returns (dA, dB) of c = a @ b^T with a:[m,k], b:[n,k]."""
    _require(a.rank() == 2 and b.rank() == 2 and g.rank() == 2 and a.shape[1] == b.shape[1]
             and g.shape == (a.shape[0], b.shape[0]), "matmulTransposeBBackward: incompatible shapes")
    m, k, n = a.shape[0], a.shape[1], b.shape[0]
    return _gemm(0, 0, g, b, m, k, n), _gemm(1, 0, g, a, n, k, m)


def _matmul_bf16(name, a, b, cache):
    _require(a.rank() == 2 and b.rank() == 2 and a.shape[1] == b.shape[0], f"{name}: incompatible shapes")
    out = DeviceTensor((a.shape[0], b.shape[1]))
    _call("bf_hip_matmul_bf16", a.ptr, b.ptr, out.ptr, a.shape[0], a.shape[1], b.shape[1], cache, None)
    return out


def matmulBf16(a, b): return _matmul_bf16("matmulBf16", a, b, 0)
def matmulBf16CachedWeight(a, b): return _matmul_bf16("matmulBf16CachedWeight", a, b, 1)


def invalidateBf16WeightCache() -> None:
    _call("bf_hip_invalidate_bf16_weight_cache")


def _matmul_bf16_bwd(name, a, b, g, cache):
    _check_mm_bwd(name, a, b, g)
    dA, dB = DeviceTensor(a.shape), DeviceTensor(b.shape)
    _call("bf_hip_matmul_bf16_backward", a.ptr, b.ptr, g.ptr, dA.ptr, dB.ptr, a.shape[0], a.shape[1], b.shape[1], cache,
          None)
    return dA, dB


def matmulBf16Backward(a, b, g): return _matmul_bf16_bwd("matmulBf16Backward", a, b, g, 0)
def matmulBf16BackwardCachedWeight(a, b, g): return _matmul_bf16_bwd("matmulBf16BackwardCachedWeight", a, b, g, 1)


def _flat2d(t: DeviceTensor):
    """A [rows, features] view descriptor (no copy): a non-owning alias used only inside one op."""
    v = DeviceTensor.__new__(DeviceTensor)
    rows, f = _rows(t)
    v.shape, v.itemsize, v._bytes, v.ptr = (rows, f), t.itemsize, 0, t.ptr  # _bytes = 0: never released
    return v


def _linear(name, x, w, bias, mm):
    _require(x.rank() >= 2, f"{name}: needs a tensor of rank >= 2")
    _require(w.rank() == 2 and x.shape[-1] == w.shape[0], f"{name}: incompatible shapes {x.shape} x {w.shape}")
    _require(bias.rank() == 1 and bias.shape[0] == w.shape[1], f"{name}: bias {bias.shape} does not match {w.shape}")
    prod = mm(_flat2d(x), w)
    out = DeviceTensor(x.shape[:-1] + (w.shape[1],))
    _call("bf_hip_add_bias", prod.ptr, bias.ptr, out.ptr, prod.shape[0], prod.shape[1], None)
    return out


def _linear_bf16(name, x, w, bias, residual, cache):
    """x w (+ bias) (+ residual) with the adds folded into the GEMM's store (bf_hip_linear_bf16)."""
    _require(x.rank() >= 2, f"{name}: needs a tensor of rank >= 2")
    _require(w.rank() == 2 and x.shape[-1] == w.shape[0], f"{name}: incompatible shapes {x.shape} x {w.shape}")
    _require(bias is None or (bias.rank() == 1 and bias.shape[0] == w.shape[1]), f"{name}: bias does not match {w.shape}")
    out = DeviceTensor(x.shape[:-1] + (w.shape[1],))
    _require(residual is None or residual.shape == out.shape, f"{name}: residual shape differs from the product")
    rows = out.elementCount() // w.shape[1] if w.shape[1] else 0
    _call("bf_hip_linear_bf16", x.ptr, w.ptr, bias.ptr if bias is not None else None, residual.ptr if residual is not None else None,
          out.ptr, rows, w.shape[0], w.shape[1], cache, None)
    return out


def linear(x, w, bias): return _linear("linear", x, w, bias, matmul)
def linearBf16(x, w, bias): return _linear_bf16("linearBf16", x, w, bias, None, 0)
def linearBf16CachedWeight(x, w, bias): return _linear_bf16("linearBf16CachedWeight", x, w, bias, None, 1)
def linearBf16Fused(x, w, bias=None, residual=None, cached=False):
    """The projection-plus-adds form the composite blocks use: bias and residual are optional."""
    return _linear_bf16("linearBf16Fused", x, w, bias, residual, 1 if cached else 0)


def _ptr_array(tensors):
    """A host array of device pointers; None entries and empty tensors become NULL."""
    return (ctypes.c_void_p * len(tensors))(*[t.ptr.value if t is not None and t.ptr else None for t in tensors])


def matmulBf16SharedInput(a, weights, cached=False):
    """[a w for w in weights] for up to three weights of one shape: one conversion of `a`, one GEMM when it can be."""
    _require(1 <= len(weights) <= 3, "matmulBf16SharedInput: one to three weights")
    _require(a.rank() == 2 and all(w.rank() == 2 and w.shape == weights[0].shape and w.shape[0] == a.shape[1] for w in weights),
             "matmulBf16SharedInput: incompatible shapes")
    outs = [DeviceTensor((a.shape[0], w.shape[1])) for w in weights]
    _call("bf_hip_matmul_bf16_shared_input", a.ptr, _ptr_array(weights), _ptr_array(outs), len(weights), a.shape[0], a.shape[1],
          weights[0].shape[1], 1 if cached else 0, None)
    return outs


def matmulBf16SharedInputBackward(a, weights, grads, cached=False, want_dA=True, want_dB=(True, True, True)):
    """dA = sum_i g_i w_i^T and dB_i = a^T g_i for the products of matmulBf16SharedInput."""
    _require(len(weights) == len(grads) and 1 <= len(weights) <= 3, "matmulBf16SharedInputBackward: one to three products")
    dA = DeviceTensor(a.shape) if want_dA else None
    dBs = [DeviceTensor(w.shape) if want_dB[i] else None for i, w in enumerate(weights)]
    _call("bf_hip_matmul_bf16_shared_input_backward", a.ptr, _ptr_array(weights), _ptr_array(grads),
          dA.ptr if dA is not None else None, _ptr_array(dBs), len(weights), a.shape[0], a.shape[1], weights[0].shape[1],
          1 if cached else 0, None)
    return dA, dBs


# ------------------------------------------------------------------------------------------------
# fused attention (fused_attention.hpp:55,73)
# ------------------------------------------------------------------------------------------------
@dataclass
class FusedAttentionForwardResult:
    output: DeviceTensor
    m: DeviceTensor
    l: DeviceTensor


@dataclass
class FusedAttentionGrad:
    dQ: DeviceTensor
    dK: DeviceTensor
    dV: DeviceTensor


def fusedAttentionForward(q, k, v, numHeads: int, scaleFactor: float, oldLen: int) -> FusedAttentionForwardResult:
    batch, newLen, dim = q.shape
    totalLen = k.shape[1]
    out = DeviceTensor((batch, newLen, dim))
    m = DeviceTensor((batch, numHeads, newLen))
    l = DeviceTensor((batch, numHeads, newLen))
    _call("bf_hip_attention_forward", q.ptr, k.ptr, v.ptr, out.ptr, m.ptr, l.ptr, batch, numHeads, newLen, totalLen, dim,
          scaleFactor, oldLen, None)
    return FusedAttentionForwardResult(out, m, l)


def fusedAttentionBackward(dOutput, q, k, v, output, m, l, numHeads: int, scaleFactor: float, oldLen: int) -> FusedAttentionGrad:
    batch, newLen, dim = q.shape
    totalLen = k.shape[1]
    dQ, dK, dV = DeviceTensor(q.shape), DeviceTensor(k.shape), DeviceTensor(v.shape)
    _call("bf_hip_attention_backward", dOutput.ptr, q.ptr, k.ptr, v.ptr, output.ptr, m.ptr, l.ptr, dQ.ptr, dK.ptr, dV.ptr,
          batch, numHeads, newLen, totalLen, dim, scaleFactor, oldLen, None)
    return FusedAttentionGrad(dQ, dK, dV)


# ------------------------------------------------------------------------------------------------
# composite blocks (ops.hpp:127-245, autodiff.hpp:117-177).  These are pass-throughs to the C++ operator
# layer (include/blackforge/backend/hip/{ops,autodiff}.hpp) through blackforge_amd/hostlayer.py: the
# orchestration (normalisation, projections, fused attention, residuals) exists once, in C++.
# `act` selects the feed-forward activation: ACT_SILU is the reference block, ACT_GELU the same block
# with gelu substituted.  `cached=True` runs the *ForwardCached / *BackwardCached pair that Model uses.
# ------------------------------------------------------------------------------------------------
def _opt(t):
    return t.ptr if t is not None else None


def feedForwardBf16Fused(x, w1, b1, w2, b2, residual=None, act: int = ACT_SILU, cached=False):
    """bf_hip_feedforward_bf16 on x:[m,d]: returns (out, z, hImage, xImage); the images are raw bf16 storage held in
    DeviceTensors of half the width."""
    _require(x.rank() == 2 and w1.rank() == 2 and w2.rank() == 2 and x.shape[1] == w1.shape[0] and w1.shape[1] == w2.shape[0]
             and w2.shape[1] == x.shape[1], "feedForwardBf16Fused: incompatible shapes")
    m, d, hidden = x.shape[0], x.shape[1], w1.shape[1]
    _require(d % 8 == 0 and hidden % 8 == 0, "feedForwardBf16Fused: d and hidden must be multiples of 8")
    z, hImage, xImage, out = DeviceTensor((m, hidden)), DeviceTensor((m, hidden // 2)), DeviceTensor((m, d // 2)), DeviceTensor((m, d))
    _call("bf_hip_feedforward_bf16", x.ptr, w1.ptr, _opt(b1), w2.ptr, _opt(b2), _opt(residual), act, z.ptr, hImage.ptr, xImage.ptr,
          out.ptr, m, d, hidden, 1 if cached else 0, None)
    return out, z, hImage, xImage


def feedForwardBf16FusedBackward(x, xImage, w1, w2, z, hImage, g, act: int = ACT_SILU, cached=False):
    """bf_hip_feedforward_bf16_backward: returns (dX, dW1, dB1, dW2, dB2); x or xImage may be None."""
    m, d, hidden = g.shape[0], g.shape[1], w1.shape[1]
    dX, dW1, dB1, dW2, dB2 = DeviceTensor((m, d)), DeviceTensor(w1.shape), DeviceTensor((hidden,)), DeviceTensor(w2.shape), DeviceTensor((d,))
    _call("bf_hip_feedforward_bf16_backward", _opt(x), _opt(xImage), w1.ptr, w2.ptr, z.ptr, hImage.ptr, g.ptr, act, dX.ptr, dW1.ptr,
          dB1.ptr, dW2.ptr, dB2.ptr, m, d, hidden, 1 if cached else 0, None)
    return dX, dW1, dB1, dW2, dB2


def _variant(useBf16: bool, cached: bool) -> int:
    return (2 if cached else 0) + (1 if useBf16 else 0)


def feedForward(x, w1, b1, w2, b2, act: int = ACT_SILU, useBf16: bool = False, cached: bool = False):
    from . import hostlayer
    return hostlayer.feedForward(x, w1, b1, w2, b2, act, _variant(useBf16, cached))


def feedForwardBf16(x, w1, b1, w2, b2, act: int = ACT_SILU):
    return feedForward(x, w1, b1, w2, b2, act, True)


@dataclass
class FeedForwardGrad:
    dInput: DeviceTensor
    dW1: DeviceTensor
    dB1: DeviceTensor
    dW2: DeviceTensor
    dB2: DeviceTensor


def feedForwardBackward(x, w1, b1, w2, b2, g, act: int = ACT_SILU, useBf16: bool = False, cached: bool = False) -> FeedForwardGrad:
    from . import hostlayer
    return FeedForwardGrad(*hostlayer.feedForwardBackward(x, w1, b1, w2, b2, g, act, _variant(useBf16, cached)))


def feedForwardBf16Backward(x, w1, b1, w2, b2, g, act: int = ACT_SILU):
    return feedForwardBackward(x, w1, b1, w2, b2, g, act, True)


def selfAttention(x, wq, wk, wv, wout, numHeads: int, useBf16: bool = False, cached: bool = False):
    from . import hostlayer
    return hostlayer.selfAttention(x, wq, wk, wv, wout, numHeads, _variant(useBf16, cached), True)


def selfAttentionBf16(x, wq, wk, wv, wout, numHeads: int):
    return selfAttention(x, wq, wk, wv, wout, numHeads, True)


def bidirectionalSelfAttention(x, wq, wk, wv, wout, numHeads: int, useBf16: bool = False, cached: bool = False):
    """The block without the causal mask (CPU backend, ops.cpp:504-507; absent from the CUDA backend, model.cu:151-160)."""
    from . import hostlayer
    return hostlayer.selfAttention(x, wq, wk, wv, wout, numHeads, _variant(useBf16, cached), False)


@dataclass
class SelfAttentionGrad:
    dInput: DeviceTensor
    dWq: DeviceTensor
    dWk: DeviceTensor
    dWv: DeviceTensor
    dWout: DeviceTensor


def selfAttentionBackward(x, wq, wk, wv, wout, numHeads: int, g, useBf16: bool = False, cached: bool = False) -> SelfAttentionGrad:
    from . import hostlayer
    return SelfAttentionGrad(*hostlayer.selfAttentionBackward(x, wq, wk, wv, wout, numHeads, g, _variant(useBf16, cached), True))


def selfAttentionBf16Backward(x, wq, wk, wv, wout, numHeads: int, g):
    return selfAttentionBackward(x, wq, wk, wv, wout, numHeads, g, True)


def bidirectionalSelfAttentionBackward(x, wq, wk, wv, wout, numHeads: int, g, useBf16: bool = False, cached: bool = False) -> SelfAttentionGrad:
    """cpu autodiff.cpp:492-496."""
    from . import hostlayer
    return SelfAttentionGrad(*hostlayer.selfAttentionBackward(x, wq, wk, wv, wout, numHeads, g, _variant(useBf16, cached), False))


def KVCache():
    """hip::KVCache (ops.hpp of the C++ layer): K/V of the positions processed so far."""
    from . import hostlayer
    return hostlayer.KVCache()


def selfAttentionIncremental(xNew, wq, wk, wv, wout, numHeads: int, cache, useBf16: bool = False):
    from . import hostlayer
    return hostlayer.selfAttentionIncremental(xNew, wq, wk, wv, wout, numHeads, cache, useBf16)


def selfAttentionIncrementalBf16(xNew, wq, wk, wv, wout, numHeads: int, cache):
    return selfAttentionIncremental(xNew, wq, wk, wv, wout, numHeads, cache, True)


# ------------------------------------------------------------------------------------------------
# losses (loss.hpp:20-70)
# ------------------------------------------------------------------------------------------------
@dataclass
class LossResult:
    value: float
    grad: DeviceTensor


def _read_scalar(t: DeviceTensor) -> float:
    return float(t.toHost().reshape(-1)[0])


def meanSquaredErrorAccumulate(pred, target, lossAccumulator: DeviceTensor) -> DeviceTensor:
    _require(pred.shape == target.shape, "meanSquaredError: incompatible shapes")
    grad = DeviceTensor(pred.shape)
    _call("bf_hip_mse", pred.ptr, target.ptr, grad.ptr, lossAccumulator.ptr, pred.elementCount(), 1, None)
    return grad


def meanSquaredError(pred, target) -> LossResult:
    _require(pred.shape == target.shape, "meanSquaredError: incompatible shapes")
    grad, total = DeviceTensor(pred.shape), DeviceTensor((1,))
    n = pred.elementCount()
    _call("bf_hip_mse", pred.ptr, target.ptr, grad.ptr, total.ptr, n, 0, None)
    return LossResult(_read_scalar(total) / n if n else 0.0, grad)


def _check_ce(name, logits, target):
    _require(logits.shape == target.shape, f"{name}: incompatible shapes")
    _require(logits.rank() >= 2, f"{name}: needs a tensor of rank >= 2")


def softmaxCrossEntropyAccumulate(logits, target, lossAccumulator: DeviceTensor) -> DeviceTensor:
    _check_ce("softmaxCrossEntropyAccumulate", logits, target)
    grad = DeviceTensor(logits.shape)
    _call("bf_hip_cross_entropy", logits.ptr, target.ptr, grad.ptr, lossAccumulator.ptr, *_rows(logits), 1, None)
    return grad


def softmaxCrossEntropy(logits, target) -> LossResult:
    _check_ce("softmaxCrossEntropy", logits, target)
    grad, total = DeviceTensor(logits.shape), DeviceTensor((1,))
    rows, classes = _rows(logits)
    _call("bf_hip_cross_entropy", logits.ptr, target.ptr, grad.ptr, total.ptr, rows, classes, 0, None)
    return LossResult(_read_scalar(total) / rows if rows else 0.0, grad)


def _check_sparse(name, logits, idx):
    _require(logits.rank() >= 2, f"{name}: needs logits of rank >= 2")
    _require(idx.elementCount() == _rows(logits)[0], f"{name}: targetIndices count does not match the logits rows")


def softmaxCrossEntropySparseAccumulate(logits, targetIndices, lossAccumulator: DeviceTensor) -> DeviceTensor:
    """Indices are the caller's precondition here (loss.hpp:59-70): no range check, no host sync."""
    _check_sparse("softmaxCrossEntropySparseAccumulate", logits, targetIndices)
    grad = DeviceTensor(logits.shape)
    _call("bf_hip_cross_entropy_sparse", logits.ptr, targetIndices.ptr, grad.ptr, lossAccumulator.ptr, *_rows(logits), 1,
          None)
    return grad


def softmaxCrossEntropySparse(logits, targetIndices) -> LossResult:
    _check_sparse("softmaxCrossEntropySparse", logits, targetIndices)
    rows, classes = _rows(logits)
    if rows:
        _validate_ids("softmaxCrossEntropySparse", targetIndices, classes, "class index")
    grad, total = DeviceTensor(logits.shape), DeviceTensor((1,))
    _call("bf_hip_cross_entropy_sparse", logits.ptr, targetIndices.ptr, grad.ptr, total.ptr, rows, classes, 0, None)
    return LossResult(_read_scalar(total) / rows if rows else 0.0, grad)


def softmaxCrossEntropyMasked(logits, targetIndices) -> LossResult:
    """cpu loss.cpp:149-215: rows whose index is -1 are ignored; loss and gradient are means over the other rows."""
    _check_sparse("softmaxCrossEntropyMasked", logits, targetIndices)
    rows, classes = _rows(logits)
    if rows:
        idx = np.rint(targetIndices.toHost()).astype(np.int64).ravel()
        bad = idx[(idx != -1) & ((idx < 0) | (idx >= classes))]
        _require(bad.size == 0, f"softmaxCrossEntropyMasked: class index {bad[0] if bad.size else 0} outside [0, {classes}) (or -1 to ignore)")
    grad, mean = DeviceTensor(logits.shape), DeviceTensor((1,))
    _call("bf_hip_cross_entropy_masked", logits.ptr, targetIndices.ptr, grad.ptr, mean.ptr, rows, classes, 0, None)
    return LossResult(_read_scalar(mean), grad)


def softmaxCrossEntropyMaskedAccumulate(logits, targetIndices, lossAccumulator: DeviceTensor) -> DeviceTensor:
    """Adds this call's mean over the rows that are not ignored to lossAccumulator; indices are the caller's precondition."""
    _check_sparse("softmaxCrossEntropyMaskedAccumulate", logits, targetIndices)
    grad = DeviceTensor(logits.shape)
    _call("bf_hip_cross_entropy_masked", logits.ptr, targetIndices.ptr, grad.ptr, lossAccumulator.ptr, *_rows(logits), 1, None)
    return grad


# ------------------------------------------------------------------------------------------------
# optimizers (optimizer.hpp:17-66)
# ------------------------------------------------------------------------------------------------
@dataclass
class Parameter:
    name: str
    value: DeviceTensor
    grad: DeviceTensor


class SGD:
    def __init__(self, learningRate: float):
        self.learningRate = learningRate

    def setLearningRate(self, learningRate: float):
        self.learningRate = learningRate

    def step(self, parameters: List[Parameter]):
        n = len(parameters)
        if n == 0:
            return
        counts = (ctypes.c_size_t * n)(*[p.value.elementCount() for p in parameters])
        _call("bf_hip_sgd_multi", _ptr_array([p.value for p in parameters]), _ptr_array([p.grad for p in parameters]),
              counts, n, self.learningRate, None)


class AdamW:
    def __init__(self, learningRate=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weightDecay=0.01):
        self.learningRate, self.beta1, self.beta2, self.eps, self.weightDecay = learningRate, beta1, beta2, eps, weightDecay
        self.stepCount = 0
        self.state: Dict[str, tuple] = {}

    def setLearningRate(self, learningRate: float):
        self.learningRate = learningRate

    def step(self, parameters: List[Parameter]):
        self.stepCount += 1
        n = len(parameters)
        if n == 0:
            return
        for p in parameters:
            if p.name not in self.state:
                self.state[p.name] = (DeviceTensor.zeros(p.value.shape), DeviceTensor.zeros(p.value.shape))
        counts = (ctypes.c_size_t * n)(*[p.value.elementCount() for p in parameters])
        _call("bf_hip_adamw_multi", _ptr_array([p.value for p in parameters]), _ptr_array([p.grad for p in parameters]),
              _ptr_array([self.state[p.name][0] for p in parameters]), _ptr_array([self.state[p.name][1] for p in parameters]),
              counts, n, self.stepCount, self.learningRate, self.beta1, self.beta2, self.eps, self.weightDecay, None)
