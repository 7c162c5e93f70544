#pragma once
// Fused causal attention (reference: include/blackforge/backend/cuda/fused_attention.hpp:42-76).
#include <cstddef>
#include <string>

#include "blackforge/backend/hip/device_tensor.hpp"

namespace blackforge::backend::hip {

struct FusedAttentionForwardResult {
    DeviceTensor output;  // [batch, newLen, dim], before the output projection
    DeviceTensor m;       // [batch, numHeads, newLen] row max of the scaled scores
    DeviceTensor l;       // [batch, numHeads, newLen] row sum of exp(score - m)
};

// q: [batch, newLen, dim], k/v: [batch, totalLen, dim]; query row i attends to keys j <= oldLen + i.
// Throws std::invalid_argument when headDim = dim / numHeads exceeds 256 (same limit as the reference).
inline FusedAttentionForwardResult fusedAttentionForward(const DeviceTensor& q, const DeviceTensor& k, const DeviceTensor& v,
                                                          std::size_t numHeads, float scaleFactor, std::size_t oldLen) {
    require(q.rank() == 3 && k.rank() == 3 && v.rank() == 3, "fusedAttentionForward: q, k, v must have rank 3");
    std::size_t batch = q.dim(0), newLen = q.dim(1), dim = q.dim(2), totalLen = k.dim(1);
    require(k.shape() == v.shape() && k.dim(0) == batch && k.dim(2) == dim, "fusedAttentionForward: k/v shape mismatch");
    FusedAttentionForwardResult r{DeviceTensor({batch, newLen, dim}), DeviceTensor({batch, numHeads, newLen}),
                                  DeviceTensor({batch, numHeads, newLen})};
    check(bf_hip_attention_forward(q.data(), k.data(), v.data(), r.output.data(), r.m.data(), r.l.data(), batch, numHeads,
                                   newLen, totalLen, dim, scaleFactor, oldLen, nullptr));
    return r;
}

struct FusedAttentionGrad {
    DeviceTensor dQ;
    DeviceTensor dK;
    DeviceTensor dV;
};

inline FusedAttentionGrad fusedAttentionBackward(const DeviceTensor& dOutput, const DeviceTensor& q, const DeviceTensor& k,
                                                  const DeviceTensor& v, const DeviceTensor& output, const DeviceTensor& m,
                                                  const DeviceTensor& l, std::size_t numHeads, float scaleFactor,
                                                  std::size_t oldLen) {
    require(q.rank() == 3 && k.rank() == 3 && v.rank() == 3, "fusedAttentionBackward: q, k, v must have rank 3");
    std::size_t batch = q.dim(0), newLen = q.dim(1), dim = q.dim(2), totalLen = k.dim(1);
    require(dOutput.shape() == q.shape() && output.shape() == q.shape() && k.shape() == v.shape(),
            "fusedAttentionBackward: shape mismatch");
    FusedAttentionGrad g{DeviceTensor(q.shape()), DeviceTensor(k.shape()), DeviceTensor(v.shape())};
    check(bf_hip_attention_backward(dOutput.data(), q.data(), k.data(), v.data(), output.data(), m.data(), l.data(),
                                    g.dQ.data(), g.dK.data(), g.dV.data(), batch, numHeads, newLen, totalLen, dim,
                                    scaleFactor, oldLen, nullptr));
    return g;
}

}  // namespace blackforge::backend::hip
