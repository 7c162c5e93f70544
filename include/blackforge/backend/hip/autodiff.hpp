#pragma once
// Backward operators with the reference's signatures (include/blackforge/backend/cuda/autodiff.hpp:18-177).
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <utility>

#include "blackforge/backend/hip/device_tensor.hpp"
#include "blackforge/backend/hip/ops.hpp"

namespace blackforge::backend::hip {

struct MatmulGrad {
    DeviceTensor dA;
    DeviceTensor dB;
};

// Where a backward pass may write parameter gradients directly: tensors of the gradients' shapes whose contents are to be
// REPLACED (a model's gradient buffers straight after zeroGrad(): writing g there equals adding g to zero).  A gradient
// written to slot i comes back as a non-owning view of that tensor instead of a tensor of its own, so callers can tell by
// the data pointer.  Slots: Linear {weight}; self-attention {wq, wk, wv, wout}; feed-forward {w1, b1, w2, b2}.
struct GradientTargets {
    DeviceTensor* slot[4] = {nullptr, nullptr, nullptr, nullptr};
};

namespace detail {
inline DeviceTensor gradientTensor(const GradientTargets* into, int i, std::vector<std::size_t> shape) {
    if (into != nullptr && into->slot[i] != nullptr && into->slot[i]->shape() == shape && into->slot[i]->data() != nullptr)
        return DeviceTensor::borrow(into->slot[i]->data(), std::move(shape));
    return DeviceTensor(std::move(shape));
}
inline void requireMatmulBackward(const char* op, const DeviceTensor& a, const DeviceTensor& b, const DeviceTensor& g) {
    require(a.rank() == 2 && b.rank() == 2 && g.rank() == 2 && a.dim(1) == b.dim(0) && g.dim(0) == a.dim(0) &&
                g.dim(1) == b.dim(1),
            std::string(op) + ": incompatible shapes on the device");
}
// Gradients of c = a(as [m,k]) * b[k,n] given g (as [m,n]); mode as in detail::projection.
inline MatmulGrad projectionBackward(const DeviceTensor& a, const DeviceTensor& b, const DeviceTensor& g, int mode,
                                     std::vector<std::size_t> dAShape, const GradientTargets* into = nullptr, int slot = 0) {
    std::size_t m = rowsOf(a), k = lastDim(a), n = b.dim(1);
    MatmulGrad r{DeviceTensor(std::move(dAShape)), gradientTensor(into, slot, {k, n})};
    if (mode == 0) {   // dA = g b^T and dB = a^T g do not depend on each other: one call
        productsF32({{0, 1, g.data(), b.data(), r.dA.data(), m, k, n}, {1, 0, a.data(), g.data(), r.dB.data(), k, n, m}});
    } else {   // a gradient that carries its bf16 image (made by the kernel that produced it) is not converted again
        check(bf_hip_matmul_bf16_backward_img(a.data(), a.image(), b.data(), g.data(), g.image(), r.dA.data(), r.dB.data(), m, k, n,
                                              mode == 2, nullptr));
    }
    return r;
}
}  // namespace detail

inline MatmulGrad matmulBackward(const DeviceTensor& a, const DeviceTensor& b, const DeviceTensor& gradOutput) {
    detail::requireMatmulBackward("matmulBackward", a, b, gradOutput);
    return detail::projectionBackward(a, b, gradOutput, 0, a.shape());
}
inline MatmulGrad matmulBf16Backward(const DeviceTensor& a, const DeviceTensor& b, const DeviceTensor& gradOutput) {
    detail::requireMatmulBackward("matmulBf16Backward", a, b, gradOutput);
    return detail::projectionBackward(a, b, gradOutput, 1, a.shape());
}
inline MatmulGrad matmulBf16BackwardCachedWeight(const DeviceTensor& a, const DeviceTensor& b, const DeviceTensor& gradOutput) {
    detail::requireMatmulBackward("matmulBf16BackwardCachedWeight", a, b, gradOutput);
    return detail::projectionBackward(a, b, gradOutput, 2, a.shape());
}

struct MatmulTransposeBGrad {
    DeviceTensor dA;
    DeviceTensor dB;
};

// Forward was a:[m,k], b:[n,k] -> a b^T:[m,n].
inline MatmulTransposeBGrad matmulTransposeBBackward(const DeviceTensor& a, const DeviceTensor& b, const DeviceTensor& gradOutput) {
    require(a.rank() == 2 && b.rank() == 2 && gradOutput.rank() == 2 && a.dim(1) == b.dim(1) && gradOutput.dim(0) == a.dim(0) &&
                gradOutput.dim(1) == b.dim(0),
            "matmulTransposeBBackward: incompatible shapes on the device");
    std::size_t m = a.dim(0), k = a.dim(1), n = b.dim(0);
    MatmulTransposeBGrad r{DeviceTensor({m, k}), DeviceTensor({n, k})};
    // dA = g b and dB = g^T a
    detail::productsF32({{0, 0, gradOutput.data(), b.data(), r.dA.data(), m, k, n}, {1, 0, gradOutput.data(), a.data(), r.dB.data(), n, k, m}});
    return r;
}

struct AddBiasGrad {
    DeviceTensor dInput;
    DeviceTensor dBias;
};

// into / slot: where the caller wants the gradient written (a model's own gradient tensor), see GradientTargets
inline DeviceTensor biasGradientOnly(const DeviceTensor& gradOutput, const GradientTargets* into = nullptr, int slot = 0) {
    require(gradOutput.rank() >= 2, "biasGradientOnly: needs a gradient of rank >= 2 on the device");
    DeviceTensor dBias = detail::gradientTensor(into, slot, {detail::lastDim(gradOutput)});
    check(bf_hip_bias_grad(gradOutput.data(), dBias.data(), detail::rowsOf(gradOutput), detail::lastDim(gradOutput), nullptr));
    return dBias;
}

inline AddBiasGrad addBiasBackward(const DeviceTensor& gradOutput) {
    require(gradOutput.rank() >= 2, "addBiasBackward: needs a gradient of rank >= 2 on the device");
    return AddBiasGrad{gradOutput.clone(), biasGradientOnly(gradOutput)};
}

struct AddBiasSiluGrad {
    DeviceTensor dGemmOutput;
    DeviceTensor dBias;
};

inline AddBiasSiluGrad addBiasActivationBackward(const DeviceTensor& gemmOutput, const DeviceTensor& bias,
                                                  const DeviceTensor& dHidden, Activation act, const GradientTargets* into = nullptr,
                                                  int slot = 0) {
    require(gemmOutput.shape() == dHidden.shape() && bias.rank() == 1 && detail::lastDim(gemmOutput) == bias.dim(0),
            "addBiasSiluBackward: incompatible shapes on the device");
    AddBiasSiluGrad r{DeviceTensor(gemmOutput.shape()), detail::gradientTensor(into, slot, {bias.dim(0)})};
    check(bf_hip_add_bias_act_backward(gemmOutput.data(), bias.data(), dHidden.data(), r.dGemmOutput.data(), r.dBias.data(),
                                       detail::rowsOf(gemmOutput), bias.dim(0), static_cast<int>(act), nullptr));
    return r;
}
inline AddBiasSiluGrad addBiasSiluBackward(const DeviceTensor& gemmOutput, const DeviceTensor& bias, const DeviceTensor& dHidden) {
    return addBiasActivationBackward(gemmOutput, bias, dHidden, Activation::Silu);
}

inline DeviceTensor activationBackward(const char* op, const DeviceTensor& input, const DeviceTensor& gradOutput, Activation act) {
    require(input.shape() == gradOutput.shape(), std::string(op) + ": incompatible shapes on the device");
    DeviceTensor out(input.shape());
    check(bf_hip_act_backward(input.data(), gradOutput.data(), out.data(), input.elementCount(), static_cast<int>(act), nullptr));
    return out;
}
inline DeviceTensor siluBackward(const DeviceTensor& input, const DeviceTensor& gradOutput) {
    return activationBackward("siluBackward", input, gradOutput, Activation::Silu);
}
inline DeviceTensor reluBackward(const DeviceTensor& input, const DeviceTensor& gradOutput) {
    return activationBackward("reluBackward", input, gradOutput, Activation::Relu);
}
inline DeviceTensor geluBackward(const DeviceTensor& input, const DeviceTensor& gradOutput) {
    return activationBackward("geluBackward", input, gradOutput, Activation::Gelu);
}

inline DeviceTensor rmsnormBackward(const DeviceTensor& input, const DeviceTensor& gradOutput) {
    require(input.shape() == gradOutput.shape(), "rmsnormBackward: incompatible shapes on the device");
    require(input.rank() >= 2, "rmsnormBackward: needs a tensor of rank >= 2 on the device");
    DeviceTensor out(input.shape());
    check(bf_hip_rmsnorm_backward(input.data(), gradOutput.data(), out.data(), detail::rowsOf(input), detail::lastDim(input), nullptr));
    return out;
}

// residualGrad + rmsnormBackward(input, gradOutput) in one pass: how both composite blocks' backward passes end
// (autodiff.cu:746,794).
// withImage: the result also carries its bf16 image (DeviceTensor::image()), for a reader that is a bf16 GEMM.
inline DeviceTensor rmsnormBackwardAdd(const DeviceTensor& input, const DeviceTensor& gradOutput, const DeviceTensor& residualGrad,
                                       bool withImage = false) {
    require(input.shape() == gradOutput.shape() && residualGrad.shape() == input.shape(), "rmsnormBackward: incompatible shapes on the device");
    require(input.rank() >= 2, "rmsnormBackward: needs a tensor of rank >= 2 on the device");
    DeviceTensor out(input.shape());
    std::uint16_t* image = withImage && detail::lastDim(input) % 8 == 0 && input.elementCount() > 0 ? out.attachImage() : nullptr;
    check(bf_hip_rmsnorm_backward_add_img(input.data(), gradOutput.data(), residualGrad.data(), out.data(), image, detail::rowsOf(input),
                                          detail::lastDim(input), nullptr));
    return out;
}

inline DeviceTensor softmaxBackward(const DeviceTensor& input, const DeviceTensor& gradOutput) {
    require(input.shape() == gradOutput.shape(), "softmaxBackward: incompatible shapes on the device");
    require(input.rank() >= 2, "softmaxBackward: needs a tensor of rank >= 2 on the device");
    DeviceTensor out(input.shape());
    check(bf_hip_softmax_backward(input.data(), gradOutput.data(), out.data(), detail::rowsOf(input), detail::lastDim(input), nullptr));
    return out;
}

inline DeviceTensor embeddingLookupBackwardPreValidated(const DeviceTensor& tokenIds, const DeviceTensor& gradOutput,
                                                         std::size_t vocabSize, const GradientTargets* into = nullptr) {
    require(tokenIds.rank() == 2 && gradOutput.rank() == 3 && tokenIds.dim(0) == gradOutput.dim(0) &&
                tokenIds.dim(1) == gradOutput.dim(1),
            "embeddingLookupBackward: incompatible shapes on the device");
    DeviceTensor dTable = detail::gradientTensor(into, 0, {vocabSize, gradOutput.dim(2)});
    check(bf_hip_embedding_backward(tokenIds.data(), gradOutput.data(), dTable.data(), tokenIds.elementCount(), vocabSize,
                                    gradOutput.dim(2), nullptr));
    return dTable;
}

inline DeviceTensor embeddingLookupBackward(const DeviceTensor& tokenIds, const DeviceTensor& gradOutput, std::size_t vocabSize,
                                            const GradientTargets* into = nullptr) {
    require(tokenIds.rank() == 2 && gradOutput.rank() == 3 && tokenIds.dim(0) == gradOutput.dim(0) &&
                tokenIds.dim(1) == gradOutput.dim(1),
            "embeddingLookupBackward: incompatible shapes on the device");
    detail::requireIdsInRange("embeddingLookupBackward", tokenIds, vocabSize, "token id");
    return embeddingLookupBackwardPreValidated(tokenIds, gradOutput, vocabSize, into);
}

struct PositionalEmbeddingGrad {
    DeviceTensor dInput;
    DeviceTensor dTable;
};

inline PositionalEmbeddingGrad addPositionalEmbeddingBackward(const DeviceTensor& gradOutput, std::size_t maxSeqLen,
                                                              const GradientTargets* into = nullptr) {
    require(gradOutput.rank() == 3, "addPositionalEmbeddingBackward: needs a gradient of rank 3 on the device");
    PositionalEmbeddingGrad r{DeviceTensor(), detail::gradientTensor(into, 0, {maxSeqLen, gradOutput.dim(2)})};
    check(bf_hip_positional_backward(gradOutput.data(), r.dTable.data(), gradOutput.dim(0), gradOutput.dim(1), gradOutput.dim(2),
                                     maxSeqLen, nullptr));
    r.dInput = gradOutput.clone();
    return r;
}

struct FeedForwardGrad {
    DeviceTensor dInput, dW1, dB1, dW2, dB2;
};

inline FeedForwardGrad feedForwardBackwardCached(const DeviceTensor& input, const DeviceTensor& w1, const DeviceTensor& b1,
                                                  const DeviceTensor& w2, const DeviceTensor& b2, const FeedForwardCache& cache,
                                                  const DeviceTensor& gradOutput, bool useBf16, Activation act = Activation::Silu,
                                                  const GradientTargets* into = nullptr, bool imageForConsumer = false) {
    (void)b2;
    require(gradOutput.shape() == input.shape(), "feedForwardBackward: gradient shape differs from the input");
    const int mode = useBf16 ? 2 : 0;
    if (cache.fused) {
        const std::size_t rows = detail::rowsOf(input), d = detail::lastDim(input), hidden = w1.dim(1);
        DeviceTensor dNormed(input.shape()), dW1 = detail::gradientTensor(into, 0, w1.shape()),
                     dB1 = detail::gradientTensor(into, 1, {hidden}), dW2 = detail::gradientTensor(into, 2, w2.shape()),
                     dB2 = detail::gradientTensor(into, 3, {d});
        check(bf_hip_feedforward_bf16_backward_img(nullptr, reinterpret_cast<const uint16_t*>(cache.normedImage.data()), w1.data(), w2.data(),
                                                   cache.gemm1.data(), reinterpret_cast<const uint16_t*>(cache.hiddenImage.data()),
                                                   gradOutput.data(), gradOutput.image(), static_cast<int>(act), dNormed.data(), dW1.data(),
                                                   dB1.data(), dW2.data(), dB2.data(), rows, d, hidden, 1, nullptr));
        DeviceTensor dInput = rmsnormBackwardAdd(input, dNormed, gradOutput, imageForConsumer);
        return FeedForwardGrad{std::move(dInput), std::move(dW1), std::move(dB1), std::move(dW2), std::move(dB2)};
    }
    DeviceTensor dB2 = biasGradientOnly(gradOutput, into, 3);
    MatmulGrad g2 = detail::projectionBackward(cache.hidden, w2, gradOutput, mode, cache.hidden.shape(), into, 2);
    AddBiasSiluGrad hiddenGrad = addBiasActivationBackward(cache.gemm1, b1, g2.dA, act, into, 1);
    MatmulGrad g1 = detail::projectionBackward(cache.normed, w1, hiddenGrad.dGemmOutput, mode, cache.normed.shape(), into, 0);
    DeviceTensor dInput = rmsnormBackwardAdd(input, g1.dA, gradOutput, imageForConsumer && useBf16);
    return FeedForwardGrad{std::move(dInput), std::move(g1.dB), std::move(hiddenGrad.dBias), std::move(g2.dB), std::move(dB2)};
}

namespace detail {
// Stateless variant: recomputes the forward first (reference: autodiff.cu:624-652).
inline FeedForwardGrad feedForwardBackwardImpl(const DeviceTensor& input, const DeviceTensor& w1, const DeviceTensor& b1,
                                               const DeviceTensor& w2, const DeviceTensor& b2, const DeviceTensor& gradOutput,
                                               int mode, Activation act) {
    FeedForwardCache cache;
    cache.normed = rmsnorm(input);
    cache.gemm1 = projection(cache.normed, w1, mode, withLastDim(input, w1.dim(1)));
    cache.hidden = addBiasActivation(cache.gemm1, b1, act);
    DeviceTensor dB2 = biasGradientOnly(gradOutput);
    MatmulGrad g2 = projectionBackward(cache.hidden, w2, gradOutput, mode, cache.hidden.shape());
    AddBiasSiluGrad hiddenGrad = addBiasActivationBackward(cache.gemm1, b1, g2.dA, act);
    MatmulGrad g1 = projectionBackward(cache.normed, w1, hiddenGrad.dGemmOutput, mode, cache.normed.shape());
    DeviceTensor dInput = rmsnormBackwardAdd(input, g1.dA, gradOutput);
    (void)b2;
    return FeedForwardGrad{std::move(dInput), std::move(g1.dB), std::move(hiddenGrad.dBias), std::move(g2.dB), std::move(dB2)};
}
}  // namespace detail

inline FeedForwardGrad feedForwardBackward(const DeviceTensor& input, const DeviceTensor& w1, const DeviceTensor& b1,
                                            const DeviceTensor& w2, const DeviceTensor& b2, const DeviceTensor& gradOutput,
                                            Activation act = Activation::Silu) {
    return detail::feedForwardBackwardImpl(input, w1, b1, w2, b2, gradOutput, 0, act);
}
inline FeedForwardGrad feedForwardBf16Backward(const DeviceTensor& input, const DeviceTensor& w1, const DeviceTensor& b1,
                                                const DeviceTensor& w2, const DeviceTensor& b2, const DeviceTensor& gradOutput,
                                                Activation act = Activation::Silu) {
    return detail::feedForwardBackwardImpl(input, w1, b1, w2, b2, gradOutput, 1, act);
}

struct SelfAttentionGrad {
    DeviceTensor dInput, dWq, dWk, dWv, dWout;
};

namespace detail {
inline SelfAttentionGrad selfAttentionBackwardFromCache(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                        const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                        const SelfAttentionCache& cache, const DeviceTensor& gradOutput, int mode,
                                                        const GradientTargets* into = nullptr, bool imageForConsumer = false) {
    require(gradOutput.shape() == input.shape(), "selfAttentionBackward: gradient shape differs from the input");
    std::size_t batch = input.dim(0), seq = input.dim(1), dim = input.dim(2);
    float scaleFactor = 1.0F / std::sqrt(static_cast<float>(dim / numHeads));
    MatmulGrad outGrad = projectionBackward(cache.attnOutput, wout, gradOutput, mode, {batch, seq, dim}, into, 3);
    if (mode != 0 && cache.normedImage.data() != nullptr) {
        // the forward pass kept bf16 images of the normalised input and of the attention output; here the attention
        // gradients go straight to one side-by-side bf16 image [rows, 3 dim] (they have no reader but the two GEMMs below)
        const std::size_t rows = batch * seq;
        DeviceTensor gradImage({rows, 3 * dim / 2});   // raw bf16 storage
        std::uint16_t* gi = reinterpret_cast<std::uint16_t*>(gradImage.data());
        check(bf_hip_attention_backward_img(outGrad.dA.data(), cache.q.data(), cache.k.data(), cache.v.data(), cache.attnOutput.data(),
                                            cache.attnM.data(), cache.attnL.data(), nullptr, nullptr, nullptr, gi, gi + dim, gi + 2 * dim, 3 * dim,
                                            batch, numHeads, seq, seq, dim, scaleFactor, cache.causal ? 0 : seq, nullptr));
        DeviceTensor dNormed({batch, seq, dim}), dWq = gradientTensor(into, 0, wq.shape()), dWk = gradientTensor(into, 1, wk.shape()),
                     dWv = gradientTensor(into, 2, wv.shape());
        const float* weights[3] = {wq.data(), wk.data(), wv.data()};
        float* weightGrads[3] = {dWq.data(), dWk.data(), dWv.data()};
        check(bf_hip_matmul_bf16_shared_input_backward_img(nullptr, reinterpret_cast<const std::uint16_t*>(cache.normedImage.data()), weights,
                                                           nullptr, gi, dNormed.data(), weightGrads, 3, rows, dim, dim, mode == 2, nullptr));
        DeviceTensor dInput = rmsnormBackwardAdd(input, dNormed, gradOutput, imageForConsumer);
        return SelfAttentionGrad{std::move(dInput), std::move(dWq), std::move(dWk), std::move(dWv), std::move(outGrad.dB)};
    }
    FusedAttentionGrad attn = fusedAttentionBackward(outGrad.dA, cache.q, cache.k, cache.v, cache.attnOutput, cache.attnM,
                                                      cache.attnL, numHeads, scaleFactor, cache.causal ? 0 : seq);
    if (mode != 0) {
        // the three projection gradients share their input: one GEMM sums dQ Wq^T + dK Wk^T + dV Wv^T, one produces
        // the three weight gradients (for widths that are multiples of 256; separate GEMMs otherwise)
        DeviceTensor dNormed({batch, seq, dim}), dWq = gradientTensor(into, 0, wq.shape()), dWk = gradientTensor(into, 1, wk.shape()),
                     dWv = gradientTensor(into, 2, wv.shape());
        const float* weights[3] = {wq.data(), wk.data(), wv.data()};
        const float* grads[3] = {attn.dQ.data(), attn.dK.data(), attn.dV.data()};
        float* weightGrads[3] = {dWq.data(), dWk.data(), dWv.data()};
        check(bf_hip_matmul_bf16_shared_input_backward(cache.normedFlat.data(), weights, grads, dNormed.data(), weightGrads, 3,
                                                       batch * seq, dim, dim, mode == 2, nullptr));
        DeviceTensor dInput = rmsnormBackwardAdd(input, dNormed, gradOutput, imageForConsumer);
        return SelfAttentionGrad{std::move(dInput), std::move(dWq), std::move(dWk), std::move(dWv), std::move(outGrad.dB)};
    }
    // the six gradient products of the three projections are independent of each other: one call, then
    // (dQ Wq^T + dK Wk^T) + dV Wv^T
    const std::size_t rows = batch * seq;
    DeviceTensor dAq({rows, dim}), dAk({rows, dim}), dAv({rows, dim});
    DeviceTensor dWq = gradientTensor(into, 0, wq.shape()), dWk = gradientTensor(into, 1, wk.shape()), dWv = gradientTensor(into, 2, wv.shape());
    productsF32({{0, 1, attn.dQ.data(), wq.data(), dAq.data(), rows, dim, dim}, {1, 0, cache.normedFlat.data(), attn.dQ.data(), dWq.data(), dim, dim, rows},
                 {0, 1, attn.dK.data(), wk.data(), dAk.data(), rows, dim, dim}, {1, 0, cache.normedFlat.data(), attn.dK.data(), dWk.data(), dim, dim, rows},
                 {0, 1, attn.dV.data(), wv.data(), dAv.data(), rows, dim, dim}, {1, 0, cache.normedFlat.data(), attn.dV.data(), dWv.data(), dim, dim, rows}});
    DeviceTensor dNormed = add(add(dAq, dAk), dAv).reshaped({batch, seq, dim});
    DeviceTensor dInput = rmsnormBackwardAdd(input, dNormed, gradOutput);
    return SelfAttentionGrad{std::move(dInput), std::move(dWq), std::move(dWk), std::move(dWv), std::move(outGrad.dB)};
}
}  // namespace detail

inline SelfAttentionGrad selfAttentionBackwardCached(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                      const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                      const SelfAttentionCache& cache, const DeviceTensor& gradOutput, bool useBf16,
                                                      const GradientTargets* into = nullptr, bool imageForConsumer = false) {
    return detail::selfAttentionBackwardFromCache(input, wq, wk, wv, wout, numHeads, cache, gradOutput, useBf16 ? 2 : 0, into,
                                                  imageForConsumer && useBf16);
}
// Stateless variants: recompute the forward first (reference: autodiff.cu:654-700).
inline SelfAttentionGrad selfAttentionBackward(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                const DeviceTensor& gradOutput) {
    SelfAttentionCache cache;
    detail::selfAttentionForwardImpl("selfAttentionBackward", input, wq, wk, wv, wout, numHeads, 0, cache);
    return detail::selfAttentionBackwardFromCache(input, wq, wk, wv, wout, numHeads, cache, gradOutput, 0);
}
inline SelfAttentionGrad selfAttentionBf16Backward(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                    const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                    const DeviceTensor& gradOutput) {
    SelfAttentionCache cache;
    detail::selfAttentionForwardImpl("selfAttentionBf16Backward", input, wq, wk, wv, wout, numHeads, 1, cache);
    return detail::selfAttentionBackwardFromCache(input, wq, wk, wv, wout, numHeads, cache, gradOutput, 1);
}
// Gradients of bidirectionalSelfAttention (src/backend/cpu/autodiff.cpp:492-496): the cache remembers that the forward
// pass was not causal, so the cached form is selfAttentionBackwardCached; these recompute the forward pass first.
inline SelfAttentionGrad bidirectionalSelfAttentionBackward(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                             const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                             const DeviceTensor& gradOutput) {
    SelfAttentionCache cache;
    detail::selfAttentionForwardImpl("bidirectionalSelfAttentionBackward", input, wq, wk, wv, wout, numHeads, 0, cache, false);
    return detail::selfAttentionBackwardFromCache(input, wq, wk, wv, wout, numHeads, cache, gradOutput, 0);
}
inline SelfAttentionGrad bidirectionalSelfAttentionBf16Backward(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                                 const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                                 const DeviceTensor& gradOutput) {
    SelfAttentionCache cache;
    detail::selfAttentionForwardImpl("bidirectionalSelfAttentionBf16Backward", input, wq, wk, wv, wout, numHeads, 1, cache, false);
    return detail::selfAttentionBackwardFromCache(input, wq, wk, wv, wout, numHeads, cache, gradOutput, 1);
}

}  // namespace blackforge::backend::hip
