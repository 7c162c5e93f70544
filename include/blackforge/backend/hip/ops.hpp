#pragma once
// Forward operators with the reference's signatures (include/blackforge/backend/cuda/ops.hpp:8-258).
// Each function validates shapes (std::invalid_argument), takes its result from the pool and makes one or
// a few calls into the C ABI; no computation happens on the host.
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <string>
#include <utility>
#include <vector>

#include "blackforge/backend/hip/device_tensor.hpp"
#include "blackforge/backend/hip/fused_attention.hpp"

namespace blackforge::backend::hip {

// Feed-forward activation: Silu is the reference block; Gelu is the same block with the reference's
// gelu / geluBackward formulas substituted.
enum class Activation : int { Silu = BF_ACT_SILU, Gelu = BF_ACT_GELU, Relu = BF_ACT_RELU };

namespace detail {
inline std::size_t lastDim(const DeviceTensor& t) { return t.shape().back(); }
inline std::size_t rowsOf(const DeviceTensor& t) { return lastDim(t) ? t.elementCount() / lastDim(t) : 0; }
inline std::vector<std::size_t> withLastDim(const DeviceTensor& t, std::size_t last) {
    std::vector<std::size_t> s = t.shape();
    s.back() = last;
    return s;
}
inline void requireBias(const char* op, const DeviceTensor& x, const DeviceTensor& bias) {
    require(x.rank() >= 2 && bias.rank() == 1 && lastDim(x) == bias.dim(0),
            std::string(op) + ": expected input [..., features] and bias [features]");
}
// c[rows(a), n] = a(as [rows, k]) * b[k, n]; bf16 = 0 fp32 MFMA, 1 bf16 MFMA, 2 bf16 with cached weight image
inline DeviceTensor projection(const DeviceTensor& a, const DeviceTensor& b, int bf16, std::vector<std::size_t> outShape) {
    std::size_t k = lastDim(a), m = rowsOf(a), n = b.dim(1);
    DeviceTensor c(std::move(outShape));
    if (bf16 == 0) check(bf_hip_gemm_f32(0, 0, a.data(), b.data(), c.data(), m, n, k, nullptr));
    else check(bf_hip_matmul_bf16(a.data(), b.data(), c.data(), m, k, n, bf16 == 2, nullptr));
    return c;
}
// Independent fp32 products in one call (one launch when they are small): {transA, transB, A, B, C, M, N, K}.
struct F32Product {
    int transA, transB;
    const float* a;
    const float* b;
    float* c;
    std::size_t m, n, k;
};
inline void productsF32(std::initializer_list<F32Product> products) {
    bf_gemm_f32_problem list[8];
    std::size_t count = 0;
    for (const F32Product& p : products) list[count++] = bf_gemm_f32_problem{p.a, p.b, p.c, nullptr, nullptr, p.m, p.n, p.k, p.transA, p.transB};
    check(bf_hip_gemm_f32_group(list, count, nullptr));
}
// A projection with the adds that follow it folded into the GEMM's store: a*b (+ bias) (+ residual).
// bf16: 0 = fp32 product, 1 = fresh weight image, 2 = cached weight image.
inline DeviceTensor projectionFused(const DeviceTensor& a, const DeviceTensor& b, const DeviceTensor* bias, const DeviceTensor* residual,
                                    int bf16, std::vector<std::size_t> outShape) {
    DeviceTensor c(std::move(outShape));
    const std::size_t k = b.dim(0), n = b.dim(1), m = n ? c.elementCount() / n : 0;
    if (bf16 == 0) {
        if (k == 0 && m != 0 && n != 0) {   // an empty contraction: the product is zero, the adds remain
            DeviceTensor zero = DeviceTensor::zeros(c.shape());
            if (bias && residual) check(bf_hip_add_bias_residual(zero.data(), bias->data(), residual->data(), c.data(), m, n, nullptr));
            else if (bias) check(bf_hip_add_bias(zero.data(), bias->data(), c.data(), m, n, nullptr));
            else if (residual) return residual->clone();
            else return zero;
            return c;
        }
        check(bf_hip_gemm_f32_adds(0, 0, a.data(), b.data(), bias ? bias->data() : nullptr, residual ? residual->data() : nullptr, c.data(),
                                   m, n, k, nullptr));
        return c;
    }
    // an input that carries its bf16 image is not converted again
    check(bf_hip_linear_bf16_img(a.data(), a.image(), b.data(), bias ? bias->data() : nullptr, residual ? residual->data() : nullptr,
                                 c.data(), m, k, n, bf16 == 2, nullptr));
    return c;
}
}  // namespace detail

inline DeviceTensor add(const DeviceTensor& a, const DeviceTensor& b) {
    require(a.shape() == b.shape(), "add: incompatible shapes on the device");
    DeviceTensor out(a.shape());
    check(bf_hip_add(a.data(), b.data(), out.data(), a.elementCount(), nullptr));
    return out;
}

inline DeviceTensor scale(const DeviceTensor& x, float factor) {
    DeviceTensor out(x.shape());
    check(bf_hip_scale(x.data(), factor, out.data(), x.elementCount(), nullptr));
    return out;
}

inline DeviceTensor addBias(const DeviceTensor& input, const DeviceTensor& bias) {
    detail::requireBias("addBias", input, bias);
    DeviceTensor out(input.shape());
    check(bf_hip_add_bias(input.data(), bias.data(), out.data(), detail::rowsOf(input), bias.dim(0), nullptr));
    return out;
}

inline DeviceTensor addBiasActivation(const DeviceTensor& gemmOutput, const DeviceTensor& bias, Activation act) {
    detail::requireBias("addBiasSilu", gemmOutput, bias);
    DeviceTensor out(gemmOutput.shape());
    check(bf_hip_add_bias_act(gemmOutput.data(), bias.data(), out.data(), detail::rowsOf(gemmOutput), bias.dim(0),
                              static_cast<int>(act), nullptr));
    return out;
}

inline DeviceTensor addBiasSilu(const DeviceTensor& gemmOutput, const DeviceTensor& bias) {
    return addBiasActivation(gemmOutput, bias, Activation::Silu);
}

inline DeviceTensor addBiasResidual(const DeviceTensor& gemmOutput, const DeviceTensor& bias, const DeviceTensor& residual) {
    detail::requireBias("addBiasResidual", gemmOutput, bias);
    require(gemmOutput.shape() == residual.shape(), "addBiasResidual: residual shape differs");
    DeviceTensor out(gemmOutput.shape());
    check(bf_hip_add_bias_residual(gemmOutput.data(), bias.data(), residual.data(), out.data(), detail::rowsOf(gemmOutput),
                                   bias.dim(0), nullptr));
    return out;
}

inline DeviceTensor matmul(const DeviceTensor& a, const DeviceTensor& b) {
    require(a.rank() == 2 && b.rank() == 2 && a.dim(1) == b.dim(0), "matmul: incompatible shapes on the device");
    return detail::projection(a, b, 0, {a.dim(0), b.dim(1)});
}

inline DeviceTensor matmulTransposeB(const DeviceTensor& a, const DeviceTensor& b) {
    require(a.rank() == 2 && b.rank() == 2 && a.dim(1) == b.dim(1), "matmulTransposeB: incompatible shapes on the device");
    DeviceTensor c({a.dim(0), b.dim(0)});
    check(bf_hip_gemm_f32(0, 1, a.data(), b.data(), c.data(), a.dim(0), b.dim(0), a.dim(1), nullptr));
    return c;
}

inline DeviceTensor matmulBf16(const DeviceTensor& a, const DeviceTensor& b) {
    require(a.rank() == 2 && b.rank() == 2 && a.dim(1) == b.dim(0), "matmulBf16: incompatible shapes on the device");
    return detail::projection(a, b, 1, {a.dim(0), b.dim(1)});
}

inline DeviceTensor matmulBf16CachedWeight(const DeviceTensor& a, const DeviceTensor& b) {
    require(a.rank() == 2 && b.rank() == 2 && a.dim(1) == b.dim(0), "matmulBf16CachedWeight: incompatible shapes on the device");
    return detail::projection(a, b, 2, {a.dim(0), b.dim(1)});
}

inline void invalidateBf16WeightCache() { check(bf_hip_invalidate_bf16_weight_cache()); }
// The same for a caller that knows which weights it has just changed in place (an optimizer step): their cached images
// are made again at once, in one launch, instead of one by one inside the next forward pass (not in the reference).
inline void refreshBf16WeightImages(const std::vector<const float*>& changed) {
    check(bf_hip_bf16_weight_cache_refresh(changed.data(), changed.size(), nullptr));
}

inline DeviceTensor activation(const DeviceTensor& input, Activation act) {
    DeviceTensor out(input.shape());
    check(bf_hip_act_forward(input.data(), out.data(), input.elementCount(), static_cast<int>(act), nullptr));
    return out;
}
inline DeviceTensor silu(const DeviceTensor& input) { return activation(input, Activation::Silu); }
inline DeviceTensor relu(const DeviceTensor& input) { return activation(input, Activation::Relu); }
inline DeviceTensor gelu(const DeviceTensor& input) { return activation(input, Activation::Gelu); }

inline DeviceTensor rmsnorm(const DeviceTensor& input) {
    require(input.rank() >= 2, "rmsnorm: needs a tensor of rank >= 2 on the device");
    DeviceTensor out(input.shape());
    check(bf_hip_rmsnorm(input.data(), out.data(), detail::rowsOf(input), detail::lastDim(input), nullptr));
    return out;
}

inline DeviceTensor softmax(const DeviceTensor& input) {
    require(input.rank() >= 2, "softmax: needs a tensor of rank >= 2 on the device");
    DeviceTensor out(input.shape());
    check(bf_hip_softmax(input.data(), out.data(), detail::rowsOf(input), detail::lastDim(input), nullptr));
    return out;
}

namespace detail {
inline void requireIdsInRange(const char* op, const DeviceTensor& ids, std::size_t limit, const char* what) {
    std::size_t bad = 0;
    long long first = 0;
    check(bf_hip_count_out_of_range(ids.data(), ids.elementCount(), limit, &bad, &first, nullptr));
    require(bad == 0, std::string(op) + ": " + what + " " + std::to_string(first) + " outside [0, " + std::to_string(limit) + ")");
}
}  // namespace detail

inline DeviceTensor embeddingLookupPreValidated(const DeviceTensor& tokenIds, const DeviceTensor& table) {
    require(tokenIds.rank() == 2, "embeddingLookup: token ids must have rank 2 [batch, seq]");
    require(table.rank() == 2, "embeddingLookup: table must have rank 2 [vocabSize, dim]");
    DeviceTensor out({tokenIds.dim(0), tokenIds.dim(1), table.dim(1)});
    check(bf_hip_embedding_forward(tokenIds.data(), table.data(), out.data(), tokenIds.elementCount(), table.dim(0),
                                   table.dim(1), nullptr));
    return out;
}

inline DeviceTensor embeddingLookup(const DeviceTensor& tokenIds, const DeviceTensor& table) {
    require(tokenIds.rank() == 2, "embeddingLookup: token ids must have rank 2 [batch, seq]");
    require(table.rank() == 2, "embeddingLookup: table must have rank 2 [vocabSize, dim]");
    detail::requireIdsInRange("embeddingLookup", tokenIds, table.dim(0), "token id");
    return embeddingLookupPreValidated(tokenIds, table);
}

inline DeviceTensor addPositionalEmbeddingAt(const DeviceTensor& input, const DeviceTensor& table, std::size_t offset) {
    require(input.rank() == 3, "addPositionalEmbedding: needs an input of rank 3 [batch, seq, dim]");
    require(table.rank() == 2 && table.dim(1) == input.dim(2), "addPositionalEmbedding: table must be [maxSeqLen, dim]");
    DeviceTensor out(input.shape());
    check(bf_hip_positional_forward(input.data(), table.data(), out.data(), input.dim(0), input.dim(1), input.dim(2),
                                    table.dim(0), offset, nullptr));
    return out;
}

inline DeviceTensor addPositionalEmbedding(const DeviceTensor& input, const DeviceTensor& table) {
    return addPositionalEmbeddingAt(input, table, 0);
}

namespace detail {
inline DeviceTensor linearImpl(const char* op, const DeviceTensor& input, const DeviceTensor& weight, const DeviceTensor& bias, int bf16) {
    require(input.rank() >= 2, std::string(op) + ": needs a tensor of rank >= 2");
    require(weight.rank() == 2 && lastDim(input) == weight.dim(0), std::string(op) + ": incompatible shapes on the device");
    require(bias.rank() == 1 && bias.dim(0) == weight.dim(1), std::string(op) + ": bias does not match the weight");
    return projectionFused(input, weight, &bias, nullptr, bf16, withLastDim(input, weight.dim(1)));
}
}  // namespace detail

inline DeviceTensor linear(const DeviceTensor& input, const DeviceTensor& weight, const DeviceTensor& bias) {
    return detail::linearImpl("linear", input, weight, bias, 0);
}
inline DeviceTensor linearBf16(const DeviceTensor& input, const DeviceTensor& weight, const DeviceTensor& bias) {
    return detail::linearImpl("linearBf16", input, weight, bias, 1);
}
inline DeviceTensor linearBf16CachedWeight(const DeviceTensor& input, const DeviceTensor& weight, const DeviceTensor& bias) {
    return detail::linearImpl("linearBf16CachedWeight", input, weight, bias, 2);
}

// ---- composite blocks ------------------------------------------------------------------------
struct FeedForwardCache {
    DeviceTensor normed;  // rmsnorm(input); empty with `fused` (only normedImage exists)
    DeviceTensor gemm1;   // normed @ w1, before bias and activation; with `fused` normed @ w1 + b1
    DeviceTensor hidden;  // act(gemm1 + b1); empty with `fused`
    // bf16 mode with widths that are multiples of 8: the activation is applied where the first GEMM stores its product and
    // only the bf16 images the later GEMMs read are kept (raw storage, two values per float)
    bool fused = false;
    DeviceTensor hiddenImage;  // bf16(act(gemm1)), [rows, hidden / 2]
    DeviceTensor normedImage;  // bf16(normed), [rows, d / 2]
};

namespace detail {
inline bool feedForwardFuses(const DeviceTensor& input, const DeviceTensor& w1, bool useBf16) {
    return useBf16 && input.elementCount() > 0 && lastDim(input) % 8 == 0 && w1.dim(1) % 8 == 0;
}
}  // namespace detail

inline DeviceTensor feedForwardForwardCached(const DeviceTensor& input, const DeviceTensor& w1, const DeviceTensor& b1,
                                              const DeviceTensor& w2, const DeviceTensor& b2, bool useBf16,
                                              FeedForwardCache& cache, Activation act = Activation::Silu) {
    require(input.rank() >= 2 && w1.rank() == 2 && w2.rank() == 2 && detail::lastDim(input) == w1.dim(0) && w1.dim(1) == w2.dim(0),
            "feedForward: incompatible shapes on the device");
    const int mode = useBf16 ? 2 : 0;
    cache.fused = detail::feedForwardFuses(input, w1, useBf16);
    if (!cache.fused) cache.normed = rmsnorm(input);
    if (cache.fused) {
        require(b1.rank() == 1 && b1.dim(0) == w1.dim(1), "addBiasSilu: expected input [..., features] and bias [features]");
        require(b2.rank() == 1 && b2.dim(0) == w2.dim(1), "addBiasResidual: expected input [..., features] and bias [features]");
        require(w2.dim(1) == detail::lastDim(input), "addBiasResidual: residual shape differs from the product");
        const std::size_t rows = detail::rowsOf(input), d = detail::lastDim(input), hidden = w1.dim(1);
        cache.gemm1 = DeviceTensor(detail::withLastDim(input, hidden));
        cache.hidden = DeviceTensor();
        cache.hiddenImage = DeviceTensor({rows, hidden / 2});
        cache.normedImage = DeviceTensor({rows, d / 2});
        cache.normed = DeviceTensor();
        // the normalised input has no reader but the GEMMs: it is written as a bf16 image only
        check(bf_hip_rmsnorm_img(input.data(), nullptr, reinterpret_cast<uint16_t*>(cache.normedImage.data()), rows, d, nullptr));
        DeviceTensor out(input.shape());
        check(bf_hip_feedforward_bf16(nullptr, w1.data(), b1.data(), w2.data(), b2.data(), input.data(), static_cast<int>(act),
                                      cache.gemm1.data(), reinterpret_cast<uint16_t*>(cache.hiddenImage.data()),
                                      reinterpret_cast<uint16_t*>(cache.normedImage.data()), out.data(), rows, d, hidden, 1, nullptr));
        return out;
    }
    cache.gemm1 = detail::projection(cache.normed, w1, mode, detail::withLastDim(input, w1.dim(1)));
    cache.hidden = addBiasActivation(cache.gemm1, b1, act);
    require(b2.rank() == 1 && b2.dim(0) == w2.dim(1), "addBiasResidual: expected input [..., features] and bias [features]");
    require(w2.dim(1) == detail::lastDim(input), "addBiasResidual: residual shape differs from the product");
    return detail::projectionFused(cache.hidden, w2, &b2, &input, mode, input.shape());
}

// The feed-forward block of an incremental step: nothing is kept for a backward pass.  With bf16 projections whose
// widths allow it (the condition of the fused training block) one library call makes the block, and for one or two
// rows that is two launches: the normalisation joins the first product's staging of its rows, the activation its store.
inline DeviceTensor feedForwardIncremental(const DeviceTensor& input, const DeviceTensor& w1, const DeviceTensor& b1, const DeviceTensor& w2,
                                            const DeviceTensor& b2, bool useBf16, Activation act = Activation::Silu) {
    require(input.rank() >= 2 && w1.rank() == 2 && w2.rank() == 2 && detail::lastDim(input) == w1.dim(0) && w1.dim(1) == w2.dim(0),
            "feedForward: incompatible shapes on the device");
    if (!useBf16 && input.elementCount() > 0) {
        require(b1.rank() == 1 && b1.dim(0) == w1.dim(1), "addBiasSilu: expected input [..., features] and bias [features]");
        require(b2.rank() == 1 && b2.dim(0) == w2.dim(1), "addBiasResidual: expected input [..., features] and bias [features]");
        require(w2.dim(1) == detail::lastDim(input), "addBiasResidual: residual shape differs from the product");
        DeviceTensor out(input.shape());
        check(bf_hip_rmsnorm_feedforward_f32(input.data(), w1.data(), b1.data(), w2.data(), b2.data(), static_cast<int>(act), out.data(),
                                             detail::rowsOf(input), detail::lastDim(input), w1.dim(1), nullptr));
        return out;
    }
    if (!detail::feedForwardFuses(input, w1, useBf16)) {
        FeedForwardCache unused;
        return feedForwardForwardCached(input, w1, b1, w2, b2, useBf16, unused, act);
    }
    require(b1.rank() == 1 && b1.dim(0) == w1.dim(1), "addBiasSilu: expected input [..., features] and bias [features]");
    require(b2.rank() == 1 && b2.dim(0) == w2.dim(1), "addBiasResidual: expected input [..., features] and bias [features]");
    require(w2.dim(1) == detail::lastDim(input), "addBiasResidual: residual shape differs from the product");
    DeviceTensor out(input.shape());
    check(bf_hip_rmsnorm_feedforward_bf16(input.data(), w1.data(), b1.data(), w2.data(), b2.data(), static_cast<int>(act), out.data(),
                                          detail::rowsOf(input), detail::lastDim(input), w1.dim(1), 1, nullptr));
    return out;
}

namespace detail {
inline DeviceTensor feedForwardImpl(const DeviceTensor& input, const DeviceTensor& w1, const DeviceTensor& b1,
                                     const DeviceTensor& w2, const DeviceTensor& b2, bool useBf16, Activation act) {
    DeviceTensor normed = rmsnorm(input);
    DeviceTensor hidden = activation(linearImpl("feedForward", normed, w1, b1, useBf16 ? 1 : 0), act);
    DeviceTensor out = linearImpl("feedForward", hidden, w2, b2, useBf16 ? 1 : 0);
    return add(input, out);
}
}  // namespace detail

inline DeviceTensor feedForward(const DeviceTensor& input, const DeviceTensor& w1, const DeviceTensor& b1,
                                 const DeviceTensor& w2, const DeviceTensor& b2, Activation act = Activation::Silu) {
    return detail::feedForwardImpl(input, w1, b1, w2, b2, false, act);
}
inline DeviceTensor feedForwardBf16(const DeviceTensor& input, const DeviceTensor& w1, const DeviceTensor& b1,
                                     const DeviceTensor& w2, const DeviceTensor& b2, Activation act = Activation::Silu) {
    return detail::feedForwardImpl(input, w1, b1, w2, b2, true, act);
}

struct SelfAttentionCache {
    // bf16 mode with a width that is a multiple of 8: the normalised input exists only as the bf16 image the projections
    // read (raw storage, [batch*seq, dim / 2]; normedFlat is empty) and attnOutput carries its own image
    DeviceTensor normedImage;
    DeviceTensor normedFlat;  // [batch*seq, dim]
    DeviceTensor q, k, v;     // [batch, seq, dim]
    DeviceTensor attnOutput;  // [batch, seq, dim], before Wout
    DeviceTensor attnM, attnL;
    bool causal = true;       // false: bidirectionalSelfAttention (every position sees the whole sequence)
};

namespace detail {
inline void requireAttention(const char* op, const DeviceTensor& input, std::size_t numHeads) {
    require(input.rank() == 3, std::string(op) + ": needs an input of rank 3 [batch, seq, dim] on the device");
    require(numHeads != 0 && input.dim(2) % numHeads == 0, std::string(op) + ": numHeads must divide dim exactly");
}
// mode: 0 fp32, 1 bf16, 2 bf16 with cached weight images
inline DeviceTensor selfAttentionForwardImpl(const char* op, const DeviceTensor& input, const DeviceTensor& wq,
                                              const DeviceTensor& wk, const DeviceTensor& wv, const DeviceTensor& wout,
                                              std::size_t numHeads, int mode, SelfAttentionCache& cache, bool causal = true) {
    requireAttention(op, input, numHeads);
    std::size_t batch = input.dim(0), seq = input.dim(1), dim = input.dim(2);
    cache.causal = causal;
    float scaleFactor = 1.0F / std::sqrt(static_cast<float>(dim / numHeads));
    cache.normedImage = DeviceTensor();
    if (mode != 0 && dim % 8 == 0 && input.elementCount() > 0) {
        // bf16 operands are written where they are produced: the normalised input only as an image, the attention output
        // with an image beside it (the fp32 copy feeds the backward pass); Q, K and V are one GEMM for widths that are
        // multiples of 256
        require(wq.rank() == 2 && wq.shape() == wk.shape() && wq.shape() == wv.shape() && wq.dim(0) == dim && wq.dim(1) == dim &&
                    wout.shape() == wq.shape(),
                std::string(op) + ": projection weights must be [dim, dim]");
        const std::size_t rows = batch * seq;
        cache.normedFlat = DeviceTensor();
        cache.normedImage = DeviceTensor({rows, dim / 2});
        const std::uint16_t* normedImage = reinterpret_cast<const std::uint16_t*>(cache.normedImage.data());
        check(bf_hip_rmsnorm_img(input.data(), nullptr, reinterpret_cast<std::uint16_t*>(cache.normedImage.data()), rows, dim, nullptr));
        cache.q = DeviceTensor({batch, seq, dim});
        cache.k = DeviceTensor({batch, seq, dim});
        cache.v = DeviceTensor({batch, seq, dim});
        const float* weights[3] = {wq.data(), wk.data(), wv.data()};
        float* outputs[3] = {cache.q.data(), cache.k.data(), cache.v.data()};
        check(bf_hip_matmul_bf16_shared_input_img(nullptr, normedImage, weights, outputs, 3, rows, dim, dim, mode == 2, nullptr));
        cache.attnOutput = DeviceTensor({batch, seq, dim});
        cache.attnM = DeviceTensor({batch, numHeads, seq});
        cache.attnL = DeviceTensor({batch, numHeads, seq});
        std::uint16_t* outImage = cache.attnOutput.attachImage();
        check(bf_hip_attention_forward_img(cache.q.data(), cache.k.data(), cache.v.data(), cache.attnOutput.data(), outImage, dim,
                                           cache.attnM.data(), cache.attnL.data(), batch, numHeads, seq, seq, dim, scaleFactor,
                                           causal ? 0 : seq, nullptr));
        DeviceTensor out({batch, seq, dim});
        check(bf_hip_linear_bf16_img(nullptr, outImage, wout.data(), nullptr, input.data(), out.data(), rows, dim, dim, mode == 2, nullptr));
        return out;
    }
    cache.normedFlat = rmsnorm(input).reshaped({batch * seq, dim});
    if (mode != 0) {
        // one conversion of the normalised input and (for widths that are multiples of 256) one GEMM for Q, K and V
        require(wq.rank() == 2 && wq.shape() == wk.shape() && wq.shape() == wv.shape() && wq.dim(0) == dim && wq.dim(1) == dim,
                std::string(op) + ": projection weights must be [dim, dim]");
        cache.q = DeviceTensor({batch, seq, dim});
        cache.k = DeviceTensor({batch, seq, dim});
        cache.v = DeviceTensor({batch, seq, dim});
        const float* weights[3] = {wq.data(), wk.data(), wv.data()};
        float* outputs[3] = {cache.q.data(), cache.k.data(), cache.v.data()};
        check(bf_hip_matmul_bf16_shared_input(cache.normedFlat.data(), weights, outputs, 3, batch * seq, dim, dim, mode == 2, nullptr));
    } else {
        // three products of one input, independent of each other: one call
        require(wq.rank() == 2 && wk.rank() == 2 && wv.rank() == 2 && wq.dim(0) == dim && wk.dim(0) == dim && wv.dim(0) == dim &&
                    wq.dim(1) == dim && wk.dim(1) == dim && wv.dim(1) == dim,
                std::string(op) + ": projection weights must be [dim, dim]");
        cache.q = DeviceTensor({batch, seq, dim});
        cache.k = DeviceTensor({batch, seq, dim});
        cache.v = DeviceTensor({batch, seq, dim});
        const std::size_t rows = batch * seq;
        productsF32({{0, 0, cache.normedFlat.data(), wq.data(), cache.q.data(), rows, dim, dim},
                     {0, 0, cache.normedFlat.data(), wk.data(), cache.k.data(), rows, dim, dim},
                     {0, 0, cache.normedFlat.data(), wv.data(), cache.v.data(), rows, dim, dim}});
    }
    // query i sees keys j <= oldLen + i: an offset of seq makes every key visible, which is the bidirectional form
    FusedAttentionForwardResult attn = fusedAttentionForward(cache.q, cache.k, cache.v, numHeads, scaleFactor, causal ? 0 : seq);
    cache.attnOutput = std::move(attn.output);
    cache.attnM = std::move(attn.m);
    cache.attnL = std::move(attn.l);
    return projectionFused(cache.attnOutput, wout, nullptr, &input, mode, {batch, seq, dim});
}
}  // namespace detail

inline DeviceTensor selfAttentionForwardCached(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                bool useBf16, SelfAttentionCache& cache) {
    return detail::selfAttentionForwardImpl("selfAttentionForwardCached", input, wq, wk, wv, wout, numHeads, useBf16 ? 2 : 0, cache);
}
inline DeviceTensor selfAttention(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                   const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads) {
    SelfAttentionCache cache;
    return detail::selfAttentionForwardImpl("selfAttention", input, wq, wk, wv, wout, numHeads, 0, cache);
}
// The same block without the causal mask (the CPU backend's bidirectionalSelfAttention, src/backend/cpu/ops.cpp:504-507;
// the CUDA backend refuses the op, model.cu:151-160).
inline DeviceTensor bidirectionalSelfAttentionForwardCached(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                             const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                             bool useBf16, SelfAttentionCache& cache) {
    return detail::selfAttentionForwardImpl("bidirectionalSelfAttentionForwardCached", input, wq, wk, wv, wout, numHeads, useBf16 ? 2 : 0,
                                            cache, false);
}
inline DeviceTensor bidirectionalSelfAttention(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads) {
    SelfAttentionCache cache;
    return detail::selfAttentionForwardImpl("bidirectionalSelfAttention", input, wq, wk, wv, wout, numHeads, 0, cache, false);
}
inline DeviceTensor bidirectionalSelfAttentionBf16(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                                    const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads) {
    SelfAttentionCache cache;
    return detail::selfAttentionForwardImpl("bidirectionalSelfAttentionBf16", input, wq, wk, wv, wout, numHeads, 1, cache, false);
}
inline DeviceTensor selfAttentionBf16(const DeviceTensor& input, const DeviceTensor& wq, const DeviceTensor& wk,
                                       const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads) {
    SelfAttentionCache cache;
    return detail::selfAttentionForwardImpl("selfAttentionBf16", input, wq, wk, wv, wout, numHeads, 1, cache);
}

// K/V of the positions processed so far, for incremental decoding.  The buffers have room to grow: k and v are
// [batch, capacity, dim] with the first `length` rows of every sequence valid, and a call appends its rows in place
// (the reference's k and v are exactly [batch, length, dim] and are re-made, old rows copied, at every call:
// ops.hpp:213, ops_transformer.cu:22-58).  keys() / values() give the [batch, length, dim] tensors.
struct KVCache {
    DeviceTensor k;
    DeviceTensor v;
    std::size_t length = 0;
    std::size_t capacity = 0;   // rows per sequence in k and v

    [[nodiscard]] DeviceTensor keys() const { return dense(k); }
    [[nodiscard]] DeviceTensor values() const { return dense(v); }

    // Room for `rows` positions per sequence: a first allocation takes 64 spare rows, later ones double.
    void reserve(std::size_t batch, std::size_t rows, std::size_t dim) {
        if (rows <= capacity && k.rank() == 3) return;
        const std::size_t grown = (std::max(rows + 64, 2 * capacity) + 63) / 64 * 64;
        DeviceTensor newK({batch, grown, dim}), newV({batch, grown, dim});
        if (length != 0) {
            check(bf_hip_copy_pitched(newK.data(), grown * dim, k.data(), capacity * dim, length * dim, batch, nullptr));
            check(bf_hip_copy_pitched(newV.data(), grown * dim, v.data(), capacity * dim, length * dim, batch, nullptr));
        }
        k = std::move(newK);
        v = std::move(newV);
        capacity = grown;
    }

private:
    [[nodiscard]] DeviceTensor dense(const DeviceTensor& store) const {
        if (length == 0 || store.rank() != 3) return DeviceTensor();
        const std::size_t batch = store.dim(0), dim = store.dim(2);
        DeviceTensor out({batch, length, dim});
        check(bf_hip_copy_pitched(out.data(), length * dim, store.data(), capacity * dim, length * dim, batch, nullptr));
        return out;
    }
};

namespace detail {
// The normalised input's three projections of an incremental step, written where `outs` point
inline void incrementalProjections(const DeviceTensor& newInput, const DeviceTensor& wq, const DeviceTensor& wk, const DeviceTensor& wv,
                                   float* const (&outs)[3], int mode) {
    const std::size_t dim = newInput.dim(2), rows = newInput.dim(0) * newInput.dim(1);
    if (mode != 0 && dim % 8 == 0 && rows > 0) {
        // the normalised rows have no reader but the three projections: one library call normalises and multiplies (for
        // one or two rows one launch: the product's kernel normalises the rows while it stages them)
        const float* weights[3] = {wq.data(), wk.data(), wv.data()};
        float* targets[3] = {outs[0], outs[1], outs[2]};
        check(bf_hip_rmsnorm_matmul_bf16_shared_input(newInput.data(), weights, targets, 3, rows, dim, dim, mode == 2, nullptr));
    } else {
        const float* weights[3] = {wq.data(), wk.data(), wv.data()};
        float* targets[3] = {outs[0], outs[1], outs[2]};
        if (mode == 0) {   // fp32: one library call as well (one or two rows: the products' kernel normalises, all three in one launch)
            check(bf_hip_rmsnorm_matmul_f32_shared_input(newInput.data(), weights, targets, 3, rows, dim, dim, nullptr));
        } else {
            DeviceTensor normedFlat = rmsnorm(newInput).reshaped({rows, dim});
            for (int i = 0; i < 3; ++i)
                check(bf_hip_linear_bf16_img(normedFlat.data(), nullptr, weights[i], nullptr, nullptr, outs[i], rows, dim, dim, mode == 2, nullptr));
        }
    }
}

// The step for a host that runs ahead of the device (Model::generateGreedy): the number of cached positions is read from
// *devicePosition by the kernels (append, attention), nothing of it is in the arguments, and the host-side cache.length
// is left alone.  The cache must already hold room for every position the steps will reach (KVCache::reserve).
inline DeviceTensor selfAttentionIncrementalOnDevicePosition(const char* op, const DeviceTensor& newInput, const DeviceTensor& wq, const DeviceTensor& wk,
                                                      const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads, KVCache& cache,
                                                      int mode, const int* devicePosition) {
    const std::size_t batch = newInput.dim(0), newLen = newInput.dim(1), dim = newInput.dim(2);
    require(cache.capacity != 0 && cache.k.rank() == 3 && cache.k.dim(0) == batch && cache.k.dim(2) == dim,
            std::string(op) + ": a step on a device-side position needs a cache that already holds the prompt, for this batch size and width");
    DeviceTensor qNew({batch, newLen, dim});
    if (mode == 0) {
        check(bf_hip_decode_projections_f32(newInput.data(), wq.data(), wk.data(), wv.data(), qNew.data(), cache.k.data(), cache.v.data(), batch,
                                            newLen, dim, cache.capacity, devicePosition, nullptr));
    } else if (dim % 8 == 0) {
        check(bf_hip_decode_projections_bf16(newInput.data(), wq.data(), wk.data(), wv.data(), qNew.data(), cache.k.data(), cache.v.data(), batch,
                                             newLen, dim, cache.capacity, devicePosition, mode == 2, nullptr));
    } else {
        DeviceTensor kNew({batch, newLen, dim}), vNew({batch, newLen, dim});
        float* const outs[3] = {qNew.data(), kNew.data(), vNew.data()};
        incrementalProjections(newInput, wq, wk, wv, outs, mode);
        check(bf_hip_kv_append_indirect(cache.k.data(), cache.v.data(), kNew.data(), vNew.data(), batch, newLen, dim, cache.capacity,
                                        devicePosition, nullptr));
    }
    const float scaleFactor = 1.0F / std::sqrt(static_cast<float>(dim / numHeads));
    const bool imageOnly = mode != 0 && dim % 8 == 0;
    DeviceTensor attnOut = imageOnly ? DeviceTensor::imageOnly({batch, newLen, dim}) : DeviceTensor({batch, newLen, dim});
    DeviceTensor m({batch, numHeads, newLen}), l({batch, numHeads, newLen});
    check(bf_hip_attention_forward_rows_indirect(qNew.data(), cache.k.data(), cache.v.data(), attnOut.data(),
                                                 imageOnly ? const_cast<std::uint16_t*>(attnOut.image()) : nullptr, imageOnly ? dim : 0, m.data(),
                                                 l.data(), batch, numHeads, newLen, cache.capacity, dim, scaleFactor, devicePosition, nullptr));
    return projectionFused(attnOut, wout, nullptr, &newInput, mode, {batch, newLen, dim});
}

inline DeviceTensor selfAttentionIncrementalImpl(const char* op, const DeviceTensor& newInput, const DeviceTensor& wq,
                                                  const DeviceTensor& wk, const DeviceTensor& wv, const DeviceTensor& wout,
                                                  std::size_t numHeads, KVCache& cache, int mode,
                                                  const int* devicePosition = nullptr) {
    requireAttention(op, newInput, numHeads);
    std::size_t batch = newInput.dim(0), newLen = newInput.dim(1), dim = newInput.dim(2);
    const std::size_t oldLen = cache.length;
    if (devicePosition != nullptr)
        return selfAttentionIncrementalOnDevicePosition(op, newInput, wq, wk, wv, wout, numHeads, cache, mode, devicePosition);
    if (cache.length != 0) require(cache.k.rank() == 3 && cache.k.dim(0) == batch && cache.k.dim(2) == dim, std::string(op) + ": the cache was filled with another batch size or width");
    cache.reserve(batch, oldLen + newLen, dim);
    // one sequence: its new keys and values are rows oldLen.. of the cache, and the projections write them there;
    // several: the projections' rows lie batch by batch and one launch spreads both over the sequences
    const bool inPlace = batch == 1;
    DeviceTensor qNew({batch, newLen, dim}), kNew, vNew;
    if (!inPlace) {
        kNew = DeviceTensor({batch, newLen, dim});
        vNew = DeviceTensor({batch, newLen, dim});
    }
    float* kRows = inPlace ? cache.k.data() + oldLen * dim : kNew.data();
    float* vRows = inPlace ? cache.v.data() + oldLen * dim : vNew.data();
    float* const outs[3] = {qNew.data(), kRows, vRows};
    incrementalProjections(newInput, wq, wk, wv, outs, mode);
    if (!inPlace) check(bf_hip_kv_append(cache.k.data(), cache.v.data(), kNew.data(), vNew.data(), batch, newLen, dim, cache.capacity, oldLen, nullptr));
    cache.length = oldLen + newLen;
    const float scaleFactor = 1.0F / std::sqrt(static_cast<float>(dim / numHeads));
    // the attention output has one reader, the output projection: in bf16 mode it is written as that product's operand image only
    const bool imageOnly = mode != 0 && dim % 8 == 0;
    DeviceTensor attnOut = imageOnly ? DeviceTensor::imageOnly({batch, newLen, dim}) : DeviceTensor({batch, newLen, dim});
    DeviceTensor m({batch, numHeads, newLen}), l({batch, numHeads, newLen});
    check(bf_hip_attention_forward_rows(qNew.data(), cache.k.data(), cache.v.data(), attnOut.data(),
                                        imageOnly ? const_cast<std::uint16_t*>(attnOut.image()) : nullptr, imageOnly ? dim : 0, m.data(), l.data(), batch,
                                        numHeads, newLen, cache.length, cache.capacity, dim, scaleFactor, oldLen, nullptr));
    return projectionFused(attnOut, wout, nullptr, &newInput, mode, {batch, newLen, dim});   // the residual joins in the product's store
}
}  // namespace detail

inline DeviceTensor selfAttentionIncremental(const DeviceTensor& newInput, const DeviceTensor& wq, const DeviceTensor& wk,
                                              const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                              KVCache& cache) {
    return detail::selfAttentionIncrementalImpl("selfAttentionIncremental", newInput, wq, wk, wv, wout, numHeads, cache, 0);
}
inline DeviceTensor selfAttentionIncrementalBf16(const DeviceTensor& newInput, const DeviceTensor& wq, const DeviceTensor& wk,
                                                  const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                  KVCache& cache) {
    return detail::selfAttentionIncrementalImpl("selfAttentionIncrementalBf16", newInput, wq, wk, wv, wout, numHeads, cache, 1);
}
// The same with the weights' bf16 images kept between calls (until invalidateBf16WeightCache): for a generation loop,
// during which the weights do not change (not part of the reference's interface).
inline DeviceTensor selfAttentionIncrementalBf16CachedWeights(const DeviceTensor& newInput, const DeviceTensor& wq, const DeviceTensor& wk,
                                                               const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads,
                                                               KVCache& cache) {
    return detail::selfAttentionIncrementalImpl("selfAttentionIncrementalBf16", newInput, wq, wk, wv, wout, numHeads, cache, 2);
}
// One incremental step that needs nothing from the host (Model::generateGreedy): the number of cached positions comes
// from *devicePosition, read by the kernels; cache.length stays as it is.
inline DeviceTensor selfAttentionIncrementalOnDevicePosition(const DeviceTensor& newInput, const DeviceTensor& wq, const DeviceTensor& wk,
                                                      const DeviceTensor& wv, const DeviceTensor& wout, std::size_t numHeads, KVCache& cache,
                                                      bool useBf16, const int* devicePosition) {
    require(devicePosition != nullptr, "selfAttentionIncrementalOnDevicePosition: no device-side position");
    return detail::selfAttentionIncrementalImpl(useBf16 ? "selfAttentionIncrementalBf16" : "selfAttentionIncremental", newInput, wq, wk, wv, wout,
                                                numHeads, cache, useBf16 ? 2 : 0, devicePosition);
}

// Greedy next-token choice over the last position of [1, seq, vocab] logits (reference: src/main.cpp:504-518),
// computed on the device; only the index crosses to the host.
inline std::size_t argmaxLastPosition(const DeviceTensor& logits) {
    require(logits.rank() >= 2, "argmaxLastPosition: needs logits of rank >= 2");
    long long index = 0;
    check(bf_hip_argmax_last_position(logits.data(), logits.dim(logits.rank() - 2), logits.dim(logits.rank() - 1), &index, nullptr));
    return static_cast<std::size_t>(index);
}

}  // namespace blackforge::backend::hip
