// C wrapper around the REAL reference CPU backend -- TEST INFRASTRUCTURE ONLY.
//
// Implements oracle/bf_oracle.h by calling blackforge::backend::cpu functions.  It is compiled
// together with the reference's own source files, where they lie, into oracle/_ref/libbf_ref.so
// (see oracle/Makefile); no reference source is copied into this repository.  The library is used
// to validate the C restatement (bf_oracle.c), to write the fixtures under tests/golden/, and as
// the benchmark's "reference" CPU baseline.  The shipped library never loads it.
//
// Functions with no counterpart in the reference's public API (the attention core, the GELU
// feed-forward variant) are expressed here as the same composition of public reference functions
// that the reference itself performs at the cited call sites.
#include "bf_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "blackforge/ast/ast.hpp"
#include "blackforge/backend/cpu/autodiff.hpp"
#include "blackforge/backend/cpu/checkpoint.hpp"
#include "blackforge/backend/cpu/train_runner.hpp"
#include "blackforge/backend/lr_schedule.hpp"
#include "blackforge/data/dataset.hpp"
#include "blackforge/backend/cpu/loss.hpp"
#include "blackforge/backend/cpu/model.hpp"
#include "blackforge/backend/cpu/ops.hpp"
#include "blackforge/backend/cpu/optimizer.hpp"
#include "blackforge/backend/cpu/quantize.hpp"
#include "blackforge/ir/module.hpp"
#include "blackforge/runtime/tensor.hpp"

namespace cpu = blackforge::backend::cpu;
namespace ir = blackforge::ir;
using blackforge::runtime::Tensor;

namespace {

Tensor wrap(const float* data, std::vector<std::size_t> shape) {
    std::size_t count = 1;
    for (std::size_t d : shape) count *= d;
    return Tensor(std::move(shape), std::vector<float>(data, data + count));
}

void store(const Tensor& t, float* out) { std::copy(t.data().begin(), t.data().end(), out); }

template <typename Fn>
int guarded(Fn&& fn) {
    try {
        fn();
        return BFO_OK;
    } catch (const std::invalid_argument&) {
        return BFO_INVALID_ARGUMENT;
    } catch (const std::out_of_range&) {
        return BFO_INVALID_ARGUMENT;
    }
}

Tensor headOf(const Tensor& full, std::size_t b, std::size_t h, std::size_t seq, std::size_t dim, std::size_t hd) {
    std::vector<float> data(seq * hd);
    for (std::size_t s = 0; s < seq; ++s)
        std::copy_n(full.data().begin() + static_cast<std::ptrdiff_t>((b * seq + s) * dim + h * hd), hd,
                    data.begin() + static_cast<std::ptrdiff_t>(s * hd));
    return Tensor({seq, hd}, std::move(data));
}

void putHead(float* full, const Tensor& head, std::size_t b, std::size_t h, std::size_t seq, std::size_t dim,
             std::size_t hd) {
    for (std::size_t s = 0; s < seq; ++s)
        std::copy_n(head.data().begin() + static_cast<std::ptrdiff_t>(s * hd), hd, full + (b * seq + s) * dim + h * hd);
}

// scale(matmulTransposeB(q, k)) then -inf above the (shifted) diagonal: ops.cpp:479-480,553-554.
Tensor maskedScores(const Tensor& qh, const Tensor& kh, float scale, std::size_t oldLen) {
    Tensor scores = cpu::scale(cpu::matmulTransposeB(qh, kh), scale);
    std::size_t newLen = scores.dim(0), totalLen = scores.dim(1);
    for (std::size_t i = 0; i < newLen; ++i)
        for (std::size_t j = oldLen + i + 1; j < totalLen; ++j)
            scores.at(i * totalLen + j) = -std::numeric_limits<float>::infinity();
    return scores;
}

Tensor activation(const Tensor& x, int act) { return act == 1 ? cpu::gelu(x) : cpu::silu(x); }

}  // namespace

extern "C" {

int bfo_is_reference(void) { return 1; }

int bfo_add(const float* a, const float* b, float* out, size_t n) {
    return guarded([&] { store(cpu::add(wrap(a, {n}), wrap(b, {n})), out); });
}
int bfo_scale(const float* x, float factor, float* out, size_t n) {
    return guarded([&] { store(cpu::scale(wrap(x, {n}), factor), out); });
}
int bfo_add_bias(const float* x, const float* bias, float* out, size_t rows, size_t features) {
    return guarded([&] { store(cpu::addBias(wrap(x, {rows, features}), wrap(bias, {features})), out); });
}
int bfo_matmul(const float* a, const float* b, float* c, size_t m, size_t k, size_t n) {
    return guarded([&] { store(cpu::matmul(wrap(a, {m, k}), wrap(b, {k, n})), c); });
}
int bfo_matmul_transpose_b(const float* a, const float* b, float* c, size_t m, size_t k, size_t n) {
    return guarded([&] { store(cpu::matmulTransposeB(wrap(a, {m, k}), wrap(b, {n, k})), c); });
}
int bfo_silu(const float* x, float* out, size_t n) {
    return guarded([&] { store(cpu::silu(wrap(x, {n})), out); });
}
int bfo_relu(const float* x, float* out, size_t n) {
    return guarded([&] { store(cpu::relu(wrap(x, {n})), out); });
}
int bfo_gelu(const float* x, float* out, size_t n) {
    return guarded([&] { store(cpu::gelu(wrap(x, {n})), out); });
}
int bfo_linear(const float* x, const float* w, const float* bias, float* out, size_t rows, size_t inF, size_t outF) {
    return guarded([&] { store(cpu::linear(wrap(x, {rows, inF}), wrap(w, {inF, outF}), wrap(bias, {outF})), out); });
}
int bfo_rmsnorm(const float* x, float* out, size_t rows, size_t features) {
    return guarded([&] { store(cpu::rmsnorm(wrap(x, {rows, features})), out); });
}
int bfo_softmax(const float* x, float* out, size_t rows, size_t features) {
    return guarded([&] { store(cpu::softmax(wrap(x, {rows, features})), out); });
}
int bfo_embedding_lookup(const float* ids, const float* table, float* out, size_t batch, size_t seq, size_t vocab,
                         size_t dim) {
    return guarded([&] { store(cpu::embeddingLookup(wrap(ids, {batch, seq}), wrap(table, {vocab, dim})), out); });
}
int bfo_add_positional_embedding_at(const float* x, const float* table, float* out, size_t batch, size_t seq,
                                    size_t dim, size_t maxSeq, size_t offset) {
    return guarded([&] {
        Tensor input = wrap(x, {batch, seq, dim});
        Tensor tab = wrap(table, {maxSeq, dim});
        store(offset == 0 ? cpu::addPositionalEmbedding(input, tab) : cpu::addPositionalEmbeddingAt(input, tab, offset),
              out);
    });
}
int bfo_feed_forward(const float* x, const float* w1, const float* b1, const float* w2, const float* b2, float* out,
                     size_t rows, size_t dim, size_t hidden, int act) {
    return guarded([&] {
        Tensor input = wrap(x, {rows, dim});
        Tensor tw1 = wrap(w1, {dim, hidden}), tb1 = wrap(b1, {hidden}), tw2 = wrap(w2, {hidden, dim}),
               tb2 = wrap(b2, {dim});
        if (act == 0) {
            store(cpu::feedForward(input, tw1, tb1, tw2, tb2), out);
        } else {
            Tensor normed = cpu::rmsnorm(input);
            Tensor hid = activation(cpu::linear(normed, tw1, tb1), act);
            store(cpu::add(input, cpu::linear(hid, tw2, tb2)), out);
        }
    });
}
int bfo_self_attention(const float* x, const float* wq, const float* wk, const float* wv, const float* wout,
                       float* out, size_t batch, size_t seq, size_t dim, size_t heads, int causal) {
    return guarded([&] {
        Tensor input = wrap(x, {batch, seq, dim});
        Tensor q = wrap(wq, {dim, dim}), k = wrap(wk, {dim, dim}), v = wrap(wv, {dim, dim}), o = wrap(wout, {dim, dim});
        store(causal ? cpu::selfAttention(input, q, k, v, o, heads)
                     : cpu::bidirectionalSelfAttention(input, q, k, v, o, heads),
              out);
    });
}
int bfo_self_attention_incremental(const float* xNew, const float* wq, const float* wk, const float* wv,
                                   const float* wout, float* out, const float* kCache, const float* vCache,
                                   float* kOut, float* vOut, size_t batch, size_t newLen, size_t oldLen, size_t dim,
                                   size_t heads) {
    return guarded([&] {
        cpu::KVCache cache;
        if (oldLen > 0) {
            cache.k = wrap(kCache, {batch, oldLen, dim});
            cache.v = wrap(vCache, {batch, oldLen, dim});
            cache.length = oldLen;
        }
        Tensor result = cpu::selfAttentionIncremental(wrap(xNew, {batch, newLen, dim}), wrap(wq, {dim, dim}),
                                                      wrap(wk, {dim, dim}), wrap(wv, {dim, dim}),
                                                      wrap(wout, {dim, dim}), heads, cache);
        store(result, out);
        store(cache.k, kOut);
        store(cache.v, vOut);
    });
}

int bfo_attention_core_forward(const float* q, const float* k, const float* v, float* out, float* m, float* l,
                               size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim, float scale,
                               size_t oldLen) {
    if (heads == 0 || dim % heads != 0) return BFO_INVALID_ARGUMENT;
    return guarded([&] {
        std::size_t hd = dim / heads;
        Tensor tq = wrap(q, {batch, newLen, dim}), tk = wrap(k, {batch, totalLen, dim}),
               tv = wrap(v, {batch, totalLen, dim});
        for (std::size_t b = 0; b < batch; ++b) {
            for (std::size_t h = 0; h < heads; ++h) {
                Tensor qh = headOf(tq, b, h, newLen, dim, hd);
                Tensor kh = headOf(tk, b, h, totalLen, dim, hd);
                Tensor vh = headOf(tv, b, h, totalLen, dim, hd);
                Tensor masked = maskedScores(qh, kh, scale, oldLen);
                Tensor probs = cpu::softmax(masked);
                putHead(out, cpu::matmul(probs, vh), b, h, newLen, dim, hd);
                for (std::size_t i = 0; i < newLen; ++i) {
                    float mx = masked.at(i * totalLen);
                    for (std::size_t j = 1; j < totalLen; ++j) mx = std::max(mx, masked.at(i * totalLen + j));
                    double sum = 0.0;
                    for (std::size_t j = 0; j < totalLen; ++j)
                        sum += std::exp(static_cast<double>(masked.at(i * totalLen + j) - mx));
                    if (m) m[(b * heads + h) * newLen + i] = mx;
                    if (l) l[(b * heads + h) * newLen + i] = static_cast<float>(sum);
                }
            }
        }
    });
}

int bfo_attention_core_backward(const float* dOut, const float* q, const float* k, const float* v, float* dQ,
                                float* dK, float* dV, size_t batch, size_t heads, size_t newLen, size_t totalLen,
                                size_t dim, float scale, size_t oldLen) {
    if (heads == 0 || dim % heads != 0) return BFO_INVALID_ARGUMENT;
    return guarded([&] {
        std::size_t hd = dim / heads;
        Tensor tq = wrap(q, {batch, newLen, dim}), tk = wrap(k, {batch, totalLen, dim}),
               tv = wrap(v, {batch, totalLen, dim}), tg = wrap(dOut, {batch, newLen, dim});
        for (std::size_t b = 0; b < batch; ++b) {
            for (std::size_t h = 0; h < heads; ++h) {
                Tensor qh = headOf(tq, b, h, newLen, dim, hd);
                Tensor kh = headOf(tk, b, h, totalLen, dim, hd);
                Tensor vh = headOf(tv, b, h, totalLen, dim, hd);
                Tensor gh = headOf(tg, b, h, newLen, dim, hd);
                Tensor masked = maskedScores(qh, kh, scale, oldLen);
                Tensor probs = cpu::softmax(masked);
                cpu::MatmulGrad pv = cpu::matmulBackward(probs, vh, gh);
                Tensor dMasked = cpu::softmaxBackward(masked, pv.dA);
                Tensor dScores = cpu::scale(dMasked, scale);
                cpu::MatmulTransposeBGrad qk = cpu::matmulTransposeBBackward(qh, kh, dScores);
                putHead(dQ, qk.dA, b, h, newLen, dim, hd);
                putHead(dK, qk.dB, b, h, totalLen, dim, hd);
                putHead(dV, pv.dB, b, h, totalLen, dim, hd);
            }
        }
    });
}

int bfo_matmul_backward(const float* a, const float* b, const float* g, float* dA, float* dB, size_t m, size_t k,
                        size_t n) {
    return guarded([&] {
        cpu::MatmulGrad r = cpu::matmulBackward(wrap(a, {m, k}), wrap(b, {k, n}), wrap(g, {m, n}));
        store(r.dA, dA);
        store(r.dB, dB);
    });
}
int bfo_matmul_transpose_b_backward(const float* a, const float* b, const float* g, float* dA, float* dB, size_t m,
                                    size_t k, size_t n) {
    return guarded([&] {
        cpu::MatmulTransposeBGrad r = cpu::matmulTransposeBBackward(wrap(a, {m, k}), wrap(b, {n, k}), wrap(g, {m, n}));
        store(r.dA, dA);
        store(r.dB, dB);
    });
}
int bfo_add_bias_backward(const float* g, float* dBias, size_t rows, size_t features) {
    return guarded([&] { store(cpu::addBiasBackward(wrap(g, {rows, features})).dBias, dBias); });
}
int bfo_silu_backward(const float* x, const float* g, float* out, size_t n) {
    return guarded([&] { store(cpu::siluBackward(wrap(x, {n}), wrap(g, {n})), out); });
}
int bfo_relu_backward(const float* x, const float* g, float* out, size_t n) {
    return guarded([&] { store(cpu::reluBackward(wrap(x, {n}), wrap(g, {n})), out); });
}
int bfo_gelu_backward(const float* x, const float* g, float* out, size_t n) {
    return guarded([&] { store(cpu::geluBackward(wrap(x, {n}), wrap(g, {n})), out); });
}
int bfo_rmsnorm_backward(const float* x, const float* g, float* out, size_t rows, size_t features) {
    return guarded([&] { store(cpu::rmsnormBackward(wrap(x, {rows, features}), wrap(g, {rows, features})), out); });
}
int bfo_softmax_backward(const float* x, const float* g, float* out, size_t rows, size_t features) {
    return guarded([&] { store(cpu::softmaxBackward(wrap(x, {rows, features}), wrap(g, {rows, features})), out); });
}
int bfo_embedding_lookup_backward(const float* ids, const float* g, float* dTable, size_t batch, size_t seq,
                                  size_t vocab, size_t dim) {
    return guarded(
        [&] { store(cpu::embeddingLookupBackward(wrap(ids, {batch, seq}), wrap(g, {batch, seq, dim}), vocab), dTable); });
}
int bfo_add_positional_embedding_backward(const float* g, float* dTable, size_t batch, size_t seq, size_t dim,
                                          size_t maxSeq) {
    return guarded([&] { store(cpu::addPositionalEmbeddingBackward(wrap(g, {batch, seq, dim}), maxSeq).dTable, dTable); });
}
int bfo_feed_forward_backward(const float* x, const float* w1, const float* b1, const float* w2, const float* b2,
                              const float* g, float* dX, float* dW1, float* dB1, float* dW2, float* dB2, size_t rows,
                              size_t dim, size_t hidden, int act) {
    return guarded([&] {
        Tensor input = wrap(x, {rows, dim}), grad = wrap(g, {rows, dim});
        Tensor tw1 = wrap(w1, {dim, hidden}), tb1 = wrap(b1, {hidden}), tw2 = wrap(w2, {hidden, dim}),
               tb2 = wrap(b2, {dim});
        if (act == 0) {
            cpu::FeedForwardGrad r = cpu::feedForwardBackward(input, tw1, tb1, tw2, tb2, grad);
            store(r.dInput, dX); store(r.dW1, dW1); store(r.dB1, dB1); store(r.dW2, dW2); store(r.dB2, dB2);
            return;
        }
        // GELU variant: the reference's feedForwardBackward sequence with gelu/geluBackward substituted.
        Tensor normed = cpu::rmsnorm(input);
        Tensor pre = cpu::linear(normed, tw1, tb1);
        Tensor hid = activation(pre, act);
        cpu::AddBiasGrad add2 = cpu::addBiasBackward(grad);
        cpu::MatmulGrad mat2 = cpu::matmulBackward(hid, tw2, add2.dInput);
        Tensor dPre = cpu::geluBackward(pre, mat2.dA);
        cpu::AddBiasGrad add1 = cpu::addBiasBackward(dPre);
        cpu::MatmulGrad mat1 = cpu::matmulBackward(normed, tw1, add1.dInput);
        Tensor dInput = cpu::add(grad, cpu::rmsnormBackward(input, mat1.dA));
        store(dInput, dX); store(mat1.dB, dW1); store(add1.dBias, dB1); store(mat2.dB, dW2); store(add2.dBias, dB2);
    });
}
int bfo_self_attention_backward(const float* x, const float* wq, const float* wk, const float* wv, const float* wout,
                                const float* g, float* dX, float* dWq, float* dWk, float* dWv, float* dWout,
                                size_t batch, size_t seq, size_t dim, size_t heads, int causal) {
    if (heads == 0 || dim % heads != 0) return BFO_INVALID_ARGUMENT;
    return guarded([&] {
        Tensor input = wrap(x, {batch, seq, dim}), grad = wrap(g, {batch, seq, dim});
        Tensor q = wrap(wq, {dim, dim}), k = wrap(wk, {dim, dim}), v = wrap(wv, {dim, dim}), o = wrap(wout, {dim, dim});
        cpu::SelfAttentionGrad r = causal ? cpu::selfAttentionBackward(input, q, k, v, o, heads, grad)
                                          : cpu::bidirectionalSelfAttentionBackward(input, q, k, v, o, heads, grad);
        store(r.dInput, dX); store(r.dWq, dWq); store(r.dWk, dWk); store(r.dWv, dWv); store(r.dWout, dWout);
    });
}

int bfo_mean_squared_error(const float* pred, const float* target, float* grad, float* value, size_t n) {
    return guarded([&] {
        cpu::LossResult r = cpu::meanSquaredError(wrap(pred, {n}), wrap(target, {n}));
        *value = r.value;
        store(r.grad, grad);
    });
}
int bfo_softmax_cross_entropy(const float* logits, const float* target, float* grad, float* value, size_t rows,
                              size_t classes) {
    return guarded([&] {
        cpu::LossResult r = cpu::softmaxCrossEntropy(wrap(logits, {rows, classes}), wrap(target, {rows, classes}));
        *value = r.value;
        store(r.grad, grad);
    });
}
int bfo_softmax_cross_entropy_sparse(const float* logits, const float* targetIdx, float* grad, float* value,
                                     size_t rows, size_t classes) {
    return guarded([&] {
        cpu::LossResult r = cpu::softmaxCrossEntropySparse(wrap(logits, {rows, classes}), wrap(targetIdx, {rows}));
        *value = r.value;
        store(r.grad, grad);
    });
}

int bfo_softmax_cross_entropy_masked(const float* logits, const float* targetIdx, float* grad, float* value,
                                     size_t rows, size_t classes) {
    return guarded([&] {
        cpu::LossResult r = cpu::softmaxCrossEntropyMasked(wrap(logits, {rows, classes}), wrap(targetIdx, {rows}));
        *value = r.value;
        store(r.grad, grad);
    });
}

int bfo_sgd_step(float* param, const float* grad, size_t n, float lr) {
    return guarded([&] {
        cpu::Parameter p{"p", wrap(param, {n}), wrap(grad, {n})};
        cpu::SGD sgd(lr);
        sgd.step({&p});
        store(p.value, param);
    });
}

// The reference keeps AdamW's moments private, so only the first step from zero moments can be
// reproduced through its public API; later steps are covered through bfo_model_adamw_step.
int bfo_adamw_step(float* param, const float* grad, float* m, float* v, size_t n, long long step, float lr,
                   float beta1, float beta2, float eps, float weightDecay) {
    if (step != 1) return BFO_INVALID_ARGUMENT;
    for (size_t i = 0; i < n; ++i)
        if (m[i] != 0.0F || v[i] != 0.0F) return BFO_INVALID_ARGUMENT;
    return guarded([&] {
        cpu::Parameter p{"p", wrap(param, {n}), wrap(grad, {n})};
        cpu::AdamW opt(lr, beta1, beta2, eps, weightDecay);
        opt.step({&p});
        store(p.value, param);
        for (size_t i = 0; i < n; ++i) {
            m[i] = (1.0F - beta1) * grad[i];
            v[i] = (1.0F - beta2) * grad[i] * grad[i];
        }
    });
}

int bfo_round_to_bf16(const float* x, float* out, size_t n) {
    return guarded([&] { store(cpu::quantize(wrap(x, {n}), blackforge::sema::DType::BF16), out); });
}

// argmaxLastPosition lives in the CLI translation unit (src/main.cpp:504-518, internal linkage), which
// cannot be linked as a library; its rule (strict '>' scan over the last position) is restated here.
int bfo_argmax_last_position(const float* logits, size_t seq, size_t vocab, long long* index) {
    if (seq == 0 || vocab == 0) return BFO_INVALID_ARGUMENT;
    const float* row = logits + (seq - 1) * vocab;
    size_t best = 0;
    for (size_t c = 1; c < vocab; ++c)
        if (row[c] > row[best]) best = c;
    *index = static_cast<long long>(best);
    return BFO_OK;
}

struct bfo_model {
    ir::ModelIR irModel;
    std::unique_ptr<cpu::Model> model;
    std::unique_ptr<cpu::AdamW> adamw;
    std::vector<std::size_t> lastOutputShape;
};

bfo_model* bfo_model_create(int numLayers, const int* kinds, const long long* arg0, const long long* arg1,
                            size_t inputFeatures) {
    try {
        auto handle = std::make_unique<bfo_model>();
        ir::ModelIR& m = handle->irModel;
        m.name = "oracle_model";
        auto makeValue = [&](std::size_t id, long long lastDim) {
            ir::Value v;
            v.id = id;
            v.dtype = blackforge::sema::DType::FP32;
            v.shape = {ir::Dim{true, "batch", 0}, ir::Dim{false, "", lastDim}};
            return v;
        };
        m.values.push_back(makeValue(0, static_cast<long long>(inputFeatures)));
        m.inputValue = 0;
        ir::Pipeline pipeline;
        pipeline.sourceValue = 0;
        long long features = static_cast<long long>(inputFeatures);
        for (int i = 0; i < numLayers; ++i) {
            ir::Operation op{};
            op.input = static_cast<std::size_t>(i);
            op.output = static_cast<std::size_t>(i + 1);
            long long a1 = arg1 ? arg1[i] : 0;
            switch (kinds[i]) {
                case BFO_LINEAR: op.kind = ir::OpKind::Linear; op.linearOutFeatures = arg0[i]; features = arg0[i]; break;
                case BFO_SILU: op.kind = ir::OpKind::Silu; break;
                case BFO_RELU: op.kind = ir::OpKind::Relu; break;
                case BFO_GELU: op.kind = ir::OpKind::Gelu; break;
                case BFO_RMSNORM: op.kind = ir::OpKind::RmsNorm; break;
                case BFO_SOFTMAX: op.kind = ir::OpKind::Softmax; break;
                case BFO_EMBEDDING:
                    op.kind = ir::OpKind::Embedding; op.embeddingVocabSize = arg0[i]; op.embeddingDim = a1; features = a1;
                    break;
                case BFO_POSITIONAL: op.kind = ir::OpKind::PositionalEmbedding; op.positionalMaxSeqLen = arg0[i]; break;
                case BFO_ATTENTION: op.kind = ir::OpKind::Attention; op.attentionNumHeads = arg0[i]; break;
                case BFO_BIDIRECTIONAL_ATTENTION: op.kind = ir::OpKind::BidirectionalAttention; op.attentionNumHeads = arg0[i]; break;
                case BFO_FEEDFORWARD:
                    if (a1 != 0) return nullptr;  // the reference's feedforward block is SiLU only
                    op.kind = ir::OpKind::FeedForward; op.feedForwardHiddenDim = arg0[i];
                    break;
                default: return nullptr;
            }
            m.values.push_back(makeValue(op.output, features));
            pipeline.operations.push_back(op);
        }
        m.pipelines.push_back(std::move(pipeline));
        handle->model = std::make_unique<cpu::Model>(m, 42U);
        // start from all-zero parameters, like the restatement; callers assign the values they want
        for (cpu::Parameter* p : handle->model->parameters()) std::fill(p->value.data().begin(), p->value.data().end(), 0.0F);
        return handle.release();
    } catch (const std::exception&) {
        return nullptr;
    }
}

void bfo_model_destroy(bfo_model* model) { delete model; }

int bfo_model_num_params(const bfo_model* model) {
    return static_cast<int>(const_cast<bfo_model*>(model)->model->parameters().size());
}

int bfo_model_param_info(const bfo_model* model, int index, char* name, size_t nameCapacity, size_t* count) {
    auto params = const_cast<bfo_model*>(model)->model->parameters();
    if (index < 0 || static_cast<size_t>(index) >= params.size()) return BFO_INVALID_ARGUMENT;
    if (name && nameCapacity) {
        std::strncpy(name, params[static_cast<size_t>(index)]->name.c_str(), nameCapacity - 1);
        name[nameCapacity - 1] = '\0';
    }
    if (count) *count = params[static_cast<size_t>(index)]->value.elementCount();
    return BFO_OK;
}

float* bfo_model_param_value(bfo_model* model, int index) {
    return model->model->parameters()[static_cast<size_t>(index)]->value.data().data();
}
float* bfo_model_param_grad(bfo_model* model, int index) {
    return model->model->parameters()[static_cast<size_t>(index)]->grad.data().data();
}

int bfo_model_forward(bfo_model* model, const float* input, int rank, const size_t* shape, float* out,
                      size_t outCapacity, size_t* outCount) {
    if (rank < 2 || rank > 3) return BFO_INVALID_ARGUMENT;
    return guarded([&] {
        std::vector<std::size_t> dims(shape, shape + rank);
        Tensor result = model->model->forward(wrap(input, dims));
        model->lastOutputShape = result.shape();
        if (outCount) *outCount = result.elementCount();
        if (result.elementCount() > outCapacity) throw std::invalid_argument("output capacity");
        store(result, out);
    });
}

int bfo_model_backward(bfo_model* model, const float* outputGrad, size_t count) {
    return guarded([&] {
        std::size_t expected = 1;
        for (std::size_t d : model->lastOutputShape) expected *= d;
        if (expected != count) throw std::invalid_argument("grad count");
        model->model->backward(wrap(outputGrad, model->lastOutputShape));
    });
}

int bfo_model_zero_grad(bfo_model* model) {
    return guarded([&] { model->model->zeroGrad(); });
}

int bfo_model_adamw_step(bfo_model* model, float lr, float beta1, float beta2, float eps, float weightDecay) {
    return guarded([&] {
        if (!model->adamw) model->adamw = std::make_unique<cpu::AdamW>(lr, beta1, beta2, eps, weightDecay);
        model->adamw->setLearningRate(lr);
        model->adamw->step(model->model->parameters());
    });
}


// ---- training run: the reference's own runTraining, dataset, checkpoint and schedule functions ----------------
int bfo_shuffle_order(size_t numExamples, unsigned seed, size_t* order) {
    return guarded([&] {
        // a dataset whose example i holds the number i: after shuffle(seed), position i holds order[i]
        std::vector<float> ids(numExamples), zeros(numExamples, 0.0F);
        for (std::size_t i = 0; i < numExamples; ++i) ids[i] = static_cast<float>(i);
        if (numExamples >= (std::size_t(1) << 24)) throw std::invalid_argument("too many examples for float indices");
        blackforge::data::Dataset d({1}, {1}, ids, zeros, numExamples);
        d.shuffle(seed);
        if (numExamples == 0) return;
        auto all = d.batch(0, numExamples);
        for (std::size_t i = 0; i < numExamples; ++i) order[i] = static_cast<std::size_t>(all.input.data()[i]);
    });
}

float bfo_cosine_learning_rate(long long epoch, long long totalEpochs, float base) {
    return blackforge::backend::cosineAnnealingLearningRate(epoch, totalEpochs, base);
}

int bfo_model_save_checkpoint(const bfo_model* model, const char* path) {
    try {
        cpu::saveCheckpoint(*model->model, path);
        return BFO_OK;
    } catch (const std::exception&) {
        return BFO_INVALID_ARGUMENT;
    }
}
int bfo_model_load_checkpoint(bfo_model* model, const char* path) {
    try {
        cpu::loadCheckpoint(*model->model, path);
        return BFO_OK;
    } catch (const std::exception&) {
        return BFO_INVALID_ARGUMENT;
    }
}
int bfo_model_write_initial_checkpoint(bfo_model* model, const char* path) {
    try {
        cpu::Model fresh(model->irModel, 42U);
        cpu::saveCheckpoint(fresh, path);
        return BFO_OK;
    } catch (const std::exception&) {
        return BFO_INVALID_ARGUMENT;
    }
}
int bfo_save_dataset(const char* path, int inputRank, const size_t* inputShape, int targetRank, const size_t* targetShape,
                     const float* inputs, const float* targets, size_t numExamples) {
    try {
        std::vector<std::size_t> inS(inputShape, inputShape + inputRank), tgS(targetShape, targetShape + targetRank);
        std::size_t inN = numExamples, tgN = numExamples;
        for (std::size_t d : inS) inN *= d;
        for (std::size_t d : tgS) tgN *= d;
        blackforge::data::saveDataset(path, inS, tgS, std::vector<float>(inputs, inputs + inN), std::vector<float>(targets, targets + tgN),
                                      numExamples);
        return BFO_OK;
    } catch (const std::exception&) {
        return BFO_INVALID_ARGUMENT;
    }
}

// The real cpu::runTraining, driven by a hand-built program: one dataset declaration (path) and one train block.
// It constructs its own cpu::Model from the IR (seed 42) and loads `fromCheckpoint` over it; the trained weights
// come back through `saveCheckpoint`, which is then loaded into this handle's model.
int bfo_model_run_training(bfo_model* model, const char* datasetPath, int lossKind, int optimizerKind, long long epochs,
                           size_t batchSize, float learningRate, int cosineSchedule, const char* fromCheckpoint,
                           const char* saveCheckpoint, double* epochLosses) {
    namespace ast = blackforge::ast;
    try {
        if (!saveCheckpoint || !saveCheckpoint[0]) return BFO_INVALID_ARGUMENT;
        ast::Program program;
        ast::DatasetDecl dataset;
        dataset.name = "data";
        dataset.fields.push_back(ast::DatasetPathField{datasetPath, {}});
        program.declarations.push_back(dataset);
        ast::TrainDecl train;
        train.fields.push_back(ast::TrainModelField{model->irModel.name, {}});
        train.fields.push_back(ast::TrainDatasetField{"data", {}});
        const char* lossNames[4] = {"mse", "cross_entropy", "cross_entropy_sparse", "cross_entropy_masked"};
        if (lossKind < 0 || lossKind > 3) return BFO_INVALID_ARGUMENT;
        train.fields.push_back(ast::TrainLossField{lossNames[lossKind], {}});
        train.fields.push_back(ast::TrainOptimizerField{optimizerKind == 0 ? "sgd" : "adamw", {}});
        train.fields.push_back(ast::TrainEpochsField{epochs, {}});
        train.fields.push_back(ast::TrainBatchSizeField{static_cast<long long>(batchSize), {}});
        train.fields.push_back(ast::TrainLearningRateField{static_cast<double>(learningRate), {}});
        if (cosineSchedule) train.fields.push_back(ast::TrainLrScheduleField{"cosine", {}});
        program.declarations.push_back(train);
        ir::Module module;
        module.models.push_back(model->irModel);
        cpu::TrainRunResult result = cpu::runTraining(program, module, fromCheckpoint ? fromCheckpoint : "", saveCheckpoint, nullptr);
        for (std::size_t i = 0; i < result.epochLosses.size(); ++i) epochLosses[i] = result.epochLosses[i];
        cpu::loadCheckpoint(*model->model, saveCheckpoint);
        return BFO_OK;
    } catch (const std::exception&) {
        return BFO_INVALID_ARGUMENT;
    }
}

}  // extern "C"
