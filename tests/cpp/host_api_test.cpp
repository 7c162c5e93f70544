// Tests of the C++ operator layer (namespace blackforge::backend::hip) written the way the reference tests
// its GPU backend: DeviceTensor::fromHost -> op -> toHost, compared with literal expectations.  The literal
// inputs and expected values are the ones the reference's own tests use; each case cites its source.
// Built by blackforge_amd/host/Makefile, run on a GPU by tests/test_gpu_host_layer.py.
#include <cmath>
#include <cstdio>
#include <functional>
#include <stdexcept>
#include <string>
#include <vector>

#include "blackforge/backend/hip/autodiff.hpp"
#include "blackforge/backend/hip/device_query.hpp"
#include "blackforge/backend/hip/fused_attention.hpp"
#include "blackforge/backend/hip/loss.hpp"
#include "blackforge/backend/hip/model.hpp"
#include "blackforge/backend/hip/ops.hpp"
#include "blackforge/backend/hip/optimizer.hpp"

namespace hip = blackforge::backend::hip;
using blackforge::runtime::Tensor;
using hip::DeviceTensor;

namespace {
int g_failures = 0;
int g_checks = 0;

#define EXPECT_TRUE(cond)                                                            \
    do {                                                                             \
        ++g_checks;                                                                  \
        if (!(cond)) { ++g_failures; std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); } \
    } while (0)
#define EXPECT_NEAR(a, b, tol)                                                       \
    do {                                                                             \
        ++g_checks;                                                                  \
        double a_ = (a), b_ = (b);                                                   \
        if (!(std::fabs(a_ - b_) <= (tol))) { ++g_failures; std::printf("  FAILED %s:%d: %s = %.9g, expected %.9g\n", __FILE__, __LINE__, #a, a_, b_); } \
    } while (0)
#define EXPECT_THROW_INVALID(stmt)                                                   \
    do {                                                                             \
        ++g_checks;                                                                  \
        bool thrown_ = false;                                                        \
        try { stmt; } catch (const std::invalid_argument&) { thrown_ = true; }       \
        if (!thrown_) { ++g_failures; std::printf("  FAILED %s:%d: %s did not throw std::invalid_argument\n", __FILE__, __LINE__, #stmt); } \
    } while (0)

DeviceTensor dev(std::vector<std::size_t> shape, std::vector<float> data) { return DeviceTensor::fromHost(Tensor(std::move(shape), std::move(data))); }

void run(const char* name, const std::function<void()>& fn) {
    int before = g_failures;
    try {
        fn();
    } catch (const std::exception& e) {
        ++g_failures;
        std::printf("  FAILED %s: unexpected exception: %s\n", name, e.what());
    }
    std::printf("[%s] %s\n", before == g_failures ? "  OK  " : "FAILED", name);
}

// shared attention fixture: tests/backend/cpu/ops_tests.cpp:328-337, tests/backend/cuda/ops_tests.cu:343-351
const std::vector<float> kWq = {0.3F, -0.1F, 0.2F, 0.05F, 0.1F, 0.4F, -0.2F, 0.15F, -0.3F, 0.2F, 0.1F, -0.05F, 0.2F, -0.1F, 0.3F, 0.1F};
const std::vector<float> kWk = {0.1F, 0.2F, -0.1F, 0.3F, -0.2F, 0.1F, 0.4F, -0.1F, 0.3F, -0.3F, 0.1F, 0.2F, -0.1F, 0.2F, -0.2F, 0.1F};
const std::vector<float> kWv = {0.2F, 0.1F, -0.1F, 0.3F, 0.1F, -0.2F, 0.3F, 0.1F, -0.1F, 0.3F, 0.2F, -0.1F, 0.3F, 0.1F, -0.2F, 0.2F};
const std::vector<float> kWout = {0.1F, -0.1F, 0.2F, 0.1F, 0.2F, 0.1F, -0.1F, 0.2F, -0.1F, 0.2F, 0.1F, -0.1F, 0.1F, 0.2F, -0.1F, 0.2F};
const std::vector<float> kAttnInput = {0.1F, -0.2F, 0.3F, 0.4F, -0.5F, 0.6F, 0.2F, -0.1F, 0.3F, 0.2F, -0.4F, 0.5F};
}  // namespace

int main() {
    if (hip::enumerateDevices().empty()) {
        std::printf("no HIP device visible\n");
        return 2;
    }
    hip::setActiveDevice(0);

    run("device selection rejects a missing index (device_query.cu:34-40)", [] { EXPECT_THROW_INVALID(hip::setActiveDevice(4096)); });

    run("DeviceTensor round trip, zeros, clone, reshaped (device_tensor.hpp:35-62)", [] {
        DeviceTensor t = dev({2, 3}, {1, 2, 3, 4, 5, 6});
        Tensor back = t.toHost();
        EXPECT_TRUE(back.shape() == (std::vector<std::size_t>{2, 3}));
        for (std::size_t i = 0; i < 6; ++i) EXPECT_NEAR(back.at(i), float(i + 1), 0.0);
        DeviceTensor c = t.clone();
        DeviceTensor r = std::move(c).reshaped({3, 2});
        EXPECT_TRUE(r.dim(0) == 3 && c.data() == nullptr);
        EXPECT_THROW_INVALID((void)std::move(r).reshaped({4, 2}));
        Tensor z = DeviceTensor::zeros({4}).toHost();
        for (std::size_t i = 0; i < 4; ++i) EXPECT_NEAR(z.at(i), 0.0, 0.0);
        DeviceTensor empty({0, 4});
        EXPECT_TRUE(empty.data() == nullptr && empty.toHost().elementCount() == 0);
    });

    run("add / addBias literals and shape errors (cpu/ops_tests.cpp:10-34)", [] {
        Tensor sum = hip::add(dev({2}, {1, 2}), dev({2}, {10, 20})).toHost();
        EXPECT_NEAR(sum.at(0), 11, 0.0);
        EXPECT_NEAR(sum.at(1), 22, 0.0);
        EXPECT_THROW_INVALID(hip::add(dev({2}, {1, 2}), dev({3}, {1, 2, 3})));
        Tensor b = hip::addBias(dev({2, 2}, {1, 2, 3, 4}), dev({2}, {10, 20})).toHost();
        EXPECT_NEAR(b.at(0), 11, 0.0);
        EXPECT_NEAR(b.at(3), 24, 0.0);
    });

    run("matmul 2x2 = 19,22,43,50 in fp32 and through bf16 (cpu/ops_tests.cpp:36-46, cuda/ops_tests.cu:85-103)", [] {
        DeviceTensor a = dev({2, 2}, {1, 2, 3, 4}), b = dev({2, 2}, {5, 6, 7, 8});
        const float expected[] = {19, 22, 43, 50};
        Tensor c = hip::matmul(a, b).toHost(), cb = hip::matmulBf16(a, b).toHost();
        for (int i = 0; i < 4; ++i) { EXPECT_NEAR(c.at(i), expected[i], 0.0); EXPECT_NEAR(cb.at(i), expected[i], 0.0); }
        EXPECT_THROW_INVALID(hip::matmul(dev({2, 3}, std::vector<float>(6, 1.0F)), dev({2, 2}, std::vector<float>(4, 1.0F))));
    });

    run("linear: identity weight and rank-3 input (cpu/ops_tests.cpp:54-63,173-184)", [] {
        Tensor r = hip::linear(dev({1, 2}, {3, 4}), dev({2, 2}, {1, 0, 0, 1}), dev({2}, {10, 20})).toHost();
        EXPECT_NEAR(r.at(0), 13, 0.0);
        EXPECT_NEAR(r.at(1), 24, 0.0);
        std::vector<float> x = {1, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6, 6};
        Tensor r3 = hip::linear(dev({2, 3, 2}, x), dev({2, 1}, {1, 1}), dev({1}, {0})).toHost();
        EXPECT_TRUE(r3.shape() == (std::vector<std::size_t>{2, 3, 1}));
        for (std::size_t i = 0; i < 6; ++i) EXPECT_NEAR(r3.at(i), x[2 * i] + x[2 * i + 1], 0.0);
    });

    run("activations (cpu/ops_tests.cpp:65-90)", [] {
        Tensor r = hip::relu(dev({3}, {-2, 0, 3})).toHost();
        EXPECT_NEAR(r.at(0), 0, 0.0); EXPECT_NEAR(r.at(2), 3, 0.0);
        Tensor s = hip::silu(dev({3}, {0, 20, -20})).toHost();
        EXPECT_NEAR(s.at(0), 0, 0.0); EXPECT_NEAR(s.at(1), 20, 0.01); EXPECT_NEAR(s.at(2), 0, 0.01);
        Tensor g = hip::gelu(dev({3}, {0, 20, -20})).toHost();
        EXPECT_NEAR(g.at(0), 0, 0.0); EXPECT_NEAR(g.at(1), 20, 0.01); EXPECT_NEAR(g.at(2), 0, 0.01);
    });

    run("rmsnorm and softmax invariants (cpu/ops_tests.cpp:92-170)", [] {
        Tensor r = hip::rmsnorm(dev({2, 4}, {1, 2, 3, 4, -1, -1, -1, -1})).toHost();
        for (int row = 0; row < 2; ++row) {
            double ss = 0;
            for (int c = 0; c < 4; ++c) ss += double(r.at(row * 4 + c)) * r.at(row * 4 + c);
            EXPECT_NEAR(std::sqrt(ss / 4), 1.0, 1e-3);
        }
        EXPECT_THROW_INVALID(hip::rmsnorm(dev({4}, {1, 2, 3, 4})));
        Tensor s = hip::softmax(dev({1, 3}, {1000, 1000, 1000})).toHost();
        for (int i = 0; i < 3; ++i) EXPECT_NEAR(s.at(i), 1.0 / 3, 1e-6);
        EXPECT_THROW_INVALID(hip::softmax(dev({4}, {1, 2, 3, 4})));
    });

    run("embedding lookup rows, range errors, scatter-add of repeated ids (cpu/ops_tests.cpp:238-262, autodiff_tests.cpp:180-199)", [] {
        DeviceTensor table = dev({3, 2}, {10, 11, 20, 21, 30, 31});
        Tensor r = hip::embeddingLookup(dev({1, 3}, {0, 2, 1}), table).toHost();
        const float expected[] = {10, 11, 30, 31, 20, 21};
        for (int i = 0; i < 6; ++i) EXPECT_NEAR(r.at(i), expected[i], 0.0);
        EXPECT_THROW_INVALID(hip::embeddingLookup(dev({1, 1}, {3}), table));
        EXPECT_THROW_INVALID(hip::embeddingLookup(dev({1, 1}, {-1}), table));
        Tensor d = hip::embeddingLookupBackward(dev({1, 3}, {0, 1, 0}), dev({1, 3, 2}, {1, 2, 10, 20, 3, 4}), 3).toHost();
        const float dexp[] = {4, 6, 10, 20, 0, 0};
        for (int i = 0; i < 6; ++i) EXPECT_NEAR(d.at(i), dexp[i], 0.0);
    });

    run("positional embedding add, offset and limits (cpu/ops_tests.cpp:264-286,435-461)", [] {
        Tensor r = hip::addPositionalEmbedding(dev({2, 2, 2}, {0, 0, 0, 0, 100, 100, 100, 100}), dev({2, 2}, {1, 2, 3, 4})).toHost();
        const float expected[] = {1, 2, 3, 4, 101, 102, 103, 104};
        for (int i = 0; i < 8; ++i) EXPECT_NEAR(r.at(i), expected[i], 0.0);
        EXPECT_THROW_INVALID(hip::addPositionalEmbedding(dev({1, 3, 2}, std::vector<float>(6, 0.0F)), dev({2, 2}, {1, 2, 3, 4})));
        Tensor at = hip::addPositionalEmbeddingAt(dev({1, 1, 2}, {0, 0}), dev({4, 2}, {1, 2, 3, 4, 5, 6, 7, 8}), 2).toHost();
        EXPECT_NEAR(at.at(0), 5, 0.0); EXPECT_NEAR(at.at(1), 6, 0.0);
        EXPECT_THROW_INVALID(hip::addPositionalEmbeddingAt(dev({1, 2, 2}, {0, 0, 0, 0}), dev({3, 2}, {1, 2, 3, 4, 5, 6}), 2));
    });

    run("zero weights give the residual identity (cpu/ops_tests.cpp:290-322)", [] {
        std::vector<float> x = {0.1F, -0.2F, 0.3F, 0.4F, -0.5F, 0.6F};
        Tensor r = hip::feedForward(dev({1, 2, 3}, x), DeviceTensor::zeros({3, 4}), DeviceTensor::zeros({4}), DeviceTensor::zeros({4, 3}),
                                    DeviceTensor::zeros({3})).toHost();
        for (std::size_t i = 0; i < 6; ++i) EXPECT_NEAR(r.at(i), x[i], 0.0);
        DeviceTensor z = DeviceTensor::zeros({4, 4});
        Tensor a = hip::selfAttention(dev({1, 3, 4}, kAttnInput), z, z, z, z, 2).toHost();
        for (std::size_t i = 0; i < 12; ++i) EXPECT_NEAR(a.at(i), kAttnInput[i], 0.0);
    });

    run("self attention respects the causal mask; heads must divide dim (cpu/ops_tests.cpp:324-357)", [] {
        DeviceTensor wq = dev({4, 4}, kWq), wk = dev({4, 4}, kWk), wv = dev({4, 4}, kWv), wo = dev({4, 4}, kWout);
        std::vector<float> perturbed = kAttnInput;
        perturbed[8] = 99.0F;
        Tensor a = hip::selfAttention(dev({1, 3, 4}, kAttnInput), wq, wk, wv, wo, 2).toHost();
        Tensor b = hip::selfAttention(dev({1, 3, 4}, perturbed), wq, wk, wv, wo, 2).toHost();
        for (std::size_t i = 0; i < 8; ++i) EXPECT_NEAR(a.at(i), b.at(i), 0.0);
        DeviceTensor w3 = DeviceTensor::zeros({3, 3});
        EXPECT_THROW_INVALID(hip::selfAttention(DeviceTensor::zeros({1, 2, 3}), w3, w3, w3, w3, 2));
    });

    run("incremental attention equals full attention position by position (cpu/ops_tests.cpp:393-425)", [] {
        DeviceTensor wq = dev({4, 4}, kWq), wk = dev({4, 4}, kWk), wv = dev({4, 4}, kWv), wo = dev({4, 4}, kWout);
        Tensor full = hip::selfAttention(dev({1, 3, 4}, kAttnInput), wq, wk, wv, wo, 2).toHost();
        hip::KVCache cache;
        for (std::size_t s = 0; s < 3; ++s) {
            std::vector<float> tok(kAttnInput.begin() + 4 * s, kAttnInput.begin() + 4 * s + 4);
            Tensor inc = hip::selfAttentionIncremental(dev({1, 1, 4}, tok), wq, wk, wv, wo, 2, cache).toHost();
            for (std::size_t d = 0; d < 4; ++d) EXPECT_NEAR(inc.at(d), full.at(s * 4 + d), 1e-5);
        }
        EXPECT_TRUE(cache.length == 3);
    });

    run("fused attention rejects headDim > 256 (fused_attention.cu:305-311)", [] {
        DeviceTensor big = DeviceTensor::zeros({1, 1, 260});
        EXPECT_THROW_INVALID(hip::fusedAttentionForward(big, big, big, 1, 1.0F, 0));
    });

    run("losses: MSE = 2.5, CE(uniform) = ln 2, sparse == dense, range error (cpu/loss_tests.cpp:10-16,51-69,115-140)", [] {
        EXPECT_NEAR(hip::meanSquaredError(dev({2}, {1, 2}), dev({2}, {0, 0})).value, 2.5, 0.0);
        hip::LossResult ce = hip::softmaxCrossEntropy(dev({1, 2}, {0, 0}), dev({1, 2}, {1, 0}));
        EXPECT_NEAR(ce.value, std::log(2.0), 1e-6);
        Tensor g = ce.grad.toHost();
        EXPECT_NEAR(g.at(0), -0.5, 1e-6); EXPECT_NEAR(g.at(1), 0.5, 1e-6);
        DeviceTensor logits = dev({2, 3}, {0.5F, -1.2F, 0.3F, 2.0F, 0.1F, -0.5F});
        hip::LossResult dense = hip::softmaxCrossEntropy(logits, dev({2, 3}, {0, 1, 0, 1, 0, 0}));
        hip::LossResult sparse = hip::softmaxCrossEntropySparse(logits, dev({2}, {1, 0}));
        EXPECT_NEAR(sparse.value, dense.value, 1e-6);
        Tensor gd = dense.grad.toHost(), gs = sparse.grad.toHost();
        for (std::size_t i = 0; i < 6; ++i) EXPECT_NEAR(gs.at(i), gd.at(i), 1e-6);
        EXPECT_THROW_INVALID(hip::softmaxCrossEntropySparse(dev({1, 3}, {0.1F, 0.2F, 0.3F}), dev({1}, {5})));
        EXPECT_THROW_INVALID(hip::meanSquaredError(dev({2}, {1, 2}), dev({3}, {1, 2, 3})));
    });

    run("optimizers: SGD and AdamW first-step closed forms, decoupled decay (cpu/optimizer_tests.cpp:10-59)", [] {
        hip::Parameter p{"p", dev({2}, {1, -2}), dev({2}, {0.5F, 0.5F})};
        hip::SGD(0.1F).step({&p});
        EXPECT_NEAR(p.value.toHost().at(0), 1.0F - 0.1F * 0.5F, 1e-7);
        EXPECT_NEAR(p.value.toHost().at(1), -2.0F - 0.1F * 0.5F, 1e-7);
        hip::Parameter q{"p", dev({1}, {1}), dev({1}, {0.2F})};
        hip::AdamW(0.1F, 0.9F, 0.999F, 1e-8F, 0.0F).step({&q});
        EXPECT_NEAR(q.value.toHost().at(0), 1.0 - 0.1 * (0.2 / (std::sqrt(0.04) + 1e-8)), 1e-5);
        hip::Parameter w{"p", dev({1}, {1}), dev({1}, {0})};
        hip::AdamW(0.1F, 0.9F, 0.999F, 1e-8F, 0.1F).step({&w});
        EXPECT_NEAR(w.value.toHost().at(0), 1.0F - 0.1F * 0.1F, 1e-7);
    });

    run("Model: tiny LM trains (loss goes down over AdamW steps), greedy argmax on device", [] {
        using hip::LayerKind;
        hip::Model model("tiny", {{LayerKind::Embedding, 16, 8}, {LayerKind::PositionalEmbedding, 4, 0}, {LayerKind::Attention, 2, 0},
                                  {LayerKind::FeedForward, 16, 0}, {LayerKind::Linear, 16, 0}}, 0, false);
        unsigned state = 12345;
        for (hip::Parameter* p : model.parameters()) {
            std::vector<float> init(p->value.elementCount());
            for (float& v : init) { state = state * 1664525u + 1013904223u; v = (float(state >> 8) / float(1u << 24) - 0.5F) * 0.2F; }
            p->value = DeviceTensor::fromHost(Tensor(p->value.shape(), init));
        }
        DeviceTensor ids = dev({2, 4}, {1, 2, 3, 4, 5, 6, 7, 8});
        DeviceTensor targets = dev({8}, {2, 3, 4, 5, 6, 7, 8, 9});
        hip::AdamW opt(1e-2F);
        float first = 0, last = 0;
        for (int step = 0; step < 30; ++step) {
            model.zeroGrad();
            DeviceTensor logits = model.forward(ids);
            hip::LossResult loss = hip::softmaxCrossEntropySparse(logits, targets);
            model.backward(loss.grad);
            opt.step(model.parameters());
            if (step == 0) first = loss.value;
            last = loss.value;
        }
        EXPECT_TRUE(last < first * 0.8F);
        EXPECT_TRUE(model.firstLayerEmbeddingVocabSize().value() == 16);
        std::size_t idx = hip::argmaxLastPosition(dev({1, 2, 4}, {0, 5, 1, 9, 1, 7, 7, 3}));
        EXPECT_TRUE(idx == 1);
    });

    run("Model: masked-language-model pipeline (bidirectional attention, masked loss) trains; no incremental generation", [] {
        using hip::LayerKind;
        hip::Model model("mlm", {{LayerKind::Embedding, 16, 8}, {LayerKind::PositionalEmbedding, 4, 0}, {LayerKind::BidirectionalAttention, 2, 0},
                                 {LayerKind::FeedForward, 16, 0}, {LayerKind::Linear, 16, 0}}, 0, false);
        unsigned state = 777;
        for (hip::Parameter* p : model.parameters()) {
            std::vector<float> init(p->value.elementCount());
            for (float& v : init) { state = state * 1664525u + 1013904223u; v = (float(state >> 8) / float(1u << 24) - 0.5F) * 0.2F; }
            p->value = DeviceTensor::fromHost(Tensor(p->value.shape(), init));
        }
        EXPECT_TRUE(model.parameters()[2]->name == "bidirectional_attention3.wq");
        DeviceTensor ids = dev({2, 4}, {1, 2, 3, 4, 5, 6, 7, 8});
        DeviceTensor targets = dev({8}, {-1, 2, -1, -1, 5, -1, -1, 8});   // loss over three of the eight positions
        hip::AdamW opt(1e-2F);
        float first = 0, last = 0;
        for (int step = 0; step < 30; ++step) {
            model.zeroGrad();
            hip::LossResult loss = hip::softmaxCrossEntropyMasked(model.forward(ids), targets);
            model.backward(loss.grad);
            opt.step(model.parameters());
            if (step == 0) first = loss.value;
            last = loss.value;
        }
        EXPECT_TRUE(last < first * 0.8F);
        EXPECT_THROW_INVALID(hip::softmaxCrossEntropyMasked(model.forward(ids), dev({8}, {-2, 2, -1, -1, 5, -1, -1, 8})));
        EXPECT_THROW_INVALID((void)model.forwardIncremental(dev({1, 1}, {3})));   // src/backend/cpu/model.cpp:365-374
    });

    // tests/backend/cuda/model_tests.cu:536-611: generating token by token gives the logits of the full forward pass
    for (bool bf16 : {false, true}) {
        run(bf16 ? "Model::forwardIncremental == forward, bf16 projections" : "Model::forwardIncremental == forward, fp32", [bf16] {
            using hip::LayerKind;
            const std::size_t vocab = 24, dim = 16, maxSeq = 8;
            hip::Model model("decode", {{LayerKind::Embedding, vocab, dim}, {LayerKind::PositionalEmbedding, maxSeq, 0}, {LayerKind::Attention, 2, 0},
                                        {LayerKind::FeedForward, 32, 0}, {LayerKind::Attention, 4, 0}, {LayerKind::Linear, vocab, 0}}, 0, bf16);
            unsigned state = 4242;
            for (hip::Parameter* p : model.parameters()) {
                std::vector<float> init(p->value.elementCount());
                for (float& v : init) { state = state * 1664525u + 1013904223u; v = (float(state >> 8) / float(1u << 24) - 0.5F) * 0.6F; }
                p->value = DeviceTensor::fromHost(Tensor(p->value.shape(), init));
            }
            const std::vector<float> tokens = {3, 17, 5, 9, 21, 0};
            const double tol = bf16 ? 2e-2 : 1e-4;
            for (int round = 0; round < 2; ++round) {   // the second round checks resetGenerationState()
                std::size_t done = 0;
                for (std::size_t newLen : {std::size_t(3), std::size_t(1), std::size_t(1), std::size_t(1)}) {
                    std::vector<float> piece(tokens.begin() + long(done), tokens.begin() + long(done + newLen));
                    Tensor inc = model.forwardIncremental(dev({1, newLen}, piece)).toHost();
                    done += newLen;
                    Tensor full = model.forward(dev({1, done}, std::vector<float>(tokens.begin(), tokens.begin() + long(done)))).toHost();
                    EXPECT_TRUE(inc.shape() == (std::vector<std::size_t>{1, newLen, vocab}));
                    double scale = 0;
                    for (float v : full.data()) scale = std::fmax(scale, std::fabs(v));
                    for (std::size_t i = 0; i < newLen * vocab; ++i)
                        EXPECT_NEAR(inc.data()[i], full.data()[(done - newLen) * vocab + i], tol * scale);
                    std::size_t choice = hip::argmaxLastPosition(DeviceTensor::fromHost(inc));
                    std::size_t best = 0;
                    for (std::size_t c = 1; c < vocab; ++c)
                        if (inc.data()[(newLen - 1) * vocab + c] > inc.data()[(newLen - 1) * vocab + best]) best = c;
                    EXPECT_TRUE(choice == best);
                }
                model.resetGenerationState();
            }
            // positions continue without a reset: 6 + 3 > maxSeq rows of the positional table
            (void)model.forwardIncremental(dev({1, 6}, tokens));
            EXPECT_THROW_INVALID((void)model.forwardIncremental(dev({1, 3}, {1, 2, 3})));

            // generateGreedy (token and position kept on the device) = the loop of the reference's generate command
            // (main.cpp:594-617): argmax of the last logits, fed back
            const std::vector<float> prompt = {3, 17, 5};
            EXPECT_TRUE(model.supportsGenerateGreedy() && model.maxPositions() == maxSeq);
            const std::vector<std::size_t> fast = model.generateGreedy(dev({1, 3}, prompt), 5);
            model.resetGenerationState();
            DeviceTensor logits = model.forwardIncremental(dev({1, 3}, prompt));
            EXPECT_TRUE(fast.size() == 5);
            for (std::size_t step = 0; step < fast.size(); ++step) {
                const Tensor host = logits.toHost();
                const std::size_t rows = host.elementCount() / vocab, best = hip::argmaxLastPosition(logits);
                const float margin = host.data()[(rows - 1) * vocab + best] - host.data()[(rows - 1) * vocab + fast[step]];
                EXPECT_TRUE(fast[step] == best || margin <= float(tol));   // a near tie may fall the other way: other kernels, other last bits
                if (step + 1 < fast.size()) logits = model.forwardIncremental(dev({1, 1}, {static_cast<float>(fast[step])}));
            }
            EXPECT_THROW_INVALID((void)model.generateGreedy(dev({1, 3}, prompt), maxSeq));   // 3 + 8 - 1 positions > 8 table rows
            EXPECT_TRUE(model.generateGreedy(dev({1, 3}, prompt), 6).size() == 6);         // the last token is not fed: 3 + 5 positions fit
        });
    }

    std::printf("%d checks, %d failures\n", g_checks, g_failures);
    return g_failures == 0 ? 0 : 1;
}
