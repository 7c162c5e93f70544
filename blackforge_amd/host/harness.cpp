// C entry points over the C++ operator layer (blackforge::backend::hip::Model, losses, optimizers) so
// that the benchmark and the Python parity tests can drive a whole training step of the C++ host layer.
// Host-only code: it calls the GPU exclusively through the C ABI of libbf_hip.so.
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "blackforge/backend/hip/captured_step.hpp"
#include "blackforge/backend/hip/loss.hpp"
#include "blackforge/backend/hip/model.hpp"
#include "blackforge/backend/hip/train_runner.hpp"
#include "blackforge/backend/hip/optimizer.hpp"

namespace hip = blackforge::backend::hip;

namespace {
thread_local std::string g_error;

struct Handle {
    std::unique_ptr<hip::Model> model;
    std::unique_ptr<hip::AdamW> adamw;
    std::unique_ptr<hip::SGD> sgd;
    hip::DeviceTensor output;
    hip::DeviceTensor lossGrad;
    hip::DeviceTensor lossAccumulator;
    std::vector<hip::Parameter*> params;
    // no parameter value has changed since the model's last forward pass: every path that changes one (optimizer steps,
    // replays, training runs, checkpoint loads, bfh_model_weights_changed for uploads through the raw pointers) clears it
    bool weightImagesCurrent = false;
};

template <typename Fn>
int guarded(Fn&& fn) {
    try {
        fn();
        return 0;
    } catch (const std::invalid_argument& e) {
        g_error = e.what();
        return 1;
    } catch (const std::exception& e) {
        g_error = e.what();
        return 2;
    }
}

// Non-owning view of caller-owned device memory as a DeviceTensor argument.
struct Borrowed {
    hip::DeviceTensor tensor;
    Borrowed(const float* ptr, std::vector<std::size_t> shape) : tensor(hip::DeviceTensor::borrow(ptr, std::move(shape))) {}
};
}  // namespace

extern "C" {

const char* bfh_last_error(void) { return g_error.c_str(); }

// kinds follow hip::LayerKind order: 0 linear, 1 silu, 2 relu, 3 gelu, 4 rmsnorm, 5 softmax, 6 embedding,
// 7 positional embedding, 8 attention, 9 feedforward (arg1: 0 SiLU, 1 GELU), 10 bidirectional attention
void* bfh_model_create(int numLayers, const int* kinds, const long long* arg0, const long long* arg1, size_t inputFeatures,
                       int useBf16) {
    Handle* handle = nullptr;
    int st = guarded([&] {
        std::vector<hip::LayerSpec> specs;
        for (int i = 0; i < numLayers; ++i)
            specs.push_back(hip::LayerSpec{static_cast<hip::LayerKind>(kinds[i]), static_cast<std::size_t>(arg0[i]),
                                           static_cast<std::size_t>(arg1 ? arg1[i] : 0)});
        auto h = std::make_unique<Handle>();
        h->model = std::make_unique<hip::Model>("harness", specs, inputFeatures, useBf16 != 0);
        h->params = h->model->parameters();
        h->lossAccumulator = hip::DeviceTensor::zeros({1});
        handle = h.release();
    });
    return st == 0 ? handle : nullptr;
}

void bfh_model_destroy(void* h) { delete static_cast<Handle*>(h); }

int bfh_model_num_params(void* h) { return static_cast<int>(static_cast<Handle*>(h)->params.size()); }

int bfh_model_param_info(void* h, int index, char* name, size_t capacity, size_t* count, float** value, float** grad) {
    Handle* handle = static_cast<Handle*>(h);
    if (index < 0 || static_cast<size_t>(index) >= handle->params.size()) return 1;
    hip::Parameter* p = handle->params[static_cast<size_t>(index)];
    if (name && capacity) {
        std::strncpy(name, p->name.c_str(), capacity - 1);
        name[capacity - 1] = '\0';
    }
    if (count) *count = p->value.elementCount();
    if (value) *value = p->value.data();
    if (grad) *grad = p->grad.data();
    return 0;
}

// input: device pointer to [shape...] floats (token ids or features).
int bfh_model_forward(void* h, const float* input, int rank, const size_t* shape, int trusted, float** output, size_t* outCount) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        Borrowed in(input, std::vector<std::size_t>(shape, shape + rank));
        handle->output = handle->model->forward(in.tensor, trusted != 0);
        handle->weightImagesCurrent = true;
        if (output) *output = handle->output.data();
        if (outCount) *outCount = handle->output.elementCount();
    });
}

}  // extern "C"

namespace {
const char* lossName(int lossKind) {
    return lossKind == 0 ? "cross_entropy_sparse" : lossKind == 2 ? "cross_entropy_masked" : lossKind == 3 ? "cross_entropy" : "mse";
}
// The loss of handle->output against `target`, accumulated on the device, and its gradient (with a bf16 image where the
// model's last layer reads one).
void accumulateLoss(Handle* handle, const float* target, int lossKind) {
    std::vector<std::size_t> shape = handle->output.shape();
    if (lossKind == 0 || lossKind == 2) shape = {handle->output.elementCount() / handle->output.shape().back()};
    Borrowed tgt(target, shape);
    handle->lossGrad = hip::lossGradientAccumulate(lossName(lossKind), handle->output, tgt.tensor, handle->lossAccumulator,
                                                   handle->model->usesBf16());
}
}  // namespace

extern "C" {

// lossKind 0: sparse cross-entropy (targets = one class index per output row), 1: mean squared error, 2: masked sparse
// cross-entropy (index -1 = row ignored), 3: dense cross-entropy (targets = one probability row per output row).  The loss
// sum (for kind 2: the mean over the rows not ignored) is accumulated on the device; bfh_model_read_loss reads and resets it.
int bfh_model_loss(void* h, const float* target, int lossKind) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] { accumulateLoss(handle, target, lossKind); });
}

int bfh_model_loss_grad(void* h, float** grad, size_t* count) {
    Handle* handle = static_cast<Handle*>(h);
    if (grad) *grad = handle->lossGrad.data();
    if (count) *count = handle->lossGrad.elementCount();
    return 0;
}

int bfh_model_backward(void* h, int trusted) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] { handle->model->backward(handle->lossGrad, trusted != 0); });
}

int bfh_model_zero_grad(void* h) {
    return guarded([&] { static_cast<Handle*>(h)->model->zeroGrad(); });
}

int bfh_model_adamw_step(void* h, float lr, float beta1, float beta2, float eps, float weightDecay) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        if (!handle->adamw) handle->adamw = std::make_unique<hip::AdamW>(lr, beta1, beta2, eps, weightDecay);
        handle->adamw->setLearningRate(lr);
        handle->weightImagesCurrent = false;
        handle->adamw->step(handle->params);
    });
}

int bfh_model_sgd_step(void* h, float lr) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        if (!handle->sgd) handle->sgd = std::make_unique<hip::SGD>(lr);
        handle->sgd->setLearningRate(lr);
        handle->weightImagesCurrent = false;
        handle->sgd->step(handle->params);
    });
}

// To be called after parameter values were changed through the pointers of bfh_model_param_info (an upload).
int bfh_model_weights_changed(void* h) {
    static_cast<Handle*>(h)->weightImagesCurrent = false;
    return 0;
}

// One whole training step with no host synchronisation: zeroGrad, forward, loss (accumulated on the
// device), backward, optimizer (0 none, 1 AdamW with the reference defaults and the given lr).
int bfh_model_train_step(void* h, const float* input, int rank, const size_t* shape, const float* target, int lossKind,
                         int optimizer, float lr) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        handle->model->zeroGrad(/*deferred=*/true);
        // the caller's input buffer outlives the step, so the model keeps a view of it instead of a copy; weight images
        // made by the previous step stay in use when nothing has changed a weight since
        Borrowed in(input, std::vector<std::size_t>(shape, shape + rank));
        handle->output = handle->model->forward(std::move(in.tensor), true, handle->weightImagesCurrent);
        handle->weightImagesCurrent = true;
        {
            std::vector<std::size_t> targetShape = handle->output.shape();
            if (lossKind == 0 || lossKind == 2) targetShape = {handle->output.elementCount() / handle->output.shape().back()};
            Borrowed tgt(target, targetShape);
            hip::lossAndBackward(*handle->model, lossName(lossKind), handle->output, tgt.tensor, handle->lossAccumulator, true);
        }
        if (optimizer == 1) {
            if (!handle->adamw) handle->adamw = std::make_unique<hip::AdamW>(lr, 0.9F, 0.999F, 1e-8F, 0.01F);
            handle->adamw->setLearningRate(lr);
            handle->adamw->step(handle->params);
            if (handle->model->usesBf16()) hip::refreshWeightImages(handle->params);   // all their images in one launch
            else handle->weightImagesCurrent = false;
        }
    });
}

// The same step recorded as a graph (hip::CapturedTrainStep) over the caller's input and target buffers: optimizer 1 =
// AdamW with the reference defaults, 2 = SGD.  The handle keeps the optimizer; *step is released with
// bfh_captured_step_destroy before the model is.
int bfh_model_capture_train_step(void* h, const float* input, int rank, const size_t* shape, const float* target, int targetRank,
                                 const size_t* targetShape, int lossKind, int optimizer, float lr, void** step) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        hip::require(optimizer == 1 || optimizer == 2, "capture_train_step: optimizer must be 1 (AdamW) or 2 (SGD)");
        hip::Optimizer* opt = nullptr;
        if (optimizer == 1) {
            if (!handle->adamw) handle->adamw = std::make_unique<hip::AdamW>(lr, 0.9F, 0.999F, 1e-8F, 0.01F);
            opt = handle->adamw.get();
        } else {
            if (!handle->sgd) handle->sgd = std::make_unique<hip::SGD>(lr);
            opt = handle->sgd.get();
        }
        opt->setLearningRate(lr);
        Borrowed in(input, std::vector<std::size_t>(shape, shape + rank));
        Borrowed tgt(target, std::vector<std::size_t>(targetShape, targetShape + targetRank));
        const char* name = lossName(lossKind);
        *step = new hip::CapturedTrainStep(*handle->model, *opt, name, in.tensor, tgt.tensor, handle->lossAccumulator);
    });
}
int bfh_captured_step_run(void* h, void* step, float lr, int optimizer) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        hip::Optimizer* opt = optimizer == 1 ? static_cast<hip::Optimizer*>(handle->adamw.get()) : handle->sgd.get();
        hip::require(opt != nullptr, "captured_step_run: no such optimizer on this model");
        opt->setLearningRate(lr);
        handle->weightImagesCurrent = false;
        static_cast<hip::CapturedTrainStep*>(step)->run();
    });
}
int bfh_captured_step_destroy(void* step) {
    return guarded([&] { delete static_cast<hip::CapturedTrainStep*>(step); });
}

// Reads the accumulated loss sum (one device->host copy) and resets the accumulator.
int bfh_model_read_loss(void* h, float* sum) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        hip::check(bf_hip_memcpy_d2h(sum, handle->lossAccumulator.data(), sizeof(float)));
        hip::check(bf_hip_fill_zero(handle->lossAccumulator.data(), sizeof(float), nullptr));
    });
}

// hip::runTraining over a BFDATA1 file (lossKind: 0 mse, 1 cross_entropy, 2 cross_entropy_sparse, 3 cross_entropy_masked; optimizerKind: 0 sgd,
// 1 adamw); epochLosses receives `epochs` values.
int bfh_model_run_training(void* h, const char* datasetPath, int lossKind, int optimizerKind, long long epochs, size_t batchSize,
                           double learningRate, int cosineSchedule, const char* fromCheckpoint, const char* saveCheckpoint,
                           double* epochLosses) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        hip::HostDataset dataset = hip::HostDataset::load(datasetPath);
        hip::TrainOptions options;
        options.loss = lossKind == 0 ? "mse" : lossKind == 1 ? "cross_entropy" : lossKind == 2 ? "cross_entropy_sparse" : "cross_entropy_masked";
        options.optimizer = optimizerKind == 0 ? "sgd" : "adamw";
        options.epochs = epochs;
        options.batchSize = batchSize;
        options.learningRate = learningRate;
        options.cosineSchedule = cosineSchedule != 0;
        options.fromCheckpointPath = fromCheckpoint ? fromCheckpoint : "";
        options.saveCheckpointPath = saveCheckpoint ? saveCheckpoint : "";
        handle->weightImagesCurrent = false;
        hip::TrainRunResult result = hip::runTraining(*handle->model, dataset, options, nullptr);
        for (std::size_t i = 0; i < result.epochLosses.size(); ++i) epochLosses[i] = result.epochLosses[i];
    });
}

int bfh_model_save_checkpoint(void* h, const char* path) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] { hip::saveCheckpoint(*handle->model, path); });
}

// Parameter buffers are re-created by the load: callers must fetch bfh_model_param_info again afterwards.
int bfh_model_load_checkpoint(void* h, const char* path) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        hip::loadCheckpoint(*handle->model, path);
        handle->weightImagesCurrent = false;
        handle->params = handle->model->parameters();
    });
}

// ---- composite blocks of the C++ operator layer, for parity tests against the CPU backend --------------------
// Every pointer is device memory owned by the caller; results are copied into the caller's buffers.
// variant: 0 the stateless fp32 operator, 1 the stateless bf16 operator, 2 the *ForwardCached / *BackwardCached pair in
// fp32, 3 the same pair with bf16 projections (cached weight images).
namespace {
void copyOut(float* dst, const hip::DeviceTensor& src) {
    if (dst != nullptr && src.elementCount() != 0)
        hip::check(bf_hip_memcpy_d2d(dst, src.data(), src.elementCount() * sizeof(float), nullptr));
}
struct AttentionWeights {
    Borrowed wq, wk, wv, wout;
    AttentionWeights(const float* q, const float* k, const float* v, const float* o, std::size_t dim)
        : wq(q, {dim, dim}), wk(k, {dim, dim}), wv(v, {dim, dim}), wout(o, {dim, dim}) {}
};
struct FeedForwardWeights {
    Borrowed w1, b1, w2, b2;
    FeedForwardWeights(const float* w1p, const float* b1p, const float* w2p, const float* b2p, std::size_t d, std::size_t hidden)
        : w1(w1p, {d, hidden}), b1(b1p, {hidden}), w2(w2p, {hidden, d}), b2(b2p, {d}) {}
};
}  // namespace

int bfh_self_attention(const float* x, const float* wq, const float* wk, const float* wv, const float* wout, size_t batch, size_t seq,
                       size_t dim, size_t heads, int variant, int causal, float* out) {
    return guarded([&] {
        Borrowed in(x, {batch, seq, dim});
        AttentionWeights w(wq, wk, wv, wout, dim);
        hip::DeviceTensor y;
        hip::SelfAttentionCache cache;
        if (variant >= 2) hip::invalidateBf16WeightCache();
        const auto &a = w.wq.tensor, &b = w.wk.tensor, &c = w.wv.tensor, &d = w.wout.tensor;
        switch (variant * 2 + (causal ? 1 : 0)) {
            case 1: y = hip::selfAttention(in.tensor, a, b, c, d, heads); break;
            case 0: y = hip::bidirectionalSelfAttention(in.tensor, a, b, c, d, heads); break;
            case 3: y = hip::selfAttentionBf16(in.tensor, a, b, c, d, heads); break;
            case 2: y = hip::bidirectionalSelfAttentionBf16(in.tensor, a, b, c, d, heads); break;
            case 5: case 7: y = hip::selfAttentionForwardCached(in.tensor, a, b, c, d, heads, variant == 3, cache); break;
            case 4: case 6: y = hip::bidirectionalSelfAttentionForwardCached(in.tensor, a, b, c, d, heads, variant == 3, cache); break;
            default: throw std::invalid_argument("bfh_self_attention: unknown variant");
        }
        copyOut(out, y);
    });
}

int bfh_self_attention_backward(const float* x, const float* wq, const float* wk, const float* wv, const float* wout, const float* g,
                                size_t batch, size_t seq, size_t dim, size_t heads, int variant, int causal, float* dInput, float* dWq,
                                float* dWk, float* dWv, float* dWout) {
    return guarded([&] {
        Borrowed in(x, {batch, seq, dim}), grad(g, {batch, seq, dim});
        AttentionWeights w(wq, wk, wv, wout, dim);
        const auto &a = w.wq.tensor, &b = w.wk.tensor, &c = w.wv.tensor, &d = w.wout.tensor;
        hip::SelfAttentionGrad r;
        if (variant >= 2) {
            hip::invalidateBf16WeightCache();
            hip::SelfAttentionCache cache;
            if (causal) hip::selfAttentionForwardCached(in.tensor, a, b, c, d, heads, variant == 3, cache);
            else hip::bidirectionalSelfAttentionForwardCached(in.tensor, a, b, c, d, heads, variant == 3, cache);
            r = hip::selfAttentionBackwardCached(in.tensor, a, b, c, d, heads, cache, grad.tensor, variant == 3);
        } else if (variant == 0) {
            r = causal ? hip::selfAttentionBackward(in.tensor, a, b, c, d, heads, grad.tensor)
                       : hip::bidirectionalSelfAttentionBackward(in.tensor, a, b, c, d, heads, grad.tensor);
        } else {
            r = causal ? hip::selfAttentionBf16Backward(in.tensor, a, b, c, d, heads, grad.tensor)
                       : hip::bidirectionalSelfAttentionBf16Backward(in.tensor, a, b, c, d, heads, grad.tensor);
        }
        copyOut(dInput, r.dInput);
        copyOut(dWq, r.dWq);
        copyOut(dWk, r.dWk);
        copyOut(dWv, r.dWv);
        copyOut(dWout, r.dWout);
    });
}

// act: 0 SiLU (the reference block), 1 GELU, 2 ReLU.  x: [shape..., d].
int bfh_feed_forward(const float* x, int rank, const size_t* shape, const float* w1, const float* b1, const float* w2, const float* b2,
                     size_t hidden, int variant, int act, float* out) {
    return guarded([&] {
        std::vector<std::size_t> dims(shape, shape + rank);
        if (dims.empty()) throw std::invalid_argument("bfh_feed_forward: rank 0");
        Borrowed in(x, dims);
        FeedForwardWeights w(w1, b1, w2, b2, dims.back(), hidden);
        const auto activation = static_cast<hip::Activation>(act);
        hip::DeviceTensor y;
        hip::FeedForwardCache cache;
        if (variant >= 2) hip::invalidateBf16WeightCache();
        if (variant == 0) y = hip::feedForward(in.tensor, w.w1.tensor, w.b1.tensor, w.w2.tensor, w.b2.tensor, activation);
        else if (variant == 1) y = hip::feedForwardBf16(in.tensor, w.w1.tensor, w.b1.tensor, w.w2.tensor, w.b2.tensor, activation);
        else y = hip::feedForwardForwardCached(in.tensor, w.w1.tensor, w.b1.tensor, w.w2.tensor, w.b2.tensor, variant == 3, cache, activation);
        copyOut(out, y);
    });
}

int bfh_feed_forward_backward(const float* x, int rank, const size_t* shape, const float* w1, const float* b1, const float* w2,
                              const float* b2, const float* g, size_t hidden, int variant, int act, float* dInput, float* dW1, float* dB1,
                              float* dW2, float* dB2) {
    return guarded([&] {
        std::vector<std::size_t> dims(shape, shape + rank);
        if (dims.empty()) throw std::invalid_argument("bfh_feed_forward_backward: rank 0");
        Borrowed in(x, dims), grad(g, dims);
        FeedForwardWeights w(w1, b1, w2, b2, dims.back(), hidden);
        const auto activation = static_cast<hip::Activation>(act);
        hip::FeedForwardGrad r;
        if (variant >= 2) {
            hip::invalidateBf16WeightCache();
            hip::FeedForwardCache cache;
            hip::feedForwardForwardCached(in.tensor, w.w1.tensor, w.b1.tensor, w.w2.tensor, w.b2.tensor, variant == 3, cache, activation);
            r = hip::feedForwardBackwardCached(in.tensor, w.w1.tensor, w.b1.tensor, w.w2.tensor, w.b2.tensor, cache, grad.tensor,
                                               variant == 3, activation);
        } else if (variant == 0) {
            r = hip::feedForwardBackward(in.tensor, w.w1.tensor, w.b1.tensor, w.w2.tensor, w.b2.tensor, grad.tensor, activation);
        } else {
            r = hip::feedForwardBf16Backward(in.tensor, w.w1.tensor, w.b1.tensor, w.w2.tensor, w.b2.tensor, grad.tensor, activation);
        }
        copyOut(dInput, r.dInput);
        copyOut(dW1, r.dW1);
        copyOut(dB1, r.dB1);
        copyOut(dW2, r.dW2);
        copyOut(dB2, r.dB2);
    });
}

// hip::KVCache behind a handle, for selfAttentionIncremental[Bf16]; k and v are reported as the dense
// [batch, length, dim] tensors, copies that live until the next call.
struct KvHandle {
    hip::KVCache cache;
    hip::DeviceTensor keys, values;
};
void* bfh_kv_cache_create(void) { return new KvHandle(); }
void bfh_kv_cache_destroy(void* cache) { delete static_cast<KvHandle*>(cache); }
int bfh_kv_cache_info(void* cache, size_t* length, size_t* capacity, float** k, float** v) {
    return guarded([&] {
        auto* c = static_cast<KvHandle*>(cache);
        if (length) *length = c->cache.length;
        if (capacity) *capacity = c->cache.capacity;
        if (k) { c->keys = c->cache.keys(); *k = c->keys.data(); }
        if (v) { c->values = c->cache.values(); *v = c->values.data(); }
    });
}
int bfh_self_attention_incremental(void* cache, const float* xNew, const float* wq, const float* wk, const float* wv, const float* wout,
                                   size_t batch, size_t newLen, size_t dim, size_t heads, int useBf16, float* out) {
    return guarded([&] {
        Borrowed in(xNew, {batch, newLen, dim});
        AttentionWeights w(wq, wk, wv, wout, dim);
        auto& kv = static_cast<KvHandle*>(cache)->cache;
        hip::DeviceTensor y = useBf16 ? hip::selfAttentionIncrementalBf16(in.tensor, w.wq.tensor, w.wk.tensor, w.wv.tensor, w.wout.tensor, heads, kv)
                                      : hip::selfAttentionIncremental(in.tensor, w.wq.tensor, w.wk.tensor, w.wv.tensor, w.wout.tensor, heads, kv);
        copyOut(out, y);
    });
}

// Model::forwardIncremental on [batch, newLen] token ids (features for a model without embedding: [batch, newLen, d]);
// the output stays owned by the handle until the next forward call.
int bfh_model_forward_incremental(void* h, const float* input, int rank, const size_t* shape, float** output, size_t* outCount) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        Borrowed in(input, std::vector<std::size_t>(shape, shape + rank));
        if (!handle->weightImagesCurrent) hip::invalidateBf16WeightCache();   // weights set or trained since the images were made
        handle->weightImagesCurrent = true;
        handle->output = handle->model->forwardIncremental(in.tensor, /*weightImagesCurrent=*/true);
        if (output) *output = handle->output.data();
        if (outCount) *outCount = handle->output.elementCount();
    });
}
// Model::generateGreedy on a [1, n] prompt of token ids (device memory); `tokens` (HOST) receives `count` ids.
int bfh_model_generate_greedy(void* h, const float* promptIds, size_t n, size_t count, long long* tokens) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        Borrowed in(promptIds, {1, n});
        if (!handle->weightImagesCurrent) hip::invalidateBf16WeightCache();
        handle->weightImagesCurrent = true;
        std::vector<std::size_t> ids = handle->model->generateGreedy(in.tensor, count, /*weightImagesCurrent=*/true);
        for (std::size_t i = 0; i < ids.size(); ++i) tokens[i] = static_cast<long long>(ids[i]);
    });
}
int bfh_model_reset_generation(void* h) {
    return guarded([&] { static_cast<Handle*>(h)->model->resetGenerationState(); });
}
// argmaxLastPosition over the handle's last output viewed as [rows, vocab].
int bfh_model_argmax_last(void* h, size_t vocab, long long* index) {
    Handle* handle = static_cast<Handle*>(h);
    return guarded([&] {
        std::size_t rows = vocab ? handle->output.elementCount() / vocab : 0;
        Borrowed view(handle->output.data(), {rows, vocab});
        *index = static_cast<long long>(hip::argmaxLastPosition(view.tensor));
    });
}

// The permutation HostDataset::shuffle(seed) applies to `numExamples` examples: order[i] = example at position i afterwards.
int bfh_shuffle_order(size_t numExamples, unsigned seed, size_t* order) {
    return guarded([&] {
        std::vector<float> ids(numExamples), zeros(numExamples, 0.0F);
        for (std::size_t i = 0; i < numExamples; ++i) ids[i] = static_cast<float>(i);
        hip::HostDataset d({1}, {1}, ids, zeros, numExamples);
        d.shuffle(seed);
        if (numExamples == 0) return;
        auto all = d.batch(0, numExamples);
        for (std::size_t i = 0; i < numExamples; ++i) order[i] = static_cast<std::size_t>(all.input.data()[i]);
    });
}

}  // extern "C"
