#pragma once
// Trainable pipeline on the GPU with the reference's Model interface
// (include/blackforge/backend/cuda/model.hpp:48-159; forward/backward src/backend/cuda/model.cu:252-383).
//
// A model is a list of layers; each layer kind corresponds to one ir::OpKind of the reference.  Inside a
// BlackForge build the constructor taking ir::ModelIR is available as well and initialises the weights
// from the project's own deterministic generator, exactly like the reference backends do.
#include <algorithm>
#include <cstddef>
#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "blackforge/backend/hip/autodiff.hpp"
#include "blackforge/backend/hip/device_tensor.hpp"
#include "blackforge/backend/hip/ops.hpp"

#if __has_include("blackforge/ir/module.hpp") && __has_include("blackforge/backend/cpu/random_init.hpp")
#include "blackforge/backend/cpu/random_init.hpp"
#include "blackforge/ir/module.hpp"
#define BLACKFORGE_HIP_HAS_IR 1
#endif

namespace blackforge::backend::hip {

struct Parameter {
    std::string name;
    DeviceTensor value;
    DeviceTensor grad;
};

enum class LayerKind { Linear, Silu, Relu, Gelu, RmsNorm, Softmax, Embedding, PositionalEmbedding, Attention, FeedForward, BidirectionalAttention };

struct LayerSpec {
    LayerKind kind;
    std::size_t arg0 = 0;  // Linear: out features; Embedding: vocab; PositionalEmbedding: maxSeqLen; [Bidirectional]Attention: heads; FeedForward: hidden
    std::size_t arg1 = 0;  // Embedding: dim; FeedForward: activation (0 SiLU = reference, 1 GELU)
};

class Model {
public:
    // inputFeatures: last dimension of the input (ignored when the first layer is an embedding).
    // Parameters start at zero; assign values through parameters().  useBf16 selects bf16 MFMA projections
    // (precision.compute == BF16 in the reference, model.cu:139-140).
    Model(std::string name, const std::vector<LayerSpec>& layers, std::size_t inputFeatures, bool useBf16)
        : name_(std::move(name)), useBf16_(useBf16) {
        std::size_t features = inputFeatures;
        std::size_t valueId = 0;
        for (const LayerSpec& spec : layers) {
            ++valueId;  // the model input is value 0; layer i writes value i+1 (names follow the reference)
            LayerState layer;
            layer.spec = spec;
            const std::string id = std::to_string(valueId);
            switch (spec.kind) {
                case LayerKind::Linear:
                    layer.params.push_back(makeParameter("linear" + id + ".weight", {features, spec.arg0}));
                    layer.params.push_back(makeParameter("linear" + id + ".bias", {spec.arg0}));
                    features = spec.arg0;
                    break;
                case LayerKind::Embedding:
                    layer.params.push_back(makeParameter("embedding" + id + ".table", {spec.arg0, spec.arg1}));
                    features = spec.arg1;
                    break;
                case LayerKind::PositionalEmbedding:
                    layer.params.push_back(makeParameter("positional_embedding" + id + ".table", {spec.arg0, features}));
                    break;
                case LayerKind::Attention:
                case LayerKind::BidirectionalAttention: {
                    // same parameters for both, named after the op (src/backend/cpu/model.cpp:124-150)
                    const std::string label = spec.kind == LayerKind::Attention ? "attention" : "bidirectional_attention";
                    require(spec.arg0 != 0 && features % spec.arg0 == 0,
                            "hip::Model: '" + label + "#" + id + "' needs " + std::to_string(spec.arg0) + " heads to divide dim=" +
                                std::to_string(features));
                    for (const char* w : {".wq", ".wk", ".wv", ".wout"})
                        layer.params.push_back(makeParameter(label + id + w, {features, features}));
                    break;
                }
                case LayerKind::FeedForward:
                    layer.params.push_back(makeParameter("feedforward" + id + ".w1", {features, spec.arg0}));
                    layer.params.push_back(makeParameter("feedforward" + id + ".b1", {spec.arg0}));
                    layer.params.push_back(makeParameter("feedforward" + id + ".w2", {spec.arg0, features}));
                    layer.params.push_back(makeParameter("feedforward" + id + ".b2", {features}));
                    break;
                default:
                    break;
            }
            layers_.push_back(std::move(layer));
        }
        planFusedTriples();
    }

#ifdef BLACKFORGE_HIP_HAS_IR
    // Same construction as cuda::Model (model.cu:137-250): first pipeline of the IR, weights from
    // cpu::randomTensor(seedFor(seed, valueId, salt)) uploaded to the device.
    explicit Model(const ir::ModelIR& modelIR, unsigned int seed = 42, std::optional<ir::PrecisionPolicy> precision = std::nullopt)
        : Model(modelIR.name, specsFromIr(modelIR), inputFeaturesFromIr(modelIR),
                precision.has_value() && precision->compute == sema::DType::BF16) {
        initialiseLikeReference(modelIR, seed);
    }
#endif

    // Runs the pipeline, keeping what backward() needs.  inputRangeTrusted: the caller has already checked
    // the token ids of a leading embedding layer on the host (train_runner.cu:210-212), so no device-side
    // range check (and no host synchronisation) is done.
    DeviceTensor forward(const DeviceTensor& input, bool inputRangeTrusted = false, bool weightImagesCurrent = false) {
        return forward(input.clone(), inputRangeTrusted, weightImagesCurrent);
    }

    // The same pass over an input the model may keep instead of copying it: `input` becomes the first layer's cached input
    // (a DeviceTensor::borrow view must stay valid and unchanged until backward() has run).  weightImagesCurrent is the
    // caller's promise that no parameter value has changed since this model's previous forward pass (no optimizer step,
    // no upload, no checkpoint load), or that whoever changed them has brought the images up to date
    // (refreshWeightImages after an optimizer step): the cached bf16 weight images are then kept instead of being
    // dropped and converted again.  Without the promise every call drops them, as the reference does per forward pass (ops_tensorcore.cu:448).
    DeviceTensor forward(DeviceTensor&& input, bool inputRangeTrusted = false, bool weightImagesCurrent = false) {
        if (!weightImagesCurrent) invalidateBf16WeightCache();   // the optimizer may have changed the weights since the last call
        DeviceTensor current = std::move(input);
        for (std::size_t li = 0; li < layers_.size(); ++li) {
            LayerState& layer = layers_[li];
            if (layer.fusedRole == 1) {
                current = forwardFusedTriple(li, current);
                li += 2;
                continue;
            }
            DeviceTensor next = applyForward(layer, current, inputRangeTrusted && li == 0);
            layer.cachedInput = std::move(current);
            current = std::move(next);
        }
        cachesValid_ = true;
        return current;
    }

    // The activation caches no longer describe a forward pass that ran (a recording into a graph walked the layers without
    // executing anything): backward() throws until forward() has run again, and gradients are added, not written.
    void invalidateCaches() {
        cachesValid_ = false;
        for (LayerState& layer : layers_) layer.gradsAreZero = false;
    }

    // True when the last layer is a bf16 linear layer on its own: its backward pass reads the output gradient only as a
    // bf16 image (both gradient products) and through its column sums (the bias gradient), so backward() accepts an
    // image-only gradient together with those sums (headBiasGrad).
    [[nodiscard]] bool headTakesImageGradient() const {
        return useBf16_ && !layers_.empty() && layers_.back().spec.kind == LayerKind::Linear && layers_.back().fusedRole == 0;
    }

    // headBiasGrad: the column sums of outputGrad, already formed by the producer of the gradient (the loss kernel); the
    // last layer, a linear one, then does not sum the gradient's columns itself, and outputGrad may be image-only.
    void backward(const DeviceTensor& outputGrad, bool inputRangeTrusted = false, const DeviceTensor* headBiasGrad = nullptr) {
        require(headBiasGrad == nullptr || headTakesImageGradient(), "hip::Model::backward: this model's last layer takes no precomputed bias gradient");
        require(cachesValid_, "hip::Model::backward: no forward pass to differentiate (none has run yet, or the last one was only "
                              "recorded into a graph)");
        // the caller's gradient is only read: no copy of it (the logits gradient of a language model is the largest
        // tensor of the step)
        const DeviceTensor* grad = &outputGrad;
        DeviceTensor owned;
        for (std::size_t li = layers_.size(); li-- > 0;) {
            // a deferred zeroGrad(): this layer's gradients are written, not added (see accumulate)
            overwriteGrads_ = zeroPending_ && layers_[li].gradsAreZero;
            if (layers_[li].fusedRole == 3) {
                overwriteGrads_ = zeroPending_ && layers_[li].gradsAreZero && layers_[li - 2].gradsAreZero;
                owned = backwardFusedTriple(li - 2, *grad);
                grad = &owned;
                li -= 2;
                continue;
            }
            // a block whose gradient goes on to another block's bf16 GEMMs writes that gradient's bf16 image with it
            const bool imageForConsumer = useBf16_ && li > 0 && isBlock(layers_[li - 1].spec.kind);
            // the gradient with respect to the model's input has no reader (backward() returns nothing): the first layer
            // does not form it
            owned = applyBackward(layers_[li], *grad, inputRangeTrusted && li == 0, imageForConsumer, /*needInputGrad=*/li > 0,
                                  li + 1 == layers_.size() ? headBiasGrad : nullptr);
            grad = &owned;
        }
        overwriteGrads_ = false;
        zeroPending_ = false;   // every layer has written its gradients
    }

    // deferred: nothing is written now.  The next backward pass WRITES every gradient it would have added to a zeroed
    // buffer (the products straight into the buffers, the rest by a copy in place of the add), which is what a training
    // step wants: the pass over all gradient buffers that zeroes them is saved.  Until that backward pass the buffers hold
    // their old values; parameters() zeroes whatever is still pending before it hands the parameters out.
    void zeroGrad(bool deferred = false) {
        for (LayerState& layer : layers_) layer.gradsAreZero = true;
        zeroPending_ = deferred;
        if (!deferred) zeroPendingGradients();
    }

    // Incremental forward for generation: only the new positions are processed, K/V of earlier positions
    // come from the per-layer cache (model.cu:385-424).
    // The weights must not change while a generation runs (the cached keys and values were made with them): in bf16
    // mode their images are converted at the first call after resetGenerationState() (or after anything else that
    // invalidated them) and kept for the calls that follow, where the reference converts them in every call.
    // weightImagesCurrent: the caller's word that no weight has changed since its images were last made (as for forward()):
    // a new generation then starts without converting them again.
    DeviceTensor forwardIncremental(const DeviceTensor& newTokenIds, bool weightImagesCurrent = false) {
        if (useBf16_ && generationPosition_ == 0 && !weightImagesCurrent) invalidateBf16WeightCache();
        std::size_t newLen = newTokenIds.rank() >= 2 ? newTokenIds.dim(1) : 0;
        DeviceTensor output = incrementalStep(newTokenIds, nullptr);
        generationPosition_ += newLen;
        return output;
    }

    // Greedy continuation of a prompt of one sequence by `count` tokens: what the reference's `generate` command does
    // from the host, one forwardIncremental and one read-back of the logits' argmax per token (main.cpp:594-617).  Here
    // the host never waits inside the loop: the prompt is processed by forwardIncremental, and every step that follows
    // (argmax of the last logits on the device, embed that token, all layers, the head, advance the position) takes the
    // position and the token from device memory, so the host launches step after step ahead of the GPU and reads the
    // tokens back once, at the end.  The caches get their room for all the tokens first.  (Replaying the step from a HIP
    // graph instead of launching it was measured at nearly twice the time per token on this runtime: not done.)
    // Starts a new generation (resetGenerationState) and leaves the model as count - 1 further calls of
    // forwardIncremental would: the last token returned has not been fed.  Needs a pipeline that starts with an
    // embedding; the ids are returned in order.  Not part of the reference's interface.
    [[nodiscard]] std::vector<std::size_t> generateGreedy(const DeviceTensor& promptIds, std::size_t count, bool weightImagesCurrent = false) {
        require(promptIds.rank() == 2 && promptIds.dim(0) == 1 && promptIds.dim(1) >= 1, "generateGreedy: the prompt must be [1, n] token ids, n >= 1");
        require(!layers_.empty() && layers_.front().spec.kind == LayerKind::Embedding, "generateGreedy: the pipeline must start with an embedding");
        const std::size_t promptLen = promptIds.dim(1), vocab = layers_.front().spec.arg0;
        for (const LayerState& layer : layers_)
            if (layer.spec.kind == LayerKind::PositionalEmbedding && count > 1)
                require(promptLen + count - 1 <= layer.params[0].value.dim(0), "generateGreedy: the positions exceed the positional table");
        resetGenerationState();
        if (count == 0) return {};
        DeviceTensor logits = forwardIncremental(promptIds, weightImagesCurrent);
        require(logits.rank() == 3 && logits.dim(2) == vocab, "generateGreedy: the pipeline must end in logits over the embedding's vocabulary");
        for (LayerState& layer : layers_)
            if (layer.spec.kind == LayerKind::Attention) layer.kvCache.reserve(1, promptLen + count, layer.kvCache.k.dim(2));
        DeviceTensor token({1, 1}), history({count}), position({1});   // position: one int, the number of positions processed
        const int start = static_cast<int>(promptLen);
        check(bf_hip_memcpy_h2d(position.data(), &start, sizeof(int)));
        int* devicePosition = reinterpret_cast<int*>(position.data());
        const long long firstSlot = -static_cast<long long>(promptLen);    // a token goes to history[*position - promptLen]
        check(bf_hip_argmax_last_position_device(logits.data(), promptLen, vocab, token.data(), history.data(), count, devicePosition, 0,
                                                 firstSlot, nullptr));
        for (std::size_t i = 1; i < count; ++i) {
            DeviceTensor next = incrementalStep(token, devicePosition);
            // the step has consumed one position: the counter moves on in the same launch that picks the next token
            check(bf_hip_argmax_last_position_device(next.data(), 1, vocab, token.data(), history.data(), count, devicePosition, 1, firstSlot,
                                                     nullptr));
        }
        generationPosition_ += count - 1;
        for (LayerState& layer : layers_)
            if (layer.spec.kind == LayerKind::Attention) layer.kvCache.length += count - 1;
        std::vector<float> ids(count);
        check(bf_hip_memcpy_d2h(ids.data(), history.data(), count * sizeof(float)));   // waits for the steps
        std::vector<std::size_t> result(count);
        for (std::size_t i = 0; i < count; ++i) result[i] = static_cast<std::size_t>(ids[i]);
        return result;
    }

    // Whether generateGreedy can run this pipeline (token ids in, logits over the same vocabulary out, no layer that
    // refuses incremental generation), and how many positions its positional tables allow (SIZE_MAX: no table).
    [[nodiscard]] bool supportsGenerateGreedy() const {
        if (layers_.empty() || layers_.front().spec.kind != LayerKind::Embedding) return false;
        std::size_t features = 0;
        for (const LayerState& layer : layers_) {
            if (layer.spec.kind == LayerKind::BidirectionalAttention) return false;
            if (layer.spec.kind == LayerKind::Embedding) features = layer.spec.arg1;
            if (layer.spec.kind == LayerKind::Linear) features = layer.spec.arg0;
        }
        return features == layers_.front().spec.arg0;
    }
    [[nodiscard]] std::size_t maxPositions() const {
        std::size_t limit = static_cast<std::size_t>(-1);
        for (const LayerState& layer : layers_)
            if (layer.spec.kind == LayerKind::PositionalEmbedding) limit = std::min(limit, layer.params[0].value.dim(0));
        return limit;
    }

    void resetGenerationState() {
        generationPosition_ = 0;
        for (LayerState& layer : layers_) layer.kvCache = KVCache{};
    }

    [[nodiscard]] std::vector<Parameter*> parameters() {
        if (zeroPending_) {   // a deferred zeroGrad() that no backward pass has made good yet
            zeroPendingGradients();
            zeroPending_ = false;
        }
        std::vector<Parameter*> result;
        for (LayerState& layer : layers_)
            for (Parameter& p : layer.params) result.push_back(&p);
        return result;
    }

    [[nodiscard]] std::optional<std::size_t> firstLayerEmbeddingVocabSize() const {
        if (layers_.empty() || layers_.front().spec.kind != LayerKind::Embedding) return std::nullopt;
        return layers_.front().spec.arg0;
    }

    [[nodiscard]] const std::string& name() const { return name_; }
    [[nodiscard]] bool usesBf16() const { return useBf16_; }

private:
    struct LayerState;
    // The layers of one incremental step.  devicePosition == nullptr: the eager step (positions from the host-side
    // counters, which the caller advances; token ids checked).  Otherwise the step that needs nothing from the host:
    // positions read from *devicePosition by the kernels, token ids trusted, host-side counters untouched.
    DeviceTensor incrementalStep(const DeviceTensor& newTokenIds, const int* devicePosition) {
        const DeviceTensor* input = &newTokenIds;
        DeviceTensor current;
        for (LayerState& layer : layers_) {
            const LayerSpec& s = layer.spec;
            const DeviceTensor& in = *input;
            switch (s.kind) {
                case LayerKind::PositionalEmbedding:
                    if (devicePosition == nullptr) {
                        current = addPositionalEmbeddingAt(in, layer.params[0].value, generationPosition_);
                    } else {
                        const DeviceTensor& table = layer.params[0].value;
                        require(in.rank() == 3 && table.rank() == 2 && table.dim(1) == in.dim(2), "addPositionalEmbedding: table must be [maxSeqLen, dim]");
                        DeviceTensor out(in.shape());
                        check(bf_hip_positional_forward_indirect(in.data(), table.data(), out.data(), in.dim(0), in.dim(1), in.dim(2), table.dim(0),
                                                                 devicePosition, nullptr));
                        current = std::move(out);
                    }
                    break;
                case LayerKind::Attention:
                    if (devicePosition != nullptr)
                        current = selfAttentionIncrementalOnDevicePosition(in, layer.params[0].value, layer.params[1].value, layer.params[2].value,
                                                                   layer.params[3].value, s.arg0, layer.kvCache, useBf16_, devicePosition);
                    else
                        current = useBf16_ ? selfAttentionIncrementalBf16CachedWeights(in, layer.params[0].value, layer.params[1].value,
                                                                                        layer.params[2].value, layer.params[3].value, s.arg0,
                                                                                        layer.kvCache)
                                           : selfAttentionIncremental(in, layer.params[0].value, layer.params[1].value, layer.params[2].value,
                                                                      layer.params[3].value, s.arg0, layer.kvCache);
                    break;
                case LayerKind::BidirectionalAttention:
                    // src/backend/cpu/model.cpp:365-374: a layer that sees the whole sequence has no next token to generate
                    throw std::invalid_argument("hip::Model::forwardIncremental: the pipeline contains 'bidirectional_attention', "
                                                "which does not support incremental generation");
                case LayerKind::FeedForward: {
                    // bias, activation and residual in the products' stores, cached weight images, nothing kept for a backward pass
                    Activation act = s.arg1 == 1 ? Activation::Gelu : Activation::Silu;
                    current = feedForwardIncremental(in, layer.params[0].value, layer.params[1].value, layer.params[2].value,
                                                     layer.params[3].value, useBf16_, act);
                    break;
                }
                case LayerKind::Linear:
                    current = useBf16_ ? linearBf16CachedWeight(in, layer.params[0].value, layer.params[1].value)
                                       : linear(in, layer.params[0].value, layer.params[1].value);
                    break;
                case LayerKind::Embedding:
                    current = devicePosition != nullptr ? embeddingLookupPreValidated(in, layer.params[0].value) : embeddingLookup(in, layer.params[0].value);
                    break;
                default: current = applyElementwise(s.kind, in); break;
            }
            input = &current;
        }
        return layers_.empty() ? newTokenIds.clone() : std::move(current);
    }

    struct LayerState {
        LayerSpec spec;
        std::vector<Parameter> params;
        DeviceTensor cachedInput;
        SelfAttentionCache attnCache;
        FeedForwardCache ffCache;
        KVCache kvCache;
        // true from zeroGrad() until this layer's next backward pass: its gradient buffers hold zeros, so that pass may
        // write the gradients there instead of adding them in
        bool gradsAreZero = true;
        // linear -> silu/gelu/relu -> linear with bf16 projections runs as one unit (1, 2, 3 = the three layers of such a
        // triple, 0 = a layer on its own): see planFusedTriples
        int fusedRole = 0;
        DeviceTensor hiddenImage;   // role 1: bf16(act(z)) of the last forward pass, raw storage [rows, hidden / 2]
    };

    static Parameter makeParameter(std::string name, std::vector<std::size_t> shape) {
        return Parameter{std::move(name), DeviceTensor::zeros(shape), DeviceTensor::zeros(shape)};
    }

    static DeviceTensor applyElementwise(LayerKind kind, const DeviceTensor& x) {
        switch (kind) {
            case LayerKind::Silu: return silu(x);
            case LayerKind::Relu: return relu(x);
            case LayerKind::Gelu: return gelu(x);
            case LayerKind::RmsNorm: return rmsnorm(x);
            case LayerKind::Softmax: return softmax(x);
            default: throw std::invalid_argument("hip::Model: not an elementwise layer");
        }
    }

    static bool isActivation(LayerKind kind) { return kind == LayerKind::Silu || kind == LayerKind::Gelu || kind == LayerKind::Relu; }
    static int activationCode(LayerKind kind) { return kind == LayerKind::Silu ? BF_ACT_SILU : kind == LayerKind::Gelu ? BF_ACT_GELU : BF_ACT_RELU; }

    // linear(d -> hidden) -> activation -> linear(hidden -> d) with bf16 projections is the feed-forward block's pair of
    // projections without its normalisation and residual: the three layers run through bf_hip_feedforward_bf16, which keeps
    // the activated hidden tensor as a bf16 image only (its sole readers are GEMMs) and, in the backward pass, forms the
    // pre-activation gradient as a bf16 image plus its column sums in one pass.  Same roundings at the same places as the
    // three layers on their own (the operands of every product, nothing else), so the same results; four passes over
    // [rows, hidden] in fp32 fewer.
    void planFusedTriples() {
        if (!useBf16_) return;
        for (std::size_t li = 0; li + 2 < layers_.size(); ++li) {
            LayerState &l1 = layers_[li], &la = layers_[li + 1], &l2 = layers_[li + 2];
            if (l1.spec.kind != LayerKind::Linear || !isActivation(la.spec.kind) || l2.spec.kind != LayerKind::Linear) continue;
            const std::size_t d = l1.params[0].value.dim(0), hidden = l1.params[0].value.dim(1);
            if (d == 0 || hidden == 0 || d % 8 != 0 || hidden % 8 != 0 || l2.params[0].value.dim(1) != d) continue;
            l1.fusedRole = 1;
            la.fusedRole = 2;
            l2.fusedRole = 3;
            li += 2;
        }
    }

    DeviceTensor forwardFusedTriple(std::size_t li, DeviceTensor& x) {
        LayerState &l1 = layers_[li], &la = layers_[li + 1], &l2 = layers_[li + 2];
        const std::size_t d = l1.params[0].value.dim(0), hidden = l1.params[0].value.dim(1);
        require(x.rank() >= 2 && detail::lastDim(x) == d, "linear: incompatible shapes on the device");
        const std::size_t rows = detail::rowsOf(x);
        DeviceTensor z(detail::withLastDim(x, hidden)), out(x.shape());
        l1.hiddenImage = DeviceTensor({rows, hidden / 2});
        if (rows > 0) {
            // x's bf16 image is kept with it for the weight gradient; a producer may have written it already
            const bool haveImage = x.image() != nullptr;
            std::uint16_t* xImage = haveImage ? const_cast<std::uint16_t*>(x.image()) : x.attachImage();
            check(bf_hip_feedforward_bf16(haveImage ? nullptr : x.data(), l1.params[0].value.data(), l1.params[1].value.data(),
                                          l2.params[0].value.data(), l2.params[1].value.data(), nullptr, activationCode(la.spec.kind), z.data(),
                                          reinterpret_cast<std::uint16_t*>(l1.hiddenImage.data()), xImage, out.data(), rows, d, hidden, 1,
                                          nullptr));
        }
        l1.cachedInput = std::move(x);
        la.cachedInput = std::move(z);
        l2.cachedInput = DeviceTensor();   // the activated hidden tensor exists as l1.hiddenImage only
        return out;
    }

    DeviceTensor backwardFusedTriple(std::size_t li, const DeviceTensor& grad) {
        LayerState &l1 = layers_[li], &la = layers_[li + 1], &l2 = layers_[li + 2];
        const DeviceTensor& x = l1.cachedInput;
        const std::size_t d = l1.params[0].value.dim(0), hidden = l1.params[0].value.dim(1), rows = detail::rowsOf(x);
        require(grad.shape() == x.shape(), "linear backward: gradient shape differs from the output");
        GradientTargets t1, t2;
        if (l1.gradsAreZero) { t1.slot[0] = &l1.params[0].grad; t1.slot[1] = &l1.params[1].grad; }
        if (l2.gradsAreZero) { t2.slot[0] = &l2.params[0].grad; t2.slot[1] = &l2.params[1].grad; }
        l1.gradsAreZero = la.gradsAreZero = l2.gradsAreZero = false;
        DeviceTensor dW1 = detail::gradientTensor(&t1, 0, l1.params[0].value.shape()), dB1 = detail::gradientTensor(&t1, 1, {hidden}),
                     dW2 = detail::gradientTensor(&t2, 0, l2.params[0].value.shape()), dB2 = detail::gradientTensor(&t2, 1, {d});
        const bool needInputGrad = li > 0;   // the model input's gradient has no reader
        DeviceTensor dX = needInputGrad ? DeviceTensor(x.shape()) : DeviceTensor();
        check(bf_hip_feedforward_bf16_backward_img(x.data(), x.image(), l1.params[0].value.data(), l2.params[0].value.data(), la.cachedInput.data(),
                                                   reinterpret_cast<const std::uint16_t*>(l1.hiddenImage.data()), grad.data(), grad.image(),
                                                   activationCode(la.spec.kind), needInputGrad ? dX.data() : nullptr, dW1.data(), dB1.data(),
                                                   dW2.data(), dB2.data(), rows, d, hidden, 1, nullptr));
        accumulate(l1.params[0].grad, dW1);
        accumulate(l1.params[1].grad, dB1);
        accumulate(l2.params[0].grad, dW2);
        accumulate(l2.params[1].grad, dB2);
        return dX;
    }

    // x is about to become the layer's cached input: a bf16 linear layer gives it the bf16 image that both its forward
    // product and, in the backward pass, its weight-gradient product read.
    DeviceTensor applyForward(LayerState& layer, DeviceTensor& x, bool trustedIds) {
        const LayerSpec& s = layer.spec;
        switch (s.kind) {
            case LayerKind::Linear:
                if (useBf16_ && x.image() == nullptr && x.rank() >= 2 && x.elementCount() > 0 && x.dim(x.rank() - 1) % 8 == 0)
                    check(bf_hip_cvt_f32_bf16(x.data(), x.attachImage(), x.elementCount(), nullptr));
                return useBf16_ ? linearBf16CachedWeight(x, layer.params[0].value, layer.params[1].value)
                                : linear(x, layer.params[0].value, layer.params[1].value);
            case LayerKind::Embedding:
                return trustedIds ? embeddingLookupPreValidated(x, layer.params[0].value) : embeddingLookup(x, layer.params[0].value);
            case LayerKind::PositionalEmbedding: return addPositionalEmbedding(x, layer.params[0].value);
            case LayerKind::Attention:
                return selfAttentionForwardCached(x, layer.params[0].value, layer.params[1].value, layer.params[2].value,
                                                  layer.params[3].value, s.arg0, useBf16_, layer.attnCache);
            case LayerKind::BidirectionalAttention:
                return bidirectionalSelfAttentionForwardCached(x, layer.params[0].value, layer.params[1].value, layer.params[2].value,
                                                               layer.params[3].value, s.arg0, useBf16_, layer.attnCache);
            case LayerKind::FeedForward:
                return feedForwardForwardCached(x, layer.params[0].value, layer.params[1].value, layer.params[2].value,
                                                layer.params[3].value, useBf16_, layer.ffCache,
                                                s.arg1 == 1 ? Activation::Gelu : Activation::Silu);
            default: return applyElementwise(s.kind, x);
        }
    }

    // The gradient buffers of every layer whose gradients still count as zero (all of them straight after zeroGrad()).
    void zeroPendingGradients() {
        std::vector<float*> ptrs;
        std::vector<std::size_t> counts;
        for (LayerState& layer : layers_) {
            if (!layer.gradsAreZero) continue;
            for (Parameter& p : layer.params) {
                ptrs.push_back(p.grad.data());
                counts.push_back(p.grad.elementCount());
            }
        }
        if (!ptrs.empty()) check(bf_hip_zero_multi(ptrs.data(), counts.data(), ptrs.size(), nullptr));
    }

    // target += delta, unless the backward pass already wrote delta into target (see GradientTargets); after a deferred
    // zeroGrad() target = delta (0 + delta without the pass that writes the zeros)
    void accumulate(DeviceTensor& target, const DeviceTensor& delta) const {
        if (delta.data() == target.data()) return;
        if (overwriteGrads_) check(bf_hip_memcpy_d2d(target.data(), delta.data(), target.elementCount() * sizeof(float), nullptr));
        else check(bf_hip_accumulate(target.data(), delta.data(), target.elementCount(), nullptr));
    }

    static bool isBlock(LayerKind kind) {
        return kind == LayerKind::Attention || kind == LayerKind::BidirectionalAttention || kind == LayerKind::FeedForward;
    }

    DeviceTensor applyBackward(LayerState& layer, const DeviceTensor& grad, bool trustedIds, bool imageForConsumer, bool needInputGrad = true,
                               const DeviceTensor* givenBiasGrad = nullptr) {
        const LayerSpec& s = layer.spec;
        const DeviceTensor& x = layer.cachedInput;
        GradientTargets targets;
        const GradientTargets* into = nullptr;
        if (layer.gradsAreZero) {
            for (std::size_t i = 0; i < layer.params.size() && i < 4; ++i) targets.slot[i] = &layer.params[i].grad;
            into = &targets;
        }
        layer.gradsAreZero = false;
        switch (s.kind) {
            case LayerKind::Linear: {
                DeviceTensor dBias = givenBiasGrad != nullptr ? DeviceTensor::borrow(givenBiasGrad->data(), givenBiasGrad->shape())
                                                              : biasGradientOnly(grad, into, 1);
                if (useBf16_ && !needInputGrad) {   // the weight gradient alone
                    const DeviceTensor& w = layer.params[0].value;
                    DeviceTensor dW = detail::gradientTensor(into, 0, w.shape());
                    check(bf_hip_matmul_bf16_backward_img(x.data(), x.image(), w.data(), grad.data(), grad.image(), nullptr, dW.data(),
                                                          detail::rowsOf(x), w.dim(0), w.dim(1), 1, nullptr));
                    accumulate(layer.params[0].grad, dW);
                    accumulate(layer.params[1].grad, dBias);
                    return DeviceTensor();
                }
                MatmulGrad g = detail::projectionBackward(x, layer.params[0].value, grad, useBf16_ ? 2 : 0, x.shape(), into, 0);
                accumulate(layer.params[0].grad, g.dB);
                accumulate(layer.params[1].grad, dBias);
                return std::move(g.dA);
            }
            case LayerKind::Silu: return siluBackward(x, grad);
            case LayerKind::Relu: return reluBackward(x, grad);
            case LayerKind::Gelu: return geluBackward(x, grad);
            case LayerKind::RmsNorm: return rmsnormBackward(x, grad);
            case LayerKind::Softmax: return softmaxBackward(x, grad);
            case LayerKind::Embedding: {
                DeviceTensor dTable = trustedIds ? embeddingLookupBackwardPreValidated(x, grad, s.arg0, into)
                                                 : embeddingLookupBackward(x, grad, s.arg0, into);
                accumulate(layer.params[0].grad, dTable);
                // token ids carry no gradient: zeros, as in the reference, for a caller that will look at them
                return needInputGrad ? DeviceTensor::zeros(x.shape()) : DeviceTensor();
            }
            case LayerKind::PositionalEmbedding: {
                PositionalEmbeddingGrad g = addPositionalEmbeddingBackward(grad, s.arg0, into);
                accumulate(layer.params[0].grad, g.dTable);
                return std::move(g.dInput);
            }
            case LayerKind::Attention:
            case LayerKind::BidirectionalAttention: {   // the cache records which of the two the forward pass was
                SelfAttentionGrad g = selfAttentionBackwardCached(x, layer.params[0].value, layer.params[1].value, layer.params[2].value,
                                                                  layer.params[3].value, s.arg0, layer.attnCache, grad, useBf16_, into,
                                                                  imageForConsumer);
                accumulate(layer.params[0].grad, g.dWq);
                accumulate(layer.params[1].grad, g.dWk);
                accumulate(layer.params[2].grad, g.dWv);
                accumulate(layer.params[3].grad, g.dWout);
                return std::move(g.dInput);
            }
            case LayerKind::FeedForward: {
                FeedForwardGrad g = feedForwardBackwardCached(x, layer.params[0].value, layer.params[1].value, layer.params[2].value,
                                                              layer.params[3].value, layer.ffCache, grad, useBf16_,
                                                              s.arg1 == 1 ? Activation::Gelu : Activation::Silu, into, imageForConsumer);
                accumulate(layer.params[0].grad, g.dW1);
                accumulate(layer.params[1].grad, g.dB1);
                accumulate(layer.params[2].grad, g.dW2);
                accumulate(layer.params[3].grad, g.dB2);
                return std::move(g.dInput);
            }
        }
        throw std::invalid_argument("hip::Model: unknown layer kind");
    }

#ifdef BLACKFORGE_HIP_HAS_IR
    static std::vector<LayerSpec> specsFromIr(const ir::ModelIR& modelIR) {
        require(!modelIR.pipelines.empty(), "hip::Model: model '" + modelIR.name + "' has no pipeline to train");
        std::vector<LayerSpec> specs;
        for (const ir::Operation& op : modelIR.pipelines.front().operations) {
            switch (op.kind) {
                case ir::OpKind::Linear: specs.push_back({LayerKind::Linear, static_cast<std::size_t>(op.linearOutFeatures), 0}); break;
                case ir::OpKind::Silu: specs.push_back({LayerKind::Silu}); break;
                case ir::OpKind::Relu: specs.push_back({LayerKind::Relu}); break;
                case ir::OpKind::Gelu: specs.push_back({LayerKind::Gelu}); break;
                case ir::OpKind::RmsNorm: specs.push_back({LayerKind::RmsNorm}); break;
                case ir::OpKind::Softmax: specs.push_back({LayerKind::Softmax}); break;
                case ir::OpKind::Embedding:
                    specs.push_back({LayerKind::Embedding, static_cast<std::size_t>(op.embeddingVocabSize), static_cast<std::size_t>(op.embeddingDim)});
                    break;
                case ir::OpKind::PositionalEmbedding:
                    specs.push_back({LayerKind::PositionalEmbedding, static_cast<std::size_t>(op.positionalMaxSeqLen), 0});
                    break;
                case ir::OpKind::Attention: specs.push_back({LayerKind::Attention, static_cast<std::size_t>(op.attentionNumHeads), 0}); break;
                case ir::OpKind::BidirectionalAttention:
                    specs.push_back({LayerKind::BidirectionalAttention, static_cast<std::size_t>(op.attentionNumHeads), 0});
                    break;
                case ir::OpKind::FeedForward: specs.push_back({LayerKind::FeedForward, static_cast<std::size_t>(op.feedForwardHiddenDim), 0}); break;
                default:
                    throw std::invalid_argument("hip::Model: operation '" + std::string(ir::opKindName(op.kind)) + "' is not implemented on this backend");
            }
        }
        return specs;
    }
    static std::size_t inputFeaturesFromIr(const ir::ModelIR& modelIR) {
        const ir::Value& v = modelIR.valueById(modelIR.pipelines.front().sourceValue);
        return v.shape.empty() || v.shape.back().isSymbolic ? 0 : static_cast<std::size_t>(v.shape.back().literalValue);
    }
    void initialiseLikeReference(const ir::ModelIR& modelIR, unsigned int seed) {
        // salts per parameter slot: src/backend/cpu/model.cpp:14-26
        static const unsigned int linearSalts[] = {0x2545F491U, 0x27D4EB2FU};
        static const unsigned int attnSalts[] = {0x27D4EB2DU, 0x165667B1U, 0xD3A2646CU, 0xFD7046C5U};
        static const unsigned int ffSalts[] = {0xB55A4F09U, 0x5BD1E995U, 0x9E3779B9U, 0x1B873593U};
        const auto& ops = modelIR.pipelines.front().operations;
        for (std::size_t li = 0; li < layers_.size(); ++li) {
            const unsigned int* salts = nullptr;
            static const unsigned int embSalt[] = {0x85EBCA6BU}, posSalt[] = {0xC2B2AE35U};
            switch (layers_[li].spec.kind) {
                case LayerKind::Linear: salts = linearSalts; break;
                case LayerKind::Embedding: salts = embSalt; break;
                case LayerKind::PositionalEmbedding: salts = posSalt; break;
                case LayerKind::Attention:
                case LayerKind::BidirectionalAttention: salts = attnSalts; break;
                case LayerKind::FeedForward: salts = ffSalts; break;
                default: break;
            }
            for (std::size_t pi = 0; pi < layers_[li].params.size(); ++pi) {
                Parameter& p = layers_[li].params[pi];
                p.name = renameForValue(p.name, ops[li].output);
                p.value = DeviceTensor::fromHost(cpu::randomTensor(p.value.shape(), cpu::seedFor(seed, ops[li].output, salts[pi])));
            }
        }
    }
    static std::string renameForValue(const std::string& name, std::size_t valueId) {
        std::size_t dot = name.find('.');
        std::size_t digits = dot;
        while (digits > 0 && name[digits - 1] >= '0' && name[digits - 1] <= '9') --digits;
        return name.substr(0, digits) + std::to_string(valueId) + name.substr(dot);
    }
#endif

    std::string name_;
    bool useBf16_ = false;
    bool cachesValid_ = false;
    bool zeroPending_ = false;     // a deferred zeroGrad() is outstanding
    bool overwriteGrads_ = false;  // during backward(): the layer at hand writes its gradients instead of adding them
    std::vector<LayerState> layers_;
    std::size_t generationPosition_ = 0;
};

}  // namespace blackforge::backend::hip
