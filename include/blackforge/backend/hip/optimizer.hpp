#pragma once
// Optimizers with the reference's interface (include/blackforge/backend/cuda/optimizer.hpp:17-66): the
// update of every parameter happens in one multi-tensor kernel launch, moments live on the device.
#include <string>
#include <unordered_map>
#include <vector>

#include "blackforge/backend/hip/model.hpp"

namespace blackforge::backend::hip {

class Optimizer {
public:
    virtual ~Optimizer() = default;
    virtual void step(const std::vector<Parameter*>& parameters) = 0;
    virtual void setLearningRate(float learningRate) = 0;

    // A step that is recorded once in a graph and replayed (CapturedTrainStep; not part of the reference's interface).
    // What changes between steps (learning rate, AdamW's bias corrections) cannot be passed by value to a recorded
    // launch, so it lives in a small device block: prepareRecording() creates the block and every per-parameter state
    // BEFORE the capture begins, recordStep() launches the update that reads the block (called inside the capture), and
    // publishStep() advances the step count and writes the block for the step about to be replayed.  The arithmetic is
    // the one step() does, value for value.
    virtual void prepareRecording(const std::vector<Parameter*>& parameters) = 0;
    virtual void recordStep(const std::vector<Parameter*>& parameters) = 0;
    virtual void publishStep(bf_stream_t stream) = 0;
};

// After an optimizer step over `updated`: the cached bf16 images of those weights are made again, all in one launch
// (refreshBf16WeightImages), so that the next Model::forward may be told that the images are current.
inline void refreshWeightImages(const std::vector<Parameter*>& updated) {
    std::vector<const float*> changed;
    for (const Parameter* param : updated) changed.push_back(param->value.data());
    refreshBf16WeightImages(changed);
}

class SGD : public Optimizer {
public:
    explicit SGD(float learningRate) : learningRate_(learningRate) {}

    void step(const std::vector<Parameter*>& parameters) override {
        std::vector<float*> p;
        std::vector<const float*> g;
        std::vector<std::size_t> n;
        for (Parameter* param : parameters) {
            p.push_back(param->value.data());
            g.push_back(param->grad.data());
            n.push_back(param->value.elementCount());
        }
        check(bf_hip_sgd_multi(p.data(), g.data(), n.data(), p.size(), learningRate_, nullptr));
    }
    void setLearningRate(float learningRate) override { learningRate_ = learningRate; }

    void prepareRecording(const std::vector<Parameter*>&) override {
        if (rateOnDevice_.elementCount() == 0) rateOnDevice_ = DeviceTensor::zeros({1});
    }
    void recordStep(const std::vector<Parameter*>& parameters) override {
        require(rateOnDevice_.elementCount() != 0, "SGD::recordStep: prepareRecording() has not been called");
        std::vector<float*> p;
        std::vector<const float*> g;
        std::vector<std::size_t> n;
        for (Parameter* param : parameters) {
            p.push_back(param->value.data());
            g.push_back(param->grad.data());
            n.push_back(param->value.elementCount());
        }
        check(bf_hip_sgd_multi_indirect(p.data(), g.data(), n.data(), p.size(), rateOnDevice_.data(), nullptr));
    }
    void publishStep(bf_stream_t stream) override { check(bf_hip_sgd_publish(rateOnDevice_.data(), learningRate_, stream)); }

private:
    float learningRate_;
    DeviceTensor rateOnDevice_;
};

class AdamW : public Optimizer {
public:
    explicit AdamW(float learningRate = 1e-3F, float beta1 = 0.9F, float beta2 = 0.999F, float eps = 1e-8F, float weightDecay = 0.01F)
        : learningRate_(learningRate), beta1_(beta1), beta2_(beta2), eps_(eps), weightDecay_(weightDecay) {}

    void step(const std::vector<Parameter*>& parameters) override {
        ++stepCount_;
        const Tensors t = gather(parameters);
        check(bf_hip_adamw_multi(t.p.data(), t.g.data(), t.m.data(), t.v.data(), t.n.data(), t.p.size(), static_cast<long long>(stepCount_),
                                 learningRate_, beta1_, beta2_, eps_, weightDecay_, nullptr));
    }
    void setLearningRate(float learningRate) override { learningRate_ = learningRate; }

    void prepareRecording(const std::vector<Parameter*>& parameters) override {
        (void)gather(parameters);   // the moments of every parameter exist (zero) before anything is recorded
        if (hyperOnDevice_.elementCount() == 0) hyperOnDevice_ = DeviceTensor::zeros({sizeof(bf_adamw_hyper) / sizeof(float)});
    }
    void recordStep(const std::vector<Parameter*>& parameters) override {
        require(hyperOnDevice_.elementCount() != 0, "AdamW::recordStep: prepareRecording() has not been called");
        const Tensors t = gather(parameters);
        check(bf_hip_adamw_multi_indirect(t.p.data(), t.g.data(), t.m.data(), t.v.data(), t.n.data(), t.p.size(),
                                          reinterpret_cast<const bf_adamw_hyper*>(hyperOnDevice_.data()), nullptr));
    }
    void publishStep(bf_stream_t stream) override {
        ++stepCount_;
        check(bf_hip_adamw_publish(reinterpret_cast<bf_adamw_hyper*>(hyperOnDevice_.data()), static_cast<long long>(stepCount_), learningRate_,
                                   beta1_, beta2_, eps_, weightDecay_, stream));
    }

private:
    struct MomentState {
        DeviceTensor m;
        DeviceTensor v;
    };
    struct Tensors {
        std::vector<float*> p, m, v;
        std::vector<const float*> g;
        std::vector<std::size_t> n;
    };
    Tensors gather(const std::vector<Parameter*>& parameters) {
        Tensors t;
        for (Parameter* param : parameters) {
            auto it = state_.find(param->name);
            if (it == state_.end())
                it = state_.emplace(param->name, MomentState{DeviceTensor::zeros(param->value.shape()),
                                                             DeviceTensor::zeros(param->value.shape())}).first;
            t.p.push_back(param->value.data());
            t.g.push_back(param->grad.data());
            t.m.push_back(it->second.m.data());
            t.v.push_back(it->second.v.data());
            t.n.push_back(param->value.elementCount());
        }
        return t;
    }
    DeviceTensor hyperOnDevice_;
    float learningRate_, beta1_, beta2_, eps_, weightDecay_;
    std::size_t stepCount_ = 0;
    std::unordered_map<std::string, MomentState> state_;  // per parameter name, survives between steps
};

}  // namespace blackforge::backend::hip
