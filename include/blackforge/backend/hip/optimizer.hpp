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
};

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

private:
    float learningRate_;
};

class AdamW : public Optimizer {
public:
    explicit AdamW(float learningRate = 1e-3F, float beta1 = 0.9F, float beta2 = 0.999F, float eps = 1e-8F, float weightDecay = 0.01F)
        : learningRate_(learningRate), beta1_(beta1), beta2_(beta2), eps_(eps), weightDecay_(weightDecay) {}

    void step(const std::vector<Parameter*>& parameters) override {
        ++stepCount_;
        std::vector<float*> p, m, v;
        std::vector<const float*> g;
        std::vector<std::size_t> n;
        for (Parameter* param : parameters) {
            auto it = state_.find(param->name);
            if (it == state_.end())
                it = state_.emplace(param->name, MomentState{DeviceTensor::zeros(param->value.shape()),
                                                             DeviceTensor::zeros(param->value.shape())}).first;
            p.push_back(param->value.data());
            g.push_back(param->grad.data());
            m.push_back(it->second.m.data());
            v.push_back(it->second.v.data());
            n.push_back(param->value.elementCount());
        }
        check(bf_hip_adamw_multi(p.data(), g.data(), m.data(), v.data(), n.data(), p.size(), static_cast<long long>(stepCount_),
                                 learningRate_, beta1_, beta2_, eps_, weightDecay_, nullptr));
    }
    void setLearningRate(float learningRate) override { learningRate_ = learningRate; }

private:
    struct MomentState {
        DeviceTensor m;
        DeviceTensor v;
    };
    float learningRate_, beta1_, beta2_, eps_, weightDecay_;
    std::size_t stepCount_ = 0;
    std::unordered_map<std::string, MomentState> state_;  // per parameter name, survives between steps
};

}  // namespace blackforge::backend::hip
