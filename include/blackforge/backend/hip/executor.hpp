#pragma once
// hip::Executor: one forward pass of a model straight from its IR, with weights generated from a seed, as
// `blackforge run --device` does (include/blackforge/backend/cuda/executor.hpp:20-33, src/backend/cuda/executor.cu:
// 28-132).  Available inside a BlackForge build only: it needs the IR and the CPU backend's seeded generators, which
// are what makes the weights (and so the outputs) equal to the CPU and CUDA executors' for the same seed.
#if __has_include("blackforge/ir/module.hpp") && __has_include("blackforge/backend/cpu/random_init.hpp")
#include <cstddef>
#include <stdexcept>
#include <vector>

#include "blackforge/backend/cpu/random_init.hpp"
#include "blackforge/backend/hip/model.hpp"
#include "blackforge/ir/module.hpp"

namespace blackforge::backend::hip {

class Executor {
public:
    explicit Executor(unsigned int seed = 42) : seed_(seed) {}

    // Random tensor of the model's declared input shape with symbolic dimensions set to batchSize: token ids in
    // [0, vocab) when the first layer is an embedding, values in [-0.1, 0.1) otherwise (executor.cu:28-45).
    [[nodiscard]] runtime::Tensor makeSyntheticInput(const ir::ModelIR& model, std::size_t batchSize) const {
        const ir::Value& inputValue = model.valueById(model.inputValue);
        std::vector<std::size_t> shape;
        shape.reserve(inputValue.shape.size());
        for (const auto& dim : inputValue.shape) shape.push_back(dim.isSymbolic ? batchSize : static_cast<std::size_t>(dim.literalValue));
        const unsigned int inputSeed = cpu::seedFor(seed_, 0, 0x9E3779B1U);
        if (!model.pipelines.empty() && !model.pipelines.front().operations.empty() &&
            model.pipelines.front().operations.front().kind == ir::OpKind::Embedding) {
            const auto vocab = static_cast<std::size_t>(model.pipelines.front().operations.front().embeddingVocabSize);
            return cpu::randomTokenIdTensor(std::move(shape), vocab, inputSeed);
        }
        return cpu::randomTensor(std::move(shape), inputSeed);
    }

    // Uploads the input, walks the first pipeline on the device in fp32 and downloads the result.  The weights are the
    // ones hip::Model draws for this seed: the same per-layer seeds and salts the executors use (executor.cu:13-24,60-125).
    [[nodiscard]] runtime::Tensor run(const ir::ModelIR& model, const runtime::Tensor& input) const {
        if (model.pipelines.empty()) throw std::invalid_argument("model '" + model.name + "' has no pipeline to run");
        Model instance(model, seed_);
        return instance.forward(DeviceTensor::fromHost(input)).toHost();
    }

private:
    unsigned int seed_;
};

}  // namespace blackforge::backend::hip
#endif
