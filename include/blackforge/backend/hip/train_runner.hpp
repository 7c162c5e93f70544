#pragma once
// hip::runTraining: the training loop of the CUDA backend's train runner (src/backend/cuda/train_runner.cu:73-259)
// on this backend: forward, loss, backward and optimizer step on the device; the dataset and the checkpoints stay on
// the host and reach the device batch by batch.  Per epoch: shuffle with the epoch number as seed, optional cosine
// learning rate (backend/lr_schedule.hpp:7-15), floor(examples / batch) steps of zeroGrad, forward, loss, backward,
// optimizer; the loss of an epoch is summed on the device and read once per epoch.  Token ids and class indices are
// validated on the host copy of the batch before the upload, so the device path runs without host round trips.
//
// Two entry points: one over a plain TrainOptions struct (any build), and, inside a BlackForge build where the
// front end's headers exist, the reference signature over ast::Program / ir::Module.
#include <cmath>
#include <memory>
#include <optional>
#include <ostream>
#include <stdexcept>
#include <string>
#include <vector>

#include "blackforge/backend/hip/captured_step.hpp"
#include "blackforge/backend/hip/checkpoint.hpp"
#include "blackforge/backend/hip/dataset.hpp"
#include "blackforge/backend/hip/loss.hpp"
#include "blackforge/backend/hip/model.hpp"
#include "blackforge/backend/hip/optimizer.hpp"

namespace blackforge::backend::hip {

struct TrainRunResult {
    std::string modelName;
    std::vector<double> epochLosses;   // mean loss per epoch, in order
};

struct TrainOptions {
    std::string loss = "mse";          // "mse", "cross_entropy", "cross_entropy_sparse", "cross_entropy_masked"
    std::string optimizer = "adamw";   // "sgd", anything else = AdamW with the reference defaults (train_runner.cu:168-173)
    long long epochs = 1;
    std::size_t batchSize = 1;
    double learningRate = 1e-3;
    bool cosineSchedule = false;
    std::string fromCheckpointPath;    // loaded over the model's values before the first step when non-empty
    std::string saveCheckpointPath;    // written after the last epoch when non-empty
};

// cosineAnnealingLearningRate (include/blackforge/backend/lr_schedule.hpp:7-15)
inline float cosineAnnealingLearningRate(long long epoch, long long totalEpochs, float baseLearningRate) {
    if (totalEpochs <= 1) return baseLearningRate;
    constexpr double kPi = 3.14159265358979323846;
    const double progress = static_cast<double>(epoch - 1) / static_cast<double>(totalEpochs - 1);
    return static_cast<float>(baseLearningRate * 0.5 * (1.0 + std::cos(kPi * progress)));
}

namespace detail {
// train_runner.cu:60-69: every element, rounded like the device kernels round it, must lie in [0, bound)
inline void validateHostIndexRange(const runtime::Tensor& host, std::size_t bound, const char* label) {
    for (std::size_t i = 0; i < host.elementCount(); ++i) {
        const long long index = static_cast<long long>(std::lround(host.at(i)));
        if (index < 0 || static_cast<std::size_t>(index) >= bound) {
            throw std::invalid_argument(std::string(label) + ": index " + std::to_string(index) + " outside [0, " + std::to_string(bound) + ")");
        }
    }
}
// src/backend/cpu/loss.cpp:171-178: -1 marks a row to ignore, every other index must lie in [0, bound)
inline void validateHostMaskedIndexRange(const runtime::Tensor& host, std::size_t bound, const char* label) {
    for (std::size_t i = 0; i < host.elementCount(); ++i) {
        const long long index = static_cast<long long>(std::lround(host.at(i)));
        if (index != -1 && (index < 0 || static_cast<std::size_t>(index) >= bound)) {
            throw std::invalid_argument(std::string(label) + ": class index " + std::to_string(index) + " outside [0, " + std::to_string(bound) +
                                        ") (or -1 to ignore)");
        }
    }
}
}  // namespace detail

// DatasetT: HostDataset, or blackforge::data::Dataset inside a BlackForge build (same batch/shuffle/numExamples members).
template <typename DatasetT>
TrainRunResult runTraining(Model& model, DatasetT& dataset, const TrainOptions& options, std::ostream* progressOutput = nullptr) {
    const bool sparse = options.loss == "cross_entropy_sparse", dense = options.loss == "cross_entropy";
    const bool maskedLoss = options.loss == "cross_entropy_masked";   // cpu/train_runner.cpp:132-133; the CUDA runner has no such loss
    const std::optional<std::size_t> vocab = model.firstLayerEmbeddingVocabSize();
    if (!options.fromCheckpointPath.empty()) {
        loadCheckpoint(model, options.fromCheckpointPath);
        if (progressOutput != nullptr) *progressOutput << "Weights loaded from '" << options.fromCheckpointPath << "' (fine-tuning)\n";
    }
    std::unique_ptr<Optimizer> optimizer;
    if (options.optimizer == "sgd") optimizer = std::make_unique<SGD>(static_cast<float>(options.learningRate));
    else optimizer = std::make_unique<AdamW>(static_cast<float>(options.learningRate));
    if (options.batchSize == 0 || dataset.numExamples() < options.batchSize) {
        throw std::runtime_error("the dataset has " + std::to_string(dataset.numExamples()) + " examples, fewer than the requested batch_size (" +
                                 std::to_string(options.batchSize) + ")");
    }
    const std::size_t batchesPerEpoch = dataset.numExamples() / options.batchSize;
    if (progressOutput != nullptr) {
        *progressOutput << "HIP training of '" << model.name() << "' on " << dataset.numExamples() << " examples (" << batchesPerEpoch
                        << " batches/epoch, batch_size=" << options.batchSize << ", loss=" << options.loss << ", optimizer=" << options.optimizer
                        << ", learning_rate=" << options.learningRate << (options.cosineSchedule ? " (schedule: cosine)" : "") << ")\n";
    }
    TrainRunResult result;
    result.modelName = model.name();
    for (long long epoch = 1; epoch <= options.epochs; ++epoch) {
        dataset.shuffle(static_cast<unsigned int>(epoch));
        if (options.cosineSchedule) {
            optimizer->setLearningRate(cosineAnnealingLearningRate(epoch, options.epochs, static_cast<float>(options.learningRate)));
        }
        DeviceTensor lossAccumulator = DeviceTensor::zeros({1});
        std::size_t lossDivisor = 0;
        // only the optimizer changes weights inside the loop; after its step it brings their bf16 images up to date
        bool weightImagesCurrent = false;
        for (std::size_t b = 0; b < batchesPerEpoch; ++b) {
            auto batch = dataset.batch(b * options.batchSize, options.batchSize);
            if (vocab.has_value()) detail::validateHostIndexRange(batch.input, *vocab, "embeddingLookup");
            DeviceTensor input = DeviceTensor::fromHost(batch.input);
            model.zeroGrad(/*deferred=*/true);
            DeviceTensor output = model.forward(input, vocab.has_value(), weightImagesCurrent);
            if (sparse) detail::validateHostIndexRange(batch.target, output.shape().back(), "softmaxCrossEntropySparse");
            if (maskedLoss) detail::validateHostMaskedIndexRange(batch.target, output.shape().back(), "softmaxCrossEntropyMasked");
            DeviceTensor target = DeviceTensor::fromHost(batch.target);
            // the masked loss adds each batch's MEAN (its divisor, the rows not ignored, differs from batch to batch),
            // so the epoch's figure is the mean of the batch means, as in cpu/train_runner.cpp:184-194
            lossDivisor += maskedLoss ? 1 : (sparse || dense) ? output.elementCount() / output.shape().back() : output.elementCount();
            lossAndBackward(model, sparse ? "cross_entropy_sparse" : maskedLoss ? "cross_entropy_masked" : dense ? "cross_entropy" : "mse", output,
                            target, lossAccumulator, vocab.has_value());
            const std::vector<Parameter*> parameters = model.parameters();
            optimizer->step(parameters);
            if (model.usesBf16()) {
                refreshWeightImages(parameters);
                weightImagesCurrent = true;
            }
        }
        const float lossSum = lossAccumulator.toHost().at(0);
        const double avgLoss = static_cast<double>(lossSum) / static_cast<double>(lossDivisor);
        result.epochLosses.push_back(avgLoss);
        if (progressOutput != nullptr) *progressOutput << "  epoch " << epoch << "/" << options.epochs << "  loss=" << avgLoss << "\n";
    }
    if (!options.saveCheckpointPath.empty()) {
        saveCheckpoint(model, options.saveCheckpointPath);
        if (progressOutput != nullptr) *progressOutput << "Weights saved to '" << options.saveCheckpointPath << "'\n";
    }
    return result;
}

}  // namespace blackforge::backend::hip

#if __has_include("blackforge/ast/ast.hpp") && __has_include("blackforge/ir/module.hpp") && __has_include("blackforge/data/dataset.hpp")
#include <variant>

#include "blackforge/ast/ast.hpp"
#include "blackforge/data/dataset.hpp"
#include "blackforge/ir/module.hpp"

namespace blackforge::backend::hip {

// The reference signature (include/blackforge/backend/cuda/train_runner.hpp:38-40): reads the first `train` block of
// the program, builds the model from the IR with seed 42 and the module's precision policy, loads the dataset the
// block names, and runs the loop above.  Like the CUDA runner it refuses a `lora` block rather than falling back.
inline TrainRunResult runTraining(const ast::Program& program, const ir::Module& module, const std::string& fromCheckpointPath,
                                  const std::string& saveCheckpointPath, std::ostream* progressOutput = nullptr) {
    const ast::TrainDecl* train = nullptr;
    for (const auto& decl : program.declarations)
        if (std::holds_alternative<ast::TrainDecl>(decl)) { train = &std::get<ast::TrainDecl>(decl); break; }
    if (train == nullptr) throw std::runtime_error("the program has no 'train' block");
    auto field = [&](auto tag) -> const decltype(tag)* {
        for (const auto& f : train->fields)
            if (std::holds_alternative<decltype(tag)>(f)) return &std::get<decltype(tag)>(f);
        return nullptr;
    };
    const auto* modelField = field(ast::TrainModelField{});
    const auto* datasetField = field(ast::TrainDatasetField{});
    const auto* lossField = field(ast::TrainLossField{});
    const auto* optimizerField = field(ast::TrainOptimizerField{});
    const auto* epochsField = field(ast::TrainEpochsField{});
    const auto* batchField = field(ast::TrainBatchSizeField{});
    const auto* lrField = field(ast::TrainLearningRateField{});
    if (!modelField || !datasetField || !lossField || !optimizerField || !epochsField || !batchField) {
        throw std::runtime_error("the 'train' block is incomplete (model/dataset/loss/optimizer/epochs/batch_size)");
    }
    if (field(ast::TrainLoraField{}) != nullptr) throw std::runtime_error("'train --device hip' does not support 'lora'; use '--device cpu'");
    const ir::ModelIR* modelIR = nullptr;
    for (const auto& m : module.models)
        if (m.name == modelField->name) modelIR = &m;
    if (modelIR == nullptr) throw std::runtime_error("model '" + modelField->name + "' not found in the IR");
    const ast::DatasetPathField* path = nullptr;
    for (const auto& decl : program.declarations) {
        if (!std::holds_alternative<ast::DatasetDecl>(decl)) continue;
        const auto& d = std::get<ast::DatasetDecl>(decl);
        if (d.name != datasetField->name) continue;
        for (const auto& f : d.fields)
            if (std::holds_alternative<ast::DatasetPathField>(f)) path = &std::get<ast::DatasetPathField>(f);
    }
    if (path == nullptr) throw std::runtime_error("dataset '" + datasetField->name + "' not found or without a 'path'");
    data::Dataset dataset = data::loadDataset(path->path);
    Model model(*modelIR, /*seed=*/42, module.precision);
    TrainOptions options;
    options.loss = lossField->name;
    options.optimizer = optimizerField->name;
    options.epochs = epochsField->value;
    options.batchSize = static_cast<std::size_t>(batchField->value);
    options.learningRate = lrField ? lrField->value : 1e-3;
    options.cosineSchedule = field(ast::TrainLrScheduleField{}) != nullptr;
    options.fromCheckpointPath = fromCheckpointPath;
    options.saveCheckpointPath = saveCheckpointPath;
    return runTraining(model, dataset, options, progressOutput);
}

}  // namespace blackforge::backend::hip
#endif
