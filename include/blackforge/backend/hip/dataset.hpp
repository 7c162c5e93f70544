#pragma once
// Host-side training data for the stand-alone build of this backend: the BFDATA1 file format and the
// batch / shuffle behaviour of blackforge::data::Dataset (include/blackforge/data/dataset.hpp:23-52,
// src/data/dataset.cpp:14,76-184).  Inside a BlackForge build the project's own class is used instead (the train
// runner is a template over the dataset type).
//   "BFDATA1\0" | u32 examples | input shape (u32 rank, u64 dims) | target shape | fp32 inputs | fp32 targets
#include <cstdint>
#include <cstring>
#include <fstream>
#include <numeric>
#include <random>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "blackforge/backend/hip/host_tensor.hpp"

namespace blackforge::backend::hip {

class HostDataset {
public:
    struct Batch {
        runtime::Tensor input;
        runtime::Tensor target;
    };

    HostDataset(std::vector<std::size_t> inputExampleShape, std::vector<std::size_t> targetExampleShape, std::vector<float> inputs,
                std::vector<float> targets, std::size_t numExamples)
        : inputShape_(std::move(inputExampleShape)), targetShape_(std::move(targetExampleShape)), inputs_(std::move(inputs)),
          targets_(std::move(targets)), numExamples_(numExamples) {
        if (inputs_.size() != numExamples_ * product(inputShape_)) throw std::invalid_argument("Dataset: input data does not match numExamples * shape");
        if (targets_.size() != numExamples_ * product(targetShape_)) throw std::invalid_argument("Dataset: target data does not match numExamples * shape");
    }

    [[nodiscard]] std::size_t numExamples() const { return numExamples_; }
    [[nodiscard]] const std::vector<std::size_t>& inputExampleShape() const { return inputShape_; }
    [[nodiscard]] const std::vector<std::size_t>& targetExampleShape() const { return targetShape_; }

    // Examples startIndex .. startIndex+batchSize-1, wrapping around the end (dataset.cpp:76-100).
    [[nodiscard]] Batch batch(std::size_t startIndex, std::size_t batchSize) const {
        if (numExamples_ == 0) throw std::invalid_argument("Dataset::batch: the dataset holds no examples");
        const std::size_t inSize = product(inputShape_), tgSize = product(targetShape_);
        std::vector<float> in(batchSize * inSize), tg(batchSize * tgSize);
        for (std::size_t i = 0; i < batchSize; ++i) {
            const std::size_t e = (startIndex + i) % numExamples_;
            std::copy_n(inputs_.begin() + static_cast<std::ptrdiff_t>(e * inSize), inSize, in.begin() + static_cast<std::ptrdiff_t>(i * inSize));
            std::copy_n(targets_.begin() + static_cast<std::ptrdiff_t>(e * tgSize), tgSize, tg.begin() + static_cast<std::ptrdiff_t>(i * tgSize));
        }
        std::vector<std::size_t> inShape{batchSize}, tgShape{batchSize};
        inShape.insert(inShape.end(), inputShape_.begin(), inputShape_.end());
        tgShape.insert(tgShape.end(), targetShape_.begin(), targetShape_.end());
        return Batch{runtime::Tensor(std::move(inShape), std::move(in)), runtime::Tensor(std::move(tgShape), std::move(tg))};
    }

    // The same permutation as data::Dataset::shuffle(seed) (dataset.cpp:102-131) when built against the same C++
    // standard library: std::mt19937 seeded with `seed`, Fisher-Yates from the last position down with one
    // std::uniform_int_distribution<std::size_t>(0, i) draw per position.
    void shuffle(unsigned int seed) {
        if (numExamples_ <= 1) return;
        std::vector<std::size_t> order(numExamples_);
        std::iota(order.begin(), order.end(), std::size_t{0});
        std::mt19937 rng(seed);
        for (std::size_t i = numExamples_ - 1; i > 0; --i) {
            std::uniform_int_distribution<std::size_t> pick(0, i);
            std::swap(order[i], order[pick(rng)]);
        }
        const std::size_t inSize = product(inputShape_), tgSize = product(targetShape_);
        std::vector<float> in(inputs_.size()), tg(targets_.size());
        for (std::size_t i = 0; i < numExamples_; ++i) {
            std::copy_n(inputs_.begin() + static_cast<std::ptrdiff_t>(order[i] * inSize), inSize, in.begin() + static_cast<std::ptrdiff_t>(i * inSize));
            std::copy_n(targets_.begin() + static_cast<std::ptrdiff_t>(order[i] * tgSize), tgSize, tg.begin() + static_cast<std::ptrdiff_t>(i * tgSize));
        }
        inputs_ = std::move(in);
        targets_ = std::move(tg);
    }

    static HostDataset load(const std::string& path) {
        std::ifstream in(path, std::ios::binary);
        if (!in) throw std::runtime_error("loadDataset: cannot open '" + path + "'");
        char magic[8];
        in.read(magic, sizeof(magic));
        static constexpr char kMagic[8] = {'B', 'F', 'D', 'A', 'T', 'A', '1', '\0'};
        if (!in || std::memcmp(magic, kMagic, sizeof(magic)) != 0) throw std::runtime_error("loadDataset: '" + path + "' is not a BlackForge dataset");
        std::uint32_t numExamples = 0;
        in.read(reinterpret_cast<char*>(&numExamples), sizeof(numExamples));
        std::vector<std::size_t> inShape = readShape(in), tgShape = readShape(in);
        if (!in) throw std::runtime_error("loadDataset: '" + path + "' is truncated or corrupt");
        std::vector<float> inputs(static_cast<std::size_t>(numExamples) * product(inShape));
        std::vector<float> targets(static_cast<std::size_t>(numExamples) * product(tgShape));
        in.read(reinterpret_cast<char*>(inputs.data()), static_cast<std::streamsize>(inputs.size() * sizeof(float)));
        in.read(reinterpret_cast<char*>(targets.data()), static_cast<std::streamsize>(targets.size() * sizeof(float)));
        if (!in) throw std::runtime_error("loadDataset: '" + path + "' is truncated or corrupt");
        return HostDataset(std::move(inShape), std::move(tgShape), std::move(inputs), std::move(targets), numExamples);
    }

private:
    static std::size_t product(const std::vector<std::size_t>& shape) {
        std::size_t n = 1;
        for (std::size_t d : shape) n *= d;
        return n;
    }
    static std::vector<std::size_t> readShape(std::istream& in) {
        std::uint32_t rank = 0;
        in.read(reinterpret_cast<char*>(&rank), sizeof(rank));
        if (!in || rank > 16) return {};
        std::vector<std::size_t> shape(rank);
        for (std::uint32_t i = 0; i < rank; ++i) {
            std::uint64_t d = 0;
            in.read(reinterpret_cast<char*>(&d), sizeof(d));
            shape[i] = static_cast<std::size_t>(d);
        }
        return shape;
    }

    std::vector<std::size_t> inputShape_, targetShape_;
    std::vector<float> inputs_, targets_;
    std::size_t numExamples_ = 0;
};

}  // namespace blackforge::backend::hip
