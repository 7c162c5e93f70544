#pragma once
// Host-side tensor used by fromHost()/toHost().  Inside a BlackForge build the project's own
// blackforge::runtime::Tensor (include/blackforge/runtime/tensor.hpp:18-48) is picked up; a stand-alone
// build of this backend gets a minimal class with the same constructor and accessors.
#if __has_include("blackforge/runtime/tensor.hpp")
#include "blackforge/runtime/tensor.hpp"
#else
#include <cstddef>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace blackforge::runtime {

class Tensor {
public:
    Tensor() = default;
    Tensor(std::vector<std::size_t> shape, std::vector<float> data) : shape_(std::move(shape)), data_(std::move(data)) {
        if (data_.size() != countOf(shape_)) throw std::invalid_argument("Tensor: data size does not match shape");
    }
    static Tensor zeros(std::vector<std::size_t> shape) {
        std::size_t n = countOf(shape);
        return Tensor(std::move(shape), std::vector<float>(n, 0.0F));
    }
    [[nodiscard]] const std::vector<std::size_t>& shape() const { return shape_; }
    [[nodiscard]] std::size_t rank() const { return shape_.size(); }
    [[nodiscard]] std::size_t dim(std::size_t axis) const { return shape_.at(axis); }
    [[nodiscard]] std::size_t elementCount() const { return data_.size(); }
    [[nodiscard]] const std::vector<float>& data() const { return data_; }
    [[nodiscard]] std::vector<float>& data() { return data_; }
    [[nodiscard]] float at(std::size_t i) const { return data_.at(i); }
    float& at(std::size_t i) { return data_.at(i); }

private:
    static std::size_t countOf(const std::vector<std::size_t>& shape) {
        std::size_t n = 1;
        for (std::size_t d : shape) n *= d;
        return n;
    }
    std::vector<std::size_t> shape_;
    std::vector<float> data_;
};

}  // namespace blackforge::runtime
#endif
