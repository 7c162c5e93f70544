#pragma once
// Loss functions with the reference's signatures (include/blackforge/backend/cuda/loss.hpp:7-70).
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <string>

#include "blackforge/backend/hip/device_tensor.hpp"
#include "blackforge/backend/hip/ops.hpp"

namespace blackforge::backend::hip {

struct LossResult {
    float value;
    DeviceTensor grad;  // dL/dprediction, same shape as the prediction
};

namespace detail {
inline float readScalar(const DeviceTensor& t) {
    float v = 0.0F;
    check(bf_hip_memcpy_d2h(&v, t.data(), sizeof(float)));
    return v;
}
inline void requireDense(const char* op, const DeviceTensor& logits, const DeviceTensor& target) {
    require(logits.shape() == target.shape(), std::string(op) + ": incompatible shapes on the device");
    require(logits.rank() >= 2, std::string(op) + ": needs a tensor of rank >= 2 on the device");
}
inline void requireSparse(const char* op, const DeviceTensor& logits, const DeviceTensor& idx) {
    require(logits.rank() >= 2, std::string(op) + ": needs logits of rank >= 2 on the device");
    require(idx.elementCount() == rowsOf(logits), std::string(op) + ": targetIndices does not have one entry per logits row");
}
}  // namespace detail

inline LossResult meanSquaredError(const DeviceTensor& prediction, const DeviceTensor& target) {
    require(prediction.shape() == target.shape(), "meanSquaredError: incompatible shapes on the device");
    std::size_t n = prediction.elementCount();
    LossResult r{0.0F, DeviceTensor(prediction.shape())};
    DeviceTensor sum({1});
    check(bf_hip_mse(prediction.data(), target.data(), r.grad.data(), sum.data(), n, 0, nullptr));
    if (n > 0) r.value = detail::readScalar(sum) / static_cast<float>(n);
    return r;
}

inline LossResult softmaxCrossEntropy(const DeviceTensor& logits, const DeviceTensor& target) {
    detail::requireDense("softmaxCrossEntropy", logits, target);
    std::size_t rows = detail::rowsOf(logits);
    LossResult r{0.0F, DeviceTensor(logits.shape())};
    DeviceTensor sum({1});
    check(bf_hip_cross_entropy(logits.data(), target.data(), r.grad.data(), sum.data(), rows, detail::lastDim(logits), 0, nullptr));
    if (rows > 0) r.value = detail::readScalar(sum) / static_cast<float>(rows);
    return r;
}

inline LossResult softmaxCrossEntropySparse(const DeviceTensor& logits, const DeviceTensor& targetIndices) {
    detail::requireSparse("softmaxCrossEntropySparse", logits, targetIndices);
    std::size_t rows = detail::rowsOf(logits), classes = detail::lastDim(logits);
    if (rows > 0) detail::requireIdsInRange("softmaxCrossEntropySparse", targetIndices, classes, "class index");
    LossResult r{0.0F, DeviceTensor(logits.shape())};
    DeviceTensor sum({1});
    check(bf_hip_cross_entropy_sparse(logits.data(), targetIndices.data(), r.grad.data(), sum.data(), rows, classes, 0, nullptr));
    if (rows > 0) r.value = detail::readScalar(sum) / static_cast<float>(rows);
    return r;
}

namespace detail {
// src/backend/cpu/loss.cpp:171-178: an index is -1 (row ignored) or lies in [0, classes); checked on a host copy
inline void requireMaskedIds(const char* op, const DeviceTensor& idx, std::size_t classes) {
    const runtime::Tensor host = idx.toHost();
    for (std::size_t i = 0; i < host.elementCount(); ++i) {
        const long long index = static_cast<long long>(std::lround(host.at(i)));
        require(index == -1 || (index >= 0 && static_cast<std::size_t>(index) < classes),
                std::string(op) + ": class index " + std::to_string(index) + " outside [0, " + std::to_string(classes) + ") (or -1 to ignore)");
    }
}
}  // namespace detail

// The masked-language-model loss of the CPU backend (src/backend/cpu/loss.cpp:149-215): rows whose index is -1 are
// ignored, loss and gradient are averaged over the others (value 0 and zero gradient when every row is ignored).
inline LossResult softmaxCrossEntropyMasked(const DeviceTensor& logits, const DeviceTensor& targetIndices) {
    detail::requireSparse("softmaxCrossEntropyMasked", logits, targetIndices);
    std::size_t rows = detail::rowsOf(logits), classes = detail::lastDim(logits);
    if (rows > 0) detail::requireMaskedIds("softmaxCrossEntropyMasked", targetIndices, classes);
    LossResult r{0.0F, DeviceTensor(logits.shape())};
    DeviceTensor mean({1});
    check(bf_hip_cross_entropy_masked(logits.data(), targetIndices.data(), r.grad.data(), mean.data(), rows, classes, 0, nullptr));
    r.value = detail::readScalar(mean);
    return r;
}

// "Accumulate" variants for the training loop: the gradient is returned, the SUM of this call's per-row
// (per-element for MSE) losses is added on the device to lossAccumulator (one element, owned by the
// caller); nothing is read back to the host.
// gradImage: as for softmaxCrossEntropySparseAccumulate below (rows whose length is a multiple of 8).
inline DeviceTensor meanSquaredErrorAccumulate(const DeviceTensor& prediction, const DeviceTensor& target, DeviceTensor& lossAccumulator,
                                               bool gradImage = false) {
    require(prediction.shape() == target.shape(), "meanSquaredErrorAccumulate: incompatible shapes on the device");
    DeviceTensor grad(prediction.shape());
    std::uint16_t* image = gradImage && prediction.rank() >= 1 && prediction.elementCount() > 0 &&
                                   prediction.dim(prediction.rank() - 1) % 8 == 0 ? grad.attachImage() : nullptr;
    check(bf_hip_mse_img(prediction.data(), target.data(), grad.data(), image, lossAccumulator.data(), prediction.elementCount(), 1, nullptr));
    return grad;
}

inline DeviceTensor softmaxCrossEntropyAccumulate(const DeviceTensor& logits, const DeviceTensor& target, DeviceTensor& lossAccumulator) {
    detail::requireDense("softmaxCrossEntropyAccumulate", logits, target);
    DeviceTensor grad(logits.shape());
    check(bf_hip_cross_entropy(logits.data(), target.data(), grad.data(), lossAccumulator.data(), detail::rowsOf(logits),
                               detail::lastDim(logits), 1, nullptr));
    return grad;
}

// PRECONDITION (caller's responsibility): every index already lies in [0, classes); no range check and no
// host round trip happen here.
// gradImage: the gradient also carries its bf16 image (DeviceTensor::image()) when the class count allows it (a multiple
// of 8): a model with bf16 projections feeds it to the GEMMs of its last layer without a conversion pass.
inline DeviceTensor softmaxCrossEntropySparseAccumulate(const DeviceTensor& logits, const DeviceTensor& targetIndices,
                                                         DeviceTensor& lossAccumulator, bool gradImage = false) {
    detail::requireSparse("softmaxCrossEntropySparseAccumulate", logits, targetIndices);
    DeviceTensor grad(logits.shape());
    std::uint16_t* image = gradImage && detail::lastDim(logits) % 8 == 0 && logits.elementCount() > 0 ? grad.attachImage() : nullptr;
    check(bf_hip_cross_entropy_sparse_img(logits.data(), targetIndices.data(), grad.data(), image, lossAccumulator.data(),
                                          detail::rowsOf(logits), detail::lastDim(logits), 1, nullptr));
    return grad;
}

// The loss of a bf16 language-model head, for a caller that hands the gradient to nothing but that head's backward pass
// (Model::backward with headBiasGrad): the gradient comes back as a bf16 image only (DeviceTensor::imageOnly) together
// with its column sums, the head's bias gradient; no fp32 gradient is written.  Same loss, same image, same precondition
// as softmaxCrossEntropySparseAccumulate(..., gradImage = true).  Returns false, and does nothing, for shapes the fused
// kernel does not serve (the caller then takes the ordinary route).
inline bool softmaxCrossEntropySparseHeadAccumulate(const DeviceTensor& logits, const DeviceTensor& targetIndices, DeviceTensor& lossAccumulator,
                                                    DeviceTensor& gradImageOnly, DeviceTensor& biasGrad) {
    detail::requireSparse("softmaxCrossEntropySparseAccumulate", logits, targetIndices);
    const std::size_t rows = detail::rowsOf(logits), classes = detail::lastDim(logits);
    if (rows == 0 || classes < 4096 || classes > (std::size_t(1) << 20)) return false;   // what the library serves (it says so itself otherwise)
    DeviceTensor grad = DeviceTensor::imageOnly(logits.shape());
    DeviceTensor bias({classes});
    const int status = bf_hip_cross_entropy_sparse_head(logits.data(), targetIndices.data(), const_cast<std::uint16_t*>(grad.image()), bias.data(),
                                                        lossAccumulator.data(), rows, classes, 1, nullptr);
    if (status == BF_ERR_UNSUPPORTED) return false;
    check(status);
    gradImageOnly = std::move(grad);
    biasGrad = std::move(bias);
    return true;
}

// Adds this call's MEAN over the rows that are not ignored (the value softmaxCrossEntropyMasked returns) to
// lossAccumulator; indices are the caller's precondition, as above.
inline DeviceTensor softmaxCrossEntropyMaskedAccumulate(const DeviceTensor& logits, const DeviceTensor& targetIndices,
                                                         DeviceTensor& lossAccumulator) {
    detail::requireSparse("softmaxCrossEntropyMaskedAccumulate", logits, targetIndices);
    DeviceTensor grad(logits.shape());
    check(bf_hip_cross_entropy_masked(logits.data(), targetIndices.data(), grad.data(), lossAccumulator.data(), detail::rowsOf(logits),
                                      detail::lastDim(logits), 1, nullptr));
    return grad;
}

}  // namespace blackforge::backend::hip
