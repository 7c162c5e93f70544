#pragma once
// RAII float32 device buffer with the reference's interface
// (include/blackforge/backend/cuda/device_tensor.hpp:19-75): move-only, fromHost/toHost/zeros/clone,
// reshaped() && transfers ownership.  Memory comes from the library's per-device pool.
#include <cstddef>
#include <cstdint>
#include <utility>
#include <vector>

#include "blackforge/backend/hip/device_pool.hpp"
#include "blackforge/backend/hip/host_tensor.hpp"

namespace blackforge::backend::hip {

class DeviceTensor {
public:
    DeviceTensor() = default;

    explicit DeviceTensor(std::vector<std::size_t> shape) : shape_(std::move(shape)) {
        data_ = static_cast<float*>(devicePoolAcquire(elementCount() * sizeof(float)));
    }

    ~DeviceTensor() { release(); }

    DeviceTensor(const DeviceTensor&) = delete;
    DeviceTensor& operator=(const DeviceTensor&) = delete;

    DeviceTensor(DeviceTensor&& other) noexcept
        : data_(other.data_), shape_(std::move(other.shape_)), owns_(other.owns_), image_(other.image_), imageBytes_(other.imageBytes_) {
        other.data_ = nullptr;
        other.shape_.clear();
        other.image_ = nullptr;
        other.imageBytes_ = 0;
    }
    DeviceTensor& operator=(DeviceTensor&& other) noexcept {
        if (this != &other) {
            release();   // the old buffer goes back to the pool, not to the driver
            data_ = other.data_;
            shape_ = std::move(other.shape_);
            owns_ = other.owns_;
            image_ = other.image_;
            imageBytes_ = other.imageBytes_;
            other.data_ = nullptr;
            other.shape_.clear();
            other.image_ = nullptr;
            other.imageBytes_ = 0;
        }
        return *this;
    }

    // A bf16 image of the same values (round to nearest even, same row-major layout, two bytes per element), for tensors
    // whose readers include bf16 GEMMs: the kernel that produces the tensor writes the image in the same pass, and the
    // GEMM entry points take it in place of a conversion pass of their own.  attachImage() gives the tensor an (unwritten)
    // image buffer from the pool; it travels with the tensor through moves and reshaped() and is returned with it.  Only
    // for tensors that are not modified after the producing call.  Not part of the reference's DeviceTensor.
    [[nodiscard]] std::uint16_t* attachImage() {
        releaseImage();
        // rows of the last dimension rounded up to 8 elements (16 bytes), the row pitch of every bf16 operand image
        const std::size_t cols = shape_.empty() ? 0 : shape_.back();
        const std::size_t rows = cols != 0 ? elementCount() / cols : 0;
        imageBytes_ = rows * ((cols + 7) / 8 * 8) * sizeof(std::uint16_t);
        image_ = static_cast<std::uint16_t*>(devicePoolAcquire(imageBytes_));
        return image_;
    }
    [[nodiscard]] const std::uint16_t* image() const { return image_; }

    // A non-owning view of device memory that belongs to someone else (an application buffer handed in
    // through a C interface): usable wherever a const DeviceTensor& is expected, never returned to the pool.
    static DeviceTensor borrow(const float* data, std::vector<std::size_t> shape) {
        DeviceTensor t;
        t.data_ = const_cast<float*>(data);
        t.shape_ = std::move(shape);
        t.owns_ = false;
        return t;
    }

    // A tensor that exists as its bf16 image only (data() is NULL): for a value whose readers are all bf16 GEMMs, written
    // by a producer that never forms the fp32 copy.  Only functions documented to accept one may be handed it.
    static DeviceTensor imageOnly(std::vector<std::size_t> shape) {
        DeviceTensor t;
        t.shape_ = std::move(shape);
        t.owns_ = false;
        (void)t.attachImage();
        return t;
    }

    static DeviceTensor fromHost(const runtime::Tensor& host) {
        DeviceTensor t(host.shape());
        check(bf_hip_memcpy_h2d(t.data_, host.data().data(), t.elementCount() * sizeof(float)));
        return t;
    }

    static DeviceTensor zeros(std::vector<std::size_t> shape) {
        DeviceTensor t(std::move(shape));
        check(bf_hip_fill_zero(t.data_, t.elementCount() * sizeof(float), nullptr));
        return t;
    }

    [[nodiscard]] runtime::Tensor toHost() const {
        std::vector<float> host(elementCount());
        check(bf_hip_memcpy_d2h(host.data(), data_, host.size() * sizeof(float)));
        return runtime::Tensor(shape_, std::move(host));
    }

    [[nodiscard]] DeviceTensor clone() const {
        DeviceTensor t(shape_);
        check(bf_hip_memcpy_d2d(t.data_, data_, elementCount() * sizeof(float), nullptr));
        return t;
    }

    [[nodiscard]] DeviceTensor reshaped(std::vector<std::size_t> newShape) && {
        std::size_t n = 1;
        for (std::size_t d : newShape) n *= d;
        require(n == elementCount(), "DeviceTensor::reshaped: the element count must not change");
        DeviceTensor t;
        t.data_ = data_;
        t.shape_ = std::move(newShape);
        t.owns_ = owns_;
        t.image_ = image_;
        t.imageBytes_ = imageBytes_;
        data_ = nullptr;
        shape_.clear();
        image_ = nullptr;
        imageBytes_ = 0;
        return t;
    }

    [[nodiscard]] float* data() { return data_; }
    [[nodiscard]] const float* data() const { return data_; }
    [[nodiscard]] const std::vector<std::size_t>& shape() const { return shape_; }
    [[nodiscard]] std::size_t rank() const { return shape_.size(); }
    [[nodiscard]] std::size_t dim(std::size_t axis) const { return shape_.at(axis); }
    [[nodiscard]] std::size_t elementCount() const {
        if (shape_.empty()) return 0;
        std::size_t n = 1;
        for (std::size_t d : shape_) n *= d;
        return n;
    }

private:
    void releaseImage() noexcept {
        if (image_ != nullptr) bf_hip_pool_release(image_, imageBytes_);
        image_ = nullptr;
        imageBytes_ = 0;
    }
    void release() noexcept {
        if (data_ != nullptr && owns_) bf_hip_pool_release(data_, elementCount() * sizeof(float));
        data_ = nullptr;
        releaseImage();
    }

    float* data_ = nullptr;
    std::vector<std::size_t> shape_;
    bool owns_ = true;
    std::uint16_t* image_ = nullptr;
    std::size_t imageBytes_ = 0;
};

}  // namespace blackforge::backend::hip
