#pragma once
// Per-device memory pool (reference: include/blackforge/backend/cuda/device_pool.hpp:47-54).
#include <cstddef>

#include "blackforge/backend/hip/hip_check.hpp"

namespace blackforge::backend::hip {

inline void* devicePoolAcquire(std::size_t bytes) {
    void* ptr = nullptr;
    check(bf_hip_pool_acquire(bytes, &ptr));
    return ptr;
}

inline void devicePoolRelease(void* ptr, std::size_t bytes) { check(bf_hip_pool_release(ptr, bytes)); }

}  // namespace blackforge::backend::hip
