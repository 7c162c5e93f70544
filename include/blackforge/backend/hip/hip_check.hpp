#pragma once
// Maps C-ABI status codes to the exception types the reference GPU backend throws
// (reference: include/blackforge/backend/cuda/cuda_check.hpp:14-53): shape/range problems are
// std::invalid_argument, runtime failures std::runtime_error carrying the library's message.
#include <stdexcept>
#include <string>

#include "bf_hip.h"

namespace blackforge::backend::hip {

inline void check(int status) {
    if (status == BF_OK) return;
    std::string message = bf_hip_last_error();
    if (status == BF_ERR_INVALID_ARGUMENT) throw std::invalid_argument(message);
    throw std::runtime_error(message);
}

inline void require(bool condition, const std::string& message) {
    if (!condition) throw std::invalid_argument(message);
}

}  // namespace blackforge::backend::hip
