#pragma once
// Device enumeration and selection (reference: include/blackforge/backend/cuda/device_query.hpp:21,33).
#include <string>
#include <vector>

#include "blackforge/backend/hip/hip_check.hpp"

namespace blackforge::backend::hip {

struct HipDeviceInfo {
    int index;
    std::string name;
    std::string arch;
    int computeUnits;
    std::size_t totalMemoryBytes;
};

// Empty when no driver or device is present (never throws for that), like the reference.
inline std::vector<HipDeviceInfo> enumerateDevices() {
    int count = 0;
    if (bf_hip_device_count(&count) != BF_OK) return {};
    std::vector<HipDeviceInfo> devices;
    for (int i = 0; i < count; ++i) {
        bf_device_props p{};
        if (bf_hip_device_props(i, &p) != BF_OK) continue;
        devices.push_back(HipDeviceInfo{i, p.name, p.arch, p.compute_units, p.total_memory});
    }
    return devices;
}

// Throws std::invalid_argument for an index that does not exist.
inline void setActiveDevice(int index) { check(bf_hip_set_device(index)); }

}  // namespace blackforge::backend::hip
