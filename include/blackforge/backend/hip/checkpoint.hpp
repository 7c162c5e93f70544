#pragma once
// Checkpoints of hip::Model in the BFCKPT1 format shared by the CPU and CUDA backends
// (src/backend/cpu/checkpoint.cpp:14,45-135; include/blackforge/backend/cuda/checkpoint.hpp): a file written by a
// CPU or CUDA training run loads here and the other way round.
//   "BFCKPT1\0" | u32 parameter count | per parameter: u32 name length, name bytes, u32 rank, u64 dims[rank], fp32 data
// Parameters are matched by NAME on load; a name the model does not have, a shape that differs, or a short file is
// a std::runtime_error, and parameters the file does not mention keep their values.
#include <cerrno>
#include <cstdint>
#include <cstring>
#include <fstream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "blackforge/backend/hip/model.hpp"

namespace blackforge::backend::hip {

namespace detail {
inline constexpr char kCheckpointMagic[8] = {'B', 'F', 'C', 'K', 'P', 'T', '1', '\0'};
template <typename T> void writeRaw(std::ostream& out, T value) { out.write(reinterpret_cast<const char*>(&value), sizeof(value)); }
template <typename T> T readRaw(std::istream& in) {
    T value{};
    in.read(reinterpret_cast<char*>(&value), sizeof(value));
    return value;
}
}  // namespace detail

inline void saveCheckpoint(Model& model, const std::string& path) {
    std::ofstream out(path, std::ios::binary | std::ios::trunc);
    if (!out) {
        throw std::runtime_error("saveCheckpoint: cannot write '" + path + "' (errno=" + std::to_string(errno) + " " + std::strerror(errno) + ")");
    }
    out.write(detail::kCheckpointMagic, sizeof(detail::kCheckpointMagic));
    std::vector<Parameter*> params = model.parameters();
    detail::writeRaw<std::uint32_t>(out, static_cast<std::uint32_t>(params.size()));
    for (const Parameter* p : params) {
        detail::writeRaw<std::uint32_t>(out, static_cast<std::uint32_t>(p->name.size()));
        out.write(p->name.data(), static_cast<std::streamsize>(p->name.size()));
        const std::vector<std::size_t>& shape = p->value.shape();
        detail::writeRaw<std::uint32_t>(out, static_cast<std::uint32_t>(shape.size()));
        for (std::size_t d : shape) detail::writeRaw<std::uint64_t>(out, static_cast<std::uint64_t>(d));
        runtime::Tensor host = p->value.toHost();   // one blocking device-to-host copy per parameter
        out.write(reinterpret_cast<const char*>(host.data().data()), static_cast<std::streamsize>(host.data().size() * sizeof(float)));
    }
    if (!out) throw std::runtime_error("saveCheckpoint: write to '" + path + "' failed");
}

inline void loadCheckpoint(Model& model, const std::string& path) {
    std::ifstream in(path, std::ios::binary);
    if (!in) throw std::runtime_error("loadCheckpoint: cannot open '" + path + "'");
    char magic[8];
    in.read(magic, sizeof(magic));
    if (!in || std::memcmp(magic, detail::kCheckpointMagic, sizeof(magic)) != 0) {
        throw std::runtime_error("loadCheckpoint: '" + path + "' is not a BlackForge checkpoint");
    }
    std::unordered_map<std::string, Parameter*> byName;
    for (Parameter* p : model.parameters()) byName[p->name] = p;
    const std::uint32_t count = detail::readRaw<std::uint32_t>(in);
    for (std::uint32_t i = 0; i < count; ++i) {
        const std::uint32_t nameLength = detail::readRaw<std::uint32_t>(in);
        if (!in || nameLength > (1U << 20)) throw std::runtime_error("loadCheckpoint: '" + path + "' is truncated or corrupt");
        std::string name(nameLength, '\0');
        in.read(name.data(), nameLength);
        const std::uint32_t rank = detail::readRaw<std::uint32_t>(in);
        if (!in || rank > 16) throw std::runtime_error("loadCheckpoint: '" + path + "' is truncated or corrupt");
        std::vector<std::size_t> shape(rank);
        std::size_t elementCount = 1;
        for (std::uint32_t d = 0; d < rank; ++d) {
            shape[d] = static_cast<std::size_t>(detail::readRaw<std::uint64_t>(in));
            elementCount *= shape[d];
        }
        auto it = byName.find(name);
        if (!in) throw std::runtime_error("loadCheckpoint: '" + path + "' is truncated or corrupt");
        if (it == byName.end()) throw std::runtime_error("loadCheckpoint: the model has no parameter called '" + name + "'");
        if (it->second->value.shape() != shape) throw std::runtime_error("loadCheckpoint: shape mismatch for '" + name + "'");
        std::vector<float> data(elementCount);
        in.read(reinterpret_cast<char*>(data.data()), static_cast<std::streamsize>(elementCount * sizeof(float)));
        if (!in) throw std::runtime_error("loadCheckpoint: '" + path + "' is truncated or corrupt");
        it->second->value = DeviceTensor::fromHost(runtime::Tensor(shape, std::move(data)));
    }
    // the next Model::forward() refreshes the bf16 weight images, as after an optimizer step
}

}  // namespace blackforge::backend::hip
