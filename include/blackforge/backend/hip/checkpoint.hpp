#pragma once
// Checkpoints of hip::Model in the BFCKPT1 format shared by the CPU and CUDA backends
// (src/backend/cpu/checkpoint.cpp:14,45-135; include/blackforge/backend/cuda/checkpoint.hpp): a file written by a
// CPU or CUDA training run loads here and the other way round.
//   "BFCKPT1\0" | u32 parameter count | per parameter: u32 name length, name bytes, u32 rank, u64 dims[rank], fp32 data
// Parameters are matched by NAME on load; a name the model does not have, a shape that differs, or a short file is
// a std::runtime_error, and parameters the file does not mention keep their values.
#include <algorithm>
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

namespace detail {

// One parameter of a checkpoint file: where its values lie, not the values.
struct CheckpointRecord {
    std::string name;
    std::vector<std::size_t> shape;
    std::size_t elementCount = 0;
    std::streamoff dataOffset = 0;
};

// The table of contents of a BFCKPT1 file.  Walks the records by seeking over their values and checks every length
// against the size of the file, so that a truncated or corrupt file is refused before anything is read into a model.
class CheckpointIndex {
public:
    explicit CheckpointIndex(const std::string& path) : path_(path), in_(path, std::ios::binary | std::ios::ate) {
        if (!in_) throw std::runtime_error("loadCheckpoint: cannot open '" + path + "'");
        fileBytes_ = static_cast<std::uint64_t>(in_.tellg());
        in_.seekg(0);
        char magic[sizeof(kCheckpointMagic)] = {};
        in_.read(magic, sizeof(magic));
        if (!in_ || std::memcmp(magic, kCheckpointMagic, sizeof(magic)) != 0)
            throw std::runtime_error("loadCheckpoint: '" + path + "' is not a BlackForge checkpoint");
        const std::uint32_t count = take<std::uint32_t>();
        records_.reserve(std::min<std::uint32_t>(count, 1U << 16));
        for (std::uint32_t i = 0; i < count; ++i) records_.push_back(nextRecord());
    }

    [[nodiscard]] const std::vector<CheckpointRecord>& records() const { return records_; }

    // The values of one record, read into `host` (resized to fit).
    void readValues(const CheckpointRecord& record, std::vector<float>& host) {
        host.resize(record.elementCount);
        in_.clear();
        in_.seekg(record.dataOffset);
        in_.read(reinterpret_cast<char*>(host.data()), static_cast<std::streamsize>(record.elementCount * sizeof(float)));
        if (!in_) corrupt();
    }

private:
    [[noreturn]] void corrupt() const { throw std::runtime_error("loadCheckpoint: '" + path_ + "' is truncated or corrupt"); }
    [[nodiscard]] std::uint64_t remaining() {
        const std::uint64_t at = static_cast<std::uint64_t>(in_.tellg());
        return at <= fileBytes_ ? fileBytes_ - at : 0;
    }
    template <typename T> T take() {
        if (remaining() < sizeof(T)) corrupt();
        return readRaw<T>(in_);
    }
    CheckpointRecord nextRecord() {
        CheckpointRecord record;
        const std::uint32_t nameLength = take<std::uint32_t>();
        if (nameLength > remaining()) corrupt();
        record.name.resize(nameLength);
        in_.read(record.name.data(), nameLength);
        const std::uint32_t rank = take<std::uint32_t>();
        if (std::uint64_t(rank) * sizeof(std::uint64_t) > remaining()) corrupt();
        record.shape.resize(rank);
        std::uint64_t elements = 1;
        for (std::size_t& extent : record.shape) {
            const std::uint64_t value = take<std::uint64_t>();
            if (value != 0 && elements > fileBytes_ / value) corrupt();   // more values than the file has bytes
            elements *= value;
            extent = static_cast<std::size_t>(value);
        }
        if (elements > remaining() / sizeof(float)) corrupt();
        record.elementCount = static_cast<std::size_t>(elements);
        record.dataOffset = in_.tellg();
        in_.seekg(static_cast<std::streamoff>(elements * sizeof(float)), std::ios::cur);
        return record;
    }

    std::string path_;
    std::ifstream in_;
    std::uint64_t fileBytes_ = 0;
    std::vector<CheckpointRecord> records_;
};

}  // namespace detail

// Loads in two phases.  First the file's table of contents is matched against the model: every record must name a
// parameter of the model with the same shape (the reference's conditions, src/backend/cpu/checkpoint.cpp:118-129), and a
// file that fails leaves the model exactly as it was.  Then the values are copied over the parameters' existing device
// buffers, so the addresses that the bf16 weight-image cache and a captured step hold stay valid.
inline void loadCheckpoint(Model& model, const std::string& path) {
    detail::CheckpointIndex index(path);
    std::unordered_map<std::string, Parameter*> byName;
    for (Parameter* p : model.parameters()) byName[p->name] = p;
    std::vector<Parameter*> targets;
    targets.reserve(index.records().size());
    for (const detail::CheckpointRecord& record : index.records()) {
        const auto found = byName.find(record.name);
        if (found == byName.end()) throw std::runtime_error("loadCheckpoint: the model has no parameter called '" + record.name + "'");
        if (found->second->value.shape() != record.shape) throw std::runtime_error("loadCheckpoint: shape mismatch for '" + record.name + "'");
        targets.push_back(found->second);
    }
    std::vector<float> staging;
    for (std::size_t i = 0; i < targets.size(); ++i) {
        const detail::CheckpointRecord& record = index.records()[i];
        if (record.elementCount == 0) continue;
        index.readValues(record, staging);
        check(bf_hip_memcpy_h2d(targets[i]->value.data(), staging.data(), record.elementCount * sizeof(float)));
    }
    invalidateBf16WeightCache();   // images of the old values must not outlive them
}

}  // namespace blackforge::backend::hip
