// Multi-tensor optimizers: SGD and AdamW over every parameter in one launch.
//
// HBM-bound: AdamW moves 28 algorithmic bytes per parameter (read p, g, m, v; write p, m, v), SGD 12.
// The host cuts every tensor into chunks of 8192 elements and launches one block per chunk, so the
// grid is balanced however unequal the tensors are (the embedding table next to a bias vector); the
// chunk table lives in device memory and is re-uploaded only when the parameter set changes.
#include "common.hpp"

#include <cmath>
#include <vector>

namespace bf {
namespace {

constexpr size_t kChunk = size_t(kBlock) * 32;

struct SgdChunk {
    float* p;
    const float* g;
    unsigned count;
    unsigned pad;
};
struct AdamChunk {
    float* p;
    const float* g;
    float* m;
    float* v;
    unsigned count;
    unsigned pad;
};

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

__global__ void __launch_bounds__(kBlock) sgdKernel(const SgdChunk* __restrict__ chunks, float lr) {
    SgdChunk c = chunks[blockIdx.x];
    bool vec = ((reinterpret_cast<uintptr_t>(c.p) | reinterpret_cast<uintptr_t>(c.g)) & 15u) == 0;
    unsigned done = 0;
    if (vec) {
        unsigned n4 = c.count / 4;
        for (unsigned i = threadIdx.x; i < n4; i += blockDim.x)
            storef4(c.p + 4 * i, loadf4(c.p + 4 * i) - loadf4(c.g + 4 * i) * lr);
        done = n4 * 4;
    }
    for (unsigned i = done + threadIdx.x; i < c.count; i += blockDim.x) c.p[i] -= lr * c.g[i];
}

struct AdamParams {
    float lr, beta1, beta2, eps, weightDecay, bias1, bias2;
};

__device__ __forceinline__ void adamOne(float& p, float g, float& m, float& v, const AdamParams& a) {
    m = a.beta1 * m + (1.0f - a.beta1) * g;
    v = a.beta2 * v + (1.0f - a.beta2) * g * g;
    float mHat = m / a.bias1;
    float vHat = v / a.bias2;
    p -= a.lr * (mHat / (sqrtf(vHat) + a.eps) + a.weightDecay * p);
}

__global__ void __launch_bounds__(kBlock) adamwKernel(const AdamChunk* __restrict__ chunks, AdamParams a) {
    AdamChunk c = chunks[blockIdx.x];
    bool vec = ((reinterpret_cast<uintptr_t>(c.p) | reinterpret_cast<uintptr_t>(c.g) | reinterpret_cast<uintptr_t>(c.m) |
                 reinterpret_cast<uintptr_t>(c.v)) & 15u) == 0;
    unsigned done = 0;
    if (vec) {
        unsigned n4 = c.count / 4;
        for (unsigned i = threadIdx.x; i < n4; i += blockDim.x) {
            float4v p = loadf4(c.p + 4 * i), g = loadf4(c.g + 4 * i), m = loadf4(c.m + 4 * i), v = loadf4(c.v + 4 * i);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float pj = p[j], mj = m[j], vj = v[j];
                adamOne(pj, g[j], mj, vj, a);
                p[j] = pj; m[j] = mj; v[j] = vj;
            }
            storef4(c.p + 4 * i, p);
            storef4(c.m + 4 * i, m);
            storef4(c.v + 4 * i, v);
        }
        done = n4 * 4;
    }
    for (unsigned i = done + threadIdx.x; i < c.count; i += blockDim.x) adamOne(c.p[i], c.g[i], c.m[i], c.v[i], a);
}

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" {

int bf_hip_sgd_multi(float* const* params, const float* const* grads, const size_t* counts, size_t numTensors, float lr,
                     bf_stream_t stream) {
    if (numTensors == 0) return BF_OK;
    BF_REQUIRE(params && grads && counts, "NULL pointer");
    std::vector<SgdChunk> chunks;
    for (size_t t = 0; t < numTensors; ++t) {
        BF_REQUIRE((params[t] && grads[t]) || counts[t] == 0, "NULL tensor pointer");
        for (size_t off = 0; off < counts[t]; off += kChunk) {
            size_t c = counts[t] - off < kChunk ? counts[t] - off : kChunk;
            chunks.push_back(SgdChunk{params[t] + off, grads[t] + off, unsigned(c), 0});
        }
    }
    if (chunks.empty()) return BF_OK;
    const void* table = nullptr;
    int st = uploadDescriptorTable(kSlotSgd, chunks.data(), chunks.size() * sizeof(SgdChunk), asStream(stream), &table);
    if (st != BF_OK) return st;
    sgdKernel<<<unsigned(chunks.size()), kBlock, 0, asStream(stream)>>>(static_cast<const SgdChunk*>(table), lr);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_adamw_multi(float* const* params, const float* const* grads, float* const* m, float* const* v,
                       const size_t* counts, size_t numTensors, long long step, float lr, float beta1, float beta2,
                       float eps, float weightDecay, bf_stream_t stream) {
    BF_REQUIRE(step >= 1, "step must be >= 1");
    if (numTensors == 0) return BF_OK;
    BF_REQUIRE(params && grads && m && v && counts, "NULL pointer");
    std::vector<AdamChunk> chunks;
    for (size_t t = 0; t < numTensors; ++t) {
        BF_REQUIRE((params[t] && grads[t] && m[t] && v[t]) || counts[t] == 0, "NULL tensor pointer");
        for (size_t off = 0; off < counts[t]; off += kChunk) {
            size_t c = counts[t] - off < kChunk ? counts[t] - off : kChunk;
            chunks.push_back(AdamChunk{params[t] + off, grads[t] + off, m[t] + off, v[t] + off, unsigned(c), 0});
        }
    }
    if (chunks.empty()) return BF_OK;
    const void* table = nullptr;
    int st = uploadDescriptorTable(kSlotAdamW, chunks.data(), chunks.size() * sizeof(AdamChunk), asStream(stream), &table);
    if (st != BF_OK) return st;
    // bias corrections on the host in float, exactly like the reference (optimizer.cu:104-107)
    float t = static_cast<float>(step);
    AdamParams a{lr, beta1, beta2, eps, weightDecay, 1.0f - std::pow(beta1, t), 1.0f - std::pow(beta2, t)};
    adamwKernel<<<unsigned(chunks.size()), kBlock, 0, asStream(stream)>>>(static_cast<const AdamChunk*>(table), a);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

}  // extern "C"
