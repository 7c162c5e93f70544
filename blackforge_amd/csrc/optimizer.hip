// Multi-tensor optimizers: SGD and AdamW over every parameter in one launch.
//
// HBM-bound: AdamW moves 28 algorithmic bytes per parameter (read p, g, m, v; write p, m, v), SGD 12.
// The launch is one flat grid over all tensors laid end to end: a block owns 1024 consecutive elements of
// one tensor (one 16-byte group per thread), finds its tensor by binary search in a small table of first
// block indices, and touches its elements once.  The grid is balanced however unequal the tensors are (the
// embedding table next to a bias vector) and walks every tensor in address order; the table (one entry per
// tensor) lives in device memory and is re-uploaded only when the parameter set changes.
#include "common.hpp"

#include <cmath>
#include <vector>

namespace bf {
namespace {

constexpr size_t kPerBlock = size_t(kBlock) * 4;

struct SgdTensor {
    float* p;
    const float* g;
    size_t count;
    unsigned firstBlock;
    unsigned pad;
};
struct AdamTensor {
    float* p;
    const float* g;
    float* m;
    float* v;
    size_t count;
    unsigned firstBlock;
    unsigned pad;
};

template <bool NT>
__global__ void __launch_bounds__(kBlock) sgdKernel(const SgdTensor* __restrict__ table, int numTensors, float lr) {
    const SgdTensor c = table[owningTensor(table, numTensors, blockIdx.x)];
    const size_t base = (size_t(blockIdx.x - c.firstBlock) * kBlock + threadIdx.x) * 4;
    if (base >= c.count) return;
    const bool vec = ((reinterpret_cast<uintptr_t>(c.p) | reinterpret_cast<uintptr_t>(c.g)) & 15u) == 0 && base + 4 <= c.count;
    if (vec) {
        stf4<NT>(c.p + base, ldf4<NT>(c.p + base) - ldf4<NT>(c.g + base) * lr);
    } else {
        for (size_t i = base; i < base + 4 && i < c.count; ++i) c.p[i] -= lr * c.g[i];
    }
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

template <bool NT>
__global__ void __launch_bounds__(kBlock) adamwKernel(const AdamTensor* __restrict__ table, int numTensors, AdamParams a) {
    const AdamTensor c = table[owningTensor(table, numTensors, blockIdx.x)];
    const size_t base = (size_t(blockIdx.x - c.firstBlock) * kBlock + threadIdx.x) * 4;
    if (base >= c.count) return;
    const bool vec = ((reinterpret_cast<uintptr_t>(c.p) | reinterpret_cast<uintptr_t>(c.g) | reinterpret_cast<uintptr_t>(c.m) |
                       reinterpret_cast<uintptr_t>(c.v)) & 15u) == 0 && base + 4 <= c.count;
    if (vec) {
        float4v p = ldf4<NT>(c.p + base), g = ldf4<NT>(c.g + base), m = ldf4<NT>(c.m + base), v = ldf4<NT>(c.v + base);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float pj = p[j], mj = m[j], vj = v[j];
            adamOne(pj, g[j], mj, vj, a);
            p[j] = pj; m[j] = mj; v[j] = vj;
        }
        stf4<NT>(c.p + base, p);
        stf4<NT>(c.m + base, m);
        stf4<NT>(c.v + base, v);
    } else {
        for (size_t i = base; i < base + 4 && i < c.count; ++i) adamOne(c.p[i], c.g[i], c.m[i], c.v[i], a);
    }
}

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" {

int bf_hip_sgd_multi(float* const* params, const float* const* grads, const size_t* counts, size_t numTensors, float lr,
                     bf_stream_t stream) {
    if (numTensors == 0) return BF_OK;
    BF_REQUIRE(params && grads && counts, "NULL pointer");
    std::vector<SgdTensor> table;
    size_t blocks = 0;
    for (size_t t = 0; t < numTensors; ++t) {
        BF_REQUIRE((params[t] && grads[t]) || counts[t] == 0, "NULL tensor pointer");
        table.push_back(SgdTensor{params[t], grads[t], counts[t], unsigned(blocks), 0});
        blocks += (counts[t] + kPerBlock - 1) / kPerBlock;
        BF_REQUIRE(blocks < (size_t(1) << 31), "too many elements for one launch");
    }
    if (blocks == 0) return BF_OK;
    const void* device = nullptr;
    int st = uploadDescriptorTable(kSlotSgd, table.data(), table.size() * sizeof(SgdTensor), asStream(stream), &device);
    if (st != BF_OK) return st;
    if (streamsPastCache(blocks * kPerBlock * 12)) sgdKernel<true><<<unsigned(blocks), kBlock, 0, asStream(stream)>>>(static_cast<const SgdTensor*>(device), int(numTensors), lr);
    else sgdKernel<false><<<unsigned(blocks), kBlock, 0, asStream(stream)>>>(static_cast<const SgdTensor*>(device), int(numTensors), lr);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_adamw_multi(float* const* params, const float* const* grads, float* const* m, float* const* v,
                       const size_t* counts, size_t numTensors, long long step, float lr, float beta1, float beta2,
                       float eps, float weightDecay, bf_stream_t stream) {
    BF_REQUIRE(step >= 1, "step must be >= 1");
    if (numTensors == 0) return BF_OK;
    BF_REQUIRE(params && grads && m && v && counts, "NULL pointer");
    std::vector<AdamTensor> table;
    size_t blocks = 0;
    for (size_t t = 0; t < numTensors; ++t) {
        BF_REQUIRE((params[t] && grads[t] && m[t] && v[t]) || counts[t] == 0, "NULL tensor pointer");
        table.push_back(AdamTensor{params[t], grads[t], m[t], v[t], counts[t], unsigned(blocks), 0});
        blocks += (counts[t] + kPerBlock - 1) / kPerBlock;
        BF_REQUIRE(blocks < (size_t(1) << 31), "too many elements for one launch");
    }
    if (blocks == 0) return BF_OK;
    const void* device = nullptr;
    int st = uploadDescriptorTable(kSlotAdamW, table.data(), table.size() * sizeof(AdamTensor), asStream(stream), &device);
    if (st != BF_OK) return st;
    // bias corrections on the host in float, exactly like the reference (optimizer.cu:104-107)
    float t = static_cast<float>(step);
    AdamParams a{lr, beta1, beta2, eps, weightDecay, 1.0f - std::pow(beta1, t), 1.0f - std::pow(beta2, t)};
    if (streamsPastCache(blocks * kPerBlock * 28)) adamwKernel<true><<<unsigned(blocks), kBlock, 0, asStream(stream)>>>(static_cast<const AdamTensor*>(device), int(numTensors), a);
    else adamwKernel<false><<<unsigned(blocks), kBlock, 0, asStream(stream)>>>(static_cast<const AdamTensor*>(device), int(numTensors), a);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

}  // extern "C"
