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

// lrDevice: when not NULL the learning rate is read from there (a launch recorded in a graph must not freeze it)
template <bool NT>
__global__ void __launch_bounds__(kBlock) sgdKernel(const SgdTensor* __restrict__ table, int numTensors, float lr,
                                                    const float* __restrict__ lrDevice) {
    if (lrDevice) lr = *lrDevice;
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

__global__ void publishHyperKernel(AdamParams* dst, AdamParams value) { *dst = value; }
__global__ void publishFloatKernel(float* dst, float value) { *dst = value; }

// hyper: when not NULL the hyper-parameters and bias corrections are read from there
template <bool NT>
__global__ void __launch_bounds__(kBlock) adamwKernel(const AdamTensor* __restrict__ table, int numTensors, AdamParams a,
                                                      const AdamParams* __restrict__ hyper) {
    if (hyper) a = *hyper;
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

static int sgdMulti(float* const* params, const float* const* grads, const size_t* counts, size_t numTensors, float lr,
                    const float* lrDevice, bf_stream_t stream) {
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
    if (streamsPastCache(blocks * kPerBlock * 12)) sgdKernel<true><<<unsigned(blocks), kBlock, 0, asStream(stream)>>>(static_cast<const SgdTensor*>(device), int(numTensors), lr, lrDevice);
    else sgdKernel<false><<<unsigned(blocks), kBlock, 0, asStream(stream)>>>(static_cast<const SgdTensor*>(device), int(numTensors), lr, lrDevice);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

static int adamwMulti(float* const* params, const float* const* grads, float* const* m, float* const* v, const size_t* counts,
                      size_t numTensors, const AdamParams& byValue, const AdamParams* hyperDevice, bf_stream_t stream) {
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
    if (streamsPastCache(blocks * kPerBlock * 28)) adamwKernel<true><<<unsigned(blocks), kBlock, 0, asStream(stream)>>>(static_cast<const AdamTensor*>(device), int(numTensors), byValue, hyperDevice);
    else adamwKernel<false><<<unsigned(blocks), kBlock, 0, asStream(stream)>>>(static_cast<const AdamTensor*>(device), int(numTensors), byValue, hyperDevice);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

// bias corrections on the host in float, exactly like the reference (optimizer.cu:104-107)
static AdamParams adamParams(long long step, float lr, float beta1, float beta2, float eps, float weightDecay) {
    const float t = static_cast<float>(step);
    return AdamParams{lr, beta1, beta2, eps, weightDecay, 1.0f - std::pow(beta1, t), 1.0f - std::pow(beta2, t)};
}

int bf_hip_sgd_multi(float* const* params, const float* const* grads, const size_t* counts, size_t numTensors, float lr,
                     bf_stream_t stream) {
    return sgdMulti(params, grads, counts, numTensors, lr, nullptr, stream);
}

int bf_hip_sgd_multi_indirect(float* const* params, const float* const* grads, const size_t* counts, size_t numTensors,
                              const float* lrDevice, bf_stream_t stream) {
    BF_REQUIRE(lrDevice != nullptr, "lrDevice is NULL");
    return sgdMulti(params, grads, counts, numTensors, 0.0f, lrDevice, stream);
}

int bf_hip_sgd_publish(float* lrDevice, float lr, bf_stream_t stream) {
    BF_REQUIRE(lrDevice != nullptr, "lrDevice is NULL");
    publishFloatKernel<<<1, 1, 0, asStream(stream)>>>(lrDevice, lr);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_adamw_multi(float* const* params, const float* const* grads, float* const* m, float* const* v,
                       const size_t* counts, size_t numTensors, long long step, float lr, float beta1, float beta2,
                       float eps, float weightDecay, bf_stream_t stream) {
    BF_REQUIRE(step >= 1, "step must be >= 1");
    return adamwMulti(params, grads, m, v, counts, numTensors, adamParams(step, lr, beta1, beta2, eps, weightDecay), nullptr, stream);
}

int bf_hip_adamw_multi_indirect(float* const* params, const float* const* grads, float* const* m, float* const* v,
                                const size_t* counts, size_t numTensors, const bf_adamw_hyper* hyperDevice, bf_stream_t stream) {
    BF_REQUIRE(hyperDevice != nullptr, "hyperDevice is NULL");
    static_assert(sizeof(bf_adamw_hyper) == sizeof(AdamParams), "the public block and the kernel's must match");
    return adamwMulti(params, grads, m, v, counts, numTensors, AdamParams{}, reinterpret_cast<const AdamParams*>(hyperDevice), stream);
}

int bf_hip_adamw_publish(bf_adamw_hyper* hyperDevice, long long step, float lr, float beta1, float beta2, float eps,
                         float weightDecay, bf_stream_t stream) {
    BF_REQUIRE(hyperDevice != nullptr, "hyperDevice is NULL");
    BF_REQUIRE(step >= 1, "step must be >= 1");
    publishHyperKernel<<<1, 1, 0, asStream(stream)>>>(reinterpret_cast<AdamParams*>(hyperDevice), adamParams(step, lr, beta1, beta2, eps, weightDecay));
    BF_LAUNCH_CHECK();
    return BF_OK;
}

}  // extern "C"
