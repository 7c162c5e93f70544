// Losses: mean squared error, dense and sparse softmax cross-entropy.
//
// HBM-bound.  Cross-entropy reads each logits row once into registers (rowcache.hpp), computes max,
// sum of exp, the row loss and the gradient from registers and writes the gradient once: 8
// algorithmic bytes per logit (12 with a dense target).  Per-row (per-block for MSE) loss terms go to
// a scratch vector that a single block then adds in a fixed order, so the reported loss is
// bit-reproducible; that block also performs the "+=" of the *Accumulate variants, so no atomics.
#include "rowcache.hpp"

namespace bf {
namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Adds `count` partial values in a fixed order and stores (or accumulates) the total.
__global__ void __launch_bounds__(1024) finishSumKernel(const float* __restrict__ partial, size_t count,
                                                        float* __restrict__ out, int accumulate) {
    __shared__ double lds[16];
    double s = 0.0;
    for (size_t i = threadIdx.x; i < count; i += blockDim.x) s += double(partial[i]);
    s = blockReduce(s, 0.0, OpSum{}, lds);
    if (threadIdx.x == 0) out[0] = accumulate ? out[0] + float(s) : float(s);
}

template <int VEC>
__global__ void __launch_bounds__(kBlock) mseKernel(const float* __restrict__ pred, const float* __restrict__ target,
                                                    float* __restrict__ grad, float* __restrict__ partial, size_t n,
                                                    float gradScale) {
    __shared__ float lds[16];
    float acc = 0.0f;
    size_t stride = size_t(gridDim.x) * blockDim.x;
    if constexpr (VEC == 4) {
        size_t n4 = n / 4;
        for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += stride) {
            float4v d = loadf4(pred + 4 * i) - loadf4(target + 4 * i);
            acc += d.x * d.x + d.y * d.y + d.z * d.z + d.w * d.w;
            storef4(grad + 4 * i, d * gradScale);
        }
        for (size_t i = n4 * 4 + size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
            float d = pred[i] - target[i];
            acc += d * d;
            grad[i] = d * gradScale;
        }
    } else {
        for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
            float d = pred[i] - target[i];
            acc += d * d;
            grad[i] = d * gradScale;
        }
    }
    acc = blockReduce(acc, 0.0f, OpSum{}, lds);
    if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}

// SPARSE: target holds one class index per row.  Otherwise a dense target row.
template <int G, int MAXE, int VEC, bool CACHED, bool SPARSE>
__global__ void __launch_bounds__(G > 256 ? G : 256) crossEntropyKernel(const float* __restrict__ logits,
                                                                         const float* __restrict__ target,
                                                                         float* __restrict__ grad, float* __restrict__ rowLoss,
                                                                         size_t rows, size_t classes, float invRows) {
    __shared__ float lds[16];
    const int t = threadIdx.x % G;
    const size_t rowsPerBlock = blockDim.x / G;
    const size_t rowStep = size_t(gridDim.x) * rowsPerBlock;
    for (size_t row = size_t(blockIdx.x) * rowsPerBlock + threadIdx.x / G; row < rows; row += rowStep) {
        const float* x = logits + row * classes;
        float* gOut = grad + row * classes;
        RowCache<G, MAXE, VEC> c;
        float mx = -INFINITY;
        if constexpr (CACHED) {
            c.load(x, classes, t, -INFINITY);
#pragma unroll
            for (int i = 0; i < MAXE; ++i) mx = fmaxf(mx, c.r[i]);
        } else {
            for (size_t e = t; e < classes; e += G) mx = fmaxf(mx, x[e]);
        }
        mx = groupMax<G>(mx, lds);
        float sum = 0.0f;
        if constexpr (CACHED) {
#pragma unroll
            for (int i = 0; i < MAXE; ++i) { c.r[i] = expf(c.r[i] - mx); sum += c.r[i]; }
        } else {
            for (size_t e = t; e < classes; e += G) sum += expf(x[e] - mx);
        }
        sum = groupSum<G>(sum, lds);
        const float inv = 1.0f / sum;

        float loss = 0.0f;  // this thread's share of the row loss
        size_t cls = 0;
        if constexpr (SPARSE) cls = size_t(lroundf(target[row]));
        auto emit = [&](float e, size_t idx) -> float {
            float p = e * inv;
            float tv;
            if constexpr (SPARSE) tv = idx == cls ? 1.0f : 0.0f;
            else tv = target[row * classes + idx];
            if (tv != 0.0f) loss += -tv * logf(fmaxf(p, 1e-12f));
            return (p - tv) * invRows;
        };
        if constexpr (CACHED) {
#pragma unroll
            for (int it = 0; it < MAXE / VEC; ++it)
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    size_t idx = RowCache<G, MAXE, VEC>::index(it, t, j);
                    if (idx < classes) c.r[it * VEC + j] = emit(c.r[it * VEC + j], idx);
                }
            c.store(gOut, classes, t);
        } else {
            for (size_t e = t; e < classes; e += G) gOut[e] = emit(expf(x[e] - mx), e);
        }
        loss = groupSum<G>(loss, lds);
        if (t == 0) rowLoss[row] = loss;
    }
}

template <bool SPARSE>
int launchCrossEntropy(const float* logits, const float* target, float* grad, float* lossSum, size_t rows,
                       size_t classes, int accumulate, hipStream_t s) {
    Scratch rowLoss(rows * sizeof(float));
    if (rowLoss.status != BF_OK) return rowLoss.status;
    float* rl = rowLoss.as<float>();
    const float invRows = 1.0f / float(rows);
    const bool vec4 = aligned16(logits) && aligned16(grad) && classes % 4 == 0;
    const unsigned cap = unsigned(computeUnits()) * 8;
#define BF_CE(G, MAXE, VEC, CACHED, threads, perBlock)                                                     \
    crossEntropyKernel<G, MAXE, VEC, CACHED, SPARSE><<<gridFor(rows, perBlock, cap), threads, 0, s>>>(      \
        logits, target, grad, rl, rows, classes, invRows)
    if (classes <= 64 * 16) { if (vec4) BF_CE(64, 16, 4, true, 256, 4); else BF_CE(64, 16, 1, true, 256, 4); }
    else if (classes <= 256 * 32) { if (vec4) BF_CE(256, 32, 4, true, 256, 1); else BF_CE(256, 32, 1, true, 256, 1); }
    else if (classes <= 1024 * 64) { if (vec4) BF_CE(1024, 64, 4, true, 1024, 1); else BF_CE(1024, 64, 1, true, 1024, 1); }
    else BF_CE(1024, 4, 1, false, 1024, 1);
#undef BF_CE
    BF_LAUNCH_CHECK();
    finishSumKernel<<<1, 1024, 0, s>>>(rl, rows, lossSum, accumulate);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" {

int bf_hip_mse(const float* pred, const float* target, float* grad, float* lossSum, size_t n, int accumulate,
               bf_stream_t stream) {
    BF_REQUIRE(lossSum != nullptr, "lossSum is NULL");
    hipStream_t s = asStream(stream);
    if (n == 0) {
        if (!accumulate) return bf_hip_fill_zero(lossSum, sizeof(float), stream);
        return BF_OK;
    }
    BF_REQUIRE(pred && target && grad, "NULL pointer");
    unsigned grid = gridFor(n, size_t(kBlock) * 8, unsigned(computeUnits()) * 8);
    Scratch partial(grid * sizeof(float));
    if (partial.status != BF_OK) return partial.status;
    float gradScale = 2.0f / float(n);
    if (aligned16(pred) && aligned16(target) && aligned16(grad))
        mseKernel<4><<<grid, kBlock, 0, s>>>(pred, target, grad, partial.as<float>(), n, gradScale);
    else
        mseKernel<1><<<grid, kBlock, 0, s>>>(pred, target, grad, partial.as<float>(), n, gradScale);
    BF_LAUNCH_CHECK();
    finishSumKernel<<<1, 1024, 0, s>>>(partial.as<float>(), grid, lossSum, accumulate);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_cross_entropy(const float* logits, const float* target, float* grad, float* lossSum, size_t rows,
                         size_t classes, int accumulate, bf_stream_t stream) {
    BF_REQUIRE(lossSum != nullptr, "lossSum is NULL");
    if (rows == 0 || classes == 0) {
        if (!accumulate) return bf_hip_fill_zero(lossSum, sizeof(float), stream);
        return BF_OK;
    }
    BF_REQUIRE(logits && target && grad, "NULL pointer");
    return launchCrossEntropy<false>(logits, target, grad, lossSum, rows, classes, accumulate, asStream(stream));
}

int bf_hip_cross_entropy_sparse(const float* logits, const float* targetIdx, float* grad, float* lossSum,
                                size_t rows, size_t classes, int accumulate, bf_stream_t stream) {
    BF_REQUIRE(lossSum != nullptr, "lossSum is NULL");
    if (rows == 0 || classes == 0) {
        if (!accumulate) return bf_hip_fill_zero(lossSum, sizeof(float), stream);
        return BF_OK;
    }
    BF_REQUIRE(logits && targetIdx && grad, "NULL pointer");
    return launchCrossEntropy<true>(logits, targetIdx, grad, lossSum, rows, classes, accumulate, asStream(stream));
}

}  // extern "C"
