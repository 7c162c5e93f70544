// Row-wise ops: rmsnorm, softmax and their backward passes.
//
// HBM-bound: 8 algorithmic bytes per element forward, 12 backward.  Each row is read once into
// registers (see rowcache.hpp), reduced with wavefront shuffles (rows up to 1024 features: one
// 64-lane wavefront per row, four rows per block) or one LDS exchange per reduction (longer rows),
// and written once.
#include "rowcache.hpp"

namespace bf {
namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }


// Visits the row either from the register cache or (CACHED == false) from global memory.
template <int G, int MAXE, int VEC, bool CACHED, bool NT = false>
struct Row {
    RowCache<G, MAXE, VEC, NT> c;
    const float* p;
    size_t n;
    int t;
    __device__ void open(const float* row, size_t features, int thread, float fill) {
        p = row; n = features; t = thread;
        if constexpr (CACHED) c.load(row, features, thread, fill);
    }
    // f(value) over every element including padding (padding holds `fill`): for reductions
    template <typename F> __device__ void reduce(F&& f) const {
        if constexpr (CACHED) {
#pragma unroll
            for (int i = 0; i < MAXE; ++i) f(c.r[i]);
        } else {
            for (size_t e = t; e < n; e += G) f(p[e]);
        }
    }
    // f(value, element index) over valid elements only
    template <typename F> __device__ void each(F&& f) const {
        if constexpr (CACHED) {
#pragma unroll
            for (int it = 0; it < MAXE / VEC; ++it)
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    size_t e = RowCache<G, MAXE, VEC, NT>::index(it, t, j);
                    if (e < n) f(c.r[it * VEC + j], e);
                }
        } else {
            for (size_t e = t; e < n; e += G) f(p[e], e);
        }
    }
    // out[e] = f(value, e), vectorised when cached
    template <typename F> __device__ void map(float* __restrict__ out, F&& f) {
        if constexpr (CACHED) {
#pragma unroll
            for (int it = 0; it < MAXE / VEC; ++it)
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    size_t e = RowCache<G, MAXE, VEC, NT>::index(it, t, j);
                    c.r[it * VEC + j] = f(c.r[it * VEC + j], e);
                }
            c.store(out, n, t);
        } else {
            for (size_t e = t; e < n; e += G) out[e] = f(p[e], e);
        }
    }
};

#define BF_ROW_PROLOGUE()                                                            \
    __shared__ float lds[16];                                                        \
    __shared__ double ldsD[16];                                                      \
    (void)lds; (void)ldsD;                                                           \
    const int t = threadIdx.x % G;                                                   \
    const size_t rowsPerBlock = blockDim.x / G;                                      \
    const size_t rowStep = size_t(gridDim.x) * rowsPerBlock;                         \
    const size_t firstRow = size_t(blockIdx.x) * rowsPerBlock + threadIdx.x / G;

// When a whole block shares a row (G > 64) every thread must take part in the LDS reductions, so
// the row loop is uniform across the block: rowsPerBlock == 1 there.

template <int G, int MAXE, int VEC, bool CACHED, bool NT = false>
__global__ void __launch_bounds__(G > 256 ? G : 256) rmsnormKernel(const float* __restrict__ x, float* __restrict__ out,
                                                                    unsigned short* __restrict__ image, size_t rows, size_t features) {
    BF_ROW_PROLOGUE();
    for (size_t row = firstRow; row < rows; row += rowStep) {
        Row<G, MAXE, VEC, CACHED, NT> rx;
        rx.open(x + row * features, features, t, 0.0f);
        // sum of squares in double and x / rms in float, as the reference does (ops.cpp:264-275)
        double ss = 0.0;
        rx.reduce([&](float v) { ss += double(v) * double(v); });
        ss = groupSum<G>(ss, ldsD);
        float rms = float(sqrt(ss / double(features) + double(kRmsNormEps)));
        // either output may be absent: the fp32 row, and its bf16 image for a consumer that is a bf16 GEMM
        if constexpr (CACHED) {
#pragma unroll
            for (int i = 0; i < MAXE; ++i) rx.c.r[i] = rx.c.r[i] / rms;
            if (out) rx.c.store(out + row * features, features, t);
            if (image) rx.c.storeBf16(image + row * features, features, t);
        } else {
            for (size_t e = t; e < features; e += G) {
                const float v = rx.p[e] / rms;
                if (out) out[row * features + e] = v;
                if (image) image[row * features + e] = toBf16Bits(v);
            }
        }
    }
}

template <int G, int MAXE, int VEC, bool CACHED, bool NT = false>
__global__ void __launch_bounds__(G > 256 ? G : 256) rmsnormBackwardKernel(const float* __restrict__ x, const float* __restrict__ g,
                                                                            const float* __restrict__ addend, float* __restrict__ out,
                                                                            unsigned short* __restrict__ outImage, size_t rows,
                                                                            size_t features) {
    BF_ROW_PROLOGUE();
    for (size_t row = firstRow; row < rows; row += rowStep) {
        Row<G, MAXE, VEC, CACHED, NT> rx, rg;
        rx.open(x + row * features, features, t, 0.0f);
        rg.open(g + row * features, features, t, 0.0f);
        // double sums and a double final formula, as the reference does (autodiff.cpp:212-229): the two
        // terms cancel almost completely for short rows, which float arithmetic cannot resolve
        double ss = 0.0, gx = 0.0;
        if constexpr (CACHED) {
#pragma unroll
            for (int i = 0; i < MAXE; ++i) { double xv = rx.c.r[i]; ss += xv * xv; gx += double(rg.c.r[i]) * xv; }
        } else {
            for (size_t e = t; e < features; e += G) { double xv = rx.p[e]; ss += xv * xv; gx += double(rg.p[e]) * xv; }
        }
        ss = groupSum<G>(ss, ldsD);
        gx = groupSum<G>(gx, ldsD);
        const double r = sqrt(ss / double(features) + double(kRmsNormEps));
        const double invR = 1.0 / r;
        const double k = gx / (double(features) * r * r * r);
        float* o = out + row * features;
        if constexpr (CACHED) {
            if (features >= 64) {   // cancellation between the two terms is at most 1/features of either: float is enough
                const float invRf = float(invR), kf = float(k);
#pragma unroll
                for (int i = 0; i < MAXE; ++i) rg.c.r[i] = rg.c.r[i] * invRf - rx.c.r[i] * kf;
            } else {
#pragma unroll
                for (int i = 0; i < MAXE; ++i) rg.c.r[i] = float(double(rg.c.r[i]) * invR - double(rx.c.r[i]) * k);
            }
            if (addend) {   // the gradient that bypassed the normalisation (a residual connection) joins here
                rx.open(addend + row * features, features, t, 0.0f);
#pragma unroll
                for (int i = 0; i < MAXE; ++i) rg.c.r[i] += rx.c.r[i];
            }
            rg.c.store(o, features, t);
            if (outImage) rg.c.storeBf16(outImage + row * features, features, t);
        } else {
            const float* a = addend ? addend + row * features : nullptr;
            for (size_t e = t; e < features; e += G) {
                float v = float(double(rg.p[e]) * invR - double(rx.p[e]) * k);
                if (a) v += a[e];
                o[e] = v;
                if (outImage) outImage[row * features + e] = toBf16Bits(v);
            }
        }
    }
}

template <int G, int MAXE, int VEC, bool CACHED, bool NT = false>
__global__ void __launch_bounds__(G > 256 ? G : 256) softmaxKernel(const float* __restrict__ x, float* __restrict__ out,
                                                                    size_t rows, size_t features) {
    BF_ROW_PROLOGUE();
    for (size_t row = firstRow; row < rows; row += rowStep) {
        Row<G, MAXE, VEC, CACHED, NT> rx;
        rx.open(x + row * features, features, t, -INFINITY);
        float mx = -INFINITY;
        rx.reduce([&](float v) { mx = fmaxf(mx, v); });
        mx = groupMax<G>(mx, lds);
        float sum = 0.0f;
        if constexpr (CACHED) {
#pragma unroll
            for (int i = 0; i < MAXE; ++i) { rx.c.r[i] = expf(rx.c.r[i] - mx); sum += rx.c.r[i]; }
        } else {
            for (size_t e = t; e < features; e += G) sum += expf(rx.p[e] - mx);
        }
        sum = groupSum<G>(sum, lds);
        float inv = 1.0f / sum;
        float* o = out + row * features;
        if constexpr (CACHED) {
#pragma unroll
            for (int i = 0; i < MAXE; ++i) rx.c.r[i] *= inv;
            rx.c.store(o, features, t);
        } else {
            for (size_t e = t; e < features; e += G) o[e] = expf(rx.p[e] - mx) * inv;
        }
    }
}

// dx = y * (g - sum(g*y)) with y = softmax(x) recomputed in registers.
template <int G, int MAXE, int VEC, bool CACHED, bool NT = false>
__global__ void __launch_bounds__(G > 256 ? G : 256) softmaxBackwardKernel(const float* __restrict__ x, const float* __restrict__ g,
                                                                            float* __restrict__ out, size_t rows, size_t features) {
    BF_ROW_PROLOGUE();
    for (size_t row = firstRow; row < rows; row += rowStep) {
        Row<G, MAXE, VEC, CACHED, NT> rx, rg;
        rx.open(x + row * features, features, t, -INFINITY);
        rg.open(g + row * features, features, t, 0.0f);
        float mx = -INFINITY;
        rx.reduce([&](float v) { mx = fmaxf(mx, v); });
        mx = groupMax<G>(mx, lds);
        float sum = 0.0f, gy = 0.0f;
        if constexpr (CACHED) {
#pragma unroll
            for (int i = 0; i < MAXE; ++i) { rx.c.r[i] = expf(rx.c.r[i] - mx); sum += rx.c.r[i]; gy += rg.c.r[i] * rx.c.r[i]; }
        } else {
            for (size_t e = t; e < features; e += G) { float ev = expf(rx.p[e] - mx); sum += ev; gy += rg.p[e] * ev; }
        }
        sum = groupSum<G>(sum, lds);
        gy = groupSum<G>(gy, lds);
        float inv = 1.0f / sum;
        float dot = gy * inv;  // sum_j g_j y_j
        float* o = out + row * features;
        if constexpr (CACHED) {
#pragma unroll
            for (int i = 0; i < MAXE; ++i) rg.c.r[i] = rx.c.r[i] * inv * (rg.c.r[i] - dot);
            rg.c.store(o, features, t);
        } else {
            for (size_t e = t; e < features; e += G) o[e] = expf(rx.p[e] - mx) * inv * (rg.p[e] - dot);
        }
    }
}

// Picks the instantiation for a row length: the smallest group (64, 256 or 1024 threads per row) and the
// smallest per-thread register count whose product holds the row, so short rows carry no padding work and
// no variant spills.  Two-input kernels get half the registers per input at 1024 threads (16 waves per CU
// leave 128 VGPRs each).  Every block takes its rows once: the grid covers all rows, which keeps the HBM
// access stream in address order.
#define BF_ROW_CASE(KERNEL, G, MAXE, limitRows)                                                                    \
    if ((features_) <= size_t(G) * MAXE) {                                                                         \
        const unsigned threads = G > 256 ? G : 256;                                                                \
        const unsigned grid = gridFor(rows_, threads / G);                                                         \
        if (vec4 && nt_) KERNEL<G, MAXE, 4, true, true><<<grid, threads, 0, stream_>>>(ARGS_);                      \
        else if (vec4) KERNEL<G, MAXE, 4, true><<<grid, threads, 0, stream_>>>(ARGS_);                             \
        else KERNEL<G, MAXE, 1, true><<<grid, threads, 0, stream_>>>(ARGS_);                                       \
        break;                                                                                                     \
    }
#define BF_ROW_LAUNCH(KERNEL, TWO_INPUTS, vecOk, rows, features, stream, ...)                                      \
    do {                                                                                                           \
        const size_t rows_ = (rows), features_ = (features);                                                       \
        hipStream_t stream_ = (stream);                                                                            \
        const bool vec4 = (vecOk) && features_ % 4 == 0;                                                           \
        const bool nt_ = !(TWO_INPUTS) && streamsPastCache(rows_ * features_ * 8);   /* measured: no gain with two inputs */ \
        BF_ROW_CASE(KERNEL, 64, 4, 0)                                                                              \
        BF_ROW_CASE(KERNEL, 64, 8, 0)                                                                              \
        BF_ROW_CASE(KERNEL, 64, 16, 0)                                                                             \
        BF_ROW_CASE(KERNEL, 256, 8, 0)                                                                             \
        BF_ROW_CASE(KERNEL, 256, 16, 0)                                                                            \
        BF_ROW_CASE(KERNEL, 256, 32, 0)                                                                            \
        BF_ROW_CASE(KERNEL, 1024, 16, 0)                                                                           \
        if (!(TWO_INPUTS)) {                                                                                       \
            BF_ROW_CASE(KERNEL, 1024, 32, 0)                                                                       \
            if (vec4) { BF_ROW_CASE(KERNEL, 1024, 52, 0) }                                                         \
        }                                                                                                          \
        KERNEL<1024, 4, 1, false><<<gridFor(rows_, 1), 1024, 0, stream_>>>(ARGS_);                                 \
    } while (0)

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" {

int bf_hip_rmsnorm_img(const float* x, float* out, uint16_t* image, size_t rows, size_t features, bf_stream_t stream) {
    if (rows == 0 || features == 0) return BF_OK;
    BF_REQUIRE(x && (out || image), "NULL pointer");
    BF_REQUIRE(image == nullptr || features % 8 == 0, "the bf16 image needs a feature count that is a multiple of 8");
    hipStream_t s = asStream(stream);
#define ARGS_ x, out, image, rows, features
    BF_ROW_LAUNCH(rmsnormKernel, false, aligned16(x) && aligned16(out) && aligned16(image), rows, features, s, x, out, image, rows, features);
#undef ARGS_
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_rmsnorm(const float* x, float* out, size_t rows, size_t features, bf_stream_t stream) {
    if (rows == 0 || features == 0) return BF_OK;
    BF_REQUIRE(x && out, "NULL pointer");
    return bf_hip_rmsnorm_img(x, out, nullptr, rows, features, stream);
}

int bf_hip_rmsnorm_backward_add_img(const float* x, const float* g, const float* addend, float* out, uint16_t* outImage, size_t rows,
                                    size_t features, bf_stream_t stream) {
    if (rows == 0 || features == 0) return BF_OK;
    BF_REQUIRE(x && g && out, "NULL pointer");
    BF_REQUIRE(addend != out, "the output must not be the addend");
    BF_REQUIRE(outImage == nullptr || features % 8 == 0, "the bf16 image needs a feature count that is a multiple of 8");
    hipStream_t s = asStream(stream);
#define ARGS_ x, g, addend, out, outImage, rows, features
    BF_ROW_LAUNCH(rmsnormBackwardKernel, true, aligned16(x) && aligned16(g) && aligned16(out) && aligned16(addend) && aligned16(outImage), rows,
                  features, s, x, g, addend, out, outImage, rows, features);
#undef ARGS_
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_rmsnorm_backward_add(const float* x, const float* g, const float* addend, float* out, size_t rows, size_t features,
                                bf_stream_t stream) {
    return bf_hip_rmsnorm_backward_add_img(x, g, addend, out, nullptr, rows, features, stream);
}

int bf_hip_rmsnorm_backward(const float* x, const float* g, float* out, size_t rows, size_t features,
                            bf_stream_t stream) {
    return bf_hip_rmsnorm_backward_add(x, g, nullptr, out, rows, features, stream);
}

int bf_hip_softmax(const float* x, float* out, size_t rows, size_t features, bf_stream_t stream) {
    if (rows == 0 || features == 0) return BF_OK;
    BF_REQUIRE(x && out, "NULL pointer");
    hipStream_t s = asStream(stream);
#define ARGS_ x, out, rows, features
    BF_ROW_LAUNCH(softmaxKernel, false, aligned16(x) && aligned16(out), rows, features, s, x, out, rows, features);
#undef ARGS_
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_softmax_backward(const float* x, const float* g, float* out, size_t rows, size_t features,
                            bf_stream_t stream) {
    if (rows == 0 || features == 0) return BF_OK;
    BF_REQUIRE(x && g && out, "NULL pointer");
    hipStream_t s = asStream(stream);
#define ARGS_ x, g, out, rows, features
    BF_ROW_LAUNCH(softmaxBackwardKernel, true, aligned16(x) && aligned16(g) && aligned16(out), rows, features, s, x, g,
                  out, rows, features);
#undef ARGS_
    BF_LAUNCH_CHECK();
    return BF_OK;
}

}  // extern "C"
