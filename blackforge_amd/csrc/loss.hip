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

// info[0] = number of entries of `target` that do not round to -1, info[1] = 1 / info[0] (0 when there is none).
__global__ void __launch_bounds__(1024) countUnmaskedKernel(const float* __restrict__ target, size_t rows, float* __restrict__ info) {
    __shared__ double lds[16];
    double n = 0.0;
    for (size_t i = threadIdx.x; i < rows; i += blockDim.x) n += lroundf(target[i]) == -1 ? 0.0 : 1.0;
    const double total = blockReduce(n, 0.0, OpSum{}, lds);
    if (threadIdx.x == 0) {
        info[0] = float(total);
        info[1] = total > 0.0 ? 1.0f / float(total) : 0.0f;
    }
}

// finishSumKernel with the total scaled by *scale (read on the device) before it is stored or accumulated.
__global__ void __launch_bounds__(1024) finishScaledSumKernel(const float* __restrict__ partial, size_t count, const float* __restrict__ scale,
                                                              float* __restrict__ out, int accumulate) {
    __shared__ double lds[16];
    double s = 0.0;
    for (size_t i = threadIdx.x; i < count; i += blockDim.x) s += double(partial[i]);
    s = blockReduce(s, 0.0, OpSum{}, lds);
    if (threadIdx.x == 0) {
        const float mean = float(s * double(scale[0]));
        out[0] = accumulate ? out[0] + mean : mean;
    }
}

// gradImage (VEC == 4 only; may be NULL): the bf16 image of the gradient, written in the same pass (8 bytes per thread
// and step), for a model whose last layer's gradient products read it.
template <int VEC, bool NT = false>
__global__ void __launch_bounds__(kBlock) mseKernel(const float* __restrict__ pred, const float* __restrict__ target,
                                                    float* __restrict__ grad, float* __restrict__ partial, size_t n,
                                                    float gradScale, unsigned short* __restrict__ gradImage = nullptr) {
    __shared__ float lds[16];
    float acc = 0.0f;
    size_t stride = size_t(gridDim.x) * blockDim.x;
    if constexpr (VEC == 4) {
        size_t n4 = n / 4;
        for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n4; i += stride) {
            float4v d = ldf4<NT>(pred + 4 * i) - ldf4<NT>(target + 4 * i);
            acc += d.x * d.x + d.y * d.y + d.z * d.z + d.w * d.w;
            const float4v gv = d * gradScale;
            stf4<NT>(grad + 4 * i, gv);
            if (gradImage) {
                const uint2v packed = {unsigned(toBf16Bits(gv.x)) | (unsigned(toBf16Bits(gv.y)) << 16),
                                       unsigned(toBf16Bits(gv.z)) | (unsigned(toBf16Bits(gv.w)) << 16)};
                stu2<NT>(gradImage + 4 * i, packed);
            }
        }
        for (size_t i = n4 * 4 + size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
            float d = pred[i] - target[i];
            acc += d * d;
            grad[i] = d * gradScale;
            if (gradImage) gradImage[i] = toBf16Bits(d * gradScale);
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

typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));   // a float4 that may start on any 4-byte boundary

// The elements of a row that is not held in registers, for thread t of the G that share it: whole groups of four as one
// 16-byte access from whatever 4-byte boundary the row starts on (global memory serves those), then the last one to
// three elements one by one.
template <int G, typename Four, typename One>
__device__ __forceinline__ void forRowElements(size_t classes, int t, Four four, One one) {
    const size_t whole = classes & ~size_t(3);
    for (size_t e = size_t(t) * 4; e < whole; e += size_t(G) * 4) four(e);
    for (size_t e = whole + t; e < classes; e += G) one(e);
}

// SPARSE: target holds one class index per row.  Otherwise a dense target row.
// SHIFTED (with VEC = 4, CACHED): rows of any length and alignment through 16-byte accesses (RowCache::loadShifted).
// AHEAD (CACHED only): a grid that fills the chip walks the rows, each block with its next row's loads in flight
// (requested into a second set of registers before the current row is reduced).  Otherwise one block per group of rows.
template <int G, int MAXE, int VEC, bool CACHED, bool SPARSE, bool SHIFTED = false, bool NT = false, bool AHEAD = false>
__global__ void __launch_bounds__(G > 256 ? G : 256) crossEntropyKernel(const float* __restrict__ logits,
                                                                         const float* __restrict__ target,
                                                                         float* __restrict__ grad, float* __restrict__ rowLoss,
                                                                         size_t rows, size_t classes, float invRows,
                                                                         const float* __restrict__ maskInfo,
                                                                         unsigned short* __restrict__ gradImage, unsigned shiftMask) {
    static_assert(CACHED || !AHEAD, "only rows held in registers are fetched ahead");
    __shared__ float lds[16];
    const int t = threadIdx.x % G;
    const size_t rowsPerBlock = blockDim.x / G;
    const size_t rowStep = size_t(gridDim.x) * rowsPerBlock;
    // masked form (sparse targets only): maskInfo[1] = 1 / (number of rows whose index is not -1) replaces 1 / rows,
    // and a row with index -1 contributes nothing: zero gradient, zero loss
    if (SPARSE && maskInfo != nullptr) invRows = maskInfo[1];
    using Row = RowCache<G, MAXE, VEC, NT>;
    RowCache<G, AHEAD ? MAXE : VEC, VEC, NT> ahead;
    const size_t firstRow = size_t(blockIdx.x) * rowsPerBlock + threadIdx.x / G;
    // the loads only: a shifted row is masked (Row::maskShifted) where it is first used, so that a row fetched ahead
    // is not waited for here
    auto fetch = [&](auto& into, size_t r) __attribute__((always_inline)) {
        const float* src = logits + r * classes;
        if constexpr (SHIFTED) into.template issueShifted<0, MAXE / VEC>(src, classes, t, Row::shiftOf(src, shiftMask));
        else into.load(src, classes, t, -INFINITY);
    };
    if constexpr (AHEAD) { if (firstRow < rows) fetch(ahead, firstRow); }
    for (size_t row = firstRow; row < rows; row += rowStep) {
        const float* x = logits + row * classes;
        float* gOut = grad + row * classes;
        Row c;
        if constexpr (AHEAD) {
            c = ahead;
            if (row + rowStep < rows) fetch(ahead, row + rowStep);
        } else if constexpr (CACHED) {
            fetch(c, row);
        }
        const int shift = SHIFTED ? Row::shiftOf(x, shiftMask) : 0;   // the same for gOut: the host checks that
        if constexpr (CACHED && SHIFTED) c.maskShifted(classes, t, -INFINITY, shift);
        // gradImage (aligned rows only; the host checks): the gradient row rounded to bf16, for the bf16 GEMMs that consume it
        unsigned short* gImg = gradImage ? gradImage + row * classes : nullptr;
        auto storeRow = [&]() __attribute__((always_inline)) {
            if constexpr (SHIFTED) c.storeShifted(gOut, classes, t, shift);
            else {
                c.store(gOut, classes, t);
                if (gImg) c.storeBf16(gImg, classes, t);
            }
        };
        if constexpr (SPARSE) {
            if (maskInfo != nullptr && lroundf(target[row]) == -1) {   // uniform over the row's group
                if constexpr (CACHED) {
#pragma unroll
                    for (int i = 0; i < MAXE; ++i) c.r[i] = 0.0f;
                    storeRow();
                } else {
                    forRowElements<G>(classes, t,
                                      [&](size_t e) {
                                          *reinterpret_cast<float4u*>(gOut + e) = float4u{0.0f, 0.0f, 0.0f, 0.0f};
                                          if (gImg) *reinterpret_cast<uint2v*>(gImg + e) = uint2v{0u, 0u};
                                      },
                                      [&](size_t e) { gOut[e] = 0.0f; if (gImg) gImg[e] = 0; });
                }
                if (t == 0) rowLoss[row] = 0.0f;
                continue;
            }
        }
        float mx = -INFINITY;
        if constexpr (CACHED) {
#pragma unroll
            for (int i = 0; i < MAXE; ++i) mx = fmaxf(mx, c.r[i]);
        } else {
            forRowElements<G>(classes, t,
                              [&](size_t e) {
                                  const float4u v = *reinterpret_cast<const float4u*>(x + e);
                                  mx = fmaxf(fmaxf(mx, fmaxf(v.x, v.y)), fmaxf(v.z, v.w));
                              },
                              [&](size_t e) { mx = fmaxf(mx, x[e]); });
        }
        mx = groupMax<G>(mx, lds);
        // exp(x - mx) as one hardware exp2 of (x - mx) * log2(e): the argument is <= 0 and the result feeds
        // a sum of up to `classes` terms, so its ~1e-6 relative error is far inside the 1e-4 bound
        constexpr float kLog2e = 1.4426950408889634f;
        float sum = 0.0f;
        if constexpr (CACHED) {
            const float top = mx * kLog2e;   // one fused multiply-add per element; its rounding is common to the row and cancels in p
#pragma unroll
            for (int i = 0; i < MAXE; ++i) { c.r[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(c.r[i], kLog2e, -top)); sum += c.r[i]; }
        } else {
            forRowElements<G>(classes, t,
                              [&](size_t e) {
                                  const float4u v = *reinterpret_cast<const float4u*>(x + e);
                                  sum += __builtin_amdgcn_exp2f((v.x - mx) * kLog2e);
                                  sum += __builtin_amdgcn_exp2f((v.y - mx) * kLog2e);
                                  sum += __builtin_amdgcn_exp2f((v.z - mx) * kLog2e);
                                  sum += __builtin_amdgcn_exp2f((v.w - mx) * kLog2e);
                              },
                              [&](size_t e) { sum += __builtin_amdgcn_exp2f((x[e] - mx) * kLog2e); });
        }
        sum = groupSum<G>(sum, lds);
        const float inv = 1.0f / sum;

        float loss = 0.0f;  // this thread's share of the row loss
        if constexpr (SPARSE) {
            // grad = (p - onehot) / rows; the one thread that holds the target class keeps its probability
            const unsigned cls = unsigned(lroundf(target[row]));
            float pTarget = -1.0f;
            if constexpr (CACHED) {
                // Element e of the row sits at position e + shift of the held row: iteration pos / (G * VEC), thread
                // (pos / VEC) % G, slot pos % VEC.  Only the iteration that holds the target looks for it (the same
                // for the whole group), every other element is one multiplication.
                const unsigned pos = cls + unsigned(shift);
                const int targetIt = cls < classes ? int(pos / unsigned(G * VEC)) : -1;
                const bool mine = int((pos / VEC) % G) == t;
                const int targetSlot = int(pos % VEC);
                const float scale = inv * invRows;
#pragma unroll
                for (int it = 0; it < MAXE / VEC; ++it) {
                    if (it == targetIt) {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) {
                            const bool hit = mine && j == targetSlot;
                            const float p = c.r[it * VEC + j] * inv;
                            pTarget = hit ? p : pTarget;
                            c.r[it * VEC + j] = hit ? (p - 1.0f) * invRows : c.r[it * VEC + j] * scale;
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < VEC; ++j) c.r[it * VEC + j] *= scale;
                    }
                }
                storeRow();
            } else {
                auto element = [&](float xe, size_t e) -> float {
                    const float p = __builtin_amdgcn_exp2f((xe - mx) * kLog2e) * inv;
                    const bool hit = e == cls;
                    pTarget = hit ? p : pTarget;
                    return (p - (hit ? 1.0f : 0.0f)) * invRows;
                };
                forRowElements<G>(classes, t,
                                  [&](size_t e) {
                                      const float4u v = *reinterpret_cast<const float4u*>(x + e);
                                      const float4u gv = {element(v.x, e), element(v.y, e + 1), element(v.z, e + 2), element(v.w, e + 3)};
                                      *reinterpret_cast<float4u*>(gOut + e) = gv;
                                      if (gImg)   // (aligned rows of a multiple of 8 classes only: an 8-byte group)
                                          *reinterpret_cast<uint2v*>(gImg + e) = uint2v{unsigned(toBf16Bits(gv.x)) | unsigned(toBf16Bits(gv.y)) << 16,
                                                                                        unsigned(toBf16Bits(gv.z)) | unsigned(toBf16Bits(gv.w)) << 16};
                                  },
                                  [&](size_t e) {
                                      const float gv = element(x[e], e);
                                      gOut[e] = gv;
                                      if (gImg) gImg[e] = toBf16Bits(gv);
                                  });
            }
            if (pTarget >= 0.0f) loss = -logf(fmaxf(pTarget, 1e-12f));
        } else {
            const float* tRow = target + row * classes;
            auto emit = [&](float e, size_t idx) -> float {
                const float p = e * inv;
                const float tv = tRow[idx];
                if (tv != 0.0f) loss += -tv * logf(fmaxf(p, 1e-12f));
                return (p - tv) * invRows;
            };
            if constexpr (CACHED) {
#pragma unroll
                for (int it = 0; it < MAXE / VEC; ++it)
#pragma unroll
                    for (int j = 0; j < VEC; ++j) {
                        const long idx = long(Row::index(it, t, j)) - shift;
                        if (idx >= 0 && size_t(idx) < classes) c.r[it * VEC + j] = emit(c.r[it * VEC + j], size_t(idx));
                    }
                storeRow();
            } else {
                for (size_t e = t; e < classes; e += G) {
                    const float gv = emit(__builtin_amdgcn_exp2f((x[e] - mx) * kLog2e), e);
                    gOut[e] = gv;
                    if (gImg) gImg[e] = toBf16Bits(gv);
                }
            }
        }
        loss = groupSum<G>(loss, lds);
        if (t == 0) rowLoss[row] = loss;
    }
}

// The sparse cross-entropy of a language-model head whose gradient has no reader but the head's own gradient products:
// the gradient row goes out as its bf16 image only (no fp32 copy is written), and its column sums, the bias gradient of
// the head, are collected on the way: a thread holds the same columns of every row its block walks, so it adds each
// gradient value (fp32, before the rounding) to a sum per column and the block writes one partial row at the end;
// columnPartialsFinishKernel adds the partial rows in index order.  Same arithmetic per element as crossEntropyKernel
// (1024 threads a row, rows in registers, the next row's loads in flight): the same loss, the same image.
template <int MAXE, bool NT>
__global__ void __launch_bounds__(1024) crossEntropyImageKernel(const float* __restrict__ logits, const float* __restrict__ target,
                                                                unsigned short* __restrict__ gradImage, float* __restrict__ rowLoss,
                                                                float* __restrict__ colPartial, size_t rows, size_t classes, float invRows) {
    constexpr int G = 1024, VEC = 4;
    __shared__ float lds[16];
    // the column sums live in LDS ([iteration][thread] groups of four: a thread touches only its own, 16 bytes at a time,
    // consecutive threads consecutive groups), so that two rows' worth of registers remain for the rows themselves
    extern __shared__ __attribute__((aligned(16))) float colSums[];
    const int t = threadIdx.x;
    using Row = RowCache<G, MAXE, VEC, NT>;
    Row ahead;
#pragma unroll
    for (int it = 0; it < MAXE / VEC; ++it) *reinterpret_cast<float4v*>(colSums + (it * G + t) * VEC) = float4v{0.0f, 0.0f, 0.0f, 0.0f};
    const size_t rowStep = gridDim.x;
    if (blockIdx.x < rows) ahead.load(logits + size_t(blockIdx.x) * classes, classes, t, -INFINITY);
    for (size_t row = blockIdx.x; row < rows; row += rowStep) {
        Row c = ahead;
        if (row + rowStep < rows) ahead.load(logits + (row + rowStep) * classes, classes, t, -INFINITY);
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < MAXE; ++i) mx = fmaxf(mx, c.r[i]);
        mx = groupMax<G>(mx, lds);
        constexpr float kLog2e = 1.4426950408889634f;
        const float top = mx * kLog2e;
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < MAXE; ++i) { c.r[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(c.r[i], kLog2e, -top)); sum += c.r[i]; }
        sum = groupSum<G>(sum, lds);
        const float inv = 1.0f / sum;
        const unsigned cls = unsigned(lroundf(target[row]));
        const int targetIt = cls < classes ? int(cls / unsigned(G * VEC)) : -1;
        const bool mine = int((cls / VEC) % G) == t;
        const int targetSlot = int(cls % VEC);
        const float scale = inv * invRows;
        float pTarget = -1.0f;
#pragma unroll
        for (int it = 0; it < MAXE / VEC; ++it) {
            if (it == targetIt) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const bool hit = mine && j == targetSlot;
                    const float p = c.r[it * VEC + j] * inv;
                    pTarget = hit ? p : pTarget;
                    c.r[it * VEC + j] = hit ? (p - 1.0f) * invRows : c.r[it * VEC + j] * scale;
                }
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) c.r[it * VEC + j] *= scale;
            }
        }
#pragma unroll
        for (int it = 0; it < MAXE / VEC; ++it) {   // slots past the row's end hold exp2(-inf) * scale = 0
            float4v* sums = reinterpret_cast<float4v*>(colSums + (it * G + t) * VEC);
            *sums = *sums + float4v{c.r[it * VEC + 0], c.r[it * VEC + 1], c.r[it * VEC + 2], c.r[it * VEC + 3]};
        }
        c.storeBf16(gradImage + row * classes, classes, t);
        float loss = pTarget >= 0.0f ? -logf(fmaxf(pTarget, 1e-12f)) : 0.0f;
        loss = groupSum<G>(loss, lds);
        if (t == 0) rowLoss[row] = loss;
    }
    Row col;
#pragma unroll
    for (int it = 0; it < MAXE / VEC; ++it) {
        const float4v v = *reinterpret_cast<const float4v*>(colSums + (it * G + t) * VEC);
        col.r[it * VEC + 0] = v.x; col.r[it * VEC + 1] = v.y; col.r[it * VEC + 2] = v.z; col.r[it * VEC + 3] = v.w;
    }
    col.store(colPartial + size_t(blockIdx.x) * classes, classes, t);
}

// out[c] = sum over p of partial[p * features + c], rows added in index order: sixteen lanes per group of four columns
// each add every sixteenth partial row, and the sixteen sums are combined in a fixed order (features % 4 == 0).
__global__ void __launch_bounds__(kBlock) columnPartialsFinishKernel(const float* __restrict__ partial, float* __restrict__ out,
                                                                     size_t parts, size_t features) {
    __shared__ float4v lds[16][17];
    const int cx = threadIdx.x & 15, part = threadIdx.x >> 4;
    const size_t c = (size_t(blockIdx.x) * 16 + cx) * 4;
    float4v s = {0.0f, 0.0f, 0.0f, 0.0f};
    if (c < features) {
#pragma unroll 8
        for (size_t p = part; p < parts; p += 16) s = s + loadf4(partial + p * features + c);
    }
    lds[part][cx] = s;
    __syncthreads();
    if (part == 0 && c < features) {
        float4v total = lds[0][cx];
        for (int i = 1; i < 16; ++i) total = total + lds[i][cx];
        storef4(out + c, total);
    }
}

// The head's loss for rows that the kernel above does not serve: more classes than its column sums have LDS for
// (up to 1024 x 52), or a class count that is not a multiple of 8 (rows that start on any 4-byte boundary; the image's
// rows are `pitch` = classes rounded up to 8 apart, the columns past the row zero).  One row at a time in 52 registers a
// thread, read with 16-byte loads from whatever boundary the row starts on (global memory serves those), the gradient
// written as its bf16 image only; same arithmetic per element as crossEntropyKernel.  The bias gradient is then the
// column sums of that image (columnSumBf16Kernel): the sum of the gradient values as the head's products see them.
template <bool NT>
__global__ void __launch_bounds__(1024) crossEntropyImageWideKernel(const float* __restrict__ logits, const float* __restrict__ target,
                                                                    unsigned short* __restrict__ gradImage, float* __restrict__ rowLoss,
                                                                    size_t rows, size_t classes, size_t pitch, float invRows) {
    constexpr int G = 1024, MAXE = 52, VEC = 4;
    __shared__ float lds[16];
    const int t = threadIdx.x;
    const int n = int(classes), wide = int(pitch);   // at most 1024 x 52
    const int tailStart = n & ~3, tailIt = (n & 3) ? tailStart / (G * VEC) : -1, tailThread = (tailStart / VEC) % G;
    for (size_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const float* __restrict__ x = logits + row * classes;
        float r[MAXE];
        // every load first, without a branch (a group that is not wholly inside the row re-reads group 0), the masking
        // afterwards; the row's last, partial group (one thread's, if the length is not a multiple of 4) element by element
#pragma unroll
        for (int it = 0; it < MAXE / VEC; ++it) {
            const int e = (it * G + t) * VEC;
            const float* src = x + (e + VEC <= n ? e : 0);
            float4u v;
            if constexpr (NT) v = __builtin_nontemporal_load(reinterpret_cast<const float4u*>(src));
            else v = *reinterpret_cast<const float4u*>(src);
            r[it * VEC + 0] = v.x; r[it * VEC + 1] = v.y; r[it * VEC + 2] = v.z; r[it * VEC + 3] = v.w;
        }
#pragma unroll
        for (int it = 0; it < MAXE / VEC; ++it) {
            const int e = (it * G + t) * VEC;
            const bool whole = e + VEC <= n;
#pragma unroll
            for (int j = 0; j < VEC; ++j) r[it * VEC + j] = whole ? r[it * VEC + j] : -INFINITY;
            if (it == tailIt && t == tailThread) {   // (the first condition is the same for the whole block)
#pragma unroll
                for (int j = 0; j < VEC - 1; ++j)
                    if (tailStart + j < n) r[it * VEC + j] = x[tailStart + j];
            }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < MAXE; ++i) mx = fmaxf(mx, r[i]);
        mx = groupMax<G>(mx, lds);
        constexpr float kLog2e = 1.4426950408889634f;
        const float top = mx * kLog2e;
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < MAXE; ++i) { r[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(r[i], kLog2e, -top)); sum += r[i]; }
        sum = groupSum<G>(sum, lds);
        const float inv = 1.0f / sum;
        const unsigned cls = unsigned(lroundf(target[row]));
        const int targetIt = cls < classes ? int(cls / unsigned(G * VEC)) : -1;
        const bool mine = int((cls / VEC) % G) == t;
        const int targetSlot = int(cls % VEC);
        const float scale = inv * invRows;
        float pTarget = -1.0f;
#pragma unroll
        for (int it = 0; it < MAXE / VEC; ++it) {
            if (it == targetIt) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) {
                    const bool hit = mine && j == targetSlot;
                    const float p = r[it * VEC + j] * inv;
                    pTarget = hit ? p : pTarget;
                    r[it * VEC + j] = hit ? (p - 1.0f) * invRows : r[it * VEC + j] * scale;
                }
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) r[it * VEC + j] *= scale;
            }
        }
        unsigned short* __restrict__ out = gradImage + row * pitch;
#pragma unroll
        for (int it = 0; it < MAXE / VEC; ++it) {   // slots past the row's end hold exp2(-inf) * scale = 0: the image's padding
            const int e = (it * G + t) * VEC;
            if (e < wide) {
                const uint2v packed = {unsigned(toBf16Bits(r[it * VEC + 0])) | unsigned(toBf16Bits(r[it * VEC + 1])) << 16,
                                       unsigned(toBf16Bits(r[it * VEC + 2])) | unsigned(toBf16Bits(r[it * VEC + 3])) << 16};
                stu2<NT>(out + e, packed);
            }
        }
        float loss = pTarget >= 0.0f ? -logf(fmaxf(pTarget, 1e-12f)) : 0.0f;
        loss = groupSum<G>(loss, lds);
        if (t == 0) rowLoss[row] = loss;
    }
}

// The same for rows too long for a block's registers (more than 1024 x 52 classes: the vocabularies of 128 256, 151 936
// or 256 000 words): the row is walked twice, the second time out of the last-level cache (a row of 256 000 floats is
// 1 MB).  First walk: the maximum and, in the same walk, the sum of exponentials about the maximum so far (the sum is
// rescaled whenever a thread's maximum moves; the threads' pairs are then combined about the row's maximum).  Second
// walk: the gradient's image.  Element by element the values are those of the kernels above up to the order of the
// additions in the sum.
template <bool NT>
__global__ void __launch_bounds__(1024) crossEntropyImageLongKernel(const float* __restrict__ logits, const float* __restrict__ target,
                                                                    unsigned short* __restrict__ gradImage, float* __restrict__ rowLoss,
                                                                    size_t rows, size_t classes, size_t pitch, float invRows) {
    constexpr int G = 1024, VEC = 4;
    constexpr float kLog2e = 1.4426950408889634f;
    __shared__ float lds[16];
    const int t = threadIdx.x;
    const size_t whole = classes & ~size_t(3);   // elements in whole groups of four
    for (size_t row = blockIdx.x; row < rows; row += gridDim.x) {
        const float* __restrict__ x = logits + row * classes;
        // base-2 logarithms throughout: y = x * log2(e)
        float mx = -INFINITY, sum = 0.0f;
        auto take = [&](float v) {
            const float y = v * kLog2e;
            if (y > mx) { sum = sum * __builtin_amdgcn_exp2f(mx - y) + 1.0f; mx = y; }   // (0 * exp2(-inf - y) = 0 for the first element)
            else sum += __builtin_amdgcn_exp2f(y - mx);
        };
        for (size_t e = size_t(t) * VEC; e < whole; e += size_t(G) * VEC) {
            const float4u v = *reinterpret_cast<const float4u*>(x + e);   // stays in the cache for the second walk
            take(v.x); take(v.y); take(v.z); take(v.w);
        }
        if (t < int(classes - whole)) take(x[whole + t]);
        const float rowMax = groupMax<G>(mx, lds);
        sum = mx > -INFINITY ? sum * __builtin_amdgcn_exp2f(mx - rowMax) : 0.0f;
        sum = groupSum<G>(sum, lds);
        const float inv = 1.0f / sum, scale = inv * invRows;
        const size_t cls = size_t(lroundf(target[row]));
        float pTarget = -1.0f;
        unsigned short* __restrict__ out = gradImage + row * pitch;
        for (size_t e = size_t(t) * VEC; e < pitch; e += size_t(G) * VEC) {
            float g[VEC];
            if (e + VEC <= classes) {
                float4u v;
                if constexpr (NT) v = __builtin_nontemporal_load(reinterpret_cast<const float4u*>(x + e));
                else v = *reinterpret_cast<const float4u*>(x + e);
                g[0] = v.x; g[1] = v.y; g[2] = v.z; g[3] = v.w;
            } else {
#pragma unroll
                for (int j = 0; j < VEC; ++j) g[j] = e + j < classes ? x[e + j] : -INFINITY;
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
                const float ex = __builtin_amdgcn_exp2f(__builtin_fmaf(g[j], kLog2e, -rowMax));
                const bool hit = e + j == cls;
                const float p = ex * inv;
                pTarget = hit ? p : pTarget;
                g[j] = hit ? (p - 1.0f) * invRows : ex * scale;
            }
            const uint2v packed = {unsigned(toBf16Bits(g[0])) | unsigned(toBf16Bits(g[1])) << 16,
                                   unsigned(toBf16Bits(g[2])) | unsigned(toBf16Bits(g[3])) << 16};
            stu2<NT>(out + e, packed);
        }
        float loss = pTarget >= 0.0f ? -logf(fmaxf(pTarget, 1e-12f)) : 0.0f;
        loss = groupSum<G>(loss, lds);
        if (t == 0) rowLoss[row] = loss;
    }
}

// partial[band * pitch + c] = sum of image[row * pitch + c] over the rows of band `blockIdx.y` (rowsPerBand each), in row
// order: a thread owns eight columns (16 bytes of a row) and keeps four rows' loads in flight.
__global__ void __launch_bounds__(kBlock) columnSumBf16Kernel(const unsigned short* __restrict__ image, float* __restrict__ partial,
                                                              size_t rows, size_t pitch, size_t rowsPerBand) {
    const size_t c = (size_t(blockIdx.x) * kBlock + threadIdx.x) * 8;
    if (c >= pitch) return;
    const size_t rowBegin = size_t(blockIdx.y) * rowsPerBand, rowEnd = rowBegin + rowsPerBand < rows ? rowBegin + rowsPerBand : rows;
    float sums[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    auto add = [&](uint4v v) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            sums[2 * j] += __builtin_bit_cast(float, v[j] << 16);
            sums[2 * j + 1] += __builtin_bit_cast(float, v[j] & 0xffff0000u);
        }
    };
    size_t row = rowBegin;
    for (; row + 4 <= rowEnd; row += 4) {
        uint4v v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(image + (row + i) * pitch + c));
#pragma unroll
        for (int i = 0; i < 4; ++i) add(v[i]);
    }
    for (; row < rowEnd; ++row) add(__builtin_nontemporal_load(reinterpret_cast<const uint4v*>(image + row * pitch + c)));
    float* __restrict__ out = partial + size_t(blockIdx.y) * pitch + c;
    storef4(out, float4v{sums[0], sums[1], sums[2], sums[3]});
    storef4(out + 4, float4v{sums[4], sums[5], sums[6], sums[7]});
}
// out[c] = sum over the bands, in band order, for the `features` columns that exist (pitch >= features)
__global__ void __launch_bounds__(kBlock) columnBandsFinishKernel(const float* __restrict__ partial, float* __restrict__ out, size_t bands,
                                                                  size_t pitch, size_t features) {
    const size_t c = size_t(blockIdx.x) * kBlock + threadIdx.x;
    if (c >= features) return;
    float total = 0.0f;
    for (size_t b = 0; b < bands; ++b) total += partial[b * pitch + c];
    out[c] = total;
}

template <bool SPARSE>
int launchCrossEntropy(const float* logits, const float* target, float* grad, float* lossSum, size_t rows,
                       size_t classes, int accumulate, hipStream_t s, bool masked = false, unsigned short* gradImage = nullptr) {
    if (gradImage != nullptr && (classes % 8 != 0 || !aligned16(logits) || !aligned16(grad) || !aligned16(gradImage)))
        return failInvalid("cross_entropy", "the bf16 gradient image needs 16-byte aligned tensors and a class count that is a multiple of 8");
    Scratch rowLoss((rows + 2) * sizeof(float));   // per-row losses, then the two words of the masked form
    if (rowLoss.status != BF_OK) return rowLoss.status;
    float* rl = rowLoss.as<float>();
    const float* maskInfo = nullptr;
    if (masked) {
        countUnmaskedKernel<<<1, 1024, 0, s>>>(target, rows, rl + rows);
        BF_LAUNCH_CHECK();
        maskInfo = rl + rows;
    }
    const float invRows = 1.0f / float(rows);
    const bool vec4 = aligned16(logits) && aligned16(grad) && classes % 4 == 0;
    // rows that are not 16-byte aligned still get 16-byte accesses (shifted) as long as a logits row and its gradient
    // row sit at the same offset within a 16-byte group; a row must then fit its registers with up to 3 elements to spare
    const bool shifted = !vec4 && ((reinterpret_cast<uintptr_t>(logits) ^ reinterpret_cast<uintptr_t>(grad)) & 15u) == 0;
    // shifted rows are addressed from the 128-byte line below their first element when logits and gradient rows sit at
    // the same offset within a line (every wavefront access then covers whole lines), else from the 16-byte group below
    // ... and only when both tensors START on a line: the first row then has shift 0 and is addressed from its own first
    // element, and every later row's line lies inside the tensor (it holds the tail of the row before), so nothing below
    // the tensor's first byte is ever read.  Past the last row's end at most the rest of its 16-byte group is read.
    const bool sameLine = ((reinterpret_cast<uintptr_t>(logits) | reinterpret_cast<uintptr_t>(grad)) & 127u) == 0;
    const bool streaming = streamsPastCache(rows * classes * (SPARSE ? 8 : 12));   // logits in, gradient out (and a dense target in)
    // smallest group and register count that hold a row (see the row kernels)
    // AHEAD as measured (8 B per logit over the launch, 16-byte aligned rows): rows of up to 8192 classes are faster
    // one block per group of rows (65536 x 2048: 5.4 against 4.9 TB/s walking, 16384 x 4096: 5.9 against 5.3), 16384
    // classes the same either way, 32000 faster walking (5.9 against 5.4-5.7), and rows past 32768, which leave no
    // registers for a second row, no faster with part of one fetched ahead on half the wavefronts
#define BF_CE(G, MAXE, AHEAD)                                                                                     \
    if (classes + (vec4 ? 0 : 3) <= size_t(G) * MAXE && (vec4 || shifted || MAXE <= 32)) {                        \
        const unsigned threads = G > 256 ? G : 256;                                                               \
        /* whole lines pay on the long rows (1024 threads a row: +5..8 %); rows of 4100 measured 12 % slower that way */ \
        const unsigned shiftMask = sameLine && G == 1024 && classes + 31 <= size_t(G) * MAXE ? 31u : 3u;           \
        const unsigned grid = gridFor(rows, threads / G, AHEAD ? unsigned(computeUnits()) * (2048 / threads) : kMaxGridX); \
        /* 16-byte aligned rows that start inside a 128-byte line go the shifted way as well, for the whole lines */ \
        /* so do the long 16-byte aligned rows of a dense target: the form without a branch per load keeps to its registers */ \
        const bool lineShift = vec4 && gradImage == nullptr &&                                                      \
                               ((classes % 32 != 0 && shiftMask == 31u) || (!SPARSE && MAXE > 32));                  \
        if (lineShift && streaming) crossEntropyKernel<G, MAXE, 4, true, SPARSE, true, true, AHEAD><<<grid, threads, 0, s>>>(logits, target, grad, rl, rows, classes, invRows, maskInfo, gradImage, shiftMask); \
        else if (lineShift) crossEntropyKernel<G, MAXE, 4, true, SPARSE, true, false, AHEAD><<<grid, threads, 0, s>>>(logits, target, grad, rl, rows, classes, invRows, maskInfo, gradImage, shiftMask); \
        else if (vec4 && streaming) crossEntropyKernel<G, MAXE, 4, true, SPARSE, false, true, AHEAD><<<grid, threads, 0, s>>>(logits, target, grad, rl, rows, classes, invRows, maskInfo, gradImage, shiftMask); \
        else if (vec4) crossEntropyKernel<G, MAXE, 4, true, SPARSE, false, false, AHEAD><<<grid, threads, 0, s>>>(logits, target, grad, rl, rows, classes, invRows, maskInfo, gradImage, shiftMask); \
        else if (shifted && streaming) crossEntropyKernel<G, MAXE, 4, true, SPARSE, true, true, AHEAD><<<grid, threads, 0, s>>>(logits, target, grad, rl, rows, classes, invRows, maskInfo, gradImage, shiftMask); \
        else if (shifted) crossEntropyKernel<G, MAXE, 4, true, SPARSE, true, false, AHEAD><<<grid, threads, 0, s>>>(logits, target, grad, rl, rows, classes, invRows, maskInfo, gradImage, shiftMask); \
        else crossEntropyKernel<G, (MAXE <= 32 ? MAXE : 4), 1, true, SPARSE, false, false, AHEAD><<<grid, threads, 0, s>>>(logits, target, grad, rl, rows, classes, invRows, maskInfo, gradImage, shiftMask); /* plans above 32 registers have no one-element form */ \
        break;                                                                                                    \
    }
    do {
        BF_CE(64, 4, false) BF_CE(64, 8, false) BF_CE(64, 16, false) BF_CE(256, 8, false) BF_CE(256, 16, false) BF_CE(256, 32, false)
        BF_CE(1024, 16, true) BF_CE(1024, 32, true) BF_CE(1024, 52, false)
        crossEntropyKernel<1024, 4, 1, false, SPARSE><<<gridFor(rows, 1), 1024, 0, s>>>(logits, target, grad, rl, rows, classes, invRows, maskInfo, gradImage, 3u);
    } while (0);
#undef BF_CE
    BF_LAUNCH_CHECK();
    if (masked) finishScaledSumKernel<<<1, 1024, 0, s>>>(rl, rows, maskInfo + 1, lossSum, accumulate);
    else finishSumKernel<<<1, 1024, 0, s>>>(rl, rows, lossSum, accumulate);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" {

int bf_hip_mse(const float* pred, const float* target, float* grad, float* lossSum, size_t n, int accumulate,
               bf_stream_t stream) {
    return bf_hip_mse_img(pred, target, grad, nullptr, lossSum, n, accumulate, stream);
}

int bf_hip_mse_img(const float* pred, const float* target, float* grad, uint16_t* gradImage, float* lossSum, size_t n, int accumulate,
                   bf_stream_t stream) {
    BF_REQUIRE(lossSum != nullptr, "lossSum is NULL");
    hipStream_t s = asStream(stream);
    if (n == 0) {
        if (!accumulate) return bf_hip_fill_zero(lossSum, sizeof(float), stream);
        return BF_OK;
    }
    BF_REQUIRE(pred && target && grad, "NULL pointer");
    unsigned grid = gridFor(n, size_t(kBlock) * 4, 65536);   // one 16-byte group per thread until the partial sums get too many
    Scratch partial(grid * sizeof(float));
    if (partial.status != BF_OK) return partial.status;
    float gradScale = 2.0f / float(n);
    const bool vec = aligned16(pred) && aligned16(target) && aligned16(grad);
    BF_REQUIRE(gradImage == nullptr || (vec && (reinterpret_cast<uintptr_t>(gradImage) & 7u) == 0),
               "a gradient image needs 16-byte aligned tensors and an 8-byte aligned image");
    if (vec && streamsPastCache(n * 12))
        mseKernel<4, true><<<grid, kBlock, 0, s>>>(pred, target, grad, partial.as<float>(), n, gradScale, gradImage);
    else if (vec)
        mseKernel<4><<<grid, kBlock, 0, s>>>(pred, target, grad, partial.as<float>(), n, gradScale, gradImage);
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

int bf_hip_cross_entropy_sparse_img(const float* logits, const float* targetIdx, float* grad, uint16_t* gradImage, float* lossSum,
                                    size_t rows, size_t classes, int accumulate, bf_stream_t stream) {
    BF_REQUIRE(lossSum != nullptr, "lossSum is NULL");
    if (rows == 0 || classes == 0) {
        if (!accumulate) return bf_hip_fill_zero(lossSum, sizeof(float), stream);
        return BF_OK;
    }
    BF_REQUIRE(logits && targetIdx && grad, "NULL pointer");
    return launchCrossEntropy<true>(logits, targetIdx, grad, lossSum, rows, classes, accumulate, asStream(stream), false, gradImage);
}

int bf_hip_cross_entropy_sparse_head(const float* logits, const float* targetIdx, uint16_t* gradImage, float* biasGrad, float* lossSum,
                                     size_t rows, size_t classes, int accumulate, bf_stream_t stream) {
    BF_REQUIRE(lossSum != nullptr, "lossSum is NULL");
    // the rows a 1024-thread block can hold in its registers, with a 16-byte aligned bf16 image
    if (rows == 0 || classes < 4096 || classes > (size_t(1) << 20) || !aligned16(gradImage)) {
        setLastError("bf_hip_cross_entropy_sparse_head: shape or alignment not served by the fused form (use bf_hip_cross_entropy_sparse_img and bf_hip_bias_grad)");
        return BF_ERR_UNSUPPORTED;
    }
    BF_REQUIRE(logits && targetIdx && gradImage && biasGrad, "NULL pointer");
    hipStream_t s = asStream(stream);
    if (classes % 8 != 0 || classes > size_t(1024) * 32 || !aligned16(logits) || !aligned16(biasGrad)) {
        // rows of any length (up to 2^20 classes) and any alignment: the loss with the image alone, then the image's column sums
        const size_t pitch = (classes + 7) / 8 * 8;
        const float invRows = 1.0f / float(rows);
        const unsigned grid = unsigned(std::min<size_t>(rows, kMaxGridX));
        Scratch rowLoss(rows * sizeof(float));
        if (rowLoss.status != BF_OK) return rowLoss.status;
        const bool streaming = streamsPastCache(rows * classes * 6);
        if (classes > size_t(1024) * 52) {   // rows that a block's registers do not hold: two walks over each row
            if (streaming) crossEntropyImageLongKernel<true><<<grid, 1024, 0, s>>>(logits, targetIdx, gradImage, rowLoss.as<float>(), rows, classes, pitch, invRows);
            else crossEntropyImageLongKernel<false><<<grid, 1024, 0, s>>>(logits, targetIdx, gradImage, rowLoss.as<float>(), rows, classes, pitch, invRows);
        } else if (streaming) {
            crossEntropyImageWideKernel<true><<<grid, 1024, 0, s>>>(logits, targetIdx, gradImage, rowLoss.as<float>(), rows, classes, pitch, invRows);
        } else {
            crossEntropyImageWideKernel<false><<<grid, 1024, 0, s>>>(logits, targetIdx, gradImage, rowLoss.as<float>(), rows, classes, pitch, invRows);
        }
        BF_LAUNCH_CHECK();
        // bands of rows so that the grid has a few thousand workgroups
        const size_t columnBlocks = (pitch / 8 + kBlock - 1) / kBlock;
        size_t bands = std::max<size_t>(1, std::min<size_t>((rows + 63) / 64, (size_t(computeUnits()) * 8 + columnBlocks - 1) / columnBlocks));
        const size_t rowsPerBand = (rows + bands - 1) / bands;
        bands = (rows + rowsPerBand - 1) / rowsPerBand;
        Scratch partial(bands * pitch * sizeof(float));
        if (partial.status != BF_OK) return partial.status;
        columnSumBf16Kernel<<<dim3(unsigned(columnBlocks), unsigned(bands)), kBlock, 0, s>>>(gradImage, partial.as<float>(), rows, pitch, rowsPerBand);
        BF_LAUNCH_CHECK();
        columnBandsFinishKernel<<<gridFor(classes, kBlock), kBlock, 0, s>>>(partial.as<float>(), biasGrad, bands, pitch, classes);
        BF_LAUNCH_CHECK();
        finishSumKernel<<<1, 1024, 0, s>>>(rowLoss.as<float>(), rows, lossSum, accumulate);
        BF_LAUNCH_CHECK();
        return BF_OK;
    }
    const unsigned grid = unsigned(std::min<size_t>(rows, size_t(computeUnits()) * 2));
    Scratch rowLoss(rows * sizeof(float));
    if (rowLoss.status != BF_OK) return rowLoss.status;
    Scratch partial(size_t(grid) * classes * sizeof(float));
    if (partial.status != BF_OK) return partial.status;
    const float invRows = 1.0f / float(rows);
    const bool streaming = streamsPastCache(rows * classes * 6);
    auto launch = [&](auto kernel, size_t ldsBytes) -> int {
        int st = allowDynamicSharedMemory(reinterpret_cast<const void*>(kernel), ldsBytes);
        if (st != BF_OK) return st;
        kernel<<<grid, 1024, ldsBytes, s>>>(logits, targetIdx, gradImage, rowLoss.as<float>(), partial.as<float>(), rows, classes, invRows);
        return BF_OK;
    };
    int st = BF_OK;
    if (classes <= size_t(1024) * 16) st = streaming ? launch(crossEntropyImageKernel<16, true>, 1024 * 16 * sizeof(float)) : launch(crossEntropyImageKernel<16, false>, 1024 * 16 * sizeof(float));
    else st = streaming ? launch(crossEntropyImageKernel<32, true>, 1024 * 32 * sizeof(float)) : launch(crossEntropyImageKernel<32, false>, 1024 * 32 * sizeof(float));
    if (st != BF_OK) return st;
    BF_LAUNCH_CHECK();
    columnPartialsFinishKernel<<<gridFor(classes / 4, 16), kBlock, 0, s>>>(partial.as<float>(), biasGrad, grid, classes);
    BF_LAUNCH_CHECK();
    finishSumKernel<<<1, 1024, 0, s>>>(rowLoss.as<float>(), rows, lossSum, accumulate);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_cross_entropy_sparse(const float* logits, const float* targetIdx, float* grad, float* lossSum,
                                size_t rows, size_t classes, int accumulate, bf_stream_t stream) {
    return bf_hip_cross_entropy_sparse_img(logits, targetIdx, grad, nullptr, lossSum, rows, classes, accumulate, stream);
}

int bf_hip_cross_entropy_masked(const float* logits, const float* targetIdx, float* grad, float* lossMean, size_t rows,
                                size_t classes, int accumulate, bf_stream_t stream) {
    BF_REQUIRE(lossMean != nullptr, "lossMean is NULL");
    if (rows == 0 || classes == 0) {
        if (!accumulate) return bf_hip_fill_zero(lossMean, sizeof(float), stream);
        return BF_OK;
    }
    BF_REQUIRE(logits && targetIdx && grad, "NULL pointer");
    return launchCrossEntropy<true>(logits, targetIdx, grad, lossMean, rows, classes, accumulate, asStream(stream), true);
}

}  // extern "C"
