// Register-resident rows for the row-wise kernels (rmsnorm, softmax, cross-entropy).
//
// A "group" of G threads (64 = one wavefront, or a whole block of 256 / 1024) owns one row and keeps
// up to MAXE elements per thread in registers, so multi-pass algorithms (max, sum, normalise) read
// the row from HBM exactly once.  Rows longer than G*MAXE fall back to re-reading global memory
// (served by L2).  VEC = 4 uses dwordx4 accesses and needs 16-byte aligned rows (features % 4 == 0
// and an aligned base); VEC = 1 handles every other shape with coalesced dword accesses.
#pragma once

#include "common.hpp"

namespace bf {

#if defined(__HIPCC__)

template <int G, int MAXE, int VEC>
struct RowCache {
    static constexpr int kIters = MAXE / VEC;
    float r[MAXE];

    // element index handled by (iteration it, vector slot j) for group-thread t
    __device__ static size_t index(int it, int t, int j) { return (size_t(it) * G + t) * VEC + j; }

    __device__ void load(const float* __restrict__ row, size_t features, int t, float fill) {
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            size_t e = index(it, t, 0);
            if constexpr (VEC == 4) {
                if (e < features) {
                    float4v v = loadf4(row + e);
                    r[it * 4 + 0] = v.x; r[it * 4 + 1] = v.y; r[it * 4 + 2] = v.z; r[it * 4 + 3] = v.w;
                } else {
                    r[it * 4 + 0] = r[it * 4 + 1] = r[it * 4 + 2] = r[it * 4 + 3] = fill;
                }
            } else {
                r[it] = e < features ? row[e] : fill;
            }
        }
    }

    __device__ void store(float* __restrict__ row, size_t features, int t) const {
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            size_t e = index(it, t, 0);
            if (e < features) {
                if constexpr (VEC == 4) {
                    float4v v = {r[it * 4 + 0], r[it * 4 + 1], r[it * 4 + 2], r[it * 4 + 3]};
                    storef4(row + e, v);
                } else {
                    row[e] = r[it];
                }
            }
        }
    }
};

// Sum / max over the G threads that share a row.  For G == 64 a wavefront shuffle; for a whole block
// an LDS exchange (`lds` must hold 16 values of T and is reused across calls).
template <int G, typename T>
__device__ __forceinline__ T groupSum(T v, T* lds) {
    if constexpr (G == 64) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
        return v;
    } else {
        return blockReduce(v, T(0), OpSum{}, lds);
    }
}
template <int G>
__device__ __forceinline__ float groupMax(float v, float* lds) {
    if constexpr (G == 64) return waveMax(v);
    else return blockReduce(v, -INFINITY, OpMaxF{}, lds);
}

#endif  // __HIPCC__

// Host-side choice of group size for a row length: the smallest group whose registers hold the row.
struct RowPlan {
    int group;        // 64, 256 or 1024 threads per row
    int rowsPerBlock; // rows handled concurrently by one block
    int threads;      // block size
    bool cached;      // whole row fits in registers
};
inline RowPlan planRows(size_t features, int maxElemsPerThread) {
    RowPlan p;
    if (features <= size_t(64) * maxElemsPerThread) { p.group = 64; p.rowsPerBlock = 4; p.threads = 256; p.cached = true; }
    else if (features <= size_t(256) * maxElemsPerThread) { p.group = 256; p.rowsPerBlock = 1; p.threads = 256; p.cached = true; }
    else { p.group = 1024; p.rowsPerBlock = 1; p.threads = 1024; p.cached = features <= size_t(1024) * maxElemsPerThread; }
    return p;
}

}  // namespace bf
