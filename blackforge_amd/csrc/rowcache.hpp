// Register-resident rows for the row-wise kernels (rmsnorm, softmax, cross-entropy).
//
// A "group" of G threads (64 = one wavefront, or a whole block of 256 / 1024) owns one row and keeps
// up to MAXE elements per thread in registers, so multi-pass algorithms (max, sum, normalise) read
// the row from HBM exactly once.  Rows longer than G*MAXE fall back to re-reading global memory
// (served by L2).  VEC = 4 uses dwordx4 accesses and needs 16-byte aligned rows (features % 4 == 0
// and an aligned base); VEC = 1 handles every other shape with coalesced dword accesses.  loadShifted /
// storeShifted give rows of ANY length and alignment the 16-byte accesses too: the row is addressed from an
// aligned boundary at or below its first element, `shift` elements earlier (the 16-byte boundary, shift 0..3, or
// the 128-byte line, shift 0..31, after which every wavefront access covers whole lines: 8 % faster on rows of
// 50 257 floats), and the elements a group holds from outside the row are masked.  A shifted access touches the bytes
// from the row's first element rounded DOWN to the boundary (16 or 128 bytes) to its end rounded UP to 16 bytes, and
// nothing else; nothing outside the row is written.  Callers use the 128-byte boundary only for tensors that start on
// a 128-byte line (the first row then has shift 0, every other row's line holds the tail of the row before it), so
// reads stay inside the tensor except for at most 12 bytes after its last element, inside the same 16-byte group.
#pragma once

// BF_ROWCACHE_HOST_MODEL: a host program (tests/cpp/rowcache_bounds_test.cpp) compiles RowCache itself with accessors
// of its own (ldf4, stf4, ...) that check every address the shifted accesses touch; it defines what common.hpp would.
#if !defined(BF_ROWCACHE_HOST_MODEL)
#include "common.hpp"
#endif

namespace bf {

#if defined(__HIPCC__) || defined(BF_ROWCACHE_HOST_MODEL)

// NT: accesses carry the non-temporal hint (rows streamed past the last-level cache, see ldf4 / stf4).
template <int G, int MAXE, int VEC, bool NT = false>
struct RowCache {
    static constexpr int kIters = MAXE / VEC;
    float r[MAXE];

    // element index handled by (iteration it, vector slot j) for group-thread t
    __device__ static size_t index(int it, int t, int j) { return (size_t(it) * G + t) * VEC + j; }

    __device__ __forceinline__ void load(const float* __restrict__ row, size_t features, int t, float fill) {
        issue<0, kIters>(row, features, t, fill);
    }

    // Iterations [B, E) of the row only: a kernel that walks rows issues the next row's loads in pieces, as registers
    // come free.
    template <int B, int E>
    __device__ __forceinline__ void issue(const float* __restrict__ row, size_t features, int t, float fill) {
#pragma unroll
        for (int it = B; it < E; ++it) {
            size_t e = index(it, t, 0);
            if constexpr (VEC == 4) {
                if (e < features) {
                    float4v v = ldf4<NT>(row + e);
                    r[it * 4 + 0] = v.x; r[it * 4 + 1] = v.y; r[it * 4 + 2] = v.z; r[it * 4 + 3] = v.w;
                } else {
                    r[it * 4 + 0] = r[it * 4 + 1] = r[it * 4 + 2] = r[it * 4 + 3] = fill;
                }
            } else {
                r[it] = e < features ? ldf1<NT>(row + e) : fill;
            }
        }
    }

    // Elements before the row's first one in the 16-byte group that holds it (mask 3), or in the 128-byte line that holds
    // it (mask 31: every wavefront access then covers whole lines).
    __device__ static int shiftOf(const float* row, unsigned mask = 3u) { return int((reinterpret_cast<uintptr_t>(row) >> 2) & mask); }

    // Rows are shorter than 2^31 - 32 elements here (G * MAXE elements at most), so 32-bit indices do.  Only the groups
    // up to the one that holds the row's first element (iteration 0) and the one that holds its last need any masking.
    __device__ __forceinline__ void loadShifted(const float* __restrict__ row, size_t features, int t, float fill, int shift) {
        // every load first (a group past the row's end re-reads group 0 instead of branching), the masking afterwards:
        // code between the loads that touches a loaded register would make each load wait for the one before it
        issueShifted<0, kIters>(row, features, t, shift);
        maskShifted(features, t, fill, shift);
    }

    // The loads of iterations [B, E) of a shifted row, unmasked: maskShifted (with the same row's shift) comes before
    // the first use, and is the first thing that waits for the loads.
    template <int B, int E>
    __device__ __forceinline__ void issueShifted(const float* __restrict__ row, size_t features, int t, int shift) {
        static_assert(VEC == 4, "shifted access is 4 wide");
        const float* base = row - shift;
        const int last = int(features) + shift;   // one past the row's last element, counted from base
#pragma unroll
        for (int it = B; it < E; ++it) {
            const int g = (it * G + t) * 4;
            const float4v v = ldf4<NT>(base + (g < last ? g : 0));
            r[it * 4 + 0] = v.x; r[it * 4 + 1] = v.y; r[it * 4 + 2] = v.z; r[it * 4 + 3] = v.w;
        }
    }

    __device__ __forceinline__ void maskShifted(size_t features, int t, float fill, int shift) {
        const int last = int(features) + shift;
        const int lo = shift - 4 * t;   // slots of this thread's first group that lie before the row (<= 0: none)
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            const int n = last - (it * G + t) * 4;   // slots of this group before the row's end (>= 4: all of them)
            const int first = it == 0 ? lo : 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) r[it * 4 + j] = (j >= first && j < n) ? r[it * 4 + j] : fill;
        }
    }

    __device__ __forceinline__ void storeShifted(float* __restrict__ row, size_t features, int t, int shift) const {
        static_assert(VEC == 4, "shifted access is 4 wide");
        float* base = row - shift;
        const int last = int(features) + shift;
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            const int g = (it * G + t) * 4;
            if (g < last) {
                const bool head = it == 0 && g < shift, tail = g + 4 > last;   // a group that starts before the row
                if (!head && !tail) {
                    stf4<NT>(base + g, float4v{r[it * 4 + 0], r[it * 4 + 1], r[it * 4 + 2], r[it * 4 + 3]});
                } else {   // a group that straddles an end of the row: its own elements one by one
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (g + j >= shift && g + j < last) base[g + j] = r[it * 4 + j];
                }
            }
        }
    }

    // The row rounded to bf16 (nearest even), for rows that are the operand of a bf16 GEMM: row[e] = bf16(r[e]).
    __device__ __forceinline__ void storeBf16(unsigned short* __restrict__ row, size_t features, int t) const {
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            size_t e = index(it, t, 0);
            if (e < features) {
                if constexpr (VEC == 4) {
                    const uint2v packed = {unsigned(toBf16Bits(r[it * 4 + 0])) | unsigned(toBf16Bits(r[it * 4 + 1])) << 16,
                                           unsigned(toBf16Bits(r[it * 4 + 2])) | unsigned(toBf16Bits(r[it * 4 + 3])) << 16};
                    stu2<NT>(row + e, packed);
                } else {
                    row[e] = toBf16Bits(r[it]);
                }
            }
        }
    }

    __device__ __forceinline__ void store(float* __restrict__ row, size_t features, int t) const {
#pragma unroll
        for (int it = 0; it < kIters; ++it) {
            size_t e = index(it, t, 0);
            if (e < features) {
                if constexpr (VEC == 4) {
                    float4v v = {r[it * 4 + 0], r[it * 4 + 1], r[it * 4 + 2], r[it * 4 + 3]};
                    stf4<NT>(row + e, v);
                } else {
                    stf1<NT>(row + e, r[it]);
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

#endif  // __HIPCC__ || BF_ROWCACHE_HOST_MODEL

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
