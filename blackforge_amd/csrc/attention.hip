// Fused causal attention, forward and backward, fp32 in and out.  Two sets of kernels for the forward pass and for
// dK/dV, chosen by bf_hip_attention_set_route: every product on the fp32 MFMA (v_mfma_f32_32x32x2_f32; the kernels
// described first), or, by default, every fp32 product as six bf16 MFMAs on operands split into three bf16 terms
// (attnForwardPipedKernel, attnBackwardDkvSplitKernel, attnBackwardDkvPipedKernel further down; same ownership, tiling
// and statistics, fp32 accuracy), and likewise for the dQ kernel that reads the stored dS
// (attnBackwardDqFromDsSplitKernel).  The dQ kernel that recomputes S and dP runs on the fp32 MFMA on both routes.
//
// Layout: q [batch,newLen,dim], k/v [batch,totalLen,dim], heads contiguous in dim.  Query row i
// (absolute position oldLen+i) attends to keys j <= oldLen+i.
//
// MFMA kernels, all with 256-thread workgroups (4 wavefronts, one per SIMD), 32 rows per wave:
//   forward : a workgroup owns 128 query rows, streams K/V tiles through LDS (double buffered, one barrier
//             per tile, next tile's global loads in flight in registers), online softmax.
//   dK/dV   : a workgroup owns 128 keys (K, V and both accumulators live in registers), streams
//             Q/dO tiles through LDS, writes dK and dV once.  On the default route it also leaves
//             dS = P o (dP - D) behind in a hand-over buffer [batch, heads, totalLen, newLen].
//   dQ      : default route: one contraction dQ = scale * dS * K over the hand-over buffer (no exp, no second
//             pass over Q and dO).  When the buffer would exceed the workspace limit, the recompute route: the
//             same ownership as forward, P rebuilt from the saved statistics, and the dK/dV kernel keeps dS to itself.
// No atomics anywhere, so gradients are bit-reproducible.  Every kernel can write a bf16 image of its result beside
// (or instead of) the fp32 tensor, for the projections that read it next.
//
// Orientation trick (what makes the softmax cheap on 64-wide waves).  With the 32x32x2 MFMA
//   A: lane l holds A[i = l%32][k = l/32]      B: lane l holds B[k = l/32][j = l%32]
//   D: lane l, reg r holds D[i = 8*(r/4) + 4*(l/32) + r%4][j = l%32]
// the query-owner kernels compute S^T = K * Q^T (M = keys, N = queries).  A lane then holds 16 keys of
// ONE query column, so row max / row sum are 16 in-register operations plus one exchange with lane^32,
// and P^T in D layout is already in B-operand layout for O^T = V^T * P^T (the k index of step r is the
// key held in register r), so P never leaves registers.  The key-owner kernel computes S = Q * K^T
// (M = queries, N = keys), whose D layout is the A-operand layout of dV = P^T * dO and dK = dS^T * Q.
// Because a dot product does not care about the order of its terms, the k index of MFMA step t is
// taken as (t, HD/2 + t) for the two lane halves, which makes every LDS operand read a contiguous
// ds_read_b128.
//
// Head dims are padded in registers/LDS to HDP in {32, 64, 128, 256}; any headDim <= 256 and any
// newLen/totalLen/oldLen are accepted (tiles are zero-filled and masked).
#include "common.hpp"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdint>

namespace bf {
namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct AttnParams {
    const float* q; const float* k; const float* v; const float* o; const float* dO;
    const float* lse2;   // [batch, heads, newLen]: m*log2(e) + log2(l)
    const float* dvec;   // [batch, heads, newLen]: dot(O, dO)
    float* out; float* m; float* l;
    float* dQ; float* dK; float* dV;
    // bf16 images (rounded to nearest even) of the outputs, for consumers that are bf16 GEMMs: row r of a [rows, dim]
    // output lies at img + r * imgLd (imgLd >= dim, so that dQ, dK and dV can be column slices of one wider image).
    // Each is optional; with an image given the fp32 tensor of the same output may be NULL.
    unsigned short* outImg; unsigned short* dQImg; unsigned short* dKImg; unsigned short* dVImg;
    size_t imgLd;
    float* ds;           // [batch*heads, nqb, nkb, 32 queries, 32 keys]: dS sub-blocks handed from dK/dV to dQ (or null)
    int nqb, nkb;        // query / key sub-blocks of 32 per (batch, head)
    int batch, heads, newLen, totalLen, dim, hd, oldLen;
    float scale;
    int numTiles;        // query tiles (forward, dQ) or key tiles (dK/dV) per (batch, head)
    // Forward pass over the keys in chunks (few queries, many keys: one step of incremental decoding): workgroup row
    // blockIdx.y takes keys [y * chunkKeys, ...), the last chunk everything that is left, and writes its normalised
    // output and its statistics `partOutStride` / `partStatStride` floats after the chunk before it (applyKeyChunk);
    // attnCombineChunksKernel puts the chunks together.  numChunks <= 1: the whole key range, as everywhere else.
    int kvRows;          // rows per batch element of the K and V tensors (totalLen, whatever the chunk)
    int chunkKeys, numChunks;
    size_t partOutStride, partStatStride;
    // attnFewQueriesKernel only: when set, the number of cached positions is read from here instead of oldLen (a step
    // launched before the host knows the position); the chunks then cover all kvRows and may be empty
    const int* oldLenPtr;
};

// A forward kernel's first statement: narrows the parameters to this workgroup's chunk of keys.  Every chunk starts at
// or before the first query's own position (the host sees to that), so every query sees a key in every chunk.
__device__ __forceinline__ void applyKeyChunk(AttnParams& p) {
    if (p.numChunks <= 1) return;
    const int c = blockIdx.y, c0 = c * p.chunkKeys;
    const size_t skip = size_t(c0) * p.dim;
    p.k += skip;
    p.v += skip;
    p.totalLen = c == p.numChunks - 1 ? p.totalLen - c0 : p.chunkKeys;
    p.oldLen -= c0;
    p.out += size_t(c) * p.partOutStride;
    p.m += size_t(c) * p.partStatStride;
    p.l += size_t(c) * p.partStatStride;
}

// A chunk whose keys all lie after the last query of a workgroup's tile (a causal pass from position 0 whose keys are
// taken in chunks: the upper right of the triangle): the tile's rows get zero output, maximum -inf and sum 0 for this
// chunk, which attnCombineChunksKernel weighs with zero.  Chunk starts are multiples of 128 like the tiles' first
// queries, so a chunk is either empty for a whole tile or holds a visible key for each of its rows.
__device__ __forceinline__ bool chunkIsEmptyFor(const AttnParams& p, int qt) {
    return p.numChunks > 1 && p.oldLen + min(p.newLen, qt * 128 + 128) <= 0;   // p.oldLen: already relative to the chunk's first key
}
__device__ __forceinline__ void writeEmptyChunk(const AttnParams& p, int b, int h, int qt) {
    const int rows = min(128, p.newLen - qt * 128);
    for (int e = threadIdx.x; e < rows * p.hd; e += 256) {
        const int r = e / p.hd, d = e - r * p.hd;
        p.out[(size_t(b) * p.newLen + qt * 128 + r) * p.dim + size_t(h) * p.hd + d] = 0.0f;
    }
    for (int r = threadIdx.x; r < rows; r += 256) {
        const size_t at = (size_t(b) * p.heads + h) * p.newLen + qt * 128 + r;
        p.m[at] = -INFINITY;
        p.l[at] = 0.0f;
    }
}

__device__ __forceinline__ float fastExp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Workgroup -> (batch*head, tile), heaviest tiles first over ALL (batch, head) pairs: causal tiles differ in
// work by up to numTiles x, and a heavy tile that starts late sets the kernel's makespan.  Consecutive
// workgroup ids walk the (batch, head) pairs at one tile level; the hardware deals workgroups round-robin to
// the 8 XCDs, so with a pair count divisible by 8 every pair stays on one XCD, and the tiles of a pair that
// are dispatched together stream through the same K/V (or Q/dO) tiles at the same time and share them in
// that XCD's L2.
__device__ __forceinline__ void decodeBlock(int numTiles, int totalBlocks, bool heavyIsLast, int& bh, int& tile) {
    const int id = blockIdx.x;
    const int numPairs = totalBlocks / numTiles;
    const int level = id / numPairs;   // 0 = heaviest
    bh = id - level * numPairs;
    tile = heavyIsLast ? numTiles - 1 - level : level;
}

// Cooperative copy of ROWS rows of one head ([row][hd] slices of a [.., dim] tensor) into LDS as
// [ROWS][HDP+4], zero-filling rows >= rowLimit and columns >= hd.  Split in two so that the global loads of
// a LATER tile are in flight while the current one is being consumed: fetchHeadTile issues the loads into
// registers, commitHeadTile writes them to LDS.
template <int HDP, int ROWS>
struct TileRegs {
    static constexpr int kSlots = (ROWS * (HDP / 4) + 255) / 256;
    float4v v[kSlots];
};

template <int HDP, int ROWS, bool VEC4>
__device__ __forceinline__ void fetchHeadTile(TileRegs<HDP, ROWS>& regs, const float* __restrict__ base, int dim, int row0,
                                              int rowLimit, int hd, int tid) {
    constexpr int V4 = HDP / 4;
    constexpr int SLOTS = ROWS * V4;
#pragma unroll
    for (int i = 0; i < TileRegs<HDP, ROWS>::kSlots; ++i) {
        int s = tid + i * 256;
        int r = s / V4, c = (s % V4) * 4;
        int row = row0 + r;
        float4v val = {0.0f, 0.0f, 0.0f, 0.0f};
        if (s < SLOTS && row < rowLimit && c < hd) {
            const float* src = base + size_t(row) * dim + c;
            if constexpr (VEC4) {
                val = loadf4(src);
            } else {
                val.x = src[0];
                if (c + 1 < hd) val.y = src[1];
                if (c + 2 < hd) val.z = src[2];
                if (c + 3 < hd) val.w = src[3];
            }
        }
        regs.v[i] = val;
    }
}

// The same tile for a caller that can take any finite values in rows past the limit (it multiplies them by zero): the
// row index is clamped instead of tested, and the column's pointer and validity are the thread's constants.  16-byte
// aligned rows only.
template <int HDP, int ROWS>
__device__ __forceinline__ void fetchRowsClamped(TileRegs<HDP, ROWS>& regs, const float* __restrict__ columnBase, bool columnValid, int dim,
                                                 int row0, int lastRow, int tid) {
    constexpr int V4 = HDP / 4;
    static_assert((ROWS * V4) % 256 == 0, "every thread takes the same number of slots");
#pragma unroll
    for (int i = 0; i < TileRegs<HDP, ROWS>::kSlots; ++i) {
        const int row = min(row0 + (tid + i * 256) / V4, lastRow);
        regs.v[i] = columnValid ? loadf4(columnBase + size_t(row) * dim) : float4v{0.0f, 0.0f, 0.0f, 0.0f};
    }
}

template <int HDP, int ROWS>
__device__ __forceinline__ void commitHeadTile(float* __restrict__ lds, const TileRegs<HDP, ROWS>& regs, int tid) {
    constexpr int LDSW = HDP + 4;
    constexpr int V4 = HDP / 4;
    constexpr int SLOTS = ROWS * V4;
#pragma unroll
    for (int i = 0; i < TileRegs<HDP, ROWS>::kSlots; ++i) {
        int s = tid + i * 256;
        if (s < SLOTS) storef4(lds + (s / V4) * LDSW + (s % V4) * 4, regs.v[i]);
    }
}

// Loads this lane's half of one head row as MFMA operand registers: reg[t] = row[half*HDP/2 + t] * mul.
template <int HDP, bool VEC4>
__device__ __forceinline__ void loadRowOperand(float (&reg)[HDP / 2], const float* __restrict__ row, bool valid, int hd,
                                               int half, float mul) {
    constexpr int HALF = HDP / 2;
#pragma unroll
    for (int t = 0; t < HALF; t += 4) {
        int d = half * HALF + t;
        float4v val = {0.0f, 0.0f, 0.0f, 0.0f};
        if (valid && d < hd) {
            if constexpr (VEC4) {
                val = loadf4(row + d);
            } else {
                val.x = row[d];
                if (d + 1 < hd) val.y = row[d + 1];
                if (d + 2 < hd) val.z = row[d + 2];
                if (d + 3 < hd) val.w = row[d + 3];
            }
        }
        reg[t] = val.x * mul; reg[t + 1] = val.y * mul; reg[t + 2] = val.z * mul; reg[t + 3] = val.w * mul;
    }
}

// acc (32x32) += A * B with A rows read from LDS (row `ldsRow`, this lane's half, ds_read_b128) and B
// from operand registers: the contraction over the head dimension.
template <int HDP>
__device__ __forceinline__ float16v headDot(const float* __restrict__ ldsRow, const float (&breg)[HDP / 2], float16v acc) {
#pragma unroll
    for (int t = 0; t < HDP / 2; t += 4) {
        float4v a = loadf4(ldsRow + t);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, breg[t], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, breg[t + 1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, breg[t + 2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, breg[t + 3], acc, 0, 0, 0);
    }
    return acc;
}
// Same contraction with the register operand on the A side (key-owner kernel).
template <int HDP>
__device__ __forceinline__ float16v headDotB(const float* __restrict__ ldsRow, const float (&areg)[HDP / 2], float16v acc) {
#pragma unroll
    for (int t = 0; t < HDP / 2; t += 4) {
        float4v a = loadf4(ldsRow + t);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, areg[t], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, areg[t + 1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, areg[t + 2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, areg[t + 3], acc, 0, 0, 0);
    }
    return acc;
}

// Two such contractions at once (S = Q K^T and dP = dO V^T of the key-owner kernel), their MFMAs alternating: a
// 32x32x2 MFMA whose accumulator is the previous instruction's result issues a few clocks late, so two independent
// accumulator chains keep the matrix pipe fuller than one chain after the other.
template <int HDP>
__device__ __forceinline__ void headDotPairB(const float* __restrict__ ldsRow0, const float* __restrict__ ldsRow1,
                                             const float (&reg0)[HDP / 2], const float (&reg1)[HDP / 2], float16v& acc0, float16v& acc1) {
#pragma unroll
    for (int t = 0; t < HDP / 2; t += 4) {
        const float4v a0 = loadf4(ldsRow0 + t), a1 = loadf4(ldsRow1 + t);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.x, reg0[t], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.x, reg1[t], acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.y, reg0[t + 1], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.y, reg1[t + 1], acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.z, reg0[t + 2], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.z, reg1[t + 2], acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.w, reg0[t + 3], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.w, reg1[t + 3], acc1, 0, 0, 0);
    }
}

// Row index inside a 32-row MFMA block held by register r of a lane in half `half`.
__device__ __forceinline__ int dRow(int r, int half) { return 8 * (r >> 2) + 4 * half + (r & 3); }

// Stores a transposed accumulator (rows = head-dim index, column = this lane's query/key row) to
// row `dst` of a [.., dim] tensor: element d = dt*32 + dRow(r, half).
template <int HDP, bool VEC4>
__device__ __forceinline__ void storeTransposed(float* __restrict__ dst, const float16v (&acc)[HDP / 32], int hd, int half,
                                                float mul) {
#pragma unroll
    for (int dt = 0; dt < HDP / 32; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            int d = dt * 32 + 8 * g + 4 * half;
            if (d < hd) {
                float4v val = {acc[dt][4 * g] * mul, acc[dt][4 * g + 1] * mul, acc[dt][4 * g + 2] * mul, acc[dt][4 * g + 3] * mul};
                if constexpr (VEC4) {
                    storef4(dst + d, val);
                } else {
                    dst[d] = val.x;
                    if (d + 1 < hd) dst[d + 1] = val.y;
                    if (d + 2 < hd) dst[d + 2] = val.z;
                    if (d + 3 < hd) dst[d + 3] = val.w;
                }
            }
        }
}

// The same accumulator as a row of a bf16 image: four consecutive head-dim elements are one 8-byte store.
template <int HDP, bool VEC4>
__device__ __forceinline__ void storeTransposedBf16(unsigned short* __restrict__ dst, const float16v (&acc)[HDP / 32], int hd, int half,
                                                    float mul) {
#pragma unroll
    for (int dt = 0; dt < HDP / 32; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            int d = dt * 32 + 8 * g + 4 * half;
            if (d < hd) {
                const unsigned short b0 = toBf16Bits(acc[dt][4 * g] * mul), b1 = toBf16Bits(acc[dt][4 * g + 1] * mul),
                                     b2 = toBf16Bits(acc[dt][4 * g + 2] * mul), b3 = toBf16Bits(acc[dt][4 * g + 3] * mul);
                if constexpr (VEC4) {
                    const uint2v packed = {unsigned(b0) | unsigned(b1) << 16, unsigned(b2) | unsigned(b3) << 16};
                    *reinterpret_cast<uint2v*>(dst + d) = packed;
                } else {
                    dst[d] = b0;
                    if (d + 1 < hd) dst[d + 1] = b1;
                    if (d + 2 < hd) dst[d + 2] = b2;
                    if (d + 3 < hd) dst[d + 3] = b3;
                }
            }
        }
}

// ---------------------------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------------------------
// One K/V tile (BC keys = BC/32 sub-blocks) for one wavefront, as straight-line code so that the
// instruction scheduler can overlap the matrix pipe with the vector pipe inside a single wave: the score
// MFMAs of sub-block sb+1 are issued BEFORE the softmax arithmetic of sub-block sb in program order, and do
// not depend on it, so exp/max/rescale run in the shadow of those MFMAs.  MASKED = false is the interior
// of the causal triangle (every key of the tile visible to every row of the wave).
//
// Lazy rescaling: exponentials are taken relative to a reference maximum `mref` that only moves when the running row
// maximum `mrow` has grown past it by more than kRescaleThreshold (in log2 units), so probabilities stay below 2^8 and
// the accumulator/row-sum rescale -- 32+ multiplies that sit between two groups of dependent MFMAs -- runs only in
// the tiles where some row of the wavefront needs it (a wave-uniform branch; for typical scores that is the first
// tile only).  The result is the same sum taken about a different reference point; the true maximum is tracked
// separately for the statistics the backward pass reads.
constexpr float kRescaleThreshold = 8.0f;
template <int HDP, int BC, bool MASKED>
__device__ __forceinline__ void forwardTile(const float* __restrict__ ks, const float* __restrict__ vs,
                                            const float (&qreg)[HDP / 2], float16v (&acc)[HDP / 32], float& mrow, float& mref,
                                            float& lrow, int kt0, int myLimit, int totalLen, int half, int li) {
    constexpr int LDSW = HDP + 4, DT = HDP / 32, NSB = BC / 32;
    float16v s[NSB];
#pragma unroll
    for (int r = 0; r < 16; ++r) s[0][r] = 0.0f;
    s[0] = headDot<HDP>(ks + li * LDSW + half * (HDP / 2), qreg, s[0]);
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
        if (sb + 1 < NSB) {
#pragma unroll
            for (int r = 0; r < 16; ++r) s[sb + 1][r] = 0.0f;
            s[sb + 1] = headDot<HDP>(ks + ((sb + 1) * 32 + li) * LDSW + half * (HDP / 2), qreg, s[sb + 1]);
        }
        float16v& sc = s[sb];   // sc[r] = log2-scaled score of (key = kt0 + sb*32 + dRow(r), this lane's query)
        if constexpr (MASKED) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                int key = kt0 + sb * 32 + dRow(r, half);
                sc[r] = (key > myLimit || key >= totalLen) ? -INFINITY : sc[r];
            }
        }
        float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
#pragma unroll
        for (int r = 4; r < 16; r += 4) mx = fmaxf(mx, fmaxf(fmaxf(sc[r], sc[r + 1]), fmaxf(sc[r + 2], sc[r + 3])));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        mrow = fmaxf(mrow, mx);
        const bool moveRef = mrow > mref + kRescaleThreshold;   // also true on the first visible key (mref = -inf)
        if (__builtin_amdgcn_ballot_w64(moveRef) != 0) {
            const float corr = moveRef ? fastExp2(mref - mrow) : 1.0f;   // 0 when the reference was still -inf
            mref = moveRef ? mrow : mref;
            lrow *= corr;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[dt][r] *= corr;
        }
        float psum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) { sc[r] = fastExp2(sc[r] - mref); psum += sc[r]; }
        lrow += psum;
        // O^T += V^T * P^T : step r contracts over key dRow(r, half)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float* vrow = vs + (sb * 32 + dRow(r, half)) * LDSW + li;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                acc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[dt * 32], sc[r], acc[dt], 0, 0, 0);
        }
    }
}

// operands of __builtin_amdgcn_global_load_lds (global memory straight into LDS)
typedef __attribute__((address_space(1))) const void* GlobalPtr;
typedef __attribute__((address_space(3))) void* LdsPtr;

// Streaming schedule shared by the three kernels (LDS double buffering, ONE barrier per tile):
//   iteration t consumes buffer t&1, then writes tile t+1 (already in registers) into buffer (t+1)&1 and
//   issues the global loads of tile t+2; the barrier at the end of the iteration both publishes tile t+1
//   and guarantees every wave is done reading buffer t&1 before iteration t+1 overwrites it with tile t+2.
template <int HDP, int BC, bool VEC4>
__global__ void __launch_bounds__(256, HDP <= 128 ? 2 : 1) attnForwardKernel(AttnParams p) {
    applyKeyChunk(p);
    constexpr int LDSW = HDP + 4, DT = HDP / 32, TILE = BC * LDSW;
    extern __shared__ float smem[];
    float* ks = smem;               // [2][BC][LDSW]
    float* vs = smem + 2 * TILE;    // [2][BC][LDSW]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    int bh, qt;
    decodeBlock(p.numTiles, gridDim.x, true, bh, qt);
    const int b = bh / p.heads, h = bh - b * p.heads;
    if (chunkIsEmptyFor(p, qt)) {                 // the same for the whole workgroup, before any barrier
        writeEmptyChunk(p, b, h, qt);
        return;
    }
    const int hd = p.hd, dim = p.dim;
    const float* qb = p.q + size_t(b) * p.newLen * dim + size_t(h) * hd;
    const float* kb = p.k + size_t(b) * p.kvRows * dim + size_t(h) * hd;
    const float* vb = p.v + size_t(b) * p.kvRows * dim + size_t(h) * hd;

    const int waveQ0 = qt * 128 + wave * 32;
    const int i = waveQ0 + li;                    // this lane's query row
    const bool rowValid = i < p.newLen;
    float qreg[HDP / 2];
    loadRowOperand<HDP, VEC4>(qreg, qb + size_t(i) * dim, rowValid, hd, half, p.scale * kLog2e);

    float16v acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.0f;
    float mrow = -INFINITY, mref = -INFINITY, lrow = 0.0f;

    const int lastQuery = min(p.newLen, qt * 128 + 128) - 1;
    const int blockKeyEnd = min(p.totalLen, p.oldLen + lastQuery + 1);   // keys >= this are invisible to the tile
    const int waveKeyEnd = p.oldLen + waveQ0 + 32;                       // keys >= this are invisible to the wave
    const int myLimit = p.oldLen + i;                                    // last visible key of this lane's row
    const int numKeyTiles = (blockKeyEnd + BC - 1) / BC;

    auto tileBody = [&](int t) __attribute__((always_inline)) {
        const int kt0 = t * BC;
        const float* kcur = ks + (t & 1) * TILE;
        const float* vcur = vs + (t & 1) * TILE;
        if (kt0 < waveKeyEnd) {   // wave-uniform: the tile holds keys some row of this wave can see
            // interior of the causal triangle: every key visible to every row of the wave, no masking arithmetic
            const bool masked = (kt0 + BC - 1 > p.oldLen + waveQ0) || (kt0 + BC > p.totalLen);
            if (masked) forwardTile<HDP, BC, true>(kcur, vcur, qreg, acc, mrow, mref, lrow, kt0, myLimit, p.totalLen, half, li);
            else forwardTile<HDP, BC, false>(kcur, vcur, qreg, acc, mrow, mref, lrow, kt0, myLimit, p.totalLen, half, li);
        }
    };
    if constexpr (VEC4 && HDP > 128) {
        // Head dims above 128: the Q rows and the accumulators leave no registers for two tiles in flight (53 spilled at 256),
        // so K and V tiles go from global memory straight into LDS (global_load_lds: one row per wavefront instruction,
        // 16 bytes a lane, lanes past the head dim switched off and their columns zeroed once), one tile ahead of its
        // use: a tile's products last several microseconds.  Rows past the sequence repeat its last row: finite values
        // under a mask.
        const int waveU = __builtin_amdgcn_readfirstlane(wave);
        const bool columnValid = 4 * lane < hd;
        const float* kBase = kb + 4 * lane;
        const float* vBase = vb + 4 * lane;
        auto issueTile = [&](int kt0, int buf) __attribute__((always_inline)) {
#pragma unroll
            for (int r4 = 0; r4 < BC / 4; ++r4) {
                const int r = waveU + 4 * r4;
                const size_t row = size_t(min(kt0 + r, p.totalLen - 1)) * dim;
                if (columnValid) {
                    __builtin_amdgcn_global_load_lds((GlobalPtr)(kBase + row), (LdsPtr)(ks + buf * TILE + r * LDSW), 16, 0, 0);
                    __builtin_amdgcn_global_load_lds((GlobalPtr)(vBase + row), (LdsPtr)(vs + buf * TILE + r * LDSW), 16, 0, 0);
                }
            }
        };
        if (hd < HDP) {   // the columns past the head dim are never loaded: zero them once (both buffers of both tiles)
            for (int z = tid; z < 4 * BC * (LDSW / 4); z += 256) storef4(ks + 4 * z, float4v{0.0f, 0.0f, 0.0f, 0.0f});
            __syncthreads();
        }
        issueTile(0, 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        for (int t = 0; t < numKeyTiles; ++t) {
            if (t + 1 < numKeyTiles) issueTile((t + 1) * BC, (t + 1) & 1);   // that buffer was last read before the barrier above
            tileBody(t);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        }
    } else {
        TileRegs<HDP, BC> kNext, vNext;
        fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, 0, p.totalLen, hd, tid);
        fetchHeadTile<HDP, BC, VEC4>(vNext, vb, dim, 0, p.totalLen, hd, tid);
        commitHeadTile<HDP, BC>(ks, kNext, tid);
        commitHeadTile<HDP, BC>(vs, vNext, tid);
        if (numKeyTiles > 1) {
            fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, BC, p.totalLen, hd, tid);
            fetchHeadTile<HDP, BC, VEC4>(vNext, vb, dim, BC, p.totalLen, hd, tid);
        }
        __syncthreads();
        for (int t = 0; t < numKeyTiles; ++t) {
            tileBody(t);
            if (t + 1 < numKeyTiles) {
                commitHeadTile<HDP, BC>(ks + ((t + 1) & 1) * TILE, kNext, tid);
                commitHeadTile<HDP, BC>(vs + ((t + 1) & 1) * TILE, vNext, tid);
                if (t + 2 < numKeyTiles) {
                    fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, t * BC + 2 * BC, p.totalLen, hd, tid);
                    fetchHeadTile<HDP, BC, VEC4>(vNext, vb, dim, t * BC + 2 * BC, p.totalLen, hd, tid);
                }
            }
            __syncthreads();
        }
    }

    lrow += __shfl_xor(lrow, 32, 64);
    if (rowValid) {
        if (p.out) storeTransposed<HDP, VEC4>(p.out + (size_t(b) * p.newLen + i) * dim + size_t(h) * hd, acc, hd, half, 1.0f / lrow);
        if (p.outImg) storeTransposedBf16<HDP, VEC4>(p.outImg + (size_t(b) * p.newLen + i) * p.imgLd + size_t(h) * hd, acc, hd, half, 1.0f / lrow);
        if (half == 0) {
            // statistics about the TRUE row maximum: l = sum exp(score - m) = (sum about mref) * 2^(mref - mrow)
            size_t idx = (size_t(b) * p.heads + h) * p.newLen + i;
            p.m[idx] = mrow * kLn2;
            p.l[idx] = lrow * fastExp2(mref - mrow);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// forward on the bf16 matrix pipe at fp32 accuracy
// ---------------------------------------------------------------------------------------------
// An fp32 value is the exact sum of three bf16 values, x = h + m + l (h = bf16(x), m = bf16(x - h), l = bf16(x - h - m);
// the remainders are exact in fp32), so a product of two fp32 operands is the sum of nine bf16 products, of which the six
// largest (h h', h m', m h', h l', l h', m m') carry everything above 2^-24 of the product: as accurate as the fp32 MFMA
// (closer to float64 in measurement), accumulated in fp32 by the same matrix unit.  v_mfma_f32_32x32x16_bf16 contracts
// sixteen elements in 32 clocks where v_mfma_f32_32x32x2_f32 contracts two in 64, so the six products cost 6/16 of the
// matrix time.  What it takes: operands as bf16 triples in the layout of that instruction (eight consecutive
// contraction elements per lane).
//   * K and V tiles are split when they are written to LDS (three bf16 images each, row-major).  S^T = K Q^T contracts
//     over the head dimension: a K fragment is 16 bytes of a row, Q fragments live in registers for the whole kernel.
//   * O^T += V^T P^T contracts over keys.  The score tile leaves the MFMA with lane (query, half) holding keys
//     8g + 4 half + 0..3; the contraction index may be permuted freely as long as both operands agree, so contraction
//     slot e of step s of a lane in `half` is DEFINED as key 16 s + 8 (e / 4) + 4 half + e % 4: the P operand is then
//     eight consecutive accumulator registers, split in place, and the V fragment is gathered for the same keys by the
//     transposing LDS read (two reads of four rows, eight rows apart).
// Everything else (online softmax, lazy rescaling, masks, statistics, stores) is the fp32 kernel's.
typedef __bf16 bf16x8a __attribute__((ext_vector_type(8)));
typedef short short4a __attribute__((ext_vector_type(4)));
typedef short short8a __attribute__((ext_vector_type(8)));

typedef __bf16 bf16x2a __attribute__((ext_vector_type(2)));
typedef float float2a __attribute__((ext_vector_type(2)));
typedef unsigned uint4a __attribute__((ext_vector_type(4)));

// two floats as a pair of bf16 (round to nearest even), the first in the low half: one v_cvt_pk_bf16_f32
__device__ __forceinline__ unsigned packBf16(float x0, float x1) {
    return __builtin_bit_cast(unsigned, __builtin_convertvector(float2a{x0, x1}, bf16x2a));
}

// x = h + m + l exactly, each term the bf16 nearest to what the terms before it leave; two values at a time so that
// every conversion fills both halves of its result (eleven instructions a pair)
__device__ __forceinline__ void splitPair3(float x0, float x1, unsigned& h, unsigned& m, unsigned& l) {
    h = packBf16(x0, x1);
    const float r0 = x0 - __builtin_bit_cast(float, h << 16), r1 = x1 - __builtin_bit_cast(float, h & 0xffff0000u);
    m = packBf16(r0, r1);
    l = packBf16(r0 - __builtin_bit_cast(float, m << 16), r1 - __builtin_bit_cast(float, m & 0xffff0000u));
}

// eight values (consecutive elements of an MFMA operand) as three operand terms
__device__ __forceinline__ void splitOperand(const float (&x)[8], bf16x8a& h, bf16x8a& m, bf16x8a& l) {
    uint4a hh, mm, ll;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        unsigned a, b, c;
        splitPair3(x[2 * e], x[2 * e + 1], a, b, c);
        hh[e] = a; mm[e] = b; ll[e] = c;
    }
    h = __builtin_bit_cast(bf16x8a, hh);
    m = __builtin_bit_cast(bf16x8a, mm);
    l = __builtin_bit_cast(bf16x8a, ll);
}

// rows p, p + pitch, p + 2 pitch, p + 3 pitch (as addressed by the lanes) and the same eight rows further down
__device__ __forceinline__ bf16x8a readTransposedApart(const unsigned short* p, int rowPitch) {
    typedef __attribute__((address_space(3))) short4a* LdsPtr;
    const short4a lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(p));
    const short4a hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(p + 8 * rowPitch));
    const short8a both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8a, both);
}

constexpr int splitKeyPitch(int hdp) { return hdp + 8; }                       // plain 16-byte fragment reads
constexpr int splitValuePitch(int hdp) { return hdp + 32 < 96 ? 96 : hdp + 32; }   // transposing reads: an odd multiple of 64 bytes

// One tile of ROWS rows from registers to three bf16 images [3][ROWS][PITCH].
template <int HDP, int ROWS, int PITCH>
__device__ __forceinline__ void commitSplitTile(unsigned short* __restrict__ img, const TileRegs<HDP, ROWS>& regs, int tid) {
    constexpr int V4 = HDP / 4, SLOTS = ROWS * V4, IMG = ROWS * PITCH;
#pragma unroll
    for (int i = 0; i < TileRegs<HDP, ROWS>::kSlots; ++i) {
        const int s = tid + i * 256;
        if (s < SLOTS) {
            unsigned h0, m0, l0, h1, m1, l1;
            splitPair3(regs.v[i][0], regs.v[i][1], h0, m0, l0);
            splitPair3(regs.v[i][2], regs.v[i][3], h1, m1, l1);
            const uint2v h = {h0, h1}, m = {m0, m1}, l = {l0, l1};
            unsigned short* dst = img + (s / V4) * PITCH + (s % V4) * 4;
            *reinterpret_cast<uint2v*>(dst) = h;
            *reinterpret_cast<uint2v*>(dst + IMG) = m;
            *reinterpret_cast<uint2v*>(dst + 2 * IMG) = l;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// backward, part 0: D = dot(O, dO) per (batch, head, row), and optionally the log2-domain
// log-sum-exp lse2 = m*log2(e) + log2(l).  16 lanes per (row, head); HBM-bound.
// ---------------------------------------------------------------------------------------------
template <bool VEC4>
__global__ void __launch_bounds__(256) attnDotKernel(const float* __restrict__ o, const float* __restrict__ dO,
                                                      const float* __restrict__ m, const float* __restrict__ l,
                                                      float* __restrict__ dvec, float* __restrict__ lse2, int batch, int heads,
                                                      int newLen, int dim, int hd) {
    const size_t groups = size_t(batch) * newLen * heads;    // (b, i, h) with h fastest: contiguous memory
    const size_t group = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) / 16;
    const int sub = threadIdx.x & 15;
    if (group >= groups) return;
    const size_t bi = group / heads;
    const int h = int(group - bi * heads);
    const float* po = o + bi * dim + size_t(h) * hd;
    const float* pg = dO + bi * dim + size_t(h) * hd;
    float acc = 0.0f;
    if constexpr (VEC4) {
        for (int d = sub * 4; d < hd; d += 64) {
            float4v a = loadf4(po + d), g = loadf4(pg + d);
            acc += a.x * g.x + a.y * g.y + a.z * g.z + a.w * g.w;
        }
    } else {
        for (int d = sub; d < hd; d += 16) acc += po[d] * pg[d];
    }
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (sub == 0) {
        const size_t b = bi / newLen, i = bi - b * newLen;
        const size_t idx = (b * heads + h) * newLen + i;
        dvec[idx] = acc;
        if (lse2) lse2[idx] = m[idx] * kLog2e + log2f(l[idx]);
    }
}

// ---------------------------------------------------------------------------------------------
// backward, part 1: dQ (query-tile owner).  Same streaming structure as the forward.
// ---------------------------------------------------------------------------------------------
// One K/V tile for one wavefront, straight-line and software-pipelined like forwardTile: the S^T and dP^T
// MFMAs of sub-block sb+1 are issued before the exp / dS arithmetic of sub-block sb.
template <int HDP, int BC, bool MASKED>
__device__ __forceinline__ void dqTile(const float* __restrict__ ks, const float* __restrict__ vs, const float (&qreg)[HDP / 2],
                                       const float (&greg)[HDP / 2], float16v (&acc)[HDP / 32], float lse, float dval, int kt0,
                                       int myLimit, int totalLen, int half, int li) {
    constexpr int LDSW = HDP + 4, DT = HDP / 32, NSB = BC / 32;
    float16v s[NSB], dp[NSB];
#pragma unroll
    for (int r = 0; r < 16; ++r) { s[0][r] = 0.0f; dp[0][r] = 0.0f; }
    // S^T = K * Q^T and dP^T = V * dO^T, their MFMAs alternating
    headDotPairB<HDP>(ks + li * LDSW + half * (HDP / 2), vs + li * LDSW + half * (HDP / 2), qreg, greg, s[0], dp[0]);
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
        if (sb + 1 < NSB) {
#pragma unroll
            for (int r = 0; r < 16; ++r) { s[sb + 1][r] = 0.0f; dp[sb + 1][r] = 0.0f; }
            headDotPairB<HDP>(ks + ((sb + 1) * 32 + li) * LDSW + half * (HDP / 2), vs + ((sb + 1) * 32 + li) * LDSW + half * (HDP / 2), qreg, greg,
                              s[sb + 1], dp[sb + 1]);
        }
        float16v& ds = s[sb];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            float prob = fastExp2(ds[r] - lse);
            if constexpr (MASKED) {
                int key = kt0 + sb * 32 + dRow(r, half);
                prob = (key > myLimit || key >= totalLen) ? 0.0f : prob;
            }
            ds[r] = prob * (dp[sb][r] - dval);   // dS^T (without the scale factor)
        }
        // dQ^T += K^T * dS^T : step r contracts over key dRow(r, half)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float* krow = ks + (sb * 32 + dRow(r, half)) * LDSW + li;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                acc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(krow[dt * 32], ds[r], acc[dt], 0, 0, 0);
        }
    }
}

template <int HDP, int BC, bool VEC4>
__global__ void __launch_bounds__(256, HDP <= 64 ? 2 : 1) attnBackwardDqKernel(AttnParams p) {
    constexpr int LDSW = HDP + 4, DT = HDP / 32, TILE = BC * LDSW;
    extern __shared__ float smem[];
    float* ks = smem;
    float* vs = smem + 2 * TILE;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    int bh, qt;
    decodeBlock(p.numTiles, gridDim.x, true, bh, qt);
    const int b = bh / p.heads, h = bh - b * p.heads;
    const int hd = p.hd, dim = p.dim;
    const size_t qOff = size_t(b) * p.newLen * dim + size_t(h) * hd;
    const float* kb = p.k + size_t(b) * p.totalLen * dim + size_t(h) * hd;
    const float* vb = p.v + size_t(b) * p.totalLen * dim + size_t(h) * hd;

    const int waveQ0 = qt * 128 + wave * 32;
    const int i = waveQ0 + li;
    const bool rowValid = i < p.newLen;
    float qreg[HDP / 2], greg[HDP / 2];
    loadRowOperand<HDP, VEC4>(qreg, p.q + qOff + size_t(i) * dim, rowValid, hd, half, p.scale * kLog2e);
    loadRowOperand<HDP, VEC4>(greg, p.dO + qOff + size_t(i) * dim, rowValid, hd, half, 1.0f);
    const size_t statIdx = (size_t(b) * p.heads + h) * p.newLen + i;
    const float lse = rowValid ? p.lse2[statIdx] : INFINITY;   // padding rows: exp2(s - inf) = 0
    const float dval = rowValid ? p.dvec[statIdx] : 0.0f;

    float16v acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.0f;

    const int lastQuery = min(p.newLen, qt * 128 + 128) - 1;
    const int blockKeyEnd = min(p.totalLen, p.oldLen + lastQuery + 1);
    const int waveKeyEnd = p.oldLen + waveQ0 + 32;
    const int myLimit = p.oldLen + i;
    const int numKeyTiles = (blockKeyEnd + BC - 1) / BC;

    TileRegs<HDP, BC> kNext, vNext;
    fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, 0, p.totalLen, hd, tid);
    fetchHeadTile<HDP, BC, VEC4>(vNext, vb, dim, 0, p.totalLen, hd, tid);
    commitHeadTile<HDP, BC>(ks, kNext, tid);
    commitHeadTile<HDP, BC>(vs, vNext, tid);
    if (numKeyTiles > 1) {
        fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, BC, p.totalLen, hd, tid);
        fetchHeadTile<HDP, BC, VEC4>(vNext, vb, dim, BC, p.totalLen, hd, tid);
    }
    __syncthreads();
    for (int t = 0; t < numKeyTiles; ++t) {
        const int kt0 = t * BC;
        const float* kcur = ks + (t & 1) * TILE;
        const float* vcur = vs + (t & 1) * TILE;
        if (kt0 < waveKeyEnd) {
            const bool masked = (kt0 + BC - 1 > p.oldLen + waveQ0) || (kt0 + BC > p.totalLen);
            if (masked) dqTile<HDP, BC, true>(kcur, vcur, qreg, greg, acc, lse, dval, kt0, myLimit, p.totalLen, half, li);
            else dqTile<HDP, BC, false>(kcur, vcur, qreg, greg, acc, lse, dval, kt0, myLimit, p.totalLen, half, li);
        }
        if (t + 1 < numKeyTiles) {
            commitHeadTile<HDP, BC>(ks + ((t + 1) & 1) * TILE, kNext, tid);
            commitHeadTile<HDP, BC>(vs + ((t + 1) & 1) * TILE, vNext, tid);
            if (t + 2 < numKeyTiles) {
                fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, kt0 + 2 * BC, p.totalLen, hd, tid);
                fetchHeadTile<HDP, BC, VEC4>(vNext, vb, dim, kt0 + 2 * BC, p.totalLen, hd, tid);
            }
        }
        __syncthreads();
    }
    if (rowValid) {
        if (p.dQ) storeTransposed<HDP, VEC4>(p.dQ + qOff + size_t(i) * dim, acc, hd, half, p.scale);
        if (p.dQImg) storeTransposedBf16<HDP, VEC4>(p.dQImg + (size_t(b) * p.newLen + i) * p.imgLd + size_t(h) * hd, acc, hd, half, p.scale);
    }
}

// ---------------------------------------------------------------------------------------------
// backward, part 1b: dQ from stored dS.  When the dK/dV kernel has left its dS sub-blocks in HBM, dQ = dS * K is a
// single contraction: a wave streams its 32 queries' row of sub-blocks (contiguous, 4 KiB each) into registers one
// tile ahead, while the K tiles go through LDS as in the kernels above.  Neither S nor dP is recomputed, so the
// backward pass executes the five products of the algorithm instead of seven.
// A sub-block is read exactly when its first key is visible to its last query; the dK/dV kernel writes all of those.
// ---------------------------------------------------------------------------------------------
constexpr int kDsPatch = 32 * 36;   // floats of LDS per staged dS sub-block

template <int HDP, int BC, bool VEC4>
__global__ void __launch_bounds__(256, HDP <= 64 ? 3 : HDP <= 128 ? 2 : 1) attnBackwardDqFromDsKernel(AttnParams p) {
    constexpr int LDSW = HDP + 4, DT = HDP / 32, TILE = BC * LDSW, NSB = BC / 32;
    extern __shared__ float smem[];
    float* ks = smem;   // [2][BC][LDSW]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    int bh, qt;
    decodeBlock(p.numTiles, gridDim.x, true, bh, qt);
    const int b = bh / p.heads, h = bh - b * p.heads;
    const int hd = p.hd, dim = p.dim;
    const size_t qOff = size_t(b) * p.newLen * dim + size_t(h) * hd;
    const float* kb = p.k + size_t(b) * p.totalLen * dim + size_t(h) * hd;

    const int waveQ0 = qt * 128 + wave * 32;
    const int i = waveQ0 + li;
    // keys below waveKeyEnd are visible to some query of this wave's sub-block row (none if the row is past newLen)
    const int waveKeyEnd = waveQ0 < p.newLen ? min(p.totalLen, p.oldLen + waveQ0 + 32) : 0;
    // A sub-block is fetched as it lies in memory (lane l takes bytes 16*l of each KiB: whole cache lines per 8 lanes)
    // and turned into B-operand layout (lane (li, half), registers 4g..4g+3 = dS[query li][keys 8g + 4*half ..+3])
    // through a wave-private LDS patch with rows padded to 36 floats; no barrier is involved, a wave's LDS
    // operations execute in order.
    const float* dsWave = p.ds + ((size_t(bh) * p.nqb + size_t(waveQ0 >> 5)) * p.nkb) * 1024 + lane * 4;
    float* stage = smem + 2 * TILE + wave * kDsPatch;   // one patch per wave, reused by its sub-blocks in turn

    float16v acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.0f;

    const int lastQuery = min(p.newLen, qt * 128 + 128) - 1;
    const int blockKeyEnd = min(p.totalLen, p.oldLen + lastQuery + 1);
    const int numKeyTiles = (blockKeyEnd + BC - 1) / BC;

    float4v dsNext[NSB][4];
    auto fetchDs = [&](int kt0) {
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
            const int k0 = kt0 + sb * 32;
            if (k0 < waveKeyEnd) {
                const float* src = dsWave + size_t(k0 >> 5) * 1024;
#pragma unroll
                for (int j = 0; j < 4; ++j) dsNext[sb][j] = __builtin_nontemporal_load(reinterpret_cast<const float4v*>(src + j * 256));
            }
        }
    };

    TileRegs<HDP, BC> kNext;
    fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, 0, p.totalLen, hd, tid);
    fetchDs(0);
    commitHeadTile<HDP, BC>(ks, kNext, tid);
    if (numKeyTiles > 1) fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, BC, p.totalLen, hd, tid);
    __syncthreads();
    for (int t = 0; t < numKeyTiles; ++t) {
        const int kt0 = t * BC;
        const float* kcur = ks + (t & 1) * TILE;
        float16v ds[NSB];
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
            if (kt0 + sb * 32 < waveKeyEnd) {
                float* patch = stage;
#pragma unroll
                for (int j = 0; j < 4; ++j) storef4(patch + (8 * j + (lane >> 3)) * 36 + (lane & 7) * 4, dsNext[sb][j]);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    float4v val = loadf4(patch + li * 36 + (2 * g + half) * 4);
                    ds[sb][4 * g] = val.x; ds[sb][4 * g + 1] = val.y; ds[sb][4 * g + 2] = val.z; ds[sb][4 * g + 3] = val.w;
                }
            }
        }
        if (t + 1 < numKeyTiles) fetchDs(kt0 + BC);
#pragma unroll
        for (int sb = 0; sb < NSB; ++sb) {
            if (kt0 + sb * 32 < waveKeyEnd) {
                // dQ^T += K^T * dS^T : step r contracts over key dRow(r, half)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float* krow = kcur + (sb * 32 + dRow(r, half)) * LDSW + li;
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
                        acc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(krow[dt * 32], ds[sb][r], acc[dt], 0, 0, 0);
                }
            }
        }
        if (t + 1 < numKeyTiles) {
            commitHeadTile<HDP, BC>(ks + ((t + 1) & 1) * TILE, kNext, tid);
            if (t + 2 < numKeyTiles) fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, kt0 + 2 * BC, p.totalLen, hd, tid);
        }
        __syncthreads();
    }
    if (i < p.newLen) {
        if (p.dQ) storeTransposed<HDP, VEC4>(p.dQ + qOff + size_t(i) * dim, acc, hd, half, p.scale);
        if (p.dQImg) storeTransposedBf16<HDP, VEC4>(p.dQImg + (size_t(b) * p.newLen + i) * p.imgLd + size_t(h) * hd, acc, hd, half, p.scale);
    }
}

// ---------------------------------------------------------------------------------------------
// backward, part 2: dK, dV (key-tile owner).  K and V of the wave's 32 keys stay in registers as MFMA
// B operands; Q/dO tiles and the per-row statistics are streamed through LDS.
// ---------------------------------------------------------------------------------------------
// One Q/dO tile (BQ queries) for one wavefront, straight-line and software-pipelined.
// stats: [0..BQ) = lse2 of the tile's queries (+inf for padding rows), [BQ..2BQ) = D.
// STORE: also writes each dS sub-block (32 queries x 32 keys, row-major) to dsLane + sb*dsStride for the dQ kernel
// that contracts it with K; dsLane already points at this lane's column and first row (li + 128*half floats in).
// AHEAD: the S / dP products of sub-block sb+1 are issued before the exp / dS arithmetic of sub-block sb (two sub-blocks
// of scores live at once).  With two waves per SIMD the other wave fills the matrix pipe during that arithmetic, and
// the 32 registers are worth more as room that keeps the kernel from spilling.
// DTP, dOff: the pass accumulates DTP 32-wide blocks of the head dim starting at element dOff (all of them unless the
// kernel takes the head dim in two passes); dsLane == nullptr: a pass that does not store dS.
template <int HDP, int BQ, bool MASKED, bool STORE, bool AHEAD, int DTP = HDP / 32>
__device__ __forceinline__ void dkvTile(const float* __restrict__ qs, const float* __restrict__ gs, const float* __restrict__ stats,
                                        const float (&kreg)[HDP / 2], const float (&vreg)[HDP / 2], float16v (&dk)[DTP],
                                        float16v (&dv)[DTP], int qt0, int key, bool keyValid, int oldLen, int half, int li,
                                        float* __restrict__ dsLane, size_t dsStride, int newLen, int dOff = 0) {
    constexpr int LDSW = HDP + 4, DT = DTP, NSB = BQ / 32, LIVE = AHEAD ? NSB : 1;
    float16v s[LIVE], dp[LIVE];
    auto scores = [&](int sb) {   // S = Q * K^T and dP = dO * V^T of sub-block sb
        float16v& sDst = s[AHEAD ? sb : 0];
        float16v& dpDst = dp[AHEAD ? sb : 0];
#pragma unroll
        for (int r = 0; r < 16; ++r) { sDst[r] = 0.0f; dpDst[r] = 0.0f; }
        headDotPairB<HDP>(qs + (sb * 32 + li) * LDSW + half * (HDP / 2), gs + (sb * 32 + li) * LDSW + half * (HDP / 2), kreg, vreg, sDst, dpDst);
    };
    if constexpr (AHEAD) scores(0);
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
        if constexpr (AHEAD) {
            if (sb + 1 < NSB) scores(sb + 1);
        } else {
            scores(sb);
        }
        // register r: query = qt0 + sb*32 + dRow(r, half), key = this lane's key
        float16v& pr = s[AHEAD ? sb : 0];
        float16v& dsv = dp[AHEAD ? sb : 0];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float4v lse4 = loadf4(stats + sb * 32 + 8 * g + 4 * half);
            float4v d4 = loadf4(stats + BQ + sb * 32 + 8 * g + 4 * half);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int r = 4 * g + c;
                float prob = fastExp2(pr[r] - lse4[c]);
                if constexpr (MASKED) {
                    int qi = qt0 + sb * 32 + dRow(r, half);
                    prob = (key > oldLen + qi || !keyValid) ? 0.0f : prob;
                }
                pr[r] = prob;                          // P
                dsv[r] = prob * (dsv[r] - d4[c]);      // dS (without the scale factor)
            }
        }
        if constexpr (STORE) {
            if (dsLane != nullptr && qt0 + sb * 32 < newLen) {   // row dRow(r, half) of the sub-block, 128 contiguous bytes per half wave
                float* dst = dsLane + sb * dsStride;
#pragma unroll
                for (int r = 0; r < 16; ++r) __builtin_nontemporal_store(dsv[r], dst + (8 * (r >> 2) + (r & 3)) * 32);
            }
        }
        // dV += P^T * dO, dK += dS^T * Q : step r contracts over query dRow(r, half)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float* grow = gs + (sb * 32 + dRow(r, half)) * LDSW + dOff + li;
            const float* qrow = qs + (sb * 32 + dRow(r, half)) * LDSW + dOff + li;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                dv[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(pr[r], grow[dt * 32], dv[dt], 0, 0, 0);
                dk[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(dsv[r], qrow[dt * 32], dk[dt], 0, 0, 0);
            }
        }
    }
}

// dk/dv[dt][r]: key = waveK0 + dRow(r, half), d = dt*32 + li  -> 128-byte coalesced rows (fp32 tensors and bf16 images)
template <int HDP, int DTP = HDP / 32>
__device__ __forceinline__ void storeKeyGradients(const AttnParams& p, const float16v (&dk)[DTP], const float16v (&dv)[DTP], int b,
                                                  int h, int waveK0, size_t kOff, int half, int li, int dOff = 0) {
    constexpr int DT = DTP;
    const int hd = p.hd, dim = p.dim;
    const bool images = p.dKImg != nullptr || p.dVImg != nullptr;
    // with an even head dim, row pitch and base every even column of an image row is 4-byte aligned and has its neighbour
    const bool pairs = (hd & 1) == 0 && (p.imgLd & 1u) == 0 && ((reinterpret_cast<uintptr_t>(p.dKImg) | reinterpret_cast<uintptr_t>(p.dVImg)) & 3u) == 0;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int d = dOff + dt * 32 + li;
        if (d < hd) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int kk = waveK0 + dRow(r, half);
                if (kk < p.totalLen) {
                    const float dkv = dk[dt][r] * p.scale, dvv = dv[dt][r];
                    if (p.dK) p.dK[kOff + size_t(kk) * dim + d] = dkv;
                    if (p.dV) p.dV[kOff + size_t(kk) * dim + d] = dvv;
                    if (images) {
                        const size_t at = (size_t(b) * p.totalLen + kk) * p.imgLd + size_t(h) * hd + d;
                        if (pairs) {   // lanes 2i and 2i+1 hold neighbouring columns: lane 2i stores both, four bytes at once
                            const float dkNext = __shfl_down(dkv, 1, 64), dvNext = __shfl_down(dvv, 1, 64);
                            if ((li & 1) == 0) {
                                if (p.dKImg) *reinterpret_cast<unsigned*>(p.dKImg + at) = unsigned(toBf16Bits(dkv)) | unsigned(toBf16Bits(dkNext)) << 16;
                                if (p.dVImg) *reinterpret_cast<unsigned*>(p.dVImg + at) = unsigned(toBf16Bits(dvv)) | unsigned(toBf16Bits(dvNext)) << 16;
                            }
                        } else {
                            if (p.dKImg) p.dKImg[at] = toBf16Bits(dkv);
                            if (p.dVImg) p.dVImg[at] = toBf16Bits(dvv);
                        }
                    }
                }
            }
        }
    }
}

// Head dims above 128 with the dS hand-over: the key-tile owner works in two passes over the query tiles that share out
// the four products instead of repeating two of them.  Pass "P" (dkvTileP) forms S = Q K^T, the probabilities P, parks
// P where dS will go (same 32 x 32 sub-blocks, the lane's own sixteen values) and accumulates dV += P^T dO over the whole
// head dim; it holds the K rows and one accumulator set.  Pass "dS" (dkvTileDs) forms dP = dO V^T, reads P back (each lane
// the values it wrote), turns it into dS = P (dP - D) in place and accumulates dK += dS^T Q; it holds the V rows and
// one accumulator set.  Every product is formed once, each output element sees the same MFMAs in the same order as in
// the one-pass kernel, and a wavefront stays inside its 512 registers, where K rows, V rows and both accumulator sets
// (512 registers by themselves) made the kernel form S and dP twice and spill half its state.
// The contraction over the head dim and the rank-one updates of an accumulator set, as fenced slices: left to itself the
// scheduler hoists every LDS read of the unrolled loop ahead of the MFMAs (128 registers of operands at head dim 256),
// which is what drove these kernels out of their registers.  One group of reads is in flight ahead of the MFMAs that
// use the group before it; a scheduling fence closes each group.
template <int HDP>
__device__ __forceinline__ float16v headDotFenced(const float* __restrict__ ldsRow, const float (&reg)[HDP / 2], float16v acc) {
    float4v a = loadf4(ldsRow);
#pragma unroll
    for (int t = 0; t < HDP / 2; t += 4) {
        float4v next = a;
        if (t + 4 < HDP / 2) next = loadf4(ldsRow + t + 4);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, reg[t], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, reg[t + 1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, reg[t + 2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, reg[t + 3], acc, 0, 0, 0);
        a = next;
        __builtin_amdgcn_sched_barrier(0);
    }
    return acc;
}
// acc[dt] += w[r] (x) row_r[(DT0 + dt)*32 + li] for the sixteen rows dRow(r, half) of a 32-row block at `rows`: the
// DT head-dim blocks from block DT0 on
template <int HDP, int DT0, int DT>
__device__ __forceinline__ void rankUpdatesFenced(const float* __restrict__ rows, const float16v& w, float16v (&acc)[DT], int half, int li) {
    constexpr int LDSW = HDP + 4;
    float cur[DT], nxt[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) cur[dt] = rows[dRow(0, half) * LDSW + li + (DT0 + dt) * 32];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        if (r + 1 < 16) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) nxt[dt] = rows[dRow(r + 1, half) * LDSW + li + (DT0 + dt) * 32];
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) acc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(w[r], cur[dt], acc[dt], 0, 0, 0);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) cur[dt] = nxt[dt];
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The sixteen values a lane parked in (or will park in) its 32 x 32 sub-block of the dS buffer; zero for rows past the sequence.
__device__ __forceinline__ float16v readParked(const float* __restrict__ src, bool stored) {
    float16v v;
#pragma unroll
    for (int r = 0; r < 16; ++r) v[r] = stored ? __builtin_nontemporal_load(src + (8 * (r >> 2) + (r & 3)) * 32) : 0.0f;
    return v;
}
// The second half of pass P or of pass dS when the accumulators take the head dim in two halves (head dim 256): the
// parked P (or dS) is read back and meets the other half of the dO (or Q) columns; no product over the head dim.
template <int HDP, int BQ, int DT0, int DTN>
__device__ __forceinline__ void dkvTileAgain(const float* __restrict__ rowsTile, float16v (&acc)[DTN], int qt0, int half, int li,
                                             const float* __restrict__ dsLane, size_t dsStride, int newLen) {
    constexpr int LDSW = HDP + 4, NSB = BQ / 32;
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
        const float16v w = readParked(dsLane + sb * dsStride, qt0 + sb * 32 < newLen);
        rankUpdatesFenced<HDP, DT0, DTN>(rowsTile + sb * 32 * LDSW, w, acc, half, li);
    }
}

template <int HDP, int BQ, bool MASKED, int DTN>
__device__ __forceinline__ void dkvTileP(const float* __restrict__ qs, const float* __restrict__ gs, const float* __restrict__ stats,
                                         const float (&kreg)[HDP / 2], float16v (&dv)[DTN], int qt0, int key, bool keyValid, int oldLen,
                                         int half, int li, float* __restrict__ dsLane, size_t dsStride, int newLen) {
    constexpr int LDSW = HDP + 4, NSB = BQ / 32;
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
        float16v pr;
#pragma unroll
        for (int r = 0; r < 16; ++r) pr[r] = 0.0f;
        pr = headDotFenced<HDP>(qs + (sb * 32 + li) * LDSW + half * (HDP / 2), kreg, pr);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4v lse4 = loadf4(stats + sb * 32 + 8 * g + 4 * half);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int r = 4 * g + c;
                float prob = fastExp2(pr[r] - lse4[c]);
                if constexpr (MASKED) {
                    const int qi = qt0 + sb * 32 + dRow(r, half);
                    prob = (key > oldLen + qi || !keyValid) ? 0.0f : prob;
                }
                pr[r] = prob;
            }
        }
        if (qt0 + sb * 32 < newLen) {
            float* dst = dsLane + sb * dsStride;
#pragma unroll
            for (int r = 0; r < 16; ++r) __builtin_nontemporal_store(pr[r], dst + (8 * (r >> 2) + (r & 3)) * 32);
        }
        rankUpdatesFenced<HDP, 0, DTN>(gs + sb * 32 * LDSW, pr, dv, half, li);
    }
}

template <int HDP, int BQ, int DTN>
__device__ __forceinline__ void dkvTileDs(const float* __restrict__ qs, const float* __restrict__ gs, const float* __restrict__ stats,
                                          const float (&vreg)[HDP / 2], float16v (&dk)[DTN], int qt0, int half, int li,
                                          float* __restrict__ dsLane, size_t dsStride, int newLen) {
    constexpr int LDSW = HDP + 4, NSB = BQ / 32;
#pragma unroll
    for (int sb = 0; sb < NSB; ++sb) {
        float* dst = dsLane + sb * dsStride;
        const bool stored = qt0 + sb * 32 < newLen;   // rows past the sequence hold no P (it is zero there)
        const float16v pr = readParked(dst, stored);
        float16v dsv;
#pragma unroll
        for (int r = 0; r < 16; ++r) dsv[r] = 0.0f;
        dsv = headDotFenced<HDP>(gs + (sb * 32 + li) * LDSW + half * (HDP / 2), vreg, dsv);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float4v d4 = loadf4(stats + BQ + sb * 32 + 8 * g + 4 * half);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int r = 4 * g + c;
                dsv[r] = pr[r] * (dsv[r] - d4[c]);      // dS (without the scale factor)
            }
        }
        if (stored) {
#pragma unroll
            for (int r = 0; r < 16; ++r) __builtin_nontemporal_store(dsv[r], dst + (8 * (r >> 2) + (r & 3)) * 32);
        }
        rankUpdatesFenced<HDP, 0, DTN>(qs + sb * 32 * LDSW, dsv, dk, half, li);
    }
}

// One pass of the key-tile owner over its query tiles for head dims above 128: Q and dO tiles (and lse2, D) through the
// double-buffered LDS stage, one barrier per tile.  MODE 0: dkvTileP with `reg` = the K rows and `acc` = dV; MODE 1:
// dkvTileDs with `reg` = the V rows and `acc` = dK; `acc` holds the first DTN head-dim blocks.  MODE 2 / MODE 3
// (dkvTileAgain, head dim 256, whose accumulators take the head dim in two halves): the parked P meets the dO columns
// of blocks DT0.. for the rest of dV / the stored dS meets the Q columns of blocks DT0.. for the rest of dK; `reg` is
// not read and only the tile that is needed is brought in.  With 16-byte aligned rows (VEC4) the tiles go from global memory
// straight into LDS (global_load_lds, one 1 KiB row per wavefront instruction, lanes past the head dim switched off: those
// columns were zeroed once), which frees the 64 registers a tile in flight would occupy; rows past the sequence repeat
// its last row (finite values that meet P = 0 and dS = 0).  Otherwise tiles are staged through registers as in
// attnBackwardDkvKernel.
template <int HDP, int BQ, bool VEC4, int MODE, int DT0, int DTN>
__device__ __forceinline__ void dkvStreamPass(const AttnParams& p, float* __restrict__ qs, float* __restrict__ gs, float* __restrict__ stats,
                                              const float (&reg)[HDP / 2], float16v (&acc)[DTN], int bh, int kt, size_t qOff,
                                              size_t statOff, int waveK0, int key, bool keyValid, int half, int li, int tid) {
    constexpr int LDSW = HDP + 4, TILE = BQ * LDSW;
    const int hd = p.hd, dim = p.dim;
    int firstQuery = kt * 128 - p.oldLen;
    if (firstQuery < 0) firstQuery = 0;
    const int q0Start = (firstQuery / BQ) * BQ;
    const int numQTiles = q0Start < p.newLen ? (p.newLen - q0Start + BQ - 1) / BQ : 0;
    const size_t dsStride = size_t(p.nkb) * 1024;
    float* const dsColumn = p.ds + (size_t(bh) * p.nqb * p.nkb + size_t(waveK0 >> 5)) * 1024;   // wave-uniform
    const int dsLaneOffset = half * 128 + li;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    auto tileBody = [&](int t, int qt0) __attribute__((always_inline)) {
        if (p.oldLen + qt0 + BQ - 1 >= waveK0 && waveK0 < p.totalLen) {
            const float* qcur = qs + (t & 1) * TILE;
            const float* gcur = gs + (t & 1) * TILE;
            const float* scur = stats + (t & 1) * 2 * BQ;
            float* dsLane = dsColumn + size_t(qt0 >> 5) * dsStride + dsLaneOffset;
            if constexpr (MODE == 0) {
                const bool masked = (waveK0 + 31 > p.oldLen + qt0) || (waveK0 + 32 > p.totalLen);
                if (masked) dkvTileP<HDP, BQ, true, DTN>(qcur, gcur, scur, reg, acc, qt0, key, keyValid, p.oldLen, half, li, dsLane, dsStride, p.newLen);
                else dkvTileP<HDP, BQ, false, DTN>(qcur, gcur, scur, reg, acc, qt0, key, keyValid, p.oldLen, half, li, dsLane, dsStride, p.newLen);
            } else if constexpr (MODE == 1) {
                dkvTileDs<HDP, BQ, DTN>(qcur, gcur, scur, reg, acc, qt0, half, li, dsLane, dsStride, p.newLen);
            } else {
                dkvTileAgain<HDP, BQ, DT0, DTN>(MODE == 2 ? gcur : qcur, acc, qt0, half, li, dsLane, dsStride, p.newLen);
            }
        }
    };
    float statNext = 0.0f;
    constexpr bool kNeedQ = MODE != 2, kNeedG = MODE != 3, kNeedStats = MODE < 2;
    auto fetchStats = [&](int qt0) __attribute__((always_inline)) {
        if constexpr (!kNeedStats) return;
        const int qi = qt0 + (tid < BQ ? tid : tid - BQ);
        if (tid < BQ) statNext = qi < p.newLen ? p.lse2[statOff + qi] : INFINITY;
        else if (tid < 2 * BQ) statNext = qi < p.newLen ? p.dvec[statOff + qi] : 0.0f;
    };
    if constexpr (VEC4) {
        // wavefront w brings rows w, w + 4, ... of either tile; lane l the 16 bytes at column 4 l
        const bool columnValid = 4 * lane < hd;
        const float* qBase = p.q + qOff + 4 * lane;
        const float* gBase = p.dO + qOff + 4 * lane;
        auto issueTile = [&](int qt0, int buf) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < BQ / 4; ++i) {
                const int r = wave + 4 * i;
                const size_t row = size_t(min(qt0 + r, p.newLen - 1)) * dim;
                if (columnValid) {
                    if constexpr (kNeedQ) __builtin_amdgcn_global_load_lds((GlobalPtr)(qBase + row), (LdsPtr)(qs + buf * TILE + r * LDSW), 16, 0, 0);
                    if constexpr (kNeedG) __builtin_amdgcn_global_load_lds((GlobalPtr)(gBase + row), (LdsPtr)(gs + buf * TILE + r * LDSW), 16, 0, 0);
                }
            }
        };
        if (hd < HDP) {   // the columns past the head dim are never loaded: zero them once (both buffers of both tiles)
            for (int i = tid; i < 4 * BQ * (LDSW / 4); i += 256) storef4(qs + 4 * i, float4v{0.0f, 0.0f, 0.0f, 0.0f});
            __syncthreads();
        }
        if (numQTiles > 0) {
            issueTile(q0Start, 0);
            fetchStats(q0Start);
            if (kNeedStats && tid < 2 * BQ) stats[tid] = statNext;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        for (int t = 0; t < numQTiles; ++t) {
            const int qt0 = q0Start + t * BQ;
            if (t + 1 < numQTiles) {   // buffer (t+1)&1 was last read before the barrier that ended the tile before
                issueTile(qt0 + BQ, (t + 1) & 1);
                fetchStats(qt0 + BQ);
            }
            tileBody(t, qt0);
            if (kNeedStats && t + 1 < numQTiles && tid < 2 * BQ) stats[((t + 1) & 1) * 2 * BQ + tid] = statNext;
            // the tile's loads have landed in LDS (the stores of the tile body, issued a hundred MFMAs ago, are long done)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();   // after the last tile too: the next pass writes the LDS buffers again
        }
    } else {
        TileRegs<HDP, BQ> qNext, gNext;
        auto fetchAll = [&](int qt0) __attribute__((always_inline)) {
            if constexpr (kNeedQ) fetchHeadTile<HDP, BQ, VEC4>(qNext, p.q + qOff, dim, qt0, p.newLen, hd, tid);
            if constexpr (kNeedG) fetchHeadTile<HDP, BQ, VEC4>(gNext, p.dO + qOff, dim, qt0, p.newLen, hd, tid);
            fetchStats(qt0);
        };
        auto commitAll = [&](int buf) __attribute__((always_inline)) {
            if constexpr (kNeedQ) commitHeadTile<HDP, BQ>(qs + buf * TILE, qNext, tid);
            if constexpr (kNeedG) commitHeadTile<HDP, BQ>(gs + buf * TILE, gNext, tid);
            if (kNeedStats && tid < 2 * BQ) stats[buf * 2 * BQ + tid] = statNext;
        };
        if (numQTiles > 0) {
            fetchAll(q0Start);
            commitAll(0);
            if (numQTiles > 1) fetchAll(q0Start + BQ);
        }
        __syncthreads();
        for (int t = 0; t < numQTiles; ++t) {
            const int qt0 = q0Start + t * BQ;
            tileBody(t, qt0);
            if (t + 1 < numQTiles) {
                commitAll((t + 1) & 1);
                if (t + 2 < numQTiles) fetchAll(qt0 + 2 * BQ);
            }
            __syncthreads();   // after the last tile too: the next pass writes the LDS buffers again
        }
    }
}

// One of the two key gradients (IS_K: dK, scaled; else dV), fp32 tensor and bf16 image, as storeKeyGradients stores them.
template <int HDP, bool IS_K, int DT0, int DTN>
__device__ __forceinline__ void storeOneKeyGradient(const AttnParams& p, const float16v (&acc)[DTN], int b, int h, int waveK0,
                                                    size_t kOff, int half, int li) {
    const int hd = p.hd, dim = p.dim;
    float* __restrict__ out = IS_K ? p.dK : p.dV;
    unsigned short* __restrict__ img = IS_K ? p.dKImg : p.dVImg;
    const float mul = IS_K ? p.scale : 1.0f;
    const bool pairs = (hd & 1) == 0 && (p.imgLd & 1u) == 0 && (reinterpret_cast<uintptr_t>(img) & 3u) == 0;
#pragma unroll
    for (int dt = 0; dt < DTN; ++dt) {
        const int d = (DT0 + dt) * 32 + li;
        if (d < hd) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int kk = waveK0 + dRow(r, half);
                if (kk < p.totalLen) {
                    const float v = acc[dt][r] * mul;
                    if (out) out[kOff + size_t(kk) * dim + d] = v;
                    if (img) {
                        const size_t at = (size_t(b) * p.totalLen + kk) * p.imgLd + size_t(h) * hd + d;
                        if (pairs) {
                            const float next = __shfl_down(v, 1, 64);
                            if ((li & 1) == 0) *reinterpret_cast<unsigned*>(img + at) = unsigned(toBf16Bits(v)) | unsigned(toBf16Bits(next)) << 16;
                        } else {
                            img[at] = toBf16Bits(v);
                        }
                    }
                }
            }
        }
    }
}

// OCC = wavefronts per SIMD the register allocation is held to.  At OCC 2 (head dims up to 64) two workgroups share
// a CU and cover each other's barriers and tile hand-overs, at the price of a handful of spilled registers; it pays
// once the grid has more workgroups than two per CU, below that one roomier workgroup per CU is faster.
template <int HDP, int BQ, bool VEC4, int OCC, bool STORE>
__global__ void __launch_bounds__(256, OCC) attnBackwardDkvKernel(AttnParams p) {
    constexpr int LDSW = HDP + 4, DT = HDP / 32, TILE = BQ * LDSW;
    extern __shared__ float smem[];
    float* qs = smem;                   // [2][BQ][LDSW]
    float* gs = smem + 2 * TILE;        // [2][BQ][LDSW]
    float* stats = smem + 4 * TILE;     // [2][2*BQ]: lse2 | D

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    int bh, kt;
    decodeBlock(p.numTiles, gridDim.x, false, bh, kt);   // the first key tile is seen by every query: heaviest
    const int b = bh / p.heads, h = bh - b * p.heads;
    const int hd = p.hd, dim = p.dim;
    const size_t qOff = size_t(b) * p.newLen * dim + size_t(h) * hd;
    const size_t kOff = size_t(b) * p.totalLen * dim + size_t(h) * hd;
    const size_t statOff = (size_t(b) * p.heads + h) * p.newLen;

    const int waveK0 = kt * 128 + wave * 32;
    const int key = waveK0 + li;                       // this lane's key (as B-operand column)
    const bool keyValid = key < p.totalLen;
    if constexpr (HDP > 128 && STORE) {
        // two passes that share out the products (dkvTileP / dkvTileDs above).  At head dim 256 an accumulator set is 128
        // registers beside the 128 of the K or V rows: each pass keeps the first half of its accumulators, and a second walk
        // over the tiles (dkvTileAgain: the parked P or dS against the other half of the columns, no K or V rows, one
        // tile instead of two) makes the rest, so that no walk leaves its registers (the one-walk form spilled 171).
        constexpr int HALVES = HDP > 192 ? 2 : 1, DTN = DT / HALVES;
        auto zero = [](float16v (&acc)[DTN]) __attribute__((always_inline)) {
#pragma unroll
            for (int dt = 0; dt < DTN; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[dt][r] = 0.0f;
        };
        {
            float kreg[HDP / 2];
            loadRowOperand<HDP, VEC4>(kreg, p.k + kOff + size_t(key) * dim, keyValid, hd, half, p.scale * kLog2e);
            float16v dv[DTN];
            zero(dv);
            dkvStreamPass<HDP, BQ, VEC4, 0, 0, DTN>(p, qs, gs, stats, kreg, dv, bh, kt, qOff, statOff, waveK0, key, keyValid, half, li, tid);
            storeOneKeyGradient<HDP, false, 0, DTN>(p, dv, b, h, waveK0, kOff, half, li);
        }
        if constexpr (HALVES == 2) {
            float none[HDP / 2];   // never read
            float16v dv[DTN];
            zero(dv);
            dkvStreamPass<HDP, BQ, VEC4, 2, DTN, DTN>(p, qs, gs, stats, none, dv, bh, kt, qOff, statOff, waveK0, key, keyValid, half, li, tid);
            storeOneKeyGradient<HDP, false, DTN, DTN>(p, dv, b, h, waveK0, kOff, half, li);
        }
        {
            float vreg[HDP / 2];
            loadRowOperand<HDP, VEC4>(vreg, p.v + kOff + size_t(key) * dim, keyValid, hd, half, 1.0f);
            float16v dk[DTN];
            zero(dk);
            dkvStreamPass<HDP, BQ, VEC4, 1, 0, DTN>(p, qs, gs, stats, vreg, dk, bh, kt, qOff, statOff, waveK0, key, keyValid, half, li, tid);
            storeOneKeyGradient<HDP, true, 0, DTN>(p, dk, b, h, waveK0, kOff, half, li);
        }
        if constexpr (HALVES == 2) {
            float none[HDP / 2];   // never read
            float16v dk[DTN];
            zero(dk);
            dkvStreamPass<HDP, BQ, VEC4, 3, DTN, DTN>(p, qs, gs, stats, none, dk, bh, kt, qOff, statOff, waveK0, key, keyValid, half, li, tid);
            storeOneKeyGradient<HDP, true, DTN, DTN>(p, dk, b, h, waveK0, kOff, half, li);
        }
        return;
    }
    float kreg[HDP / 2], vreg[HDP / 2];
    loadRowOperand<HDP, VEC4>(kreg, p.k + kOff + size_t(key) * dim, keyValid, hd, half, p.scale * kLog2e);
    loadRowOperand<HDP, VEC4>(vreg, p.v + kOff + size_t(key) * dim, keyValid, hd, half, 1.0f);

    // Head dim 256: K and V rows (256 registers) and both accumulators (256 more) do not fit a wavefront's 512 registers,
    // so the accumulators take the head dim in two passes of 128, each over all the query tiles (S and dP are formed
    // again in the second pass: half again as many MFMAs, against spilling most of the accumulators).
    constexpr int PASSES = HDP > 128 ? 2 : 1, DTP = DT / PASSES;
    float16v dk[DTP], dv[DTP];

    // first query that can see any key of this workgroup's tile: oldLen + i >= kt*128
    int firstQuery = kt * 128 - p.oldLen;
    if (firstQuery < 0) firstQuery = 0;
    const int q0Start = (firstQuery / BQ) * BQ;
    const int numQTiles = q0Start < p.newLen ? (p.newLen - q0Start + BQ - 1) / BQ : 0;

    // this lane's corner of the wave's column of dS sub-blocks: key sub-block waveK0/32, row 4*half, column li
    const size_t dsStride = size_t(p.nkb) * 1024;
    float* const dsColumn = STORE ? p.ds + (size_t(bh) * p.nqb * p.nkb + size_t(waveK0 >> 5)) * 1024 : nullptr;   // wave-uniform
    const int dsLaneOffset = half * 128 + li;

    for (int pass = 0; pass < PASSES; ++pass) {
    const int dOff = pass * DTP * 32;
#pragma unroll
    for (int dt = 0; dt < DTP; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk[dt][r] = 0.0f; dv[dt][r] = 0.0f; }
    TileRegs<HDP, BQ> qNext, gNext;
    float statNext = 0.0f;
    auto fetchStats = [&](int qt0) {   // thread t < BQ: lse2 of query qt0+t; BQ <= t < 2BQ: D of query qt0+t-BQ
        const int j = tid < BQ ? tid : tid - BQ;
        const int qi = qt0 + j;
        if (tid < BQ) statNext = qi < p.newLen ? p.lse2[statOff + qi] : INFINITY;
        else if (tid < 2 * BQ) statNext = qi < p.newLen ? p.dvec[statOff + qi] : 0.0f;
    };
    auto commitAll = [&](int buf) {
        commitHeadTile<HDP, BQ>(qs + buf * TILE, qNext, tid);
        commitHeadTile<HDP, BQ>(gs + buf * TILE, gNext, tid);
        if (tid < 2 * BQ) stats[buf * 2 * BQ + tid] = statNext;
    };
    auto fetchAll = [&](int qt0) {
        fetchHeadTile<HDP, BQ, VEC4>(qNext, p.q + qOff, dim, qt0, p.newLen, hd, tid);
        fetchHeadTile<HDP, BQ, VEC4>(gNext, p.dO + qOff, dim, qt0, p.newLen, hd, tid);
        fetchStats(qt0);
    };
    if (numQTiles > 0) {
        fetchAll(q0Start);
        commitAll(0);
        if (numQTiles > 1) fetchAll(q0Start + BQ);
    }
    __syncthreads();
    for (int t = 0; t < numQTiles; ++t) {
        const int qt0 = q0Start + t * BQ;
        // the wave's keys [waveK0, waveK0+32) are visible to some query of the tile?
        if (p.oldLen + qt0 + BQ - 1 >= waveK0 && waveK0 < p.totalLen) {
            const bool masked = (waveK0 + 31 > p.oldLen + qt0) || (waveK0 + 32 > p.totalLen);
            const float* qcur = qs + (t & 1) * TILE;
            const float* gcur = gs + (t & 1) * TILE;
            const float* scur = stats + (t & 1) * 2 * BQ;
            float* dsLane = STORE && pass == 0 ? dsColumn + size_t(qt0 >> 5) * dsStride + dsLaneOffset : nullptr;   // dS once
            if (masked)
                dkvTile<HDP, BQ, true, STORE, OCC == 1, DTP>(qcur, gcur, scur, kreg, vreg, dk, dv, qt0, key, keyValid, p.oldLen, half, li, dsLane,
                                                             dsStride, p.newLen, dOff);
            else
                dkvTile<HDP, BQ, false, STORE, OCC == 1, DTP>(qcur, gcur, scur, kreg, vreg, dk, dv, qt0, key, keyValid, p.oldLen, half, li, dsLane,
                                                              dsStride, p.newLen, dOff);
        }
        if (t + 1 < numQTiles) {
            commitAll((t + 1) & 1);
            if (t + 2 < numQTiles) fetchAll(qt0 + 2 * BQ);
        }
        __syncthreads();   // after the last tile too: the next pass writes the LDS buffers again
    }

    storeKeyGradients<HDP, DTP>(p, dk, dv, b, h, waveK0, kOff, half, li, dOff);
    }
}

// ---------------------------------------------------------------------------------------------
// backward, part 2 on the bf16 matrix pipe at fp32 accuracy: dK, dV (key-tile owner) with every product as six bf16
// MFMAs on operands split into three bf16 terms (see the forward kernel above).  The wavefront's K and V rows are split
// once into register fragments (B operands of S = Q K^T and dP = dO V^T, eight head-dim elements per lane and step);
// Q and dO tiles are split when they are written to LDS and read two ways: 16 bytes of a row as the A operand of S and
// dP, and through the transposing read as the B operand of dV += P^T dO and dK += dS^T Q, whose contraction runs over
// queries in the permuted order that makes P^T and dS^T (the A operands) eight consecutive accumulator registers.
// One wavefront per SIMD: the fragments of K and V alone take 96 registers at head dim 64 and 192 at 128.
// ---------------------------------------------------------------------------------------------
template <int HDP, bool MASKED, bool STORE>
__device__ __forceinline__ void dkvSplitTile(const unsigned short* __restrict__ qimg, const unsigned short* __restrict__ gimg,
                                             const float* __restrict__ stats, const bf16x8a (&kf)[HDP / 16][3],
                                             const bf16x8a (&vf)[HDP / 16][3], float16v (&dk)[HDP / 32], float16v (&dv)[HDP / 32], int qt0,
                                             int key, bool keyValid, int oldLen, int lane, float* __restrict__ dsLane) {
    constexpr int QP = splitKeyPitch(HDP), IMG = 32 * QP, DT = HDP / 32, KS = HDP / 16;
    const int half = lane >> 5, li = lane & 31;
    // S = Q K^T and dP = dO V^T in two accumulator chains each: the products of the two high terms, and everything
    // smaller (at most 2^-7 of the first), whose own rounding is then far below the first chain's
    float16v s0, s1, p0, p1;
#pragma unroll
    for (int r = 0; r < 16; ++r) { s0[r] = 0.0f; s1[r] = 0.0f; p0[r] = 0.0f; p1[r] = 0.0f; }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const unsigned short* qrow = qimg + li * QP + ks * 16 + half * 8;
        const unsigned short* grow = gimg + li * QP + ks * 16 + half * 8;
        bf16x8a a[3], g[3];
#pragma unroll
        for (int im = 0; im < 3; ++im) {
            a[im] = *reinterpret_cast<const bf16x8a*>(qrow + im * IMG);
            g[im] = *reinterpret_cast<const bf16x8a*>(grow + im * IMG);
        }
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], kf[ks][1], s1, 0, 0, 0);
        p1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(g[1], vf[ks][1], p1, 0, 0, 0);
        s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], kf[ks][0], s0, 0, 0, 0);
        p0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(g[0], vf[ks][0], p0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[2], kf[ks][0], s1, 0, 0, 0);
        p1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(g[2], vf[ks][0], p1, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], kf[ks][2], s1, 0, 0, 0);
        p1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(g[0], vf[ks][2], p1, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], kf[ks][0], s1, 0, 0, 0);
        p1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(g[1], vf[ks][0], p1, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], kf[ks][1], s1, 0, 0, 0);
        p1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(g[0], vf[ks][1], p1, 0, 0, 0);
    }
    // register r: query = qt0 + dRow(r, half), key = this lane's key
    float16v pr, dsv;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const float4v lse4 = loadf4(stats + 8 * g + 4 * half);
        const float4v d4 = loadf4(stats + 32 + 8 * g + 4 * half);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int r = 4 * g + c;
            float prob = fastExp2((s1[r] + s0[r]) - lse4[c]);
            if constexpr (MASKED) {
                const int qi = qt0 + dRow(r, half);
                prob = (key > oldLen + qi || !keyValid) ? 0.0f : prob;
            }
            pr[r] = prob;                                      // P
            dsv[r] = prob * ((p1[r] + p0[r]) - d4[c]);         // dS (without the scale factor)
        }
    }
    if constexpr (STORE) {   // row dRow(r, half) of the sub-block, 128 contiguous bytes per half wave (every tile a caller
                             // passes starts inside the sequence, and the buffer holds whole sub-blocks)
#pragma unroll
        for (int r = 0; r < 16; ++r) __builtin_nontemporal_store(dsv[r], dsLane + (8 * (r >> 2) + (r & 3)) * 32);
    }
    // dV += P^T dO, dK += dS^T Q: step st contracts over queries 16 st + 8 (e / 4) + 4 half + e % 4 = registers 8 st + e
    const int fragRow = 4 * (lane >> 5) + ((lane & 15) >> 2), fragCol = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    constexpr int order[6][2] = {{1, 1}, {2, 0}, {0, 2}, {1, 0}, {0, 1}, {0, 0}};   // (register term, LDS term), small products first
#pragma unroll
    for (int st = 0; st < 2; ++st) {
        bf16x8a pf[3], df[3];
        {
            float x[8], y[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) { x[e] = pr[8 * st + e]; y[e] = dsv[8 * st + e]; }
            splitOperand(x, pf[0], pf[1], pf[2]);
            splitOperand(y, df[0], df[1], df[2]);
        }
        // two 32-wide blocks of the head dim at a time: four accumulator chains alternate, and twelve operand fragments
        // are live instead of six per block of the head dim
        constexpr int DG = DT >= 2 ? 2 : 1;
#pragma unroll
        for (int d0 = 0; d0 < DT; d0 += DG) {
            bf16x8a gfr[DG][3], qfr[DG][3];
#pragma unroll
            for (int dt = 0; dt < DG; ++dt)
#pragma unroll
                for (int im = 0; im < 3; ++im) {
                    gfr[dt][im] = readTransposedApart(gimg + im * IMG + (16 * st + fragRow) * QP + (d0 + dt) * 32 + fragCol, QP);
                    qfr[dt][im] = readTransposedApart(qimg + im * IMG + (16 * st + fragRow) * QP + (d0 + dt) * 32 + fragCol, QP);
                }
#pragma unroll
            for (int pr6 = 0; pr6 < 6; ++pr6)
#pragma unroll
                for (int dt = 0; dt < DG; ++dt) {
                    dv[d0 + dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[order[pr6][0]], gfr[dt][order[pr6][1]], dv[d0 + dt], 0, 0, 0);
                    dk[d0 + dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(df[order[pr6][0]], qfr[dt][order[pr6][1]], dk[d0 + dt], 0, 0, 0);
                }
        }
    }
}

// The wavefront's K or V rows as split register fragments: step s of a lane in `half` holds head-dim elements
// 16 s + 8 half + 0..7 of the lane's key, times `mul`, as three bf16 terms.
template <int HDP, bool VEC4>
__device__ __forceinline__ void loadSplitFragments(bf16x8a (&dst)[HDP / 16][3], const float* __restrict__ row, float mul, bool keyValid,
                                                   int hd, int half) {
#pragma unroll
    for (int s = 0; s < HDP / 16; ++s) {
        float x[8];
#pragma unroll
        for (int c = 0; c < 8; c += 4) {
            const int d = 16 * s + 8 * half + c;
            float4v val = {0.0f, 0.0f, 0.0f, 0.0f};
            if (keyValid && d < hd) {
                if constexpr (VEC4) {
                    val = loadf4(row + d);
                } else {
                    val.x = row[d];
                    if (d + 1 < hd) val.y = row[d + 1];
                    if (d + 2 < hd) val.z = row[d + 2];
                    if (d + 3 < hd) val.w = row[d + 3];
                }
            }
            x[c] = val.x * mul; x[c + 1] = val.y * mul; x[c + 2] = val.z * mul; x[c + 3] = val.w * mul;
        }
        splitOperand(x, dst[s][0], dst[s][1], dst[s][2]);
    }
}

template <int HDP, bool VEC4, bool STORE>
__global__ void __launch_bounds__(256, 1) attnBackwardDkvSplitKernel(AttnParams p) {
    constexpr int BQ = 32, QP = splitKeyPitch(HDP), TILE = 3 * BQ * QP, DT = HDP / 32, KS = HDP / 16;
    extern __shared__ __attribute__((aligned(16))) unsigned short smemSplit[];
    unsigned short* qs = smemSplit;                 // [2][3][BQ][QP]
    unsigned short* gs = smemSplit + 2 * TILE;      // [2][3][BQ][QP]
    float* stats = reinterpret_cast<float*>(smemSplit + 4 * TILE);   // [2][2*BQ]: lse2 | D

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    int bh, kt;
    decodeBlock(p.numTiles, gridDim.x, false, bh, kt);   // the first key tile is seen by every query: heaviest
    const int b = bh / p.heads, h = bh - b * p.heads;
    const int hd = p.hd, dim = p.dim;
    const size_t qOff = size_t(b) * p.newLen * dim + size_t(h) * hd;
    const size_t kOff = size_t(b) * p.totalLen * dim + size_t(h) * hd;
    const size_t statOff = (size_t(b) * p.heads + h) * p.newLen;

    const int waveK0 = kt * 128 + wave * 32;
    const int key = waveK0 + li;                       // this lane's key (as B-operand column)
    const bool keyValid = key < p.totalLen;
    // K (scaled) and V fragments: step ks of a lane in `half` holds head-dim elements 16 ks + 8 half + 0..7 of its key
    bf16x8a kf[KS][3], vf[KS][3];
    loadSplitFragments<HDP, VEC4>(kf, p.k + kOff + size_t(key) * dim, p.scale * kLog2e, keyValid, hd, half);
    loadSplitFragments<HDP, VEC4>(vf, p.v + kOff + size_t(key) * dim, 1.0f, keyValid, hd, half);

    float16v dk[DT], dv[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk[dt][r] = 0.0f; dv[dt][r] = 0.0f; }

    // first query that can see any key of this workgroup's tile: oldLen + i >= kt*128
    int firstQuery = kt * 128 - p.oldLen;
    if (firstQuery < 0) firstQuery = 0;
    const int q0Start = (firstQuery / BQ) * BQ;
    const int numQTiles = q0Start < p.newLen ? (p.newLen - q0Start + BQ - 1) / BQ : 0;

    const size_t dsStride = size_t(p.nkb) * 1024;
    float* const dsColumn = STORE ? p.ds + (size_t(bh) * p.nqb * p.nkb + size_t(waveK0 >> 5)) * 1024 : nullptr;   // wave-uniform
    const int dsLaneOffset = half * 128 + li;

    // a tile's loads are issued one tile before it is written to LDS and two before it is read
    TileRegs<HDP, BQ> qStage, gStage;
    float statStage = 0.0f;
    auto fetchAll = [&](int qt0) {
        fetchHeadTile<HDP, BQ, VEC4>(qStage, p.q + qOff, dim, qt0, p.newLen, hd, tid);
        fetchHeadTile<HDP, BQ, VEC4>(gStage, p.dO + qOff, dim, qt0, p.newLen, hd, tid);
        const int j = tid < BQ ? tid : tid - BQ;
        const int qi = qt0 + j;
        if (tid < BQ) statStage = qi < p.newLen ? p.lse2[statOff + qi] : INFINITY;
        else if (tid < 2 * BQ) statStage = qi < p.newLen ? p.dvec[statOff + qi] : 0.0f;
    };
    auto commitAll = [&](int buf) {
        commitSplitTile<HDP, BQ, QP>(qs + buf * TILE, qStage, tid);
        commitSplitTile<HDP, BQ, QP>(gs + buf * TILE, gStage, tid);
        if (tid < 2 * BQ) stats[buf * 2 * BQ + tid] = statStage;
    };
    if (numQTiles > 0) {
        fetchAll(q0Start);
        commitAll(0);
        if (numQTiles > 1) fetchAll(q0Start + BQ);
    }
    __syncthreads();
    for (int t = 0; t < numQTiles; ++t) {
        const int qt0 = q0Start + t * BQ, u = t & 1;
        // the wave's keys [waveK0, waveK0+32) are visible to some query of the tile?
        if (p.oldLen + qt0 + BQ - 1 >= waveK0 && waveK0 < p.totalLen) {
            const bool masked = (waveK0 + 31 > p.oldLen + qt0) || (waveK0 + 32 > p.totalLen);
            const unsigned short* qcur = qs + u * TILE;
            const unsigned short* gcur = gs + u * TILE;
            const float* scur = stats + u * 2 * BQ;
            float* dsLane = STORE ? dsColumn + size_t(qt0 >> 5) * dsStride + dsLaneOffset : nullptr;
            if (masked) dkvSplitTile<HDP, true, STORE>(qcur, gcur, scur, kf, vf, dk, dv, qt0, key, keyValid, p.oldLen, lane, dsLane);
            else dkvSplitTile<HDP, false, STORE>(qcur, gcur, scur, kf, vf, dk, dv, qt0, key, keyValid, p.oldLen, lane, dsLane);
        }
        if (t + 1 < numQTiles) {
            commitAll(u ^ 1);
            if (t + 2 < numQTiles) fetchAll(qt0 + 2 * BQ);
        }
        __syncthreads();
    }
    storeKeyGradients<HDP>(p, dk, dv, b, h, waveK0, kOff, half, li);
}

// ---------------------------------------------------------------------------------------------
// The same dK/dV kernel as a two-stage pipeline over query tiles (head dims up to 64).  A wavefront per SIMD has nobody to
// hide behind, so the matrix pipe and the vector unit take turns unless one instruction stream feeds both: here the
// products of two neighbouring tiles are interleaved.  While S and dP of tile t run on the matrix pipe the vector unit
// splits P and dS of tile t-1 into their bf16 terms; while dV and dK of tile t-1 run, it makes P and dS of tile t from
// the finished S and dP and stores dS.  LDS reads are issued a step ahead of the MFMAs that consume them.  The order is
// given to the scheduler as groups (sched_group_barrier); the data flow alone would let it put each kind of work in one
// run.  Tile t-1 is read (transposed) while tile t is read (plain) and tile t+1 is written: three LDS buffers.
// ---------------------------------------------------------------------------------------------
template <int HDP>
__device__ __forceinline__ void readSplitTransposed(bf16x8a (&gfr)[HDP / 32][3], bf16x8a (&qfr)[HDP / 32][3],
                                                    const unsigned short* __restrict__ qimg, const unsigned short* __restrict__ gimg,
                                                    int st, int lane) {
    constexpr int QP = splitKeyPitch(HDP), IMG = 32 * QP;
    const int fragRow = 4 * (lane >> 5) + ((lane & 15) >> 2), fragCol = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
#pragma unroll
    for (int dt = 0; dt < HDP / 32; ++dt)
#pragma unroll
        for (int im = 0; im < 3; ++im) {
            gfr[dt][im] = readTransposedApart(gimg + im * IMG + (16 * st + fragRow) * QP + dt * 32 + fragCol, QP);
            qfr[dt][im] = readTransposedApart(qimg + im * IMG + (16 * st + fragRow) * QP + dt * 32 + fragCol, QP);
        }
}

// (register term, LDS term) of the six products of dV += P^T dO and dK += dS^T Q: the LDS terms retire in the order low,
// middle, high, so that their registers are free for the next fragments; the largest product comes last
__device__ constexpr int kSplitOrder[6][2] = {{0, 2}, {1, 1}, {0, 1}, {2, 0}, {1, 0}, {0, 0}};

// One step of the pipeline on an unmasked tile: S, dP, P and dS of the tile in (qimg, gimg, stats); dV and dK of the
// tile before it (qprev, gprev), whose P and dS come in through (pr, dsv) and are replaced by this tile's.  The source
// is laid out in slices of three MFMAs and a share of the vector work, with a scheduling fence after each.
template <int HDP, bool STORE>
__device__ __forceinline__ void dkvSplitStep(const unsigned short* __restrict__ qimg, const unsigned short* __restrict__ gimg,
                                             const float* __restrict__ stats, const unsigned short* __restrict__ qprev,
                                             const unsigned short* __restrict__ gprev, const bf16x8a (&kf)[HDP / 16][3],
                                             const bf16x8a (&vf)[HDP / 16][3], float16v (&dk)[HDP / 32], float16v (&dv)[HDP / 32],
                                             float16v& pr, float16v& dsv, int lane, float* __restrict__ dsLane) {
    constexpr int QP = splitKeyPitch(HDP), IMG = 32 * QP, DT = HDP / 32, KS = HDP / 16;
    static_assert(KS == 2 || KS == 4, "the pipelined form is laid out for head dims 32 and 64");
    const int half = lane >> 5, li = lane & 31;
    float16v s, dp;
#pragma unroll
    for (int r = 0; r < 16; ++r) { s[r] = 0.0f; dp[r] = 0.0f; }
    uint4a pf[2][3], df[2][3];   // bf16 pairs; an operand is one of these as eight bf16
    // sixteen pairs of neighbouring registers: P first, then dS; step st contracts over registers 8 st + e
    // The split of pair i in three parts (high term and what it leaves; middle term and what it leaves; low term), one
    // after each MFMA of a slice; `rest` carries the remainders from part to part.
    float rest[2][2];
    auto splitPairPart = [&](int i, int c, int part) {
        const int st = (i >> 2) & 1, e = i & 3;
        uint4a(&dst)[3] = i < 8 ? pf[st] : df[st];
        if (part == 0) {
            const float x0 = i < 8 ? pr[8 * st + 2 * e] : dsv[8 * st + 2 * e], x1 = i < 8 ? pr[8 * st + 2 * e + 1] : dsv[8 * st + 2 * e + 1];
            const unsigned h = packBf16(x0, x1);
            dst[0][e] = h;
            rest[c][0] = x0 - __builtin_bit_cast(float, h << 16);
            rest[c][1] = x1 - __builtin_bit_cast(float, h & 0xffff0000u);
        } else if (part == 1) {
            const unsigned m = packBf16(rest[c][0], rest[c][1]);
            dst[1][e] = m;
            rest[c][0] -= __builtin_bit_cast(float, m << 16);
            rest[c][1] -= __builtin_bit_cast(float, m & 0xffff0000u);
        } else {
            dst[2][e] = packBf16(rest[c][0], rest[c][1]);
        }
    };

    // Stage one: S = Q K^T and dP = dO V^T, one accumulator chain each, the products in the order of their size: the
    // three small ones (middle x middle, low x high, high x low) of every head-dim step, then the two middle ones, then
    // high x high, so that a small product is never added to a sum of large ones.  The chains take turns, so an MFMA
    // never waits for the one before it.  The products come in groups (a size class of one head-dim step); a group's
    // Q and dO terms are read from LDS while the group before it runs, and read again by a later group rather than
    // kept: registers are what limits this kernel, LDS bandwidth is not.
    constexpr int groups1 = 3 * KS;
    bf16x8a fa[2][3], fg[2][3];
    auto readGroup1 = [&](int gi) {
        const int ks = gi % KS, cls = gi / KS;   // 0 small (terms 0, 1, 2), 1 middle (0, 1), 2 large (0)
        const unsigned short* qrow = qimg + li * QP + ks * 16 + half * 8;
        const unsigned short* grow = gimg + li * QP + ks * 16 + half * 8;
#pragma unroll
        for (int im = 0; im < 3 - cls; ++im) {
            fa[gi & 1][im] = *reinterpret_cast<const bf16x8a*>(qrow + im * IMG);
            fg[gi & 1][im] = *reinterpret_cast<const bf16x8a*>(grow + im * IMG);
        }
    };
    // Stage two's operands: the transposed reads of one LDS term of one half (st) at a time, two groups ahead
    bf16x8a tg[3][DT], tq[3][DT];
    auto readGroup2 = [&](int gi) {
        const int st = gi / 3, im = 2 - gi % 3;   // LDS terms in the order low, middle, high
        const int fragRow = 4 * (lane >> 5) + ((lane & 15) >> 2), fragCol = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            tg[gi % 3][dt] = readTransposedApart(gprev + im * IMG + (16 * st + fragRow) * QP + dt * 32 + fragCol, QP);
            tq[gi % 3][dt] = readTransposedApart(qprev + im * IMG + (16 * st + fragRow) * QP + dt * 32 + fragCol, QP);
        }
    };
    constexpr int pairsPerSlice = 4 / KS;   // 16 pairs over the 4 KS slices of stage one
    readGroup1(0);
#pragma unroll
    for (int i = 0; i < 12 * KS; ++i) {
        int gi, at, bt;
        bool first;
        if (i < 6 * KS) {
            gi = i / 6;
            first = i % 6 == 0;
            const int pair = (i % 6) >> 1;
            at = pair == 0 ? 1 : pair == 1 ? 2 : 0;
            bt = pair == 0 ? 1 : pair == 1 ? 0 : 2;
        } else if (i < 10 * KS) {
            gi = KS + (i - 6 * KS) / 4;
            first = (i - 6 * KS) % 4 == 0;
            const int pair = ((i - 6 * KS) % 4) >> 1;
            at = pair == 0 ? 1 : 0;
            bt = pair == 0 ? 0 : 1;
        } else {
            gi = 2 * KS + (i - 10 * KS) / 2;
            first = (i - 10 * KS) % 2 == 0;
            at = 0;
            bt = 0;
        }
        const int ks = gi % KS;
        if (first) {
            if (gi + 1 < groups1) readGroup1(gi + 1);
            if (gi == groups1 - 2) readGroup2(0);
            if (gi == groups1 - 1) readGroup2(1);
        }
        if (i & 1) dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fg[gi & 1][at], vf[ks][bt], dp, 0, 0, 0);
        else s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[gi & 1][at], kf[ks][bt], s, 0, 0, 0);
        // a third of a pair's split after every MFMA, and a fence: nothing moves across, so the matrix pipe (32 clocks an
        // MFMA) and the vector unit (a wavefront alone on its SIMD issues an instruction every five clocks or so) alternate
#pragma unroll
        for (int c = 0; c < pairsPerSlice; ++c) splitPairPart((i / 3) * pairsPerSlice + c, c, i % 3);
        __builtin_amdgcn_sched_barrier(0);
    }

    // Stage two: dV += P^T dO, dK += dS^T Q of the previous tile; P and dS of this one.
    // register r: query = tile start + dRow(r, half), key = this lane's key
    float4v lse4[2], d4[2];
    auto readStats = [&](int grp) {
        lse4[grp & 1] = loadf4(stats + 8 * grp + 4 * half);
        d4[grp & 1] = loadf4(stats + 32 + 8 * grp + 4 * half);
    };
    // P and dS of register r in three parts, one after each MFMA of a slice
    auto softmaxPart = [&](int r, int part) {
        const int grp = r >> 2, c = r & 3;
        if (part == 0) {
            pr[r] = fastExp2(s[r] - lse4[grp & 1][c]);            // P
        } else if (part == 1) {
            dsv[r] = pr[r] * (dp[r] - d4[grp & 1][c]);            // dS (without the scale factor)
        } else {
            if constexpr (STORE)   // row dRow(r, half) of the sub-block, 128 contiguous bytes per half wave
                __builtin_nontemporal_store(dsv[r], dsLane + (8 * (r >> 2) + (r & 3)) * 32);
        }
    };
    constexpr int slices = 4 * DT;                  // slices of three MFMAs in each half of stage two
    constexpr int registersPerSlice = 2 / DT;       // 16 registers over the 8 DT slices
    static_assert(DT == 1 || DT == 2, "the pipelined form is laid out for head dims 32 and 64");
    readStats(0);
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
        for (int q = 0; q < 12 * DT; ++q) {
            const int pr6 = q / (2 * DT), dt = (q / 2) % DT;
            const int regTerm = kSplitOrder[pr6][0], ldsTerm = kSplitOrder[pr6][1];
            const int gi = 3 * st + (2 - ldsTerm);
            const bool first = q == 0 || kSplitOrder[(q - 1) / (2 * DT)][1] != ldsTerm;
            if (first && gi + 2 < 6) readGroup2(gi + 2);
            if (q & 1) dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8a, df[st][regTerm]), tq[gi % 3][dt], dk[dt], 0, 0, 0);
            else dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8a, pf[st][regTerm]), tg[gi % 3][dt], dv[dt], 0, 0, 0);
#pragma unroll
            for (int c = 0; c < registersPerSlice; ++c) {
                const int r = (st * slices + q / 3) * registersPerSlice + c;
                if (q % 3 == 0 && (r & 3) == 0 && r + 4 < 16) readStats((r >> 2) + 1);
                softmaxPart(r, q % 3);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// The last pending tile's dV and dK (no tile follows to share the step with).
template <int HDP>
__device__ __forceinline__ void dkvSplitDrain(const unsigned short* __restrict__ qprev, const unsigned short* __restrict__ gprev,
                                              float16v (&dk)[HDP / 32], float16v (&dv)[HDP / 32], const float16v& pr, const float16v& dsv,
                                              int lane) {
    constexpr int DT = HDP / 32;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
        bf16x8a pf[3], df[3];
        {
            float x[8], y[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) { x[e] = pr[8 * st + e]; y[e] = dsv[8 * st + e]; }
            splitOperand(x, pf[0], pf[1], pf[2]);
            splitOperand(y, df[0], df[1], df[2]);
        }
        bf16x8a gfr[DT][3], qfr[DT][3];
        readSplitTransposed<HDP>(gfr, qfr, qprev, gprev, st, lane);
#pragma unroll
        for (int pr6 = 0; pr6 < 6; ++pr6)
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                dv[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pf[kSplitOrder[pr6][0]], gfr[dt][kSplitOrder[pr6][1]], dv[dt], 0, 0, 0);
                dk[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(df[kSplitOrder[pr6][0]], qfr[dt][kSplitOrder[pr6][1]], dk[dt], 0, 0, 0);
            }
    }
}

template <int HDP, bool VEC4, bool STORE>
__global__ void __launch_bounds__(256, 1) attnBackwardDkvPipedKernel(AttnParams p) {
    constexpr int BQ = 32, QP = splitKeyPitch(HDP), TILE = 3 * BQ * QP, DT = HDP / 32, KS = HDP / 16;
    extern __shared__ __attribute__((aligned(16))) unsigned short smemSplit[];
    unsigned short* qs = smemSplit;                 // [3][3][BQ][QP]
    unsigned short* gs = smemSplit + 3 * TILE;      // [3][3][BQ][QP]
    float* stats = reinterpret_cast<float*>(smemSplit + 6 * TILE);   // [3][2*BQ]: lse2 | D

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    int bh, kt;
    decodeBlock(p.numTiles, gridDim.x, false, bh, kt);   // the first key tile is seen by every query: heaviest
    const int b = bh / p.heads, h = bh - b * p.heads;
    const int hd = p.hd, dim = p.dim;
    const size_t qOff = size_t(b) * p.newLen * dim + size_t(h) * hd;
    const size_t kOff = size_t(b) * p.totalLen * dim + size_t(h) * hd;
    const size_t statOff = (size_t(b) * p.heads + h) * p.newLen;

    const int waveK0 = kt * 128 + wave * 32;
    const int key = waveK0 + li;                       // this lane's key (as B-operand column)
    const bool keyValid = key < p.totalLen;
    bf16x8a kf[KS][3], vf[KS][3];
    loadSplitFragments<HDP, VEC4>(kf, p.k + kOff + size_t(key) * dim, p.scale * kLog2e, keyValid, hd, half);
    loadSplitFragments<HDP, VEC4>(vf, p.v + kOff + size_t(key) * dim, 1.0f, keyValid, hd, half);

    float16v dk[DT], dv[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk[dt][r] = 0.0f; dv[dt][r] = 0.0f; }

    // first query that can see any key of this workgroup's tile: oldLen + i >= kt*128
    int firstQuery = kt * 128 - p.oldLen;
    if (firstQuery < 0) firstQuery = 0;
    const int q0Start = (firstQuery / BQ) * BQ;
    const int numQTiles = q0Start < p.newLen ? (p.newLen - q0Start + BQ - 1) / BQ : 0;

    const size_t dsStride = size_t(p.nkb) * 1024;
    float* const dsColumn = STORE ? p.ds + (size_t(bh) * p.nqb * p.nkb + size_t(waveK0 >> 5)) * 1024 : nullptr;   // wave-uniform
    const int dsLaneOffset = half * 128 + li;

    // a tile's loads are issued one step before it is written to LDS and two before it is read.  Rows past the last
    // query repeat it: their statistic is +inf, so their P and dS are zero whatever Q and dO hold there.
    TileRegs<HDP, BQ> qStage, gStage;
    float statStage = 0.0f;
    const int fetchColumn = (tid % (HDP / 4)) * 4;
    const float* const qColumn = p.q + qOff + fetchColumn;
    const float* const gColumn = p.dO + qOff + fetchColumn;
    auto fetchAll = [&](int qt0) {
        if constexpr (VEC4) {
            fetchRowsClamped<HDP, BQ>(qStage, qColumn, fetchColumn < hd, dim, qt0, p.newLen - 1, tid);
            fetchRowsClamped<HDP, BQ>(gStage, gColumn, fetchColumn < hd, dim, qt0, p.newLen - 1, tid);
        } else {
            fetchHeadTile<HDP, BQ, false>(qStage, p.q + qOff, dim, qt0, p.newLen, hd, tid);
            fetchHeadTile<HDP, BQ, false>(gStage, p.dO + qOff, dim, qt0, p.newLen, hd, tid);
        }
        const int j = tid < BQ ? tid : tid - BQ;
        const int qi = qt0 + j;
        if (tid < BQ) statStage = qi < p.newLen ? p.lse2[statOff + qi] : INFINITY;
        else if (tid < 2 * BQ) statStage = qi < p.newLen ? p.dvec[statOff + qi] : 0.0f;
    };
    auto commitAll = [&](int buf) {
        commitSplitTile<HDP, BQ, QP>(qs + buf * TILE, qStage, tid);
        commitSplitTile<HDP, BQ, QP>(gs + buf * TILE, gStage, tid);
        if (tid < 2 * BQ) stats[buf * 2 * BQ + tid] = statStage;
    };
    if (numQTiles > 0) {
        fetchAll(q0Start);
        commitAll(0);
        if (numQTiles > 1) fetchAll(q0Start + BQ);
    }
    __syncthreads();
    float16v pr, dsv;       // P and dS of the tile whose dV and dK products are still to come
#pragma unroll
    for (int r = 0; r < 16; ++r) { pr[r] = 0.0f; dsv[r] = 0.0f; }
    int cur = 0, prev = 0;   // LDS buffers of tile t and tile t-1 (at t = 0 any initialised buffer); tile t+1 goes to a third
    int t = 0;
    // the end of every tile's step: the next tile goes to LDS, the loads of the one after it are issued, buffers turn
    auto advance = [&]() {
        const int next = cur == 2 ? 0 : cur + 1;
        if (t + 1 < numQTiles) {
            commitAll(next);
            if (t + 2 < numQTiles) fetchAll(q0Start + (t + 2) * BQ);
        }
        prev = cur;
        cur = next;
        ++t;
        __syncthreads();
    };
    // A wavefront's tiles come in three runs: tiles none of whose queries sees its keys, masked tiles (the diagonal;
    // every tile when the key block runs past the sequence), unmasked tiles.  Both conditions fall as the queries
    // advance, so the runs follow each other.  The first two go through one loop with the unpiped form, the third
    // through the pipeline; each loop has the one barrier per tile, so the wavefronts of a workgroup stay in step
    // although they change loops at different tiles.
    const bool waveHasKeys = waveK0 < p.totalLen;
    const bool tailBlock = waveK0 + 32 > p.totalLen;
    for (; t < numQTiles; advance()) {
        const int qt0 = q0Start + t * BQ;
        const bool visible = waveHasKeys && p.oldLen + qt0 + BQ - 1 >= waveK0;
        const bool masked = tailBlock || waveK0 + 31 > p.oldLen + qt0;
        if (visible && !masked) break;
        if (visible) {
            float* dsLane = STORE ? dsColumn + size_t(qt0 >> 5) * dsStride + dsLaneOffset : nullptr;
            dkvSplitTile<HDP, true, STORE>(qs + cur * TILE, gs + cur * TILE, stats + cur * 2 * BQ, kf, vf, dk, dv, qt0, key, keyValid, p.oldLen, lane,
                                           dsLane);
        }
    }
    if (t == numQTiles) {   // no unmasked tile; the stores appear on both paths so that neither loop copies registers for the other
        storeKeyGradients<HDP>(p, dk, dv, b, h, waveK0, kOff, half, li);
        return;
    }
    for (; t < numQTiles; advance()) {
        // with nothing pending P and dS are zero and the second stage adds zeros (the operands it reads are finite)
        const int qt0 = q0Start + t * BQ;
        float* dsLane = STORE ? dsColumn + size_t(qt0 >> 5) * dsStride + dsLaneOffset : nullptr;
        dkvSplitStep<HDP, STORE>(qs + cur * TILE, gs + cur * TILE, stats + cur * 2 * BQ, qs + prev * TILE, gs + prev * TILE, kf, vf, dk, dv, pr, dsv,
                                 lane, dsLane);
    }
    dkvSplitDrain<HDP>(qs + prev * TILE, gs + prev * TILE, dk, dv, pr, dsv, lane);
    storeKeyGradients<HDP>(p, dk, dv, b, h, waveK0, kOff, half, li);
}

// ---------------------------------------------------------------------------------------------
// dQ from stored dS on the split route: dQ^T += K^T dS^T with both operands as three bf16 terms.  K tiles (32 keys) are
// split when they are written to LDS (images [3][32][pitch], read through the transposing LDS read as A operands: eight
// consecutive keys per lane); a dS sub-block goes through the wave's LDS patch as in the fp32 kernel and is split in
// registers (B operand: lane (query, half) holds keys 16 ks + 8 half + 0..7).  Several sub-blocks of the wave's row are
// kept in flight in registers: the kernel is bound by that stream, which is why it gains less than the others.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ bf16x8a readTransposedNear(const unsigned short* p, int rowPitch) {
    typedef __attribute__((address_space(3))) short4a* LdsPtr;
    const short4a lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(p));
    const short4a hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(p + 4 * rowPitch));
    const short8a both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8a, both);
}

template <int HDP, bool VEC4>
__global__ void __launch_bounds__(256, HDP <= 128 ? 2 : 1) attnBackwardDqFromDsSplitKernel(AttnParams p) {
    constexpr int DEPTH = HDP <= 64 ? 3 : 2;   // dS sub-blocks in flight per wavefront
    constexpr int BC = 32, PITCH = splitValuePitch(HDP), IMG = BC * PITCH, KTILE = 3 * IMG, DT = HDP / 32;
    extern __shared__ __attribute__((aligned(16))) unsigned short smemSplit[];
    unsigned short* kimg = smemSplit;                                          // [2][3][BC][PITCH]
    float* patches = reinterpret_cast<float*>(smemSplit + 2 * KTILE);          // [4][kDsPatch]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    int bh, qt;
    decodeBlock(p.numTiles, gridDim.x, true, bh, qt);
    const int b = bh / p.heads, h = bh - b * p.heads;
    const int hd = p.hd, dim = p.dim;
    const size_t qOff = size_t(b) * p.newLen * dim + size_t(h) * hd;
    const float* kb = p.k + size_t(b) * p.totalLen * dim + size_t(h) * hd;

    const int waveQ0 = qt * 128 + wave * 32;
    const int i = waveQ0 + li;
    // keys below waveKeyEnd are visible to some query of this wave's sub-block row (none if the row is past newLen)
    const int waveKeyEnd = waveQ0 < p.newLen ? min(p.totalLen, p.oldLen + waveQ0 + 32) : 0;
    const float* dsWave = p.ds + ((size_t(bh) * p.nqb + size_t(waveQ0 >> 5)) * p.nkb) * 1024 + lane * 4;
    float* patch = patches + wave * kDsPatch;

    // small term products in one accumulator, large ones in the other where the head dim alone gives too few independent chains
    constexpr int NACC = DT >= 4 ? 1 : 2, SM = NACC - 1;
    float16v acc[NACC][DT];
#pragma unroll
    for (int a = 0; a < NACC; ++a)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][dt][r] = 0.0f;

    const int lastQuery = min(p.newLen, qt * 128 + 128) - 1;
    const int blockKeyEnd = min(p.totalLen, p.oldLen + lastQuery + 1);
    const int numKeyTiles = (blockKeyEnd + BC - 1) / BC;

    float4v dsStage[DEPTH][4];
    auto fetchDs = [&](int t, float4v (&dst)[4]) {
        if (t * BC < waveKeyEnd) {
            const float* src = dsWave + size_t(t) * 1024;
#pragma unroll
            for (int j = 0; j < 4; ++j) dst[j] = __builtin_nontemporal_load(reinterpret_cast<const float4v*>(src + j * 256));
        }
    };
    const int fragRow = (lane >> 5) * 8 + ((lane & 15) >> 2), fragCol = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;

    TileRegs<HDP, BC> kNext;
    fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, 0, p.totalLen, hd, tid);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
        if (d < numKeyTiles) fetchDs(d, dsStage[d]);
    commitSplitTile<HDP, BC, PITCH>(kimg, kNext, tid);
    if (numKeyTiles > 1) fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, BC, p.totalLen, hd, tid);
    __syncthreads();
    for (int t0 = 0; t0 < numKeyTiles; t0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int t = t0 + d;
            if (t >= numKeyTiles) break;
            const unsigned short* kcur = kimg + (t & 1) * KTILE;
            const bool live = t * BC < waveKeyEnd;
            bf16x8a b3[2][3];
            if (live) {
#pragma unroll
                for (int j = 0; j < 4; ++j) storef4(patch + (8 * j + (lane >> 3)) * 36 + (lane & 7) * 4, dsStage[d][j]);
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const float4v lo = loadf4(patch + li * 36 + ks * 16 + half * 8);
                    const float4v hi = loadf4(patch + li * 36 + ks * 16 + half * 8 + 4);
                    const float x[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                    splitOperand(x, b3[ks][0], b3[ks][1], b3[ks][2]);
                }
            }
            if (t + DEPTH < numKeyTiles) fetchDs(t + DEPTH, dsStage[d]);
            if (live) {
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    bf16x8a a3[DT][3];
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                        for (int im = 0; im < 3; ++im) a3[dt][im] = readTransposedNear(kcur + im * IMG + (ks * 16 + fragRow) * PITCH + dt * 32 + fragCol, PITCH);
                    // (K term, dS term): consecutive MFMAs alternate accumulators
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        acc[SM][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[dt][1], b3[ks][1], acc[SM][dt], 0, 0, 0);
                        acc[0][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[dt][0], b3[ks][0], acc[0][dt], 0, 0, 0);
                    }
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        acc[SM][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[dt][2], b3[ks][0], acc[SM][dt], 0, 0, 0);
                        acc[0][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[dt][1], b3[ks][0], acc[0][dt], 0, 0, 0);
                    }
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        acc[SM][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[dt][0], b3[ks][2], acc[SM][dt], 0, 0, 0);
                        acc[0][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a3[dt][0], b3[ks][1], acc[0][dt], 0, 0, 0);
                    }
                }
            }
            if (t + 1 < numKeyTiles) {
                commitSplitTile<HDP, BC, PITCH>(kimg + ((t + 1) & 1) * KTILE, kNext, tid);
                if (t + 2 < numKeyTiles) fetchHeadTile<HDP, BC, VEC4>(kNext, kb, dim, (t + 2) * BC, p.totalLen, hd, tid);
            }
            __syncthreads();
        }
    }
    if constexpr (NACC == 2) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[0][dt][r] += acc[SM][dt][r];
    }
    if (i < p.newLen) {
        if (p.dQ) storeTransposed<HDP, VEC4>(p.dQ + qOff + size_t(i) * dim, acc[0], hd, half, p.scale);
        if (p.dQImg) storeTransposedBf16<HDP, VEC4>(p.dQImg + (size_t(b) * p.newLen + i) * p.imgLd + size_t(h) * hd, acc[0], hd, half, p.scale);
    }
}

// ---------------------------------------------------------------------------------------------
// The forward kernel on the split route as a two-stage pipeline over key tiles (the scheme of the dK/dV pipeline
// above).  While S^T of tile t+1 runs on the matrix pipe the vector unit splits P of tile t; while O^T += V^T P^T of
// tile t runs, it takes the row maximum, the exponentials and the row sum of tile t+1.  One MFMA and one part of the
// vector work at a time, a scheduling fence after each.  A move of the reference maximum found while the products of
// the tile before are still in flight is applied to the accumulator after them.  K tiles are written to LDS two tiles
// ahead of their products and V tiles one tile ahead, so two buffers of each suffice.  A wavefront's masked tiles are
// its last ones, so it passes from the loop with unmasked next tiles to the loop with masked ones, then to the last
// tile's products alone, then waits out the workgroup's remaining tiles; every loop has the one barrier per tile.
// ---------------------------------------------------------------------------------------------
template <int HDP>
__device__ __forceinline__ float16v forwardSplitScores(const unsigned short* __restrict__ kimg, const bf16x8a (&qf)[HDP / 16][3], int lane) {
    constexpr int KP = splitKeyPitch(HDP), KIMG = 32 * KP, KS = HDP / 16;
    const int half = lane >> 5, li = lane & 31;
    float16v s0, s1, s2;
#pragma unroll
    for (int r = 0; r < 16; ++r) { s0[r] = 0.0f; s1[r] = 0.0f; s2[r] = 0.0f; }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const unsigned short* krow = kimg + li * KP + ks * 16 + half * 8;
        bf16x8a a[3];
#pragma unroll
        for (int im = 0; im < 3; ++im) a[im] = *reinterpret_cast<const bf16x8a*>(krow + im * KIMG);
        s2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], qf[ks][1], s2, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], qf[ks][0], s1, 0, 0, 0);
        s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], qf[ks][0], s0, 0, 0, 0);
        s2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[2], qf[ks][0], s2, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], qf[ks][1], s1, 0, 0, 0);
        s2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], qf[ks][2], s2, 0, 0, 0);
    }
    float16v sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = (s2[r] + s1[r]) + s0[r];
    return sc;
}

// Scores of the first tile to probabilities about a fresh reference maximum (nothing accumulated yet).
template <bool MASKED>
__device__ __forceinline__ void forwardFirstSoftmax(float16v& sc, float& mrow, float& mref, float& lrow, int kt0, int myLimit, int totalLen,
                                                    int lane) {
    const int half = lane >> 5;
    if constexpr (MASKED) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = kt0 + dRow(r, half);
            sc[r] = (key > myLimit || key >= totalLen) ? -INFINITY : sc[r];
        }
    }
    float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
#pragma unroll
    for (int r = 4; r < 16; r += 4) mx = fmaxf(mx, fmaxf(fmaxf(sc[r], sc[r + 1]), fmaxf(sc[r + 2], sc[r + 3])));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    mrow = mx;
    mref = mx;   // key 0 is visible to every query, so this is finite
    float psum = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) { sc[r] = fastExp2(sc[r] - mref); psum += sc[r]; }
    lrow = psum;
}

// One step: `pc` comes in as P of the current tile (probabilities about mref, accumulator layout) and leaves as P of the
// next one; knext = K images of the next tile, vcur = V images of the current one.
template <int HDP, bool MASKED, bool HAS_NEXT>
__device__ __forceinline__ void forwardPipedStep(const unsigned short* __restrict__ knext, const unsigned short* __restrict__ vcur,
                                                 const bf16x8a (&qf)[HDP / 16][3], float16v (&acc)[HDP / 32], float16v& pc, float& mrow,
                                                 float& mref, float& lrow, int ktNext0, int myLimit, int totalLen, int lane) {
    constexpr int KP = splitKeyPitch(HDP), VP = splitValuePitch(HDP), KIMG = 32 * KP, VIMG = 32 * VP, DT = HDP / 32, KS = HDP / 16;
    const int half = lane >> 5, li = lane & 31;
    uint4a pf[2][3];   // bf16 pairs; an operand is one of these as eight bf16
    float rest[2];
    // the split of pair i of P (registers 2 i, 2 i + 1; step st = i / 4 contracts over registers 8 st + e) in three parts
    auto splitPart = [&](int i, int part) {
        const int st = i >> 2, e = i & 3;
        if (part == 0) {
            const float x0 = pc[2 * i], x1 = pc[2 * i + 1];
            const unsigned h = packBf16(x0, x1);
            pf[st][0][e] = h;
            rest[0] = x0 - __builtin_bit_cast(float, h << 16);
            rest[1] = x1 - __builtin_bit_cast(float, h & 0xffff0000u);
        } else if (part == 1) {
            const unsigned m = packBf16(rest[0], rest[1]);
            pf[st][1][e] = m;
            rest[0] -= __builtin_bit_cast(float, m << 16);
            rest[1] -= __builtin_bit_cast(float, m & 0xffff0000u);
        } else {
            pf[st][2][e] = packBf16(rest[0], rest[1]);
        }
    };
    // V^T operands of stage two: the transposed reads of one LDS term of one half (st) at a time, two groups ahead
    bf16x8a tv[3][DT];
    auto readV = [&](int gi) {
        const int st = gi / 3, im = 2 - gi % 3;   // LDS terms in the order low, middle, high
        const int fragRow = 4 * (lane >> 5) + ((lane & 15) >> 2), fragCol = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) tv[gi % 3][dt] = readTransposedApart(vcur + im * VIMG + (16 * st + fragRow) * VP + dt * 32 + fragCol, VP);
    };

    // stage one: S^T = K Q^T of the next tile, one chain, the products in the order of their size (see the dK/dV pipeline)
    float16v s;
    if constexpr (HAS_NEXT) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.0f;
        bf16x8a a[KS][3];
        auto readK = [&](int ks) {
            const unsigned short* krow = knext + li * KP + ks * 16 + half * 8;
#pragma unroll
            for (int im = 0; im < 3; ++im) a[ks][im] = *reinterpret_cast<const bf16x8a*>(krow + im * KIMG);
        };
        readK(0);
        if (KS > 1) readK(1);
#pragma unroll
        for (int j = 0; j < 6 * KS; ++j) {
            int ks, at, bt;
            if (j < 3 * KS) {
                ks = j / 3;
                at = j % 3 == 0 ? 1 : j % 3 == 1 ? 2 : 0;
                bt = j % 3 == 0 ? 1 : j % 3 == 1 ? 0 : 2;
                if (j % 3 == 0 && ks + 2 < KS) readK(ks + 2);
            } else if (j < 5 * KS) {
                ks = (j - 3 * KS) / 2;
                at = (j - 3 * KS) % 2 == 0 ? 1 : 0;
                bt = (j - 3 * KS) % 2 == 0 ? 0 : 1;
                if (j == 3 * KS) readV(0);
            } else {
                ks = j - 5 * KS;
                at = 0;
                bt = 0;
                if (j == 5 * KS) readV(1);
            }
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ks][at], qf[ks][bt], s, 0, 0, 0);
            // 24 parts of the split over 6 KS MFMAs
#pragma unroll
            for (int c = (24 * j) / (6 * KS); c < (24 * (j + 1)) / (6 * KS); ++c) splitPart(c / 3, c % 3);
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
        readV(0);
        readV(1);
#pragma unroll
        for (int c = 0; c < 24; ++c) splitPart(c / 3, c % 3);
    }

    // stage two: O^T += V^T P^T of the current tile; maximum, exponentials and sum of the next one in 22 parts
    float mx4[4], mrefNew = mref, psum = 0.0f;
    bool moved = false;
    auto softmaxPart = [&](int part) {
        if (part < 4) {          // mask and maximum of four registers
            if constexpr (MASKED) {
#pragma unroll
                for (int r = 4 * part; r < 4 * part + 4; ++r) {
                    const int key = ktNext0 + dRow(r, half);
                    s[r] = (key > myLimit || key >= totalLen) ? -INFINITY : s[r];
                }
            }
            mx4[part] = fmaxf(fmaxf(s[4 * part], s[4 * part + 1]), fmaxf(s[4 * part + 2], s[4 * part + 3]));
        } else if (part == 4) {  // row maximum; the reference moves when the maximum has outgrown it
            float mx = fmaxf(fmaxf(mx4[0], mx4[1]), fmaxf(mx4[2], mx4[3]));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            mrow = fmaxf(mrow, mx);
            moved = mrow > mref + kRescaleThreshold;
            mrefNew = moved ? mrow : mref;
        } else if (part < 21) {  // one exponential
            const int r = part - 5;
            pc[r] = fastExp2(s[r] - mrefNew);
            psum += pc[r];
        }
    };
    constexpr int slots = 12 * DT;
#pragma unroll
    for (int st = 0; st < 2; ++st) {
#pragma unroll
        for (int q = 0; q < 6 * DT; ++q) {
            const int pr6 = q / DT, dt = q % DT;
            const int regTerm = kSplitOrder[pr6][0], ldsTerm = kSplitOrder[pr6][1];
            const int gi = 3 * st + (2 - ldsTerm);
            const bool first = q == 0 || kSplitOrder[(q - 1) / DT][1] != ldsTerm;
            if (first && gi + 2 < 6) readV(gi + 2);
            acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tv[gi % 3][dt], __builtin_bit_cast(bf16x8a, pf[st][regTerm]), acc[dt], 0, 0, 0);
            if constexpr (HAS_NEXT) {
                const int n = st * 6 * DT + q;
#pragma unroll
                for (int c = (21 * n) / slots; c < (21 * (n + 1)) / slots; ++c) softmaxPart(c);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if constexpr (HAS_NEXT) {
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {   // the products above used the old reference: rescale what they left
            const float corr = moved ? fastExp2(mref - mrefNew) : 1.0f;
            lrow *= corr;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[dt][r] *= corr;
        }
        mref = mrefNew;
        lrow += psum;
    }
}

template <int HDP, bool VEC4>
__global__ void __launch_bounds__(256, HDP <= 64 ? 2 : 1) attnForwardPipedKernel(AttnParams p) {
    applyKeyChunk(p);
    constexpr int BC = 32, KP = splitKeyPitch(HDP), VP = splitValuePitch(HDP), KTILE = 3 * BC * KP, VTILE = 3 * BC * VP, DT = HDP / 32, KS = HDP / 16;
    extern __shared__ __attribute__((aligned(16))) unsigned short smemSplit[];
    unsigned short* ks = smemSplit;               // [2][3][BC][KP]
    unsigned short* vs = smemSplit + 2 * KTILE;   // [2][3][BC][VP]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    int bh, qt;
    decodeBlock(p.numTiles, gridDim.x, true, bh, qt);
    const int b = bh / p.heads, h = bh - b * p.heads;
    if (chunkIsEmptyFor(p, qt)) {                 // the same for the whole workgroup, before any barrier
        writeEmptyChunk(p, b, h, qt);
        return;
    }
    const int hd = p.hd, dim = p.dim;
    const float* qb = p.q + size_t(b) * p.newLen * dim + size_t(h) * hd;
    const float* kb = p.k + size_t(b) * p.kvRows * dim + size_t(h) * hd;
    const float* vb = p.v + size_t(b) * p.kvRows * dim + size_t(h) * hd;

    const int waveQ0 = qt * 128 + wave * 32;
    const int i = waveQ0 + li;                    // this lane's query row
    const bool rowValid = i < p.newLen;
    // Q fragments: step ks of a lane in `half` holds head-dim elements 16 ks + 8 half + 0..7 of its query, scaled
    bf16x8a qf[KS][3];
    loadSplitFragments<HDP, VEC4>(qf, qb + size_t(i) * dim, p.scale * kLog2e, rowValid, hd, half);

    float16v acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.0f;
    float mrow = -INFINITY, mref = -INFINITY, lrow = 0.0f;

    const int lastQuery = min(p.newLen, qt * 128 + 128) - 1;
    const int blockKeyEnd = min(p.totalLen, p.oldLen + lastQuery + 1);   // keys >= this are invisible to the tile
    const int waveKeyEnd = p.oldLen + waveQ0 + 32;                       // keys >= this are invisible to the wave
    const int myLimit = p.oldLen + i;                                    // last visible key of this lane's row
    const int numKeyTiles = (blockKeyEnd + BC - 1) / BC;
    const int waveTiles = min(numKeyTiles, (waveKeyEnd + BC - 1) / BC);  // the wave's tiles are the first waveTiles ones
    auto maskedTile = [&](int t) { return (t * BC + BC - 1 > p.oldLen + waveQ0) || (t * BC + BC > p.totalLen); };

    // K tiles 0 and 1 and V tile 0 to LDS; K tile 2 and V tile 1 on their way in registers
    TileRegs<HDP, BC> kStage, vStage;
    fetchHeadTile<HDP, BC, VEC4>(kStage, kb, dim, 0, p.totalLen, hd, tid);
    fetchHeadTile<HDP, BC, VEC4>(vStage, vb, dim, 0, p.totalLen, hd, tid);
    commitSplitTile<HDP, BC, KP>(ks, kStage, tid);
    commitSplitTile<HDP, BC, VP>(vs, vStage, tid);
    if (numKeyTiles > 1) {
        fetchHeadTile<HDP, BC, VEC4>(kStage, kb, dim, BC, p.totalLen, hd, tid);
        commitSplitTile<HDP, BC, KP>(ks + KTILE, kStage, tid);
        fetchHeadTile<HDP, BC, VEC4>(vStage, vb, dim, BC, p.totalLen, hd, tid);
    }
    if (numKeyTiles > 2) fetchHeadTile<HDP, BC, VEC4>(kStage, kb, dim, 2 * BC, p.totalLen, hd, tid);
    __syncthreads();
    // the first tile's scores and probabilities (every wavefront has a first tile: key 0 is visible to every query)
    float16v pc = forwardSplitScores<HDP>(ks, qf, lane);
    if (maskedTile(0)) forwardFirstSoftmax<true>(pc, mrow, mref, lrow, 0, myLimit, p.totalLen, lane);
    else forwardFirstSoftmax<false>(pc, mrow, mref, lrow, 0, myLimit, p.totalLen, lane);
    __syncthreads();   // K tile 0's buffer is written again in the first step

    int t = 0;
    // the end of every tile's step: K tile t+2 and V tile t+1 go to LDS, the loads of K tile t+3 and V tile t+2 are issued
    auto advance = [&]() {
        if (t + 2 < numKeyTiles) commitSplitTile<HDP, BC, KP>(ks + (t & 1) * KTILE, kStage, tid);
        if (t + 1 < numKeyTiles) commitSplitTile<HDP, BC, VP>(vs + ((t + 1) & 1) * VTILE, vStage, tid);
        if (t + 3 < numKeyTiles) fetchHeadTile<HDP, BC, VEC4>(kStage, kb, dim, (t + 3) * BC, p.totalLen, hd, tid);
        if (t + 2 < numKeyTiles) fetchHeadTile<HDP, BC, VEC4>(vStage, vb, dim, (t + 2) * BC, p.totalLen, hd, tid);
        ++t;
        __syncthreads();
    };
    for (; t + 1 < waveTiles && !maskedTile(t + 1); advance())
        forwardPipedStep<HDP, false, true>(ks + ((t + 1) & 1) * KTILE, vs + (t & 1) * VTILE, qf, acc, pc, mrow, mref, lrow, (t + 1) * BC, myLimit, p.totalLen, lane);
    for (; t + 1 < waveTiles; advance())
        forwardPipedStep<HDP, true, true>(ks + ((t + 1) & 1) * KTILE, vs + (t & 1) * VTILE, qf, acc, pc, mrow, mref, lrow, (t + 1) * BC, myLimit, p.totalLen, lane);
    forwardPipedStep<HDP, false, false>(nullptr, vs + (t & 1) * VTILE, qf, acc, pc, mrow, mref, lrow, 0, myLimit, p.totalLen, lane);
    for (advance(); t < numKeyTiles; advance()) {}

    lrow += __shfl_xor(lrow, 32, 64);
    if (rowValid) {
        if (p.out) storeTransposed<HDP, VEC4>(p.out + (size_t(b) * p.newLen + i) * dim + size_t(h) * hd, acc, hd, half, 1.0f / lrow);
        if (p.outImg) storeTransposedBf16<HDP, VEC4>(p.outImg + (size_t(b) * p.newLen + i) * p.imgLd + size_t(h) * hd, acc, hd, half, 1.0f / lrow);
        if (half == 0) {
            size_t idx = (size_t(b) * p.heads + h) * p.newLen + i;
            p.m[idx] = mrow * kLn2;
            p.l[idx] = lrow * fastExp2(mref - mrow);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
int paddedHeadDim(int hd) { return hd <= 32 ? 32 : hd <= 64 ? 64 : hd <= 128 ? 128 : hd <= 192 ? 192 : 256; }

template <typename K>
int launchAttn(K kernel, size_t smemBytes, unsigned grid, const AttnParams& p, hipStream_t s) {
    int st = allowDynamicSharedMemory(reinterpret_cast<const void*>(kernel), smemBytes);
    if (st != BF_OK) return st;
    kernel<<<dim3(grid, unsigned(p.numChunks > 1 ? p.numChunks : 1)), 256, smemBytes, s>>>(p);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

// The chunks of a forward pass over the keys in chunks, put together: with chunk c's row maximum m_c, sum l_c of
// exp(score - m_c) and normalised output O_c, the row's maximum is M = max m_c, its sum L = sum_c l_c exp(m_c - M), and
// its output sum_c (l_c exp(m_c - M) / L) O_c.  One workgroup per (batch, query, head): the threads read the chunks'
// statistics side by side, and each of the four wavefronts adds every fourth chunk's output (head dims up to 256: four
// columns a lane), the four sums joined in wavefront order.
__global__ void __launch_bounds__(256) attnCombineChunksKernel(const float* __restrict__ partOut, const float* __restrict__ partM,
                                                               const float* __restrict__ partL, float* __restrict__ out,
                                                               unsigned short* __restrict__ outImg, size_t imgLd, float* __restrict__ m,
                                                               float* __restrict__ l, int heads, int newLen, int dim, int hd, int numChunks,
                                                               size_t partOutStride, size_t partStatStride) {
    __shared__ float sReduce[4];
    __shared__ float sWeight[256];
    __shared__ float sAcc[4][256];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const size_t group = blockIdx.x;                                    // (b, i, h), h fastest
    const int h = int(group % heads);
    const size_t bi = group / heads;                                    // b * newLen + i
    const size_t b = bi / newLen, i = bi - b * newLen;
    const size_t stat = (b * heads + h) * newLen + i;

    float rowMax = -INFINITY;
    for (int c = t; c < numChunks; c += 256) rowMax = fmaxf(rowMax, partM[c * partStatStride + stat]);
    for (int o = 32; o > 0; o >>= 1) rowMax = fmaxf(rowMax, __shfl_xor(rowMax, o, 64));
    if (lane == 0) sReduce[wave] = rowMax;
    __syncthreads();
    rowMax = fmaxf(fmaxf(sReduce[0], sReduce[1]), fmaxf(sReduce[2], sReduce[3]));
    __syncthreads();
    float total = 0.0f;
    for (int c = t; c < numChunks; c += 256) total += partL[c * partStatStride + stat] * expf(partM[c * partStatStride + stat] - rowMax);
    for (int o = 32; o > 0; o >>= 1) total += __shfl_xor(total, o, 64);
    if (lane == 0) sReduce[wave] = total;
    __syncthreads();
    total = (sReduce[0] + sReduce[1]) + (sReduce[2] + sReduce[3]);

    const size_t at = bi * dim + size_t(h) * hd;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c0 = 0; c0 < numChunks; c0 += 256) {
        __syncthreads();                                                // the previous round's weights have been read
        if (c0 + t < numChunks) sWeight[t] = partL[(c0 + t) * partStatStride + stat] * expf(partM[(c0 + t) * partStatStride + stat] - rowMax);
        __syncthreads();
        const int count = min(256, numChunks - c0);
#pragma unroll 4
        for (int c = wave; c < count; c += 4) {
            const float w = sWeight[c];
            const float* src = partOut + (c0 + c) * partOutStride + at;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (lane + 64 * j < hd) acc[j] += w * src[lane + 64 * j];
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) sAcc[wave][lane + 64 * j] = acc[j];
    __syncthreads();
    if (t < hd) {
        const float value = ((sAcc[0][t] + sAcc[1][t]) + (sAcc[2][t] + sAcc[3][t])) / total;
        if (out) out[at + t] = value;
        if (outImg) outImg[bi * imgLd + size_t(h) * hd + t] = toBf16Bits(value);
    }
    if (t == 0) { m[stat] = rowMax; l[stat] = total; }
}

// Forward pass of at most a few queries per sequence (a step of incremental decoding) without tiles: a 128-query tile
// would hold one live row, and the pass is a walk over the cached keys and values anyway.  LPK lanes share a key: each
// holds four of the head's columns (16 bytes of the key's row, the same of the value's), the dot product is a butterfly
// over those lanes, and each such group of lanes walks every (256 / LPK)-th key of the workgroup's chunk, eight keys a
// round, with its own running maximum, sum and output; the groups of a wavefront are joined by a butterfly, the four
// wavefronts in order through LDS.  blockIdx.x is the chunk of keys, blockIdx.y the (batch, head, query).  Head dims that
// are multiples of 4, 16-byte aligned operands.  Chunk c of numChunks > 1 writes its normalised output and statistics as
// the tile kernels do (attnCombineChunksKernel joins them); a single chunk writes the results themselves.
// The same for many rows of few chunks (a prompt's pass: thousands of (batch, query, head) rows, at most eight chunks): a
// wavefront per row, every lane with the row's chunk weights, four head columns a lane.
__global__ void __launch_bounds__(256) attnCombineRowsKernel(const float* __restrict__ partOut, const float* __restrict__ partM,
                                                             const float* __restrict__ partL, float* __restrict__ out,
                                                             unsigned short* __restrict__ outImg, size_t imgLd, float* __restrict__ m,
                                                             float* __restrict__ l, size_t groups, int heads, int newLen, int dim, int hd,
                                                             int numChunks, size_t partOutStride, size_t partStatStride) {
    const int lane = threadIdx.x & 63;
    const size_t group = size_t(blockIdx.x) * 4 + (threadIdx.x >> 6);   // (b, i, h), h fastest
    if (group >= groups) return;
    const int h = int(group % heads);
    const size_t bi = group / heads;
    const size_t b = bi / newLen, i = bi - b * newLen;
    const size_t stat = (b * heads + h) * newLen + i;
    float ms[8], ls[8];
    float rowMax = -INFINITY;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        ms[c] = c < numChunks ? partM[c * partStatStride + stat] : -INFINITY;
        ls[c] = c < numChunks ? partL[c * partStatStride + stat] : 0.0f;
        rowMax = fmaxf(rowMax, ms[c]);
    }
    float total = 0.0f;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        ls[c] = c < numChunks ? ls[c] * expf(ms[c] - rowMax) : 0.0f;   // the chunk's weight before the division
        total += ls[c];
    }
    const size_t at = bi * dim + size_t(h) * hd;
    for (int d = lane; d < hd; d += 64) {
        float acc = 0.0f;
#pragma unroll
        for (int c = 0; c < 8; ++c)
            if (c < numChunks && ls[c] != 0.0f) acc += ls[c] * partOut[c * partOutStride + at + d];
        const float value = acc / total;
        if (out) out[at + d] = value;
        if (outImg) outImg[bi * imgLd + size_t(h) * hd + d] = toBf16Bits(value);
    }
    if (lane == 0) { m[stat] = rowMax; l[stat] = total; }
}

// exp(x) for x <= 0 as the hardware's 2^(x log2 e): the walk below is a chain of a few dozen dependent steps on one
// wavefront, where the library routine's forty instructions apiece are a large part of the kernel's time
__device__ __forceinline__ float expFast(float x) { return fastExp2(x * kLog2e); }
template <int LPK>
__global__ void __launch_bounds__(256) attnFewQueriesKernel(AttnParams p) {
    constexpr int GROUPS = 256 / LPK, KEYS = LPK <= 8 ? 4 : 8;   // keys a group of lanes has in flight per round
    __shared__ float sM[4], sL[4];
    __shared__ float4v sAcc[4][LPK];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int sub = t % LPK, group = t / LPK;
    const int c = blockIdx.x;
    const int h = int(blockIdx.y) % p.heads, bi = int(blockIdx.y) / p.heads;   // bi = b * newLen + i
    const int b = bi / p.newLen, i = bi - b * p.newLen;
    const int hd = p.hd, dim = p.dim, d0 = sub * 4;
    const bool live = d0 < hd;                                 // lanes past the head's columns carry zeros
    const size_t column = size_t(h) * hd + (live ? d0 : 0);
    const float* kb = p.k + size_t(b) * p.kvRows * dim + column;
    const float* vb = p.v + size_t(b) * p.kvRows * dim + column;
    const float4v zero = {0.0f, 0.0f, 0.0f, 0.0f};
    const float4v q4 = live ? loadf4(p.q + size_t(bi) * dim + column) : zero;
    const int oldLen = p.oldLenPtr ? *p.oldLenPtr : p.oldLen;
    const int limit = min(oldLen + i + 1, p.kvRows);           // keys 0 .. oldLen + i are visible to query i
    const int start = c * p.chunkKeys;
    const int end = c == p.numChunks - 1 ? limit : min(start + p.chunkKeys, limit);

    float m = -INFINITY, l = 0.0f;
    float4v acc = zero;
    for (int j0 = start + group; j0 < end; j0 += KEYS * GROUPS) {
        float4v k4[KEYS], v4[KEYS];
#pragma unroll
        for (int u = 0; u < KEYS; ++u) {
            const int j = j0 + u * GROUPS;
            const bool in = live && j < end;
            k4[u] = in ? loadf4(kb + size_t(j) * dim) : zero;
            v4[u] = in ? loadf4(vb + size_t(j) * dim) : zero;
        }
        float sc[KEYS];
        float roundMax = m;
#pragma unroll
        for (int u = 0; u < KEYS; ++u) {
            float dot = (q4.x * k4[u].x + q4.y * k4[u].y) + (q4.z * k4[u].z + q4.w * k4[u].w);
#pragma unroll
            for (int o = LPK / 2; o > 0; o >>= 1) dot += __shfl_xor(dot, o, 64);
            sc[u] = j0 + u * GROUPS < end ? dot * p.scale : -INFINITY;
            roundMax = fmaxf(roundMax, sc[u]);
        }
        const float keep = expFast(m - roundMax);                 // m = -inf at the first round: 0 (key j0 itself is below `end`)
        l *= keep;
        acc = acc * keep;
#pragma unroll
        for (int u = 0; u < KEYS; ++u) {
            const float w = expFast(sc[u] - roundMax);
            l += w;
            acc = acc + v4[u] * w;
        }
        m = roundMax;
    }
    // join two running states: (m, l, acc) with the lanes' partners at distance `o`
    auto join = [&](float om, float ol, float4v oacc) {
        const float mm = fmaxf(m, om);
        if (mm == -INFINITY) return;                           // neither side has seen a key
        const float mine = expFast(m - mm), theirs = expFast(om - mm);
        l = l * mine + ol * theirs;
        acc = acc * mine + oacc * theirs;
        m = mm;
    };
#pragma unroll
    for (int o = LPK; o < 64; o <<= 1) {
        const float om = __shfl_xor(m, o, 64), ol = __shfl_xor(l, o, 64);
        float4v oacc;
        oacc.x = __shfl_xor(acc.x, o, 64); oacc.y = __shfl_xor(acc.y, o, 64);
        oacc.z = __shfl_xor(acc.z, o, 64); oacc.w = __shfl_xor(acc.w, o, 64);
        join(om, ol, oacc);
    }
    if (lane < LPK) {
        sAcc[wave][lane] = acc;
        if (lane == 0) { sM[wave] = m; sL[wave] = l; }
    }
    __syncthreads();
    if (t < LPK) {
        m = sM[0]; l = sL[0]; acc = sAcc[0][t];
#pragma unroll
        for (int w = 1; w < 4; ++w) join(sM[w], sL[w], sAcc[w][t]);
        const float inv = l > 0.0f ? 1.0f / l : 0.0f;          // an empty chunk (a cache read by its device-side length) gives zeros
        const float4v o4 = acc * inv;
        const size_t stat = (size_t(b) * p.heads + h) * p.newLen + i;
        const size_t at = size_t(bi) * dim + size_t(h) * hd + d0;
        const bool whole = p.numChunks <= 1;
        float* out = whole ? p.out : p.out + size_t(c) * p.partOutStride;
        if (live) {
            if (out) storef4(out + at, o4);
            if (whole && p.outImg) {
                uint2v packed = {unsigned(toBf16Bits(o4.x)) | unsigned(toBf16Bits(o4.y)) << 16,
                                 unsigned(toBf16Bits(o4.z)) | unsigned(toBf16Bits(o4.w)) << 16};
                *reinterpret_cast<uint2v*>(p.outImg + size_t(bi) * p.imgLd + size_t(h) * hd + d0) = packed;
            }
        }
        if (t == 0) {
            const size_t off = whole ? 0 : size_t(c) * p.partStatStride;
            p.m[off + stat] = m;
            p.l[off + stat] = l;
        }
    }
}

bool vec4Ok(const AttnParams& p, std::initializer_list<const void*> ptrs) {
    if (p.hd % 4 != 0 || p.dim % 4 != 0) return false;
    for (const void* q : ptrs)
        if (q && (reinterpret_cast<uintptr_t>(q) & 15u)) return false;
    return true;
}

// The walk over the cache for at most eight queries per sequence: what it asks of the operands
bool fewQueriesFit(const AttnParams& p, size_t batch, size_t heads, size_t newLen) {
    return newLen <= 8 && batch * heads * newLen <= 65535 && vec4Ok(p, {p.q, p.k, p.v, p.out});
}
// p: the whole problem, outputs included; the keys in numChunks chunks of chunkKeys
int launchFewQueries(const AttnParams& p, size_t batch, size_t heads, size_t newLen, size_t chunkKeys, size_t numChunks, hipStream_t s) {
    const size_t rows = batch * heads * newLen;
    AttnParams c = p;
    c.chunkKeys = int(chunkKeys);
    c.numChunks = int(numChunks);
    const size_t outFloats = batch * newLen * size_t(p.dim), statFloats = batch * heads * newLen;
    Scratch part(numChunks > 1 ? numChunks * (outFloats + 2 * statFloats) * sizeof(float) : 0);
    if (part.status != BF_OK) return part.status;
    if (numChunks > 1) {
        c.partOutStride = outFloats;
        c.partStatStride = statFloats;
        c.out = part.as<float>();
        c.m = c.out + numChunks * outFloats;
        c.l = c.m + numChunks * statFloats;
    }
    const dim3 g{unsigned(numChunks), unsigned(rows), 1u};
    const int lanes = p.hd <= 32 ? 8 : p.hd <= 64 ? 16 : p.hd <= 128 ? 32 : 64;
    switch (lanes) {
        case 8: attnFewQueriesKernel<8><<<g, 256, 0, s>>>(c); break;
        case 16: attnFewQueriesKernel<16><<<g, 256, 0, s>>>(c); break;
        case 32: attnFewQueriesKernel<32><<<g, 256, 0, s>>>(c); break;
        default: attnFewQueriesKernel<64><<<g, 256, 0, s>>>(c); break;
    }
    BF_LAUNCH_CHECK();
    if (numChunks > 1) {
        attnCombineChunksKernel<<<unsigned(rows), 256, 0, s>>>(c.out, c.m, c.l, p.out, p.outImg, p.imgLd, p.m, p.l, int(heads), int(newLen), p.dim, p.hd,
                                                            int(numChunks), outFloats, statFloats);
        BF_LAUNCH_CHECK();
    }
    return BF_OK;
}

// KIND 0 forward, 1 dQ, 2 dK/dV, 3 dK/dV that also stores dS, 4 dQ from stored dS
template <int HDP, int TILE, bool VEC4, bool STORE>
int launchDkv(const AttnParams& p, size_t smem, unsigned grid, hipStream_t s) {
    if (HDP <= 64 && grid > 2u * unsigned(computeUnits()))
        return launchAttn(attnBackwardDkvKernel<HDP, TILE, VEC4, (HDP <= 64 ? 2 : 1), STORE>, smem, grid, p, s);
    return launchAttn(attnBackwardDkvKernel<HDP, TILE, VEC4, 1, STORE>, smem, grid, p, s);
}

// bit 0: the forward kernel's products as six bf16 MFMAs each; bit 1: the dK/dV kernel's; bit 2: those of the dQ kernel
// that reads the stored dS (head dims up to 128 all three); 0 = every product on the fp32 MFMA
thread_local int gAttnRoute = BF_ATTN_ROUTE_SPLIT;   // per host thread: a test naming kernels does not change other threads' calls

template <int KIND, int HDP, int TILE>
int dispatchVec(const AttnParams& p, bool vec4, unsigned grid, hipStream_t s) {
    constexpr size_t operandBytes = size_t(2) * TILE * (HDP + 4) * sizeof(float);   // one operand, double buffered
    if constexpr (KIND == 0 && HDP <= 128) {
        if (gAttnRoute & 1) {
            constexpr size_t splitBytes = size_t(2) * 3 * 32 * (splitKeyPitch(HDP) + splitValuePitch(HDP)) * sizeof(unsigned short);
            return vec4 ? launchAttn(attnForwardPipedKernel<HDP, true>, splitBytes, grid, p, s)
                        : launchAttn(attnForwardPipedKernel<HDP, false>, splitBytes, grid, p, s);
        }
    }
    if constexpr (KIND == 0) {
        return vec4 ? launchAttn(attnForwardKernel<HDP, TILE, true>, 2 * operandBytes, grid, p, s)
                    : launchAttn(attnForwardKernel<HDP, TILE, false>, 2 * operandBytes, grid, p, s);
    } else if constexpr (KIND == 1) {
        return vec4 ? launchAttn(attnBackwardDqKernel<HDP, TILE, true>, 2 * operandBytes, grid, p, s)
                    : launchAttn(attnBackwardDqKernel<HDP, TILE, false>, 2 * operandBytes, grid, p, s);
    } else if constexpr (KIND == 4) {
        if constexpr (HDP <= 128) {
            if (gAttnRoute & BF_ATTN_ROUTE_SPLIT_DQ) {
                constexpr size_t splitBytes = size_t(2) * 3 * 32 * splitValuePitch(HDP) * sizeof(unsigned short) + size_t(4) * kDsPatch * sizeof(float);
                return vec4 ? launchAttn(attnBackwardDqFromDsSplitKernel<HDP, true>, splitBytes, grid, p, s)
                            : launchAttn(attnBackwardDqFromDsSplitKernel<HDP, false>, splitBytes, grid, p, s);
            }
        }
        constexpr size_t need = operandBytes + size_t(4) * kDsPatch * sizeof(float);   // K tiles + a dS patch per wave
        // Three workgroups per CU pay once the grid keeps refilling them; a grid that fits in one round is better spread
        // two per CU, which asking for more LDS than needed (over a third of the CU's 160 KiB) enforces.
        const size_t smem = grid > 3u * unsigned(computeUnits()) ? need : std::max(need, size_t(56) * 1024);
        return vec4 ? launchAttn(attnBackwardDqFromDsKernel<HDP, TILE, true>, smem, grid, p, s)
                    : launchAttn(attnBackwardDqFromDsKernel<HDP, TILE, false>, smem, grid, p, s);
    } else {
        if constexpr (HDP <= 128) {
            if (gAttnRoute & 2) {
                if constexpr (HDP <= 64) {   // Q and dO images in three buffers, statistics likewise
                    constexpr size_t pipedBytes = size_t(6) * 3 * 32 * splitKeyPitch(HDP) * sizeof(unsigned short) + size_t(3) * 64 * sizeof(float);
                    return vec4 ? launchAttn(attnBackwardDkvPipedKernel<HDP, true, KIND == 3>, pipedBytes, grid, p, s)
                                : launchAttn(attnBackwardDkvPipedKernel<HDP, false, KIND == 3>, pipedBytes, grid, p, s);
                } else {
                    constexpr size_t splitBytes = size_t(4) * 3 * 32 * splitKeyPitch(HDP) * sizeof(unsigned short) + size_t(2) * 64 * sizeof(float);
                    return vec4 ? launchAttn(attnBackwardDkvSplitKernel<HDP, true, KIND == 3>, splitBytes, grid, p, s)
                                : launchAttn(attnBackwardDkvSplitKernel<HDP, false, KIND == 3>, splitBytes, grid, p, s);
                }
            }
        }
        constexpr size_t smem = 2 * operandBytes + 4 * TILE * sizeof(float);
        return vec4 ? launchDkv<HDP, TILE, true, KIND == 3>(p, smem, grid, s) : launchDkv<HDP, TILE, false, KIND == 3>(p, smem, grid, s);
    }
}

template <int KIND>
int dispatch(const AttnParams& p, bool vec4, unsigned grid, hipStream_t s) {
    switch (paddedHeadDim(p.hd)) {
        case 32: return dispatchVec<KIND, 32, 64>(p, vec4, grid, s);
        case 64: return dispatchVec<KIND, 64, 64>(p, vec4, grid, s);
        case 128: return dispatchVec<KIND, 128, 32>(p, vec4, grid, s);
        case 192: return dispatchVec<KIND, 192, 32>(p, vec4, grid, s);
        default: return dispatchVec<KIND, 256, 32>(p, vec4, grid, s);
    }
}

// Bytes of the dS hand-over buffer: one 32x32 fp32 sub-block per (query sub-block, key sub-block) of every (batch, head).
size_t dsBytes(size_t batch, size_t heads, size_t newLen, size_t totalLen) {
    return batch * heads * ((newLen + 31) / 32) * ((totalLen + 31) / 32) * 1024 * sizeof(float);
}

// Upper limit of the hand-over buffer that bf_hip_attention_backward may take from the pool; SIZE_MAX = an eighth of
// the device's memory.  Above the limit the backward pass recomputes S and dP in the dQ kernel instead.
thread_local size_t gDsLimit = SIZE_MAX;   // per host thread, as the route

size_t dsLimit() {
    size_t limit = gDsLimit;
    if (limit != SIZE_MAX) return limit;
    return deviceMemoryBytes() / 8;
}

int checkShapes(const char* fn, size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim, size_t oldLen) {
    if (heads == 0 || dim % heads != 0)
        return failInvalid(fn, "numHeads (" + std::to_string(heads) + ") must divide dim (" + std::to_string(dim) + ")");
    size_t hd = dim / heads;
    if (hd > 256)
        return failInvalid(fn, "headDim (" + std::to_string(hd) + ") exceeds the supported limit of the fused kernel (256)");
    if (newLen > 0 && batch > 0 && totalLen == 0) return failInvalid(fn, "totalLen is 0");
    if (batch * heads * ((newLen + 127) / 128 + (totalLen + 127) / 128) >= (size_t(1) << 31) || totalLen + oldLen + newLen >= (size_t(1) << 30) ||
        dim >= (size_t(1) << 24))
        return failInvalid(fn, "shape too large");
    return BF_OK;
}

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" {

static int checkImages(const char* fn, std::initializer_list<const void*> images, size_t imageLd, size_t dim) {
    bool any = false;
    for (const void* img : images) {
        any = any || img != nullptr;
        if (reinterpret_cast<uintptr_t>(img) & 15u) return failInvalid(fn, "bf16 images must be 16-byte aligned");
    }
    if (any && (imageLd < dim || imageLd % 8 != 0 || dim % 8 != 0))
        return failInvalid(fn, "bf16 images need dim and the image row pitch to be multiples of 8, and a pitch of at least dim");
    return BF_OK;
}

int bf_hip_attention_forward_rows(const float* q, const float* k, const float* v, float* out, uint16_t* outImage, size_t imageLd, float* m,
                                  float* l, size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t kvRows, size_t dim, float scale,
                                  size_t oldLen, bf_stream_t stream) {
    int st = checkShapes(__func__, batch, heads, newLen, totalLen, dim, oldLen);
    if (st != BF_OK) return st;
    if (batch == 0 || newLen == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(q && k && v && (out || outImage) && m && l, "NULL pointer");
    if (kvRows < totalLen || kvRows >= (size_t(1) << 31)) return failInvalid(__func__, "kvRows must be at least totalLen");
    st = checkImages(__func__, {outImage}, imageLd, dim);
    if (st != BF_OK) return st;
    AttnParams p{};
    p.outImg = outImage; p.imgLd = imageLd;
    p.q = q; p.k = k; p.v = v; p.out = out; p.m = m; p.l = l;
    p.batch = int(batch); p.heads = int(heads); p.newLen = int(newLen); p.totalLen = int(totalLen);
    p.dim = int(dim); p.hd = int(dim / heads); p.oldLen = int(oldLen); p.scale = scale;
    p.numTiles = int((newLen + 127) / 128);
    p.kvRows = int(kvRows);
    unsigned grid = unsigned(batch * heads * size_t(p.numTiles));
    hipStream_t s = asStream(stream);
    const size_t cus = size_t(computeUnits());
    // At most eight queries per sequence (incremental decoding): the walk over the cache, LPK lanes a key
    if (fewQueriesFit(p, batch, heads, newLen) && (gAttnRoute & BF_ATTN_ROUTE_TILES_ONLY) == 0) {
        const size_t rows = batch * heads * newLen;
        const size_t wanted = std::max<size_t>(1, (4 * cus + rows - 1) / rows);   // about four workgroups per compute unit
        const size_t chunkKeys = std::max<size_t>(128, ((totalLen + wanted - 1) / wanted + 127) / 128 * 128);
        // a chunk starts at or before the first query's own position, so that every query sees a key in every chunk
        const size_t numChunks = std::max<size_t>(1, std::min((totalLen + chunkKeys - 1) / chunkKeys, oldLen / chunkKeys + 1));
        return launchFewQueries(p, batch, heads, newLen, chunkKeys, numChunks, s);
    }
    // Keys in chunks over the workgroups, each chunk with its own statistics, a second kernel putting the chunks together.
    //  * Cached positions (oldLen > 0) and so few (batch, head, tile) triples that half the compute units would idle: one
    //    workgroup per head would walk all the keys alone.  A chunk starts at or before the first query's own position,
    //    so that every query sees a key in every chunk; the last chunk takes everything from the last such start.
    //  * A causal pass from position 0 (a prompt, a small batch) whose heaviest tile, all T key tiles of the last query
    //    tile in a row, is at least two and a half times what a workgroup slot would get if the triangle's work were dealt
    //    evenly: the chunks cut that row; those that lie wholly after a tile's queries are skipped by that tile's
    //    workgroup (chunkIsEmptyFor).  Measured, 12 heads of 64: batch 1 at 1024 / 2048 / 4000 positions (ratios 9.5, 5, 2.6)
    //    66 -> 52, 126 -> 89, 257 -> 226 us; batch 4 at 1024 (2.4) would lose, 74 -> 90 us, and stays whole, like the
    //    GPT-small training pass (1.2) and the headline shape (0.5).
    size_t chunkKeys = 0, numChunks = 1;
    if (oldLen > 0 && size_t(grid) * 2 <= cus && totalLen >= 1024) {
        const size_t wanted = (4 * cus + grid - 1) / grid;   // about four workgroups per compute unit
        chunkKeys = std::max<size_t>(128, ((totalLen + wanted - 1) / wanted + 127) / 128 * 128);
        numChunks = std::min((totalLen + chunkKeys - 1) / chunkKeys, oldLen / chunkKeys + 1);
    } else if (oldLen == 0 && totalLen >= 1024 && newLen == totalLen) {
        const double tiles = double(p.numTiles);
        const double even = std::max(1.0, double(batch * heads) * tiles * (tiles + 1.0) / 2.0 / double(2 * cus));
        if (tiles >= 2.5 * even) {
            const size_t cuts = std::min<size_t>(8, size_t(std::ceil(tiles / even)));
            chunkKeys = std::max<size_t>(128, ((totalLen + cuts - 1) / cuts + 127) / 128 * 128);
            numChunks = (totalLen + chunkKeys - 1) / chunkKeys;
        }
    }
    if (numChunks > 1) {
        const size_t outFloats = batch * newLen * dim, statFloats = batch * heads * newLen;
        Scratch part(numChunks * (outFloats + 2 * statFloats) * sizeof(float));
        if (part.status != BF_OK) return part.status;
        AttnParams c = p;
        c.chunkKeys = int(chunkKeys);
        c.numChunks = int(numChunks);
        c.partOutStride = outFloats;
        c.partStatStride = statFloats;
        c.out = part.as<float>();
        c.m = c.out + numChunks * outFloats;
        c.l = c.m + numChunks * statFloats;
        c.outImg = nullptr;
        st = dispatch<0>(c, vec4Ok(c, {q, k, v, c.out}), grid, s);
        if (st != BF_OK) return st;
        const size_t groups = batch * newLen * heads;
        if (groups >= 2048 && numChunks <= 8) {   // many rows, few chunks: a wavefront per row
            attnCombineRowsKernel<<<unsigned((groups + 3) / 4), 256, 0, s>>>(c.out, c.m, c.l, out, outImage, imageLd, m, l, groups, int(heads), int(newLen),
                                                                          int(dim), p.hd, int(numChunks), outFloats, statFloats);
        } else {
            attnCombineChunksKernel<<<unsigned(groups), 256, 0, s>>>(c.out, c.m, c.l, out, outImage, imageLd, m, l, int(heads), int(newLen), int(dim), p.hd,
                                                                  int(numChunks), outFloats, statFloats);
        }
        BF_LAUNCH_CHECK();
        return BF_OK;
    }
    return dispatch<0>(p, vec4Ok(p, {q, k, v, out}), grid, s);
}

int bf_hip_attention_forward_rows_indirect(const float* q, const float* k, const float* v, float* out, uint16_t* outImage, size_t imageLd,
                                           float* m, float* l, size_t batch, size_t heads, size_t newLen, size_t kvRows, size_t dim, float scale,
                                           const int* oldLen, bf_stream_t stream) {
    int st = checkShapes(__func__, batch, heads, newLen, kvRows, dim, 0);
    if (st != BF_OK) return st;
    if (batch == 0 || newLen == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(q && k && v && (out || outImage) && m && l && oldLen, "NULL pointer");
    BF_REQUIRE(kvRows < (size_t(1) << 31), "kvRows too large");
    st = checkImages(__func__, {outImage}, imageLd, dim);
    if (st != BF_OK) return st;
    AttnParams p{};
    p.outImg = outImage; p.imgLd = imageLd;
    p.q = q; p.k = k; p.v = v; p.out = out; p.m = m; p.l = l;
    p.batch = int(batch); p.heads = int(heads); p.newLen = int(newLen); p.totalLen = int(kvRows);
    p.dim = int(dim); p.hd = int(dim / heads); p.scale = scale;
    p.kvRows = int(kvRows);
    p.oldLenPtr = oldLen;
    if (!fewQueriesFit(p, batch, heads, newLen))
        return failInvalid(__func__, "at most eight queries per sequence, a head dim that is a multiple of 4 and 16-byte aligned operands");
    const size_t rows = batch * heads * newLen, cus = size_t(computeUnits());
    const size_t wanted = std::max<size_t>(1, (4 * cus + rows - 1) / rows);
    const size_t chunkKeys = std::max<size_t>(128, ((kvRows + wanted - 1) / wanted + 127) / 128 * 128);
    return launchFewQueries(p, batch, heads, newLen, chunkKeys, (kvRows + chunkKeys - 1) / chunkKeys, asStream(stream));
}

int bf_hip_attention_forward_img(const float* q, const float* k, const float* v, float* out, uint16_t* outImage, size_t imageLd, float* m,
                                 float* l, size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim, float scale,
                                 size_t oldLen, bf_stream_t stream) {
    return bf_hip_attention_forward_rows(q, k, v, out, outImage, imageLd, m, l, batch, heads, newLen, totalLen, totalLen, dim, scale, oldLen, stream);
}

int bf_hip_attention_forward(const float* q, const float* k, const float* v, float* out, float* m, float* l,
                             size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim, float scale,
                             size_t oldLen, bf_stream_t stream) {
    if (batch != 0 && newLen != 0 && dim != 0) BF_REQUIRE(out != nullptr, "NULL pointer");
    return bf_hip_attention_forward_img(q, k, v, out, nullptr, 0, m, l, batch, heads, newLen, totalLen, dim, scale, oldLen, stream);
}

int bf_hip_attention_dot_o_do(const float* out, const float* dOut, float* D, size_t batch, size_t heads, size_t newLen,
                              size_t dim, bf_stream_t stream) {
    BF_REQUIRE(heads != 0 && dim % heads == 0, "numHeads must divide dim");
    if (batch == 0 || newLen == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(out && dOut && D, "NULL pointer");
    size_t groups = batch * newLen * heads;
    int hd = int(dim / heads);
    bool vec4 = hd % 4 == 0 && dim % 4 == 0 && ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(dOut)) & 15u) == 0;
    unsigned grid = gridFor(groups * 16, 256, 1u << 30);
    if (vec4) attnDotKernel<true><<<grid, 256, 0, asStream(stream)>>>(out, dOut, nullptr, nullptr, D, nullptr, int(batch), int(heads), int(newLen), int(dim), hd);
    else attnDotKernel<false><<<grid, 256, 0, asStream(stream)>>>(out, dOut, nullptr, nullptr, D, nullptr, int(batch), int(heads), int(newLen), int(dim), hd);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

static int fillParams(AttnParams& p, size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim, float scale,
                      size_t oldLen) {
    p.batch = int(batch); p.heads = int(heads); p.newLen = int(newLen); p.totalLen = int(totalLen);
    p.dim = int(dim); p.hd = int(dim / heads); p.oldLen = int(oldLen); p.scale = scale;
    p.nqb = int((newLen + 31) / 32); p.nkb = int((totalLen + 31) / 32);
    return BF_OK;
}

int bf_hip_attention_backward_prepare(const float* out, const float* dOut, const float* m, const float* l, float* lse2,
                                      float* D, size_t batch, size_t heads, size_t newLen, size_t dim,
                                      bf_stream_t stream) {
    BF_REQUIRE(heads != 0 && dim % heads == 0, "numHeads must divide dim");
    if (batch == 0 || newLen == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(out && dOut && m && l && lse2 && D, "NULL pointer");
    const int hd = int(dim / heads);
    const size_t stats = batch * heads * newLen;
    const bool vec4 = hd % 4 == 0 && dim % 4 == 0 && ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(dOut)) & 15u) == 0;
    const unsigned grid = gridFor(stats * 16, 256, 1u << 30);
    hipStream_t s = asStream(stream);
    if (vec4) attnDotKernel<true><<<grid, 256, 0, s>>>(out, dOut, m, l, D, lse2, int(batch), int(heads), int(newLen), int(dim), hd);
    else attnDotKernel<false><<<grid, 256, 0, s>>>(out, dOut, m, l, D, lse2, int(batch), int(heads), int(newLen), int(dim), hd);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

// bf16 images of the gradients (each optional; with an image the fp32 tensor of the same gradient may be NULL)
struct GradImages {
    uint16_t* dQ = nullptr;
    uint16_t* dK = nullptr;
    uint16_t* dV = nullptr;
    size_t ld = 0;
};

// dK, dV from the key-tile owner; dS != NULL also leaves the dS sub-blocks behind for dqFromDs
static int dkvStage(const char* fn, const float* dOut, const float* q, const float* k, const float* v, const float* lse2, const float* D,
                    float* dK, float* dV, float* dS, const GradImages& img, size_t batch, size_t heads, size_t newLen, size_t totalLen,
                    size_t dim, float scale, size_t oldLen, bf_stream_t stream) {
    int st = checkShapes(fn, batch, heads, newLen, totalLen, dim, oldLen);
    if (st != BF_OK) return st;
    if (batch == 0 || dim == 0 || totalLen == 0) return BF_OK;
    if (!(dK || img.dK) || !(dV || img.dV)) return failInvalid(fn, "NULL pointer");
    if (newLen == 0) {   // no query: key/value gradients are zero
        if (img.dK || img.dV) return failInvalid(fn, "bf16 gradient images need at least one query row");
        st = bf_hip_fill_zero(dK, batch * totalLen * dim * sizeof(float), stream);
        if (st != BF_OK) return st;
        return bf_hip_fill_zero(dV, batch * totalLen * dim * sizeof(float), stream);
    }
    if (!(dOut && q && k && v && lse2 && D)) return failInvalid(fn, "NULL pointer");
    if (dS != nullptr && (reinterpret_cast<uintptr_t>(dS) & 15u) != 0) return failInvalid(fn, "dS must be 16-byte aligned");
    AttnParams p{};
    p.q = q; p.k = k; p.v = v; p.dO = dOut; p.dK = dK; p.dV = dV; p.lse2 = lse2; p.dvec = D; p.ds = dS;
    p.dKImg = img.dK; p.dVImg = img.dV; p.imgLd = img.ld;
    fillParams(p, batch, heads, newLen, totalLen, dim, scale, oldLen);
    p.numTiles = int((totalLen + 127) / 128);
    const unsigned grid = unsigned(batch * heads * size_t(p.numTiles));
    return dS ? dispatch<3>(p, vec4Ok(p, {q, k, v, dOut}), grid, asStream(stream)) : dispatch<2>(p, vec4Ok(p, {q, k, v, dOut}), grid, asStream(stream));
}

int bf_hip_attention_backward_dkv(const float* dOut, const float* q, const float* k, const float* v, const float* lse2,
                                  const float* D, float* dK, float* dV, size_t batch, size_t heads, size_t newLen,
                                  size_t totalLen, size_t dim, float scale, size_t oldLen, bf_stream_t stream) {
    if (batch != 0 && dim != 0 && totalLen != 0) BF_REQUIRE(dK && dV, "NULL pointer");
    return dkvStage(__func__, dOut, q, k, v, lse2, D, dK, dV, nullptr, GradImages{}, batch, heads, newLen, totalLen, dim, scale, oldLen, stream);
}

int bf_hip_attention_ds_bytes(size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t* bytes) {
    BF_REQUIRE(bytes != nullptr, "bytes is NULL");
    *bytes = dsBytes(batch, heads, newLen, totalLen);
    return BF_OK;
}

int bf_hip_attention_set_workspace_limit(size_t bytes) {
    gDsLimit = bytes;
    return BF_OK;
}

int bf_hip_attention_backward_dkv_ds(const float* dOut, const float* q, const float* k, const float* v, const float* lse2,
                                     const float* D, float* dK, float* dV, float* dS, size_t batch, size_t heads,
                                     size_t newLen, size_t totalLen, size_t dim, float scale, size_t oldLen,
                                     bf_stream_t stream) {
    if (batch != 0 && dim != 0 && totalLen != 0) BF_REQUIRE(dK && dV && (dS || newLen == 0), "NULL pointer");
    return dkvStage(__func__, dOut, q, k, v, lse2, D, dK, dV, newLen == 0 ? nullptr : dS, GradImages{}, batch, heads, newLen, totalLen, dim,
                    scale, oldLen, stream);
}

static int dqFromDsStage(const char* fn, const float* dS, const float* k, float* dQ, const GradImages& img, size_t batch, size_t heads,
                         size_t newLen, size_t totalLen, size_t dim, float scale, size_t oldLen, bf_stream_t stream);

int bf_hip_attention_backward_dq_from_ds(const float* dS, const float* k, float* dQ, size_t batch, size_t heads, size_t newLen,
                                         size_t totalLen, size_t dim, float scale, size_t oldLen, bf_stream_t stream) {
    if (batch != 0 && dim != 0 && newLen != 0) BF_REQUIRE(dQ != nullptr, "NULL pointer");
    return dqFromDsStage(__func__, dS, k, dQ, GradImages{}, batch, heads, newLen, totalLen, dim, scale, oldLen, stream);
}

static int dqFromDsStage(const char* fn, const float* dS, const float* k, float* dQ, const GradImages& img, size_t batch, size_t heads,
                         size_t newLen, size_t totalLen, size_t dim, float scale, size_t oldLen, bf_stream_t stream) {
    int st = checkShapes(fn, batch, heads, newLen, totalLen, dim, oldLen);
    if (st != BF_OK) return st;
    if (batch == 0 || dim == 0 || newLen == 0) return BF_OK;
    if (!(dS && k && (dQ || img.dQ))) return failInvalid(fn, "NULL pointer");
    if ((reinterpret_cast<uintptr_t>(dS) & 15u) != 0) return failInvalid(fn, "dS must be 16-byte aligned");
    AttnParams p{};
    p.dQImg = img.dQ; p.imgLd = img.ld;
    p.k = k; p.dQ = dQ; p.ds = const_cast<float*>(dS);
    fillParams(p, batch, heads, newLen, totalLen, dim, scale, oldLen);
    p.numTiles = int((newLen + 127) / 128);
    return dispatch<4>(p, vec4Ok(p, {k, dQ}), unsigned(batch * heads * size_t(p.numTiles)), asStream(stream));
}

static int dqStage(const char* fn, const float* dOut, const float* q, const float* k, const float* v, const float* lse2, const float* D,
                   float* dQ, const GradImages& img, size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim, float scale,
                   size_t oldLen, bf_stream_t stream) {
    int st = checkShapes(fn, batch, heads, newLen, totalLen, dim, oldLen);
    if (st != BF_OK) return st;
    if (batch == 0 || dim == 0 || newLen == 0) return BF_OK;
    if (!(dOut && q && k && v && lse2 && D && (dQ || img.dQ))) return failInvalid(fn, "NULL pointer");
    AttnParams p{};
    p.q = q; p.k = k; p.v = v; p.dO = dOut; p.dQ = dQ; p.lse2 = lse2; p.dvec = D;
    p.dQImg = img.dQ; p.imgLd = img.ld;
    fillParams(p, batch, heads, newLen, totalLen, dim, scale, oldLen);
    p.numTiles = int((newLen + 127) / 128);
    return dispatch<1>(p, vec4Ok(p, {q, k, v, dOut, dQ}), unsigned(batch * heads * size_t(p.numTiles)), asStream(stream));
}

int bf_hip_attention_backward_dq(const float* dOut, const float* q, const float* k, const float* v, const float* lse2,
                                 const float* D, float* dQ, size_t batch, size_t heads, size_t newLen, size_t totalLen,
                                 size_t dim, float scale, size_t oldLen, bf_stream_t stream) {
    if (batch != 0 && dim != 0 && newLen != 0) BF_REQUIRE(dQ != nullptr, "NULL pointer");
    return dqStage(__func__, dOut, q, k, v, lse2, D, dQ, GradImages{}, batch, heads, newLen, totalLen, dim, scale, oldLen, stream);
}

int bf_hip_attention_backward_img(const float* dOut, const float* q, const float* k, const float* v, const float* out, const float* m,
                                  const float* l, float* dQ, float* dK, float* dV, uint16_t* dQImage, uint16_t* dKImage,
                                  uint16_t* dVImage, size_t imageLd, size_t batch, size_t heads, size_t newLen, size_t totalLen,
                                  size_t dim, float scale, size_t oldLen, bf_stream_t stream) {
    int st = checkShapes(__func__, batch, heads, newLen, totalLen, dim, oldLen);
    if (st != BF_OK) return st;
    if (batch == 0 || dim == 0) return BF_OK;
    st = checkImages(__func__, {dQImage, dKImage, dVImage}, imageLd, dim);
    if (st != BF_OK) return st;
    const GradImages img{dQImage, dKImage, dVImage, imageLd};
    // workspace: lse2 | D, each [batch, heads, newLen]
    const size_t stats = batch * heads * newLen;
    Scratch work(2 * stats * sizeof(float));
    if (work.status != BF_OK) return work.status;
    float* lse2 = work.as<float>();
    float* dvec = lse2 + stats;
    st = bf_hip_attention_backward_prepare(out, dOut, m, l, lse2, dvec, batch, heads, newLen, dim, stream);
    if (st != BF_OK) return st;
    // With room for the dS hand-over buffer the dK/dV kernel leaves dS behind and dQ is one contraction over it.
    const size_t handOver = dsBytes(batch, heads, newLen, totalLen);
    Scratch ds(newLen > 0 && totalLen > 0 && handOver <= dsLimit() ? handOver : 0);
    if (ds.status != BF_OK) (void)hipGetLastError();   // no room for the buffer after all: recompute instead
    if (ds.status == BF_OK && ds.ptr != nullptr) {
        st = dkvStage(__func__, dOut, q, k, v, lse2, dvec, dK, dV, ds.as<float>(), img, batch, heads, newLen, totalLen, dim, scale, oldLen, stream);
        if (st != BF_OK) return st;
        return dqFromDsStage(__func__, ds.as<float>(), k, dQ, img, batch, heads, newLen, totalLen, dim, scale, oldLen, stream);
    }
    st = dkvStage(__func__, dOut, q, k, v, lse2, dvec, dK, dV, nullptr, img, batch, heads, newLen, totalLen, dim, scale, oldLen, stream);
    if (st != BF_OK) return st;
    return dqStage(__func__, dOut, q, k, v, lse2, dvec, dQ, img, batch, heads, newLen, totalLen, dim, scale, oldLen, stream);
}

int bf_hip_attention_backward(const float* dOut, const float* q, const float* k, const float* v, const float* out,
                              const float* m, const float* l, float* dQ, float* dK, float* dV, size_t batch,
                              size_t heads, size_t newLen, size_t totalLen, size_t dim, float scale, size_t oldLen,
                              bf_stream_t stream) {
    if (batch != 0 && dim != 0) BF_REQUIRE((dQ || newLen == 0) && ((dK && dV) || totalLen == 0), "NULL pointer");
    return bf_hip_attention_backward_img(dOut, q, k, v, out, m, l, dQ, dK, dV, nullptr, nullptr, nullptr, 0, batch, heads, newLen, totalLen, dim,
                                         scale, oldLen, stream);
}

int bf_hip_attention_set_route(int route) {
    BF_REQUIRE(route >= 0 && route <= (BF_ATTN_ROUTE_SPLIT | BF_ATTN_ROUTE_TILES_ONLY), "unknown route");
    bf::gAttnRoute = route;
    return BF_OK;
}

}  // extern "C"
