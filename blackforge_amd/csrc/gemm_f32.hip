// fp32 GEMM on the fp32 MFMA pipe (v_mfma_f32_32x32x2_f32): C[M,N] = op(A) * op(B), any shape.
//
// Serves the fp32 `matmul`, `matmulTransposeB` and their backward passes.  A workgroup of four
// wavefronts owns a BM x BN tile of C; A and B tiles are staged through LDS in k-major order
// (As[k][m], Bs[k][n]) so that both MFMA operands are read with unit-stride, bank-conflict-free
// ds_read_b32, whatever the transposition of the global operands; the transposition is absorbed by
// the global->LDS copy, which always walks global memory along its contiguous dimension.
//
// MFMA operand layout used throughout (wave64, 32x32x2 fp32):
//   A: lane l holds A[i = l % 32][k = l / 32]        B: lane l holds B[k = l / 32][j = l % 32]
//   D: lane l, register r holds D[i = 8*(r/4) + 4*(l/32) + r%4][j = l % 32]
#include "common.hpp"

#include <algorithm>
#include <cstdint>

namespace bf {
namespace {

constexpr int BK = 32;

// One thread's share of a [BK x BT] operand tile: element e = tid + 256*i of the tile, walked so that consecutive
// threads read consecutive global addresses (along k when the tile dimension t is a row of X, along t otherwise).
template <int BT, int BKT = BK>
struct TileRegs {
    static constexpr int kPer = BKT * BT / 256;
    float v[kPer];
};

// Issues the global loads of the tile of op(X) at (k0, t0) into registers, zero outside the matrix or the K slice.
// op(X)[k][t] = X[t*ld + k] when t is the row of X (T_IS_ROW), or X[k*ld + t] when t is its column.
template <int BT, bool T_IS_ROW, int BKT = BK>
__device__ __forceinline__ void fetchTile(TileRegs<BT, BKT>& regs, const float* __restrict__ X, size_t ld, size_t tExtent,
                                          size_t kEnd, size_t t0, size_t k0, int tid) {
#pragma unroll
    for (int i = 0; i < TileRegs<BT, BKT>::kPer; ++i) {
        const int e = tid + 256 * i;
        int k, t;
        if constexpr (T_IS_ROW) { k = e % BKT; t = e / BKT; }
        else { t = e % BT; k = e / BT; }
        const size_t gt = t0 + t, gk = k0 + k;
        regs.v[i] = (gt < tExtent && gk < kEnd) ? (T_IS_ROW ? X[gt * ld + gk] : X[gk * ld + gt]) : 0.0f;
    }
}
template <int BT, bool T_IS_ROW, int BKT = BK, int PAD = 4>
__device__ __forceinline__ void commitTile(float (*lds)[BT + PAD], const TileRegs<BT, BKT>& regs, int tid) {
#pragma unroll
    for (int i = 0; i < TileRegs<BT, BKT>::kPer; ++i) {
        const int e = tid + 256 * i;
        int k, t;
        if constexpr (T_IS_ROW) { k = e % BKT; t = e / BKT; }
        else { t = e % BT; k = e / BT; }
        lds[k][t] = regs.v[i];
    }
}

// What the store adds to a finished product: an optional bias row, then an optional residual matrix (which may be the
// output itself: each element is read and written by one thread), in the order the separate add kernels use.
__device__ __forceinline__ float withAdds(float v, const float* __restrict__ bias, const float* residual, size_t index, size_t col) {
    if (bias) v += bias[col];
    if (residual) v += residual[index];
    return v;
}

template <int BM, int BN>
struct GemmTile {
    static constexpr int kPad = 4;
    float as[BK][BM + kPad];
    float bs[BK][BN + kPad];
};

// TRANS_A: A stored [K,M] (op(A)[m][k] = A[k*M + m]); otherwise A stored [M,K].
// TRANS_B: B stored [N,K] (op(B)[k][n] = B[n*K + k]); otherwise B stored [K,N].
// blockIdx.z selects a slice [z*kPerSlice, (z+1)*kPerSlice) of the contraction; slice z writes its partial product
// to C + z*sliceStride.  The global loads of the next K step are in flight (in registers) while the current one is
// multiplied out of LDS.
template <int BM, int BN, bool TRANS_A, bool TRANS_B>
__global__ void __launch_bounds__(256) gemmF32Kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                      float* C, size_t M, size_t N, size_t K, size_t kPerSlice,
                                                      size_t sliceStride, const float* __restrict__ bias, const float* residual) {
    constexpr int WM = BM / 2, WN = BN / 2;      // 2 x 2 wavefronts
    constexpr int TM = WM / 32, TN = WN / 32;    // 32x32 MFMA tiles per wavefront
    __shared__ GemmTile<BM, BN> tile;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const size_t m0 = size_t(blockIdx.y) * BM, n0 = size_t(blockIdx.x) * BN;
    const int li = lane & 31, lk = lane >> 5;
    const size_t kBegin = size_t(blockIdx.z) * kPerSlice, kEnd = kBegin + kPerSlice < K ? kBegin + kPerSlice : K;
    C += size_t(blockIdx.z) * sliceStride;

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    TileRegs<BM> aNext;
    TileRegs<BN> bNext;
    auto fetch = [&](size_t k0) {
        // A tile: tile dimension m.  A stored [M,K] -> m is the row (contiguous along k).
        if constexpr (TRANS_A) fetchTile<BM, false>(aNext, A, M, M, kEnd, m0, k0, tid);
        else fetchTile<BM, true>(aNext, A, K, M, kEnd, m0, k0, tid);
        // B tile: tile dimension n.  B stored [K,N] -> n is the column (contiguous along n).
        if constexpr (TRANS_B) fetchTile<BN, true>(bNext, B, K, N, kEnd, n0, k0, tid);
        else fetchTile<BN, false>(bNext, B, N, N, kEnd, n0, k0, tid);
    };
    if (kBegin < kEnd) fetch(kBegin);
    for (size_t k0 = kBegin; k0 < kEnd; k0 += BK) {
        commitTile<BM, !TRANS_A>(tile.as, aNext, tid);
        commitTile<BN, TRANS_B>(tile.bs, bNext, tid);
        __syncthreads();
        if (k0 + BK < kEnd) fetch(k0 + BK);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = tile.as[kk + lk][wm0 + i * 32 + li];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = tile.bs[kk + lk][wn0 + j * 32 + li];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            size_t col = n0 + wn0 + j * 32 + li;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                size_t row = m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * lk + (r % 4);
                if (row < M && col < N) C[row * N + col] = withAdds(acc[i][j][r], bias, residual, row * N + col, col);
            }
        }
}

// Small products (a model a few hundred wide: every product of it is a handful of 64 x 64 tiles whose four K steps
// each wait a full round trip to memory): 32 x 32 tiles, four wavefronts with a 16 x 16 share each on the
// 16x16x4 fp32 MFMA, and K steps of 128, so that a contraction up to 128 long is ONE round of loads and one barrier
// and a workgroup's MFMA chain is 32 instructions long.  Two accumulators alternate so that consecutive MFMAs do not
// depend on each other; they are added at the end (a fixed order: results are reproducible).
//   A: lane l holds A[i = l % 16][k = l / 16]   B: lane l holds B[k = l / 16][j = l % 16]
//   D: lane l, register r holds D[i = 4*(l/16) + r][j = l % 16]
// An operand tile lies in LDS the way it lies in memory, so that the copy writes consecutive words: [t][k] with rows of
// 132 floats when k is the contiguous dimension (the 16 rows x 4 k a wavefront reads cover all 64 banks), [k][t] with
// rows of 48 floats otherwise (4 k rows x 16 t: likewise).
constexpr int SBK = 128, SBT = 32;
constexpr int SROW_K = SBK + 4, SROW_T = SBT + 16;
constexpr int SWORDS = SBK * SROW_T > SBT * SROW_K ? SBK * SROW_T : SBT * SROW_K;

// VEC = 4: every access is 16 bytes (the contiguous extent and the row pitch are multiples of 4 and the base is 16-byte
// aligned; a group of four is then wholly inside or wholly outside the matrix); VEC = 1 takes any shape.
template <bool K_CONTIG, int VEC>
struct SmallOperand {
    static constexpr int kPer = SBK * SBT / 256 / VEC;
    static constexpr int kGroupsK = SBK / VEC, kGroupsT = SBT / VEC;
    float v[kPer * VEC];
    // X[t*ld + k] when k is contiguous, X[k*ld + t] otherwise; zero outside the matrix or the K slice
    __device__ __forceinline__ void fetch(const float* __restrict__ X, size_t ld, size_t tExtent, size_t kEnd, size_t t0, size_t k0, int tid) {
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int e = tid + 256 * i;
            const int k = K_CONTIG ? (e % kGroupsK) * VEC : e / kGroupsT, t = K_CONTIG ? e / kGroupsK : (e % kGroupsT) * VEC;
            const size_t gt = t0 + t, gk = k0 + k;
            const bool inside = gt < tExtent && gk < kEnd;
            const float* src = K_CONTIG ? X + gt * ld + gk : X + gk * ld + gt;
            if constexpr (VEC == 4) {
                const float4v q = inside ? loadf4(src) : float4v{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int j = 0; j < 4; ++j) v[4 * i + j] = q[j];
            } else {
                v[i] = inside ? *src : 0.0f;
            }
        }
    }
    __device__ __forceinline__ void commit(float* lds, int tid) const {
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int e = tid + 256 * i;
            float* dst = K_CONTIG ? lds + (e / kGroupsK) * SROW_K + (e % kGroupsK) * VEC : lds + (e / kGroupsT) * SROW_T + (e % kGroupsT) * VEC;
            if constexpr (VEC == 4) storef4(dst, float4v{v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]});
            else *dst = v[i];
        }
    }
    // element (t, k) of the tile
    static __device__ __forceinline__ float at(const float* lds, int t, int k) {
        return K_CONTIG ? lds[t * SROW_K + k] : lds[k * SROW_T + t];
    }
};

// DEPTH register stages hold the K steps that follow the one being multiplied: a contraction of up to DEPTH steps has
// all its loads in flight at once (a 512-token weight gradient waits for memory once, not four times).
template <bool TRANS_A, bool TRANS_B, int VEC, int DEPTH>
__global__ void __launch_bounds__(256) gemmF32SmallKernel(const float* __restrict__ A, const float* __restrict__ B,
                                                           float* C, size_t M, size_t N, size_t K, size_t kPerSlice,
                                                           size_t sliceStride, const float* __restrict__ bias, const float* residual) {
    __shared__ __attribute__((aligned(16))) float as[SWORDS];
    __shared__ __attribute__((aligned(16))) float bs[SWORDS];
    using OpA = SmallOperand<!TRANS_A, VEC>;   // A stored [M,K]: k contiguous
    using OpB = SmallOperand<TRANS_B, VEC>;    // B stored [N,K]: k contiguous
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave >> 1) * 16, wn0 = (wave & 1) * 16;
    const size_t m0 = size_t(blockIdx.y) * SBT, n0 = size_t(blockIdx.x) * SBT;
    const int li = lane & 15, lk = lane >> 4;
    const size_t kBegin = size_t(blockIdx.z) * kPerSlice, kEnd = kBegin + kPerSlice < K ? kBegin + kPerSlice : K;
    C += size_t(blockIdx.z) * sliceStride;
    float4v acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
    OpA aStage[DEPTH];
    OpB bStage[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
        if (kBegin + size_t(d) * SBK < kEnd) {
            aStage[d].fetch(A, TRANS_A ? M : K, M, kEnd, m0, kBegin + size_t(d) * SBK, tid);
            bStage[d].fetch(B, TRANS_B ? K : N, N, kEnd, n0, kBegin + size_t(d) * SBK, tid);
        }
    for (size_t base = kBegin; base < kEnd; base += size_t(DEPTH) * SBK) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const size_t k0 = base + size_t(d) * SBK;
            if (k0 >= kEnd) break;
            aStage[d].commit(as, tid);
            bStage[d].commit(bs, tid);
            __syncthreads();
            if (k0 + size_t(DEPTH) * SBK < kEnd) {
                aStage[d].fetch(A, TRANS_A ? M : K, M, kEnd, m0, k0 + size_t(DEPTH) * SBK, tid);
                bStage[d].fetch(B, TRANS_B ? K : N, N, kEnd, n0, k0 + size_t(DEPTH) * SBK, tid);
            }
#pragma unroll
            for (int kk = 0; kk < SBK; kk += 8) {
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(OpA::at(as, wm0 + li, kk + lk), OpB::at(bs, wn0 + li, kk + lk), acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(OpA::at(as, wm0 + li, kk + 4 + lk), OpB::at(bs, wn0 + li, kk + 4 + lk), acc1, 0, 0, 0);
            }
            __syncthreads();
        }
    }
    const size_t col = n0 + wn0 + li;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const size_t row = m0 + wm0 + 4 * lk + r;
        if (row < M && col < N) C[row * N + col] = withAdds(acc0[r] + acc1[r], bias, residual, row * N + col, col);
    }
}

template <int VEC, int DEPTH>
int launchSmallGemmAs(int transA, int transB, const float* A, const float* B, float* C, size_t M, size_t N, size_t K, size_t slices,
                      size_t kPerSlice, size_t sliceStride, const float* bias, const float* residual, hipStream_t s) {
    dim3 grid(unsigned((N + SBT - 1) / SBT), unsigned((M + SBT - 1) / SBT), unsigned(slices));
    if (!transA && !transB) gemmF32SmallKernel<false, false, VEC, DEPTH><<<grid, 256, 0, s>>>(A, B, C, M, N, K, kPerSlice, sliceStride, bias, residual);
    else if (!transA && transB) gemmF32SmallKernel<false, true, VEC, DEPTH><<<grid, 256, 0, s>>>(A, B, C, M, N, K, kPerSlice, sliceStride, bias, residual);
    else if (transA && !transB) gemmF32SmallKernel<true, false, VEC, DEPTH><<<grid, 256, 0, s>>>(A, B, C, M, N, K, kPerSlice, sliceStride, bias, residual);
    else gemmF32SmallKernel<true, true, VEC, DEPTH><<<grid, 256, 0, s>>>(A, B, C, M, N, K, kPerSlice, sliceStride, bias, residual);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int launchSmallGemm(int transA, int transB, const float* A, const float* B, float* C, size_t M, size_t N, size_t K, size_t slices,
                    size_t kPerSlice, size_t sliceStride, const float* bias, const float* residual, hipStream_t s) {
    // 16-byte accesses need the contiguous extent of either operand (K, or M / N for an operand stored with K as its rows)
    // to be a multiple of 4 and 16-byte aligned bases
    auto aligned16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    const bool vec = aligned16(A) && aligned16(B) && (transA ? M : K) % 4 == 0 && (transB ? K : N) % 4 == 0;
    if (vec) return launchSmallGemmAs<4, 4>(transA, transB, A, B, C, M, N, K, slices, kPerSlice, sliceStride, bias, residual, s);
    return launchSmallGemmAs<1, 1>(transA, transB, A, B, C, M, N, K, slices, kPerSlice, sliceStride, bias, residual, s);
}

// Several independent small products in ONE launch (blockIdx.z selects the product): the two gradient products of a
// projection, or the Q, K and V projections of one input.  A small model's step is a chain of launches of a few
// microseconds each, most of that the launch and one round trip to memory; products that do not depend on each other
// share both.  The orientation of the operands is a run-time property of each product here.
constexpr int kMaxGroup = 8;
struct GroupProblem {
    const float* A;
    const float* B;
    float* C;
    const float* bias;
    const float* residual;
    unsigned M, N, K;
    int transA, transB;
};
struct GroupArgs {
    GroupProblem p[kMaxGroup];
};

template <int VEC>
struct SmallOperandRt {
    float v[SBK * SBT / 256];
    __device__ __forceinline__ void fetch(bool kContig, const float* __restrict__ X, size_t ld, size_t tExtent, size_t kEnd, size_t t0, size_t k0,
                                          int tid) {
        if (kContig) reinterpret_cast<SmallOperand<true, VEC>*>(this)->fetch(X, ld, tExtent, kEnd, t0, k0, tid);
        else reinterpret_cast<SmallOperand<false, VEC>*>(this)->fetch(X, ld, tExtent, kEnd, t0, k0, tid);
    }
    __device__ __forceinline__ void commit(bool kContig, float* lds, int tid) const {
        if (kContig) reinterpret_cast<const SmallOperand<true, VEC>*>(this)->commit(lds, tid);
        else reinterpret_cast<const SmallOperand<false, VEC>*>(this)->commit(lds, tid);
    }
};

template <int VEC, int DEPTH>
__global__ void __launch_bounds__(256) gemmF32SmallGroupKernel(GroupArgs args) {
    __shared__ __attribute__((aligned(16))) float as[SWORDS];
    __shared__ __attribute__((aligned(16))) float bs[SWORDS];
    const GroupProblem& g = args.p[blockIdx.z];
    const size_t M = g.M, N = g.N, kEnd = g.K;
    const size_t m0 = size_t(blockIdx.y) * SBT, n0 = size_t(blockIdx.x) * SBT;
    if (m0 >= M || n0 >= N) return;   // the grid covers the largest product of the group
    const bool aContig = !g.transA, bContig = g.transB != 0;
    const float* A = g.A;
    const float* B = g.B;
    const size_t lda = g.transA ? M : kEnd, ldb = g.transB ? kEnd : N;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave >> 1) * 16, wn0 = (wave & 1) * 16;
    const int li = lane & 15, lk = lane >> 4;
    // where a lane finds element (t, k) of either tile: base + k * stride
    const int aBase = aContig ? (wm0 + li) * SROW_K : wm0 + li, aStep = aContig ? 1 : SROW_T;
    const int bBase = bContig ? (wn0 + li) * SROW_K : wn0 + li, bStep = bContig ? 1 : SROW_T;
    float4v acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
    SmallOperandRt<VEC> aStage[DEPTH], bStage[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
        if (size_t(d) * SBK < kEnd) {
            aStage[d].fetch(aContig, A, lda, M, kEnd, m0, size_t(d) * SBK, tid);
            bStage[d].fetch(bContig, B, ldb, N, kEnd, n0, size_t(d) * SBK, tid);
        }
    for (size_t base = 0; base < kEnd; base += size_t(DEPTH) * SBK) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const size_t k0 = base + size_t(d) * SBK;
            if (k0 >= kEnd) break;
            aStage[d].commit(aContig, as, tid);
            bStage[d].commit(bContig, bs, tid);
            __syncthreads();
            if (k0 + size_t(DEPTH) * SBK < kEnd) {
                aStage[d].fetch(aContig, A, lda, M, kEnd, m0, k0 + size_t(DEPTH) * SBK, tid);
                bStage[d].fetch(bContig, B, ldb, N, kEnd, n0, k0 + size_t(DEPTH) * SBK, tid);
            }
#pragma unroll
            for (int kk = 0; kk < SBK; kk += 8) {
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(as[aBase + (kk + lk) * aStep], bs[bBase + (kk + lk) * bStep], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(as[aBase + (kk + 4 + lk) * aStep], bs[bBase + (kk + 4 + lk) * bStep], acc1, 0, 0, 0);
            }
            __syncthreads();
        }
    }
    const size_t col = n0 + wn0 + li;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const size_t row = m0 + wm0 + 4 * lk + r;
        if (row < M && col < N) g.C[row * N + col] = withAdds(acc0[r] + acc1[r], g.bias, g.residual, row * N + col, col);
    }
}

// C[i] = sum over slices of partial[s*stride + i], slices added in index order (deterministic).
__global__ void __launch_bounds__(kBlock) sliceSumKernel(const float* __restrict__ partial, float* C, size_t count,
                                                         size_t stride, int slices, size_t N, const float* __restrict__ bias,
                                                         const float* residual) {
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float sum = partial[i];
    for (int s0 = 1; s0 < slices; s0 += 8) {   // eight loads in flight, added in index order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = s0 + u < slices ? partial[size_t(s0 + u) * stride + i] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (s0 + u < slices) sum += v[u];
    }
    C[i] = withAdds(sum, bias, residual, i, i % N);
}

// up to three products of one shape in one launch of the few-row kernel, and of the kernel that sums their K slices
struct FewRowsProducts {
    const float* A[3];
    const float* B[3];
    float* out[3];          // with K slices: the product's first slice in the scratch buffer
    const float* bias[3];
    const float* residual[3];
    // one or two rows only: A[] is ignored and the rows are those of rmsnorm(normInput) ([M, K], dense), normalised while
    // the kernel stages its slice of them (a decoding step's projections and feed-forward block)
    const float* normInput;
    int act;                // BF_ACT_* applied after the adds, or -1
    // products 1 and 2 are stored *rowShift rows further down, as long as the row stays below rowLimit (a decoding step's
    // new keys and values, placed at the cache's device-side length)
    const int* rowShift;
    int rowLimit;
};
__device__ __forceinline__ float actOrNot(int act, float v) {
    return act < 0 ? v : act == BF_ACT_SILU ? siluF(v) : act == BF_ACT_GELU ? geluF(v) : reluF(v);
}
// sliceSumKernel for product blockIdx.y: partial sums at partial[y], `slices` of them `stride` floats apart, to C[y]
__global__ void __launch_bounds__(kBlock) sliceSumProductsKernel(FewRowsProducts g, float* const C0, float* const C1, float* const C2, size_t count,
                                                                 size_t stride, int slices, size_t N) {
    const int which = blockIdx.y;
    const float* partial = which == 0 ? g.out[0] : which == 1 ? g.out[1] : g.out[2];
    float* C = which == 0 ? C0 : which == 1 ? C1 : C2;
    const float* bias = which == 0 ? g.bias[0] : which == 1 ? g.bias[1] : g.bias[2];
    const float* residual = which == 0 ? g.residual[0] : which == 1 ? g.residual[1] : g.residual[2];
    const size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= count) return;
    float sum = partial[i];
    for (int s0 = 1; s0 < slices; s0 += 8) {   // eight loads in flight, added in index order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = s0 + u < slices ? partial[size_t(s0 + u) * stride + i] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (s0 + u < slices) sum += v[u];
    }
    const float value = actOrNot(g.act, withAdds(sum, bias, residual, i, i % N));
    if (g.rowShift != nullptr && which >= 1) {
        const size_t row = i / N + size_t(*g.rowShift);
        if (row < size_t(g.rowLimit)) C[row * N + i % N] = value;
    } else {
        C[i] = value;
    }
}

// Products of at most eight rows, C[M, N] = A[M, K] B[K, N] (a step of incremental decoding: one new token per sequence),
// as a walk over B: a lane owns VEC adjacent columns, the WAVES wavefronts of a workgroup take every WAVES-th row of the
// workgroup's K slice, eight rows loaded before any is used, and multiply them with the slice's elements of A, which the
// workgroup holds in LDS (read as broadcasts).  The wavefronts' sums are added in order through LDS; with several K
// slices (blockIdx.y) a slice writes its sums `sliceStride` floats after the slice before it and sliceSumKernel adds them,
// with one slice the adds of the epilogue are made here.  VEC 4: N a multiple of 4 and B 16-byte aligned.
template <int MR, int VEC, int WAVES>
__global__ void __launch_bounds__(64 * WAVES) gemmF32FewRowsKernel(FewRowsProducts g, int M, int N, int K, int kPer, size_t sliceStride) {
    // blockIdx.z: which of up to three products of one shape (the Q, K and V projections of a decoding step)
    const int which = blockIdx.z;
    const float* __restrict__ A = which == 0 ? g.A[0] : which == 1 ? g.A[1] : g.A[2];
    const float* __restrict__ B = which == 0 ? g.B[0] : which == 1 ? g.B[1] : g.B[2];
    float* out = which == 0 ? g.out[0] : which == 1 ? g.out[1] : g.out[2];
    const float* __restrict__ bias = which == 0 ? g.bias[0] : which == 1 ? g.bias[1] : g.bias[2];
    const float* residual = which == 0 ? g.residual[0] : which == 1 ? g.residual[1] : g.residual[2];   // may be `out`
    extern __shared__ float fewRowsLds[];
    constexpr int U = 8, WIDTH = 64 * VEC;
    float* aRows = fewRowsLds;                      // [MR][kPer]
    float* sums = fewRowsLds + MR * kPer;           // [WAVES][MR][WIDTH]
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int col = (int(blockIdx.x) * 64 + lane) * VEC;
    const int kBeg = int(blockIdx.y) * kPer, kEnd = min(K, kBeg + kPer), kLen = kEnd - kBeg;
    float b[U][VEC];
    auto loadRows = [&](int k0) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = k0 + WAVES * u;
            const bool in = k < kEnd && col < N;
            if constexpr (VEC == 4) {
                const float4v v = in ? __builtin_nontemporal_load(reinterpret_cast<const float4v*>(B + size_t(k) * N + col)) : float4v{0.0f, 0.0f, 0.0f, 0.0f};
                b[u][0] = v.x; b[u][1] = v.y; b[u][2] = v.z; b[u][3] = v.w;
            } else {
                b[u][0] = in ? __builtin_nontemporal_load(B + size_t(k) * N + col) : 0.0f;
            }
        }
    };
    int k0 = kBeg + wave;
    loadRows(k0);                                   // in flight while A is staged
    if (g.normInput == nullptr) {
        for (int i = t; i < M * kLen; i += 64 * WAVES) {
            const int r = i / kLen, k = i - r * kLen;
            aRows[r * kPer + k] = A[size_t(r) * K + kBeg + k];
        }
    } else {
        // x / sqrt(mean(x^2) + eps), sum of squares in double, division in float (the row kernel's arithmetic, ops.cpp:264-275);
        // every workgroup sums whole rows for itself and stages its K slice of them
        __shared__ double squares[WAVES][MR];
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            double ss = 0.0;
            if (r < M)
                for (int k = t; k < K; k += 64 * WAVES) {
                    const double v = double(g.normInput[size_t(r) * K + k]);
                    ss += v * v;
                }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
            if (lane == 0) squares[wave][r] = ss;
        }
        __syncthreads();
        for (int i = t; i < M * kLen; i += 64 * WAVES) {
            const int r = i / kLen, k = i - r * kLen;
            double ss = 0.0;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) ss += squares[w][r];
            const float rms = float(sqrt(ss / double(K) + double(kRmsNormEps)));
            aRows[r * kPer + k] = g.normInput[size_t(r) * K + kBeg + k] / rms;
        }
    }
    __syncthreads();
    float acc[MR][VEC];
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[r][v] = 0.0f;
    while (k0 < kEnd) {                             // the same for every lane of a wavefront
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = k0 + WAVES * u;
            if (k < kEnd) {
#pragma unroll
                for (int r = 0; r < MR; ++r) {
                    if (r < M) {
                        const float a = aRows[r * kPer + (k - kBeg)];
#pragma unroll
                        for (int v = 0; v < VEC; ++v) acc[r][v] = fmaf(a, b[u][v], acc[r][v]);
                    }
                }
            }
        }
        k0 += WAVES * U;
        if (k0 < kEnd) loadRows(k0);
    }
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
        for (int v = 0; v < VEC; ++v) sums[((wave * MR + r) * 64 + lane) * VEC + v] = acc[r][v];
    __syncthreads();
    float* dst = out + size_t(blockIdx.y) * sliceStride;
    for (int i = t; i < M * WIDTH; i += 64 * WAVES) {
        const int r = i / WIDTH, c = i - r * WIDTH, column = int(blockIdx.x) * WIDTH + c;
        if (column < N) {
            float total = sums[r * WIDTH + c];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) total += sums[(w * MR + r) * WIDTH + c];
            const size_t at = size_t(r) * N + column;
            if (gridDim.y > 1) {
                dst[at] = total;
            } else {
                const float value = actOrNot(g.act, withAdds(total, bias, residual, at, size_t(column)));
                size_t row = size_t(r);
                if (g.rowShift != nullptr && which >= 1) row += size_t(*g.rowShift);
                if (g.rowShift == nullptr || which == 0 || row < size_t(g.rowLimit)) dst[row * N + column] = value;
            }
        }
    }
}
// `products` (1 to 3) of one shape: p.out = where each product goes, p.bias / p.residual its adds
template <int MR>
int launchFewRowsF32(const FewRowsProducts& p, size_t products, size_t M, size_t N, size_t K, hipStream_t s, bool* served) {
    *served = false;
    constexpr int WAVES = MR <= 4 ? 8 : 4;          // WAVES * MR * 256 sums in LDS
    bool vec = N % 4 == 0;
    for (size_t i = 0; i < products; ++i) vec = vec && (reinterpret_cast<uintptr_t>(p.B[i]) & 15u) == 0;
    const size_t width = vec ? 256 : 64, colBlocks = (N + width - 1) / width;
    // K slices of at least one round of loads per wavefront (8 * WAVES rows), at most 32 of them, about two workgroups
    // per compute unit and product (the same cut whatever the number of products, so that a product's bits do not depend on
    // what it is launched with); the slices are summed by a second kernel
    const size_t cus = size_t(computeUnits()), round = size_t(8) * WAVES;
    size_t slices = std::max<size_t>(1, std::min<size_t>(std::min<size_t>((K + round - 1) / round, 32), 2 * cus / colBlocks));
    size_t kPer = ((K + slices - 1) / slices + 3) / 4 * 4;
    slices = (K + kPer - 1) / kPer;
    const size_t smem = (size_t(MR) * kPer + size_t(WAVES) * MR * width) * sizeof(float);
    if (smem > 96 * 1024) return BF_OK;             // rows of A too long for the LDS: the tile kernels serve
    const size_t count = M * N;
    Scratch partial(slices > 1 ? products * slices * count * sizeof(float) : 0);
    if (partial.status != BF_OK) return partial.status;
    FewRowsProducts g = p;
    if (slices > 1)
        for (size_t i = 0; i < products; ++i) {
            g.out[i] = partial.as<float>() + i * slices * count;
            g.bias[i] = g.residual[i] = nullptr;    // added when the slices are summed
        }
    const dim3 grid{unsigned(colBlocks), unsigned(slices), unsigned(products)};
    int st;
    if (vec) {
        auto kernel = gemmF32FewRowsKernel<MR, 4, WAVES>;
        st = allowDynamicSharedMemory(reinterpret_cast<const void*>(kernel), smem);
        if (st != BF_OK) return st;
        kernel<<<grid, 64 * WAVES, smem, s>>>(g, int(M), int(N), int(K), int(kPer), count);
    } else {
        auto kernel = gemmF32FewRowsKernel<MR, 1, WAVES>;
        st = allowDynamicSharedMemory(reinterpret_cast<const void*>(kernel), smem);
        if (st != BF_OK) return st;
        kernel<<<grid, 64 * WAVES, smem, s>>>(g, int(M), int(N), int(K), int(kPer), count);
    }
    BF_LAUNCH_CHECK();
    if (slices > 1) {
        FewRowsProducts sums = g;                   // out[i]: the partial sums; bias, residual and activation from the caller
        for (size_t i = 0; i < products; ++i) { sums.bias[i] = p.bias[i]; sums.residual[i] = p.residual[i]; }
        const dim3 sumGrid{unsigned((count + kBlock - 1) / kBlock), unsigned(products), 1u};
        sliceSumProductsKernel<<<sumGrid, kBlock, 0, s>>>(sums, p.out[0], p.out[1], p.out[2], count, count, int(slices), N);
        BF_LAUNCH_CHECK();
    }
    *served = true;
    return BF_OK;
}
inline int launchFewRowsF32Any(const FewRowsProducts& p, size_t products, size_t M, size_t N, size_t K, hipStream_t s, bool* served) {
    return M == 1 ? launchFewRowsF32<1>(p, products, M, N, K, s, served) : M == 2 ? launchFewRowsF32<2>(p, products, M, N, K, s, served)
         : M <= 4 ? launchFewRowsF32<4>(p, products, M, N, K, s, served) : launchFewRowsF32<8>(p, products, M, N, K, s, served);
}

template <int BM, int BN>
int launchGemm(int transA, int transB, const float* A, const float* B, float* C, size_t M, size_t N, size_t K, size_t slices,
               size_t kPerSlice, size_t sliceStride, const float* bias, const float* residual, hipStream_t s) {
    dim3 grid(unsigned((N + BN - 1) / BN), unsigned((M + BM - 1) / BM), unsigned(slices));
    if (!transA && !transB) gemmF32Kernel<BM, BN, false, false><<<grid, 256, 0, s>>>(A, B, C, M, N, K, kPerSlice, sliceStride, bias, residual);
    else if (!transA && transB) gemmF32Kernel<BM, BN, false, true><<<grid, 256, 0, s>>>(A, B, C, M, N, K, kPerSlice, sliceStride, bias, residual);
    else if (transA && !transB) gemmF32Kernel<BM, BN, true, false><<<grid, 256, 0, s>>>(A, B, C, M, N, K, kPerSlice, sliceStride, bias, residual);
    else gemmF32Kernel<BM, BN, true, true><<<grid, 256, 0, s>>>(A, B, C, M, N, K, kPerSlice, sliceStride, bias, residual);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

}  // namespace
}  // namespace bf

using namespace bf;

namespace bf {
namespace {
// C = op(A) op(B) (+ bias per column) (+ residual); with K slices the adds move to the kernel that sums the slices.
int gemmF32(int transA, int transB, const float* A, const float* B, float* C, size_t M, size_t N, size_t K, const float* bias,
            const float* residual, bf_stream_t stream) {
    if (M == 0 || N == 0) return BF_OK;
    BF_REQUIRE(C != nullptr, "NULL output");
    if (K == 0) {
        BF_REQUIRE(!bias && !residual, "an empty contraction with a bias or residual is not supported");
        return bf_hip_fill_zero(C, M * N * sizeof(float), stream);
    }
    BF_REQUIRE(A && B, "NULL operand");
    BF_REQUIRE((M + 63) / 64 <= 65535, "M too large");
    hipStream_t s = asStream(stream);
    if (!transA && !transB && M <= 8 && N < (size_t(1) << 31) && K < (size_t(1) << 31)) {   // a walk over B, no tiles
        bool served = false;
        const FewRowsProducts one{{A, nullptr, nullptr}, {B, nullptr, nullptr}, {C, nullptr, nullptr}, {bias, nullptr, nullptr}, {residual, nullptr, nullptr}, nullptr, -1};
        int st = launchFewRowsF32Any(one, 1, M, N, K, s, &served);
        if (st != BF_OK || served) return st;
    }
    // Large tiles once they alone can fill the chip twice over; small tiles otherwise.
    const size_t cus = size_t(computeUnits());
    size_t bigTiles = ((M + 127) / 128) * ((N + 127) / 128);
    if (bigTiles >= 2 * cus) return launchGemm<128, 128>(transA, transB, A, B, C, M, N, K, 1, K, 0, bias, residual, s);
    // Few tiles and a long contraction (the weight gradients of a small model: a [features x features] product
    // over all tokens): cut K into slices so that more workgroups share it; a second kernel adds the slices in
    // order.
    // The second launch must pay for itself: with a workgroup alone on its compute unit a K step of 32 takes about a
    // microsecond (nothing hides its latencies) and a dependent launch about five, so contractions under 256 stay whole
    // (a small model's step is bounded by its launch count) and longer ones are cut into slices of at least two steps.
    const size_t tiles = ((M + 63) / 64) * ((N + 63) / 64);
    // Fewer 64 x 64 tiles than half the chip: 32 x 32 tiles with K steps of 128.  A contraction is cut into slices (of
    // at least four steps) only when it is long enough for a second launch to pay: 2048 and up.
    if (tiles * 2 <= cus && (M + SBT - 1) / SBT <= 65535) {
        const size_t smallTiles = ((M + SBT - 1) / SBT) * ((N + SBT - 1) / SBT);
        size_t cut = 1;
        if (K >= 16 * SBK && smallTiles < cus) cut = std::min<size_t>(std::min<size_t>(16, 2 * cus / smallTiles), K / (4 * SBK));
        if (cut > 1) {
            const size_t steps = (K + SBK - 1) / SBK, kPer = (steps + cut - 1) / cut * SBK;
            cut = (K + kPer - 1) / kPer;
            const size_t count = M * N;
            Scratch partial(cut * count * sizeof(float));
            if (partial.status != BF_OK) return partial.status;
            int st = launchSmallGemm(transA, transB, A, B, partial.as<float>(), M, N, K, cut, kPer, count, nullptr, nullptr, s);
            if (st != BF_OK) return st;
            sliceSumKernel<<<gridFor(count, kBlock), kBlock, 0, s>>>(partial.as<float>(), C, count, count, int(cut), N, bias, residual);
            BF_LAUNCH_CHECK();
            return BF_OK;
        }
        return launchSmallGemm(transA, transB, A, B, C, M, N, K, 1, K, 0, bias, residual, s);
    }
    size_t slices = 1;
    if (tiles < cus && K >= 8 * BK) slices = std::min<size_t>(std::min<size_t>(16, cus / tiles), K / (2 * BK));
    if (slices > 1) {
        const size_t steps = (K + BK - 1) / BK, kPer = (steps + slices - 1) / slices * BK;
        slices = (K + kPer - 1) / kPer;
        const size_t count = M * N;
        Scratch partial(slices * count * sizeof(float));
        if (partial.status != BF_OK) return partial.status;
        int st = launchGemm<64, 64>(transA, transB, A, B, partial.as<float>(), M, N, K, slices, kPer, count, nullptr, nullptr, s);
        if (st != BF_OK) return st;
        sliceSumKernel<<<gridFor(count, kBlock), kBlock, 0, s>>>(partial.as<float>(), C, count, count, int(slices), N, bias, residual);
        BF_LAUNCH_CHECK();
        return BF_OK;
    }
    return launchGemm<64, 64>(transA, transB, A, B, C, M, N, K, 1, K, 0, bias, residual, s);
}
}  // namespace
}  // namespace bf

extern "C" int bf_hip_gemm_f32(int transA, int transB, const float* A, const float* B, float* C, size_t M, size_t N,
                               size_t K, bf_stream_t stream) {
    return gemmF32(transA, transB, A, B, C, M, N, K, nullptr, nullptr, stream);
}

extern "C" int bf_hip_gemm_f32_adds(int transA, int transB, const float* A, const float* B, const float* bias, const float* residual,
                                    float* C, size_t M, size_t N, size_t K, bf_stream_t stream) {
    return gemmF32(transA, transB, A, B, C, M, N, K, bias, residual, stream);
}

// c[i] = rmsnorm(x) b[i] in fp32 for up to three weights [k, n]: the projections of an attention block's normalised input
// (ops_transformer.cu:107-111) for a caller that keeps nothing for a backward pass.  One or two rows: the normalisation is
// made by the products' kernel while it stages the rows; otherwise the row kernel runs first.
extern "C" int bf_hip_rmsnorm_matmul_f32_shared_input(const float* x, const float* const* b, float* const* c, size_t count, size_t m, size_t k,
                                                      size_t n, bf_stream_t stream) {
    BF_REQUIRE(count >= 1 && count <= 3, "count must be 1, 2 or 3");
    BF_REQUIRE(b && c, "NULL pointer array");
    if (m == 0 || n == 0) return BF_OK;
    BF_REQUIRE(k > 0 && x != nullptr, "NULL or empty input");
    for (size_t i = 0; i < count; ++i) BF_REQUIRE(b[i] != nullptr && c[i] != nullptr, "NULL operand");
    if (m <= 2 && n < (size_t(1) << 31) && k < (size_t(1) << 31)) {
        FewRowsProducts g = {};
        g.act = -1;
        g.normInput = x;
        for (size_t i = 0; i < count; ++i) { g.B[i] = b[i]; g.out[i] = c[i]; }
        bool served = false;
        int st = launchFewRowsF32Any(g, count, m, n, k, asStream(stream), &served);
        if (st != BF_OK || served) return st;
    }
    Scratch normed(m * k * sizeof(float));
    if (normed.status != BF_OK) return normed.status;
    int st = bf_hip_rmsnorm(x, normed.as<float>(), m, k, stream);
    if (st != BF_OK) return st;
    bf_gemm_f32_problem problems[3];
    for (size_t i = 0; i < count; ++i) problems[i] = bf_gemm_f32_problem{normed.as<float>(), b[i], c[i], nullptr, nullptr, m, n, k, 0, 0};
    return bf_hip_gemm_f32_group(problems, count, stream);
}

// The projections of a decoding step whose position lives on the device, in fp32: q = rmsnorm(x) wq, and the rows of
// rmsnorm(x) wk and ... wv appended to caches of `capacity` rows a sequence at row *position.  One sequence of one or two new
// rows: the three products in one walk that stores the keys and values where they belong; anything else: the products
// into scratch rows, then bf_hip_kv_append_indirect.
extern "C" int bf_hip_decode_projections_f32(const float* x, const float* wq, const float* wk, const float* wv, float* q, float* kCache,
                                             float* vCache, size_t batch, size_t newLen, size_t dim, size_t capacity, const int* position,
                                             bf_stream_t stream) {
    if (batch == 0 || newLen == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(x && wq && wk && wv && q && kCache && vCache && position, "NULL pointer");
    BF_REQUIRE(newLen <= capacity && capacity < (size_t(1) << 31), "more new rows than the cache holds");
    const size_t rows = batch * newLen;
    if (batch == 1 && rows <= 2 && dim < (size_t(1) << 31)) {
        FewRowsProducts g = {};
        g.act = -1;
        g.normInput = x;
        g.rowShift = position;
        g.rowLimit = int(capacity);
        g.B[0] = wq; g.B[1] = wk; g.B[2] = wv;
        g.out[0] = q; g.out[1] = kCache; g.out[2] = vCache;
        bool served = false;
        int st = launchFewRowsF32Any(g, 3, rows, dim, dim, asStream(stream), &served);
        if (st != BF_OK || served) return st;
    }
    Scratch fresh(2 * rows * dim * sizeof(float));
    if (fresh.status != BF_OK) return fresh.status;
    const float* weights[3] = {wq, wk, wv};
    float* outs[3] = {q, fresh.as<float>(), fresh.as<float>() + rows * dim};
    int st = bf_hip_rmsnorm_matmul_f32_shared_input(x, weights, outs, 3, rows, dim, dim, stream);
    if (st != BF_OK) return st;
    return bf_hip_kv_append_indirect(kCache, vCache, outs[1], outs[2], batch, newLen, dim, capacity, position, stream);
}

// out = input + act(rmsnorm(input) w1 + b1) w2 + b2 in fp32: the feed-forward block (ops_transformer.cu:182-215) for a caller
// that keeps nothing for a backward pass.  One or two rows: the first product normalises while it stages its rows and the
// activation is applied where its K slices are summed.
extern "C" int bf_hip_rmsnorm_feedforward_f32(const float* input, const float* w1, const float* b1, const float* w2, const float* b2, int act,
                                              float* out, size_t m, size_t d, size_t hidden, bf_stream_t stream) {
    if (m == 0) return BF_OK;
    BF_REQUIRE(d > 0 && hidden > 0, "d and hidden must be positive");
    BF_REQUIRE(act == BF_ACT_SILU || act == BF_ACT_GELU || act == BF_ACT_RELU, "unknown activation");
    BF_REQUIRE(input && w1 && b1 && w2 && b2 && out, "NULL pointer");
    Scratch h(m * hidden * sizeof(float));
    if (h.status != BF_OK) return h.status;
    bool served = false;
    if (m <= 2 && d < (size_t(1) << 31) && hidden < (size_t(1) << 31)) {
        FewRowsProducts g = {};
        g.act = act;
        g.normInput = input;
        g.B[0] = w1; g.out[0] = h.as<float>(); g.bias[0] = b1;
        int st = launchFewRowsF32Any(g, 1, m, hidden, d, asStream(stream), &served);
        if (st != BF_OK) return st;
    }
    if (!served) {
        Scratch normed(m * d * sizeof(float)), z(m * hidden * sizeof(float));
        if (normed.status != BF_OK) return normed.status;
        if (z.status != BF_OK) return z.status;
        int st = bf_hip_rmsnorm(input, normed.as<float>(), m, d, stream);
        if (st == BF_OK) st = bf_hip_gemm_f32(0, 0, normed.as<float>(), w1, z.as<float>(), m, hidden, d, stream);
        if (st == BF_OK) st = bf_hip_add_bias_act(z.as<float>(), b1, h.as<float>(), m, hidden, act, stream);
        if (st != BF_OK) return st;
    }
    return bf_hip_gemm_f32_adds(0, 0, h.as<float>(), w2, b2, input, out, m, d, hidden, stream);
}

extern "C" int bf_hip_gemm_f32_group(const bf_gemm_f32_problem* problems, size_t count, bf_stream_t stream) {
    if (count == 0) return BF_OK;
    BF_REQUIRE(problems != nullptr, "NULL problem list");
    // one launch when every product is small enough for the 32 x 32 form without K slices (the form bf_hip_gemm_f32 itself
    // would pick); otherwise, or beyond eight products, the products are launched one after the other
    // two or three products of at most eight rows and one shape (the Q, K and V projections of a decoding step): one walk
    if (count >= 2 && count <= 3) {
        const bf_gemm_f32_problem& f = problems[0];
        bool alike = f.M >= 1 && f.M <= 8 && f.N >= 1 && f.K >= 1 && f.N < (size_t(1) << 31) && f.K < (size_t(1) << 31);
        FewRowsProducts g = {};
        g.act = -1;
        for (size_t i = 0; i < count && alike; ++i) {
            const bf_gemm_f32_problem& p = problems[i];
            alike = !p.transA && !p.transB && p.M == f.M && p.N == f.N && p.K == f.K && p.A && p.B && p.C;
            g.A[i] = p.A; g.B[i] = p.B; g.out[i] = p.C; g.bias[i] = p.bias; g.residual[i] = p.residual;
        }
        if (alike) {
            bool served = false;
            int st = launchFewRowsF32Any(g, count, f.M, f.N, f.K, asStream(stream), &served);
            if (st != BF_OK || served) return st;
        }
    }
    const size_t cus = size_t(computeUnits());
    auto aligned16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    bool together = count <= size_t(kMaxGroup) && count > 1, vec = true;
    size_t tilesM = 0, tilesN = 0;
    for (size_t i = 0; i < count && together; ++i) {
        const bf_gemm_f32_problem& p = problems[i];
        if (p.M == 0 || p.N == 0) continue;
        BF_REQUIRE(p.C != nullptr, "NULL output");
        const size_t tiles = ((p.M + 63) / 64) * ((p.N + 63) / 64);
        together = p.K > 0 && p.K < size_t(16) * SBK && tiles * 2 <= cus && p.M < (size_t(1) << 31) && p.N < (size_t(1) << 31) && p.A && p.B &&
                   (p.transA || p.transB || p.M > 8);   // a product of a few rows is a walk when launched alone: the same here
        vec = vec && aligned16(p.A) && aligned16(p.B) && (p.transA ? p.M : p.K) % 4 == 0 && (p.transB ? p.K : p.N) % 4 == 0;
        tilesM = std::max(tilesM, (p.M + SBT - 1) / SBT);
        tilesN = std::max(tilesN, (p.N + SBT - 1) / SBT);
    }
    if (!together || tilesM == 0 || tilesM > 65535) {
        for (size_t i = 0; i < count; ++i) {
            const bf_gemm_f32_problem& p = problems[i];
            int st = gemmF32(p.transA, p.transB, p.A, p.B, p.C, p.M, p.N, p.K, p.bias, p.residual, stream);
            if (st != BF_OK) return st;
        }
        return BF_OK;
    }
    GroupArgs args = {};
    for (size_t i = 0; i < count; ++i) {
        const bf_gemm_f32_problem& p = problems[i];
        args.p[i] = GroupProblem{p.A, p.B, p.C, p.bias, p.residual, unsigned(p.M), unsigned(p.N), unsigned(p.K), p.transA, p.transB};
    }
    const dim3 grid = dim3(static_cast<unsigned>(tilesN), static_cast<unsigned>(tilesM), static_cast<unsigned>(count));
    if (vec) gemmF32SmallGroupKernel<4, 4><<<grid, 256, 0, asStream(stream)>>>(args);
    else gemmF32SmallGroupKernel<1, 1><<<grid, 256, 0, asStream(stream)>>>(args);
    BF_LAUNCH_CHECK();
    return BF_OK;
}
