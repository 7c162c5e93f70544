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

namespace bf {
namespace {

constexpr int BK = 16;

template <int BM, int BN>
struct GemmTile {
    static constexpr int kPad = 4;
    float as[BK][BM + kPad];
    float bs[BK][BN + kPad];
};

// Copies the [BK x BT] tile of op(X) starting at (k0, t0) into lds[k][t], zero-filling outside the
// matrix.  op(X)[k][t] = X[t*ld + k] when the tile dimension t is the row of X (contiguous along k),
// or X[k*ld + t] when t is the column of X (contiguous along t).
template <int BT, bool T_IS_ROW>
__device__ __forceinline__ void loadTile(float (*lds)[BT + 4], const float* __restrict__ X, size_t ld, size_t tExtent,
                                         size_t kExtent, size_t t0, size_t k0, int tid) {
    constexpr int kElems = BK * BT;
#pragma unroll
    for (int e = tid; e < kElems; e += 256) {
        int k, t;
        if constexpr (T_IS_ROW) { k = e % BK; t = e / BK; }   // consecutive threads walk k (contiguous)
        else { t = e % BT; k = e / BT; }                       // consecutive threads walk t (contiguous)
        size_t gt = t0 + t, gk = k0 + k;
        float v = 0.0f;
        if (gt < tExtent && gk < kExtent) v = T_IS_ROW ? X[gt * ld + gk] : X[gk * ld + gt];
        lds[k][t] = v;
    }
}

// TRANS_A: A stored [K,M] (op(A)[m][k] = A[k*M + m]); otherwise A stored [M,K].
// TRANS_B: B stored [N,K] (op(B)[k][n] = B[n*K + k]); otherwise B stored [K,N].
template <int BM, int BN, bool TRANS_A, bool TRANS_B>
__global__ void __launch_bounds__(256) gemmF32Kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                      float* __restrict__ C, size_t M, size_t N, size_t K) {
    constexpr int WM = BM / 2, WN = BN / 2;      // 2 x 2 wavefronts
    constexpr int TM = WM / 32, TN = WN / 32;    // 32x32 MFMA tiles per wavefront
    __shared__ GemmTile<BM, BN> tile;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const size_t m0 = size_t(blockIdx.y) * BM, n0 = size_t(blockIdx.x) * BN;
    const int li = lane & 31, lk = lane >> 5;

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    for (size_t k0 = 0; k0 < K; k0 += BK) {
        // A tile: tile dimension m.  A stored [M,K] -> m is the row (contiguous along k).
        if constexpr (TRANS_A) loadTile<BM, false>(tile.as, A, M, M, K, m0, k0, tid);
        else loadTile<BM, true>(tile.as, A, K, M, K, m0, k0, tid);
        // B tile: tile dimension n.  B stored [K,N] -> n is the column (contiguous along n).
        if constexpr (TRANS_B) loadTile<BN, true>(tile.bs, B, K, N, K, n0, k0, tid);
        else loadTile<BN, false>(tile.bs, B, N, N, K, n0, k0, tid);
        __syncthreads();
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
                if (row < M && col < N) C[row * N + col] = acc[i][j][r];
            }
        }
}

template <int BM, int BN>
int launchGemm(int transA, int transB, const float* A, const float* B, float* C, size_t M, size_t N, size_t K,
               hipStream_t s) {
    dim3 grid(unsigned((N + BN - 1) / BN), unsigned((M + BM - 1) / BM));
    if (!transA && !transB) gemmF32Kernel<BM, BN, false, false><<<grid, 256, 0, s>>>(A, B, C, M, N, K);
    else if (!transA && transB) gemmF32Kernel<BM, BN, false, true><<<grid, 256, 0, s>>>(A, B, C, M, N, K);
    else if (transA && !transB) gemmF32Kernel<BM, BN, true, false><<<grid, 256, 0, s>>>(A, B, C, M, N, K);
    else gemmF32Kernel<BM, BN, true, true><<<grid, 256, 0, s>>>(A, B, C, M, N, K);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" int bf_hip_gemm_f32(int transA, int transB, const float* A, const float* B, float* C, size_t M, size_t N,
                               size_t K, bf_stream_t stream) {
    if (M == 0 || N == 0) return BF_OK;
    BF_REQUIRE(C != nullptr, "NULL output");
    if (K == 0) return bf_hip_fill_zero(C, M * N * sizeof(float), stream);
    BF_REQUIRE(A && B, "NULL operand");
    BF_REQUIRE((M + 63) / 64 <= 65535, "M too large");
    // Large tiles once they alone can fill the chip twice over; small tiles otherwise.
    size_t bigTiles = ((M + 127) / 128) * ((N + 127) / 128);
    if (bigTiles >= size_t(2) * size_t(computeUnits()))
        return launchGemm<128, 128>(transA, transB, A, B, C, M, N, K, asStream(stream));
    return launchGemm<64, 64>(transA, transB, A, B, C, M, N, K, asStream(stream));
}
