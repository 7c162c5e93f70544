// bf16 GEMM with fp32 accumulation on the bf16 MFMA pipe (v_mfma_f32_32x32x16_bf16), and the
// fp32 -> bf16 operand conversion around it.
//
// The operator contract is fp32 in, fp32 out with both operands rounded to bf16 (nearest even)
// before the product.  Every product is run in one form only, C[M,N] = A[M,K] * Bt[N,K]^T with both
// operands contiguous along K, which is the layout the MFMA wants (a lane's 8 consecutive k values
// are one 16-byte LDS read).  The three products of a linear layer map onto it through the conversion
// pass, which can also transpose:
//     forward  c = a b      : A = bf16(a)        Bt = bf16(b)^T  (transposing convert, cacheable)
//     dA = g b^T            : A = bf16(g)        Bt = bf16(b)    (plain convert, cacheable)
//     dB = a^T g            : A = bf16(a)^T      Bt = bf16(g)^T  (transposing converts)
// Converted operands are padded with zeros to a multiple of 8 along K so the GEMM needs no K tail.
//
// Kernel: 256 threads (2 x 2 wavefronts), 128 x 128 tile of C per workgroup, 64 x 64 per wavefront
// (four 32x32 accumulators), K step 64.  Global loads of the next K step are issued into registers
// before the MFMAs of the current one and written to LDS afterwards (register double buffering).
// LDS rows are padded by 16 bytes so the 16-byte operand reads of 8 consecutive lanes cover all banks.
#include "common.hpp"

#include <map>
#include <unordered_map>

namespace bf {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short ushort8 __attribute__((ext_vector_type(8)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned short toBf16Bits(float x) {
    __bf16 h = static_cast<__bf16>(x);   // round to nearest even, NaN preserved
    return __builtin_bit_cast(unsigned short, h);
}

inline size_t pad8(size_t n) { return (n + 7) / 8 * 8; }

// out[r, 0..colsPad) = bf16(x[r, 0..cols)), zero padded.
__global__ void __launch_bounds__(kBlock) convertKernel(const float* __restrict__ x, unsigned short* __restrict__ out,
                                                        size_t rows, size_t cols, size_t colsPad, int vec) {
    const size_t groupsPerRow = colsPad / 8;
    const size_t total = rows * groupsPerRow;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (size_t gidx = size_t(blockIdx.x) * blockDim.x + threadIdx.x; gidx < total; gidx += stride) {
        size_t r = gidx / groupsPerRow, c = (gidx - r * groupsPerRow) * 8;
        const float* src = x + r * cols + c;
        ushort8 v;
        if (vec && c + 8 <= cols) {
            float4v a = loadf4(src), b = loadf4(src + 4);
            v[0] = toBf16Bits(a.x); v[1] = toBf16Bits(a.y); v[2] = toBf16Bits(a.z); v[3] = toBf16Bits(a.w);
            v[4] = toBf16Bits(b.x); v[5] = toBf16Bits(b.y); v[6] = toBf16Bits(b.z); v[7] = toBf16Bits(b.w);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = c + j < cols ? toBf16Bits(src[j]) : (unsigned short)0;
        }
        *reinterpret_cast<ushort8*>(out + r * colsPad + c) = v;
    }
}

// out[c, 0..rowsPad) = bf16(x[0..rows, c]), zero padded: 64 x 64 tiles through LDS.
__global__ void __launch_bounds__(kBlock) convertTransposeKernel(const float* __restrict__ x, unsigned short* __restrict__ out,
                                                                 size_t rows, size_t cols, size_t rowsPad) {
    __shared__ unsigned short tile[64][66];
    const size_t r0 = size_t(blockIdx.y) * 64, c0 = size_t(blockIdx.x) * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;   // 64 x 4
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        int r = ty + 4 * i;
        size_t gr = r0 + r, gc = c0 + tx;
        tile[r][tx] = (gr < rows && gc < cols) ? toBf16Bits(x[gr * cols + gc]) : (unsigned short)0;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        int c = ty + 4 * i;
        size_t gc = c0 + c, gr = r0 + tx;
        if (gc < cols && gr < rowsPad) out[gc * rowsPad + gr] = tile[tx][c];
    }
}

// ---- the GEMM ----------------------------------------------------------------------------------
// C[M,N] = A[M,K] * Bt[N,K]^T.  A workgroup of WAVES_M x WAVES_N wavefronts owns a BM x BN tile; each
// wavefront a (BM/WAVES_M) x (BN/WAVES_N) sub-tile made of 32x32 MFMA accumulators.  K advances in steps
// of 64 through a double-buffered LDS stage with one barrier per step: while step t is being multiplied
// out of buffer t&1, the registers holding step t+1 are written to the other buffer and the global loads
// of step t+2 are issued.
constexpr int BKK = 64;
constexpr int LDS_ROW = BKK + 8;   // bf16 elements per LDS row: 128 B of data + 16 B pad (conflict-free b128 reads)

template <int BM, int BN, int WAVES_M, int WAVES_N>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64) gemmBf16NtKernel(const unsigned short* __restrict__ A,
                                                                            const unsigned short* __restrict__ Bt,
                                                                            float* __restrict__ C, int M, int N, int K, int lda,
                                                                            int ldb) {
    constexpr int THREADS = WAVES_M * WAVES_N * 64;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;     // per-wave tile
    constexpr int TM = WM / 32, TN = WN / 32;               // 32x32 accumulators per wave
    constexpr int ROWS_PER_PASS = THREADS / 8;              // 8 threads (16 B each) cover one 128-byte row
    constexpr int A_PASSES = BM / ROWS_PER_PASS, B_PASSES = BN / ROWS_PER_PASS;
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "tile rows must be a multiple of the rows loaded per pass");
    extern __shared__ __attribute__((aligned(16))) unsigned short lds[];
    unsigned short* as = lds;                              // [2][BM][LDS_ROW]
    unsigned short* bs = lds + 2 * BM * LDS_ROW;           // [2][BN][LDS_ROW]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    // Tile order: groups of 8 tile-rows are walked column-first so that the tiles in flight at any time
    // share A and Bt panels in L2; workgroups go round-robin to the 8 XCDs.
    const int tilesM = (M + BM - 1) / BM, tilesN = (N + BN - 1) / BN;
    int tm, tn;
    {
        constexpr int GROUP = 8;
        const int id = blockIdx.x;
        const int perGroup = GROUP * tilesN;
        const int g = id / perGroup, rem = id - g * perGroup;
        const int rowsInGroup = min(GROUP, tilesM - g * GROUP);
        tm = g * GROUP + rem % rowsInGroup;
        tn = rem / rowsInGroup;
    }
    const int m0 = tm * BM, n0 = tn * BN;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;

    const int lr = tid >> 3, lc = (tid & 7) * 8;
    uint4v aReg[A_PASSES], bReg[B_PASSES];
    auto loadGlobal = [&](int k0) {
        const uint4v z = {0u, 0u, 0u, 0u};
        const bool kOk = k0 + lc < K;
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i) {
            int r = m0 + lr + ROWS_PER_PASS * i;
            aReg[i] = (r < M && kOk) ? *reinterpret_cast<const uint4v*>(A + size_t(r) * lda + k0 + lc) : z;
        }
#pragma unroll
        for (int i = 0; i < B_PASSES; ++i) {
            int r = n0 + lr + ROWS_PER_PASS * i;
            bReg[i] = (r < N && kOk) ? *reinterpret_cast<const uint4v*>(Bt + size_t(r) * ldb + k0 + lc) : z;
        }
    };
    auto storeLds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i)
            *reinterpret_cast<uint4v*>(as + (buf * BM + lr + ROWS_PER_PASS * i) * LDS_ROW + lc) = aReg[i];
#pragma unroll
        for (int i = 0; i < B_PASSES; ++i)
            *reinterpret_cast<uint4v*>(bs + (buf * BN + lr + ROWS_PER_PASS * i) * LDS_ROW + lc) = bReg[i];
    };

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int steps = (K + BKK - 1) / BKK;
    loadGlobal(0);
    storeLds(0);
    if (steps > 1) loadGlobal(BKK);
    __syncthreads();
    for (int t = 0; t < steps; ++t) {
        const unsigned short* ac = as + ((t & 1) * BM + wm0 + li) * LDS_ROW + 8 * half;
        const unsigned short* bc = bs + ((t & 1) * BN + wn0 + li) * LDS_ROW + 8 * half;
#pragma unroll
        for (int kk = 0; kk < BKK; kk += 16) {
            bf16x8 a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = *reinterpret_cast<const bf16x8*>(ac + i * 32 * LDS_ROW + kk);
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = *reinterpret_cast<const bf16x8*>(bc + j * 32 * LDS_ROW + kk);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (t + 1 < steps) {
            storeLds((t + 1) & 1);
            if (t + 2 < steps) loadGlobal((t + 2) * BKK);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = n0 + wn0 + j * 32 + li;
            if (col < N) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                    if (row < M) C[size_t(row) * N + col] = acc[i][j][r];
                }
            }
        }
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
int launchTile(const unsigned short* A, const unsigned short* Bt, float* C, size_t M, size_t N, size_t K, size_t lda, size_t ldb,
               hipStream_t s) {
    size_t tiles = ((M + BM - 1) / BM) * ((N + BN - 1) / BN);
    if (tiles >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
    constexpr size_t smem = size_t(2) * (BM + BN) * LDS_ROW * sizeof(unsigned short);
    auto kernel = gemmBf16NtKernel<BM, BN, WAVES_M, WAVES_N>;
    if (smem > 48 * 1024)
        BF_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
    kernel<<<unsigned(tiles), WAVES_M * WAVES_N * 64, smem, s>>>(A, Bt, C, int(M), int(N), int(K), int(lda), int(ldb));
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int launchGemmNt(const unsigned short* A, const unsigned short* Bt, float* C, size_t M, size_t N, size_t K, size_t lda,
                 size_t ldb, hipStream_t s) {
    if (M >= (size_t(1) << 31) || N >= (size_t(1) << 31) || K >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
    // 256x256 tiles (8 wavefronts) once they give every CU at least one tile; otherwise 128x128 (4 wavefronts)
    const size_t bigTiles = ((M + 255) / 256) * ((N + 255) / 256);
    if (bigTiles >= size_t(computeUnits()) * 3 / 4) return launchTile<256, 256, 2, 4>(A, Bt, C, M, N, K, lda, ldb, s);
    return launchTile<128, 128, 2, 2>(A, Bt, C, M, N, K, lda, ldb, s);
}

int convertPlain(const float* x, unsigned short* out, size_t rows, size_t cols, hipStream_t s) {
    size_t colsPad = pad8(cols);
    size_t groups = rows * (colsPad / 8);
    if (groups == 0) return BF_OK;
    int vec = (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && cols % 4 == 0;
    convertKernel<<<gridFor(groups, kBlock, unsigned(computeUnits()) * 16), kBlock, 0, s>>>(x, out, rows, cols, colsPad, vec);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int convertTransposed(const float* x, unsigned short* out, size_t rows, size_t cols, hipStream_t s, bool padRows = true) {
    if (rows == 0 || cols == 0) return BF_OK;
    size_t rowsPad = padRows ? pad8(rows) : rows;   // length of an output row
    dim3 grid(unsigned((cols + 63) / 64), unsigned((rowsPad + 63) / 64));
    if (grid.y > 65535) return failInvalid("cvt_f32_bf16_transpose", "too many rows");
    convertTransposeKernel<<<grid, kBlock, 0, s>>>(x, out, rows, cols, rowsPad);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

// ---- bf16 images of weights, kept per (device, pointer, layout) until invalidated -------------------
struct CachedWeight {
    size_t generation;
    void* buffer;
    size_t bytes;
};
size_t g_generation = 0;
std::map<std::tuple<int, const float*, int>, CachedWeight>& weightCache() {
    static std::map<std::tuple<int, const float*, int>, CachedWeight> cache;
    return cache;
}

// Returns a bf16 image of w[rows, cols]: transposed ([cols, pad8(rows)]) or plain ([rows, pad8(cols)]).
// With `cache` the image is kept; otherwise it is a scratch buffer the caller releases with releaseImage.
int weightImage(const float* w, size_t rows, size_t cols, bool transposed, bool cache, hipStream_t s, unsigned short** image,
                size_t* imageBytes) {
    size_t bytes = (transposed ? cols * pad8(rows) : rows * pad8(cols)) * sizeof(unsigned short);
    *imageBytes = bytes;
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    if (cache) {
        auto key = std::make_tuple(dev, w, transposed ? 1 : 0);
        auto it = weightCache().find(key);
        if (it != weightCache().end() && it->second.generation == g_generation && it->second.bytes == bytes) {
            *image = static_cast<unsigned short*>(it->second.buffer);
            return BF_OK;
        }
        void* buf = nullptr;
        if (it != weightCache().end() && it->second.bytes == bytes) buf = it->second.buffer;   // refresh in place
        else {
            if (it != weightCache().end()) bf_hip_pool_release(it->second.buffer, it->second.bytes);
            int st = bf_hip_pool_acquire(bytes, &buf);
            if (st != BF_OK) return st;
        }
        weightCache()[key] = CachedWeight{g_generation, buf, bytes};
        *image = static_cast<unsigned short*>(buf);
    } else {
        void* buf = nullptr;
        int st = bf_hip_pool_acquire(bytes, &buf);
        if (st != BF_OK) return st;
        *image = static_cast<unsigned short*>(buf);
    }
    return transposed ? convertTransposed(w, *image, rows, cols, s) : convertPlain(w, *image, rows, cols, s);
}

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" {

int bf_hip_cvt_f32_bf16(const float* x, uint16_t* out, size_t n, bf_stream_t stream) {
    if (n == 0) return BF_OK;
    BF_REQUIRE(x && out, "NULL pointer");
    // a flat vector is one row; the padded tail (if any) must not be written past n
    size_t body = n / 8 * 8;
    int st = BF_OK;
    if (body) st = convertPlain(x, out, 1, body, asStream(stream));
    if (st != BF_OK) return st;
    if (body < n) {
        // tail of fewer than 8 values: convert into a scratch group and copy what is needed
        Scratch tmp(8 * sizeof(unsigned short));
        if (tmp.status != BF_OK) return tmp.status;
        st = convertPlain(x + body, tmp.as<unsigned short>(), 1, n - body, asStream(stream));
        if (st != BF_OK) return st;
        BF_HIP_TRY(hipMemcpyAsync(out + body, tmp.ptr, (n - body) * sizeof(unsigned short), hipMemcpyDeviceToDevice,
                                  asStream(stream)));
    }
    return BF_OK;
}

int bf_hip_cvt_f32_bf16_transpose(const float* x, uint16_t* out, size_t rows, size_t cols, bf_stream_t stream) {
    if (rows == 0 || cols == 0) return BF_OK;
    BF_REQUIRE(x && out, "NULL pointer");
    return convertTransposed(x, out, rows, cols, asStream(stream), /*padRows=*/false);
}

int bf_hip_gemm_bf16_nt(const uint16_t* A, const uint16_t* Bt, float* C, size_t M, size_t N, size_t K, bf_stream_t stream) {
    if (M == 0 || N == 0) return BF_OK;
    BF_REQUIRE(C != nullptr, "NULL output");
    if (K == 0) return bf_hip_fill_zero(C, M * N * sizeof(float), stream);
    BF_REQUIRE(A && Bt, "NULL operand");
    BF_REQUIRE(K % 8 == 0, "K must be a multiple of 8 (16-byte operand rows)");
    BF_REQUIRE(((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(Bt)) & 15u) == 0, "operands must be 16-byte aligned");
    return launchGemmNt(A, Bt, C, M, N, K, K, K, asStream(stream));
}

int bf_hip_matmul_bf16(const float* a, const float* b, float* c, size_t m, size_t k, size_t n, int cacheWeight,
                       bf_stream_t stream) {
    if (m == 0 || n == 0) return BF_OK;
    BF_REQUIRE(c != nullptr, "NULL output");
    if (k == 0) return bf_hip_fill_zero(c, m * n * sizeof(float), stream);
    BF_REQUIRE(a && b, "NULL operand");
    hipStream_t s = asStream(stream);
    const size_t kp = pad8(k);
    Scratch aImg(m * kp * sizeof(unsigned short));
    if (aImg.status != BF_OK) return aImg.status;
    int st = convertPlain(a, aImg.as<unsigned short>(), m, k, s);
    if (st != BF_OK) return st;
    unsigned short* bImg = nullptr;
    size_t bBytes = 0;
    st = weightImage(b, k, n, /*transposed=*/true, cacheWeight != 0, s, &bImg, &bBytes);
    if (st != BF_OK) return st;
    st = launchGemmNt(aImg.as<unsigned short>(), bImg, c, m, n, kp, kp, kp, s);
    if (!cacheWeight) bf_hip_pool_release(bImg, bBytes);
    return st;
}

int bf_hip_matmul_bf16_backward(const float* a, const float* b, const float* g, float* dA, float* dB, size_t m,
                                size_t k, size_t n, int cacheWeight, bf_stream_t stream) {
    hipStream_t s = asStream(stream);
    if (m == 0 || k == 0 || n == 0) {   // degenerate: gradients are zero (ops_tensorcore.cu:412-415)
        int st = BF_OK;
        if (dA && m * k) st = bf_hip_fill_zero(dA, m * k * sizeof(float), stream);
        if (st == BF_OK && dB && k * n) st = bf_hip_fill_zero(dB, k * n * sizeof(float), stream);
        return st;
    }
    BF_REQUIRE(a && b && g, "NULL operand");
    int st = BF_OK;
    if (dA) {   // dA[m,k] = g[m,n] * b[k,n]^T : contraction over n
        const size_t np = pad8(n);
        Scratch gImg(m * np * sizeof(unsigned short));
        if (gImg.status != BF_OK) return gImg.status;
        st = convertPlain(g, gImg.as<unsigned short>(), m, n, s);
        if (st != BF_OK) return st;
        unsigned short* bImg = nullptr;
        size_t bBytes = 0;
        st = weightImage(b, k, n, /*transposed=*/false, cacheWeight != 0, s, &bImg, &bBytes);
        if (st != BF_OK) return st;
        st = launchGemmNt(gImg.as<unsigned short>(), bImg, dA, m, k, np, np, np, s);
        if (!cacheWeight) bf_hip_pool_release(bImg, bBytes);
        if (st != BF_OK) return st;
    }
    if (dB) {   // dB[k,n] = a[m,k]^T * g[m,n] : contraction over m
        const size_t mp = pad8(m);
        Scratch aT(k * mp * sizeof(unsigned short));
        Scratch gT(n * mp * sizeof(unsigned short));
        if (aT.status != BF_OK) return aT.status;
        if (gT.status != BF_OK) return gT.status;
        st = convertTransposed(a, aT.as<unsigned short>(), m, k, s);
        if (st != BF_OK) return st;
        st = convertTransposed(g, gT.as<unsigned short>(), m, n, s);
        if (st != BF_OK) return st;
        st = launchGemmNt(aT.as<unsigned short>(), gT.as<unsigned short>(), dB, k, n, mp, mp, mp, s);
    }
    return st;
}

int bf_hip_invalidate_bf16_weight_cache(void) {
    ++g_generation;
    return BF_OK;
}

}  // extern "C"
