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
// Two kernels, picked by tile count: a 256x256-tile kernel whose eight wavefronts alternate between moving
// data and multiplying (large products), and a 128x128-tile kernel with one barrier per K step, optionally
// cutting K into slices that a second kernel adds up in a fixed order (small products).
#include "common.hpp"

#include <algorithm>
#include <atomic>
#include <type_traits>
#include <map>
#include <set>
#include <tuple>
#include <unordered_map>
#include <vector>

namespace bf {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned short ushort8 __attribute__((ext_vector_type(8)));
typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));   // a float4 that may start on any 4-byte boundary


inline size_t pad8(size_t n) { return (n + 7) / 8 * 8; }

// out[r*ld + 0..colsPad) = bf16(x[r, 0..cols)), zero padded.
template <bool NT>
__global__ void __launch_bounds__(kBlock) convertKernel(const float* __restrict__ x, unsigned short* __restrict__ out,
                                                        size_t rows, size_t cols, size_t colsPad, size_t ld) {
    const size_t groupsPerRow = colsPad / 8;
    const size_t total = rows * groupsPerRow;
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    for (size_t gidx = size_t(blockIdx.x) * blockDim.x + threadIdx.x; gidx < total; gidx += stride) {
        size_t r = gidx / groupsPerRow, c = (gidx - r * groupsPerRow) * 8;
        const float* src = x + r * cols + c;
        ushort8 v;
        if (c + 8 <= cols) {
            // two 16-byte loads; global memory serves them from any 4-byte boundary, so rows of an odd width (which do
            // not start on 16-byte boundaries) take the same path
            float4u a, b;
            if constexpr (NT) { a = __builtin_nontemporal_load(reinterpret_cast<const float4u*>(src)); b = __builtin_nontemporal_load(reinterpret_cast<const float4u*>(src + 4)); }
            else { a = *reinterpret_cast<const float4u*>(src); b = *reinterpret_cast<const float4u*>(src + 4); }
            v[0] = toBf16Bits(a.x); v[1] = toBf16Bits(a.y); v[2] = toBf16Bits(a.z); v[3] = toBf16Bits(a.w);
            v[4] = toBf16Bits(b.x); v[5] = toBf16Bits(b.y); v[6] = toBf16Bits(b.z); v[7] = toBf16Bits(b.w);
        } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = c + j < cols ? toBf16Bits(src[j]) : (unsigned short)0;
        }
        if constexpr (NT) __builtin_nontemporal_store(v, reinterpret_cast<ushort8*>(out + r * ld + c));
        else *reinterpret_cast<ushort8*>(out + r * ld + c) = v;
    }
}

// out[c, 0..rowsPad) = bf16(x[0..rows, c]), zero padded: 64 x 64 tiles through LDS.  With `vec` (x 16-byte
// aligned, cols a multiple of 4, rowsPad a multiple of 8) a thread reads four consecutive columns of a row as
// one 16-byte load and writes eight consecutive rows of an output row as one 16-byte store, so both sides move
// whole 128-byte lines; otherwise elements go one by one.  When `plain` is not NULL the same pass also writes
// the untransposed image plain[r*ldPlain + 0..pad8(cols)) = bf16(x[r, :]), zero padded: a gradient that feeds
// both the input-gradient GEMM (plain) and the weight-gradient GEMM (transposed) is read from HBM once.
// Up to three matrices of one shape in one launch (blockIdx.z): matrix z is read from xs.p[z] and written `outStep`
// (and `plainStep`) elements after the one before.
struct ConvertSources { const float* p[3]; };
// One 64 x 64 tile (rows r0.., columns c0..) of that conversion; `tile` is the workgroup's [64][72] LDS array.
// `out` may be NULL when `plain` is not: the plain image alone is written.
__device__ __forceinline__ void convertTransposeTile(const float* __restrict__ x, unsigned short* __restrict__ out, size_t rows,
                                                     size_t cols, size_t rowsPad, int vec, unsigned short* __restrict__ plain,
                                                     size_t ldPlain, size_t r0, size_t c0, unsigned short (*tile)[72]) {
    const size_t colsPad = (cols + 7) / 8 * 8;
    if (vec) {
        const int cg = threadIdx.x & 15, rr = threadIdx.x >> 4;   // 16 column groups x 16 rows per pass
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = rr + 16 * i;
            const size_t gr = r0 + r, gc = c0 + 4 * cg;
            float4u v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (gr < rows && gc + 4 <= cols) {
                v = *reinterpret_cast<const float4u*>(x + gr * cols + gc);   // from any 4-byte boundary (rows of odd length)
            } else if (gr < rows && gc < cols) {   // the last, partial group of a row
                const float* src = x + gr * cols + gc;
                v.x = src[0];
                if (gc + 1 < cols) v.y = src[1];
                if (gc + 2 < cols) v.z = src[2];
            }
            const unsigned short b0 = toBf16Bits(v.x), b1 = toBf16Bits(v.y), b2 = toBf16Bits(v.z), b3 = toBf16Bits(v.w);
            tile[4 * cg + 0][r] = b0;
            tile[4 * cg + 1][r] = b1;
            tile[4 * cg + 2][r] = b2;
            tile[4 * cg + 3][r] = b3;
            if (plain && gr < rows && gc < colsPad) {   // ldPlain % 8 == 0 and gc % 4 == 0: an aligned 8-byte store
                uint2v packed = {unsigned(b0) | (unsigned(b1) << 16), unsigned(b2) | (unsigned(b3) << 16)};
                *reinterpret_cast<uint2v*>(plain + gr * ldPlain + gc) = packed;
            }
        }
        if (!out) return;   // (uniform) the plain image alone was asked for
        __syncthreads();
        const int chunk = threadIdx.x & 7, cc = threadIdx.x >> 3;   // 8 chunks of 8 rows x 32 columns per pass
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = cc + 32 * i;
            const size_t gc = c0 + c, gr = r0 + 8 * chunk;
            if (gc < cols && gr < rowsPad)    // rowsPad % 8 == 0: the whole chunk is in range
                *reinterpret_cast<uint4v*>(out + gc * rowsPad + gr) = *reinterpret_cast<const uint4v*>(&tile[c][8 * chunk]);
        }
        return;
    }
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;   // 64 x 4
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        int r = ty + 4 * i;
        size_t gr = r0 + r, gc = c0 + tx;
        const unsigned short b = (gr < rows && gc < cols) ? toBf16Bits(x[gr * cols + gc]) : (unsigned short)0;
        tile[tx][r] = b;
        if (plain && gr < rows && gc < colsPad) plain[gr * ldPlain + gc] = b;
    }
    if (!out) return;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        int c = ty + 4 * i;
        size_t gc = c0 + c, gr = r0 + tx;
        if (gc < cols && gr < rowsPad) out[gc * rowsPad + gr] = tile[c][tx];
    }
}
__global__ void __launch_bounds__(kBlock) convertTransposeKernel(ConvertSources xs, unsigned short* __restrict__ out,
                                                                 size_t rows, size_t cols, size_t rowsPad, int vec,
                                                                 unsigned short* __restrict__ plain, size_t ldPlain, size_t outStep,
                                                                 size_t plainStep) {
    __shared__ __attribute__((aligned(16))) unsigned short tile[64][72];   // [column][row], 144-byte pitch
    const float* __restrict__ x = blockIdx.z == 0 ? xs.p[0] : blockIdx.z == 1 ? xs.p[1] : xs.p[2];
    convertTransposeTile(x, out + blockIdx.z * outStep, rows, cols, rowsPad, vec, plain ? plain + blockIdx.z * plainStep : nullptr, ldPlain,
                         size_t(blockIdx.y) * 64, size_t(blockIdx.x) * 64, tile);
}

// The same conversion for a list of matrices of any shapes in one launch (every weight of a model after an optimizer
// step): the tiles of all matrices are laid end to end, a workgroup finds its matrix in the table (owningTensor) and
// its tile inside it, column tiles fastest.
struct ConvertEntry {
    const float* x;
    unsigned short* out;
    unsigned short* plain;
    unsigned rows, cols, rowsPad, ldPlain;
    unsigned firstBlock, tilesX;
    int vec;
    unsigned pad;
};
__global__ void __launch_bounds__(kBlock) convertTransposeMultiKernel(const ConvertEntry* __restrict__ table, int numEntries) {
    __shared__ __attribute__((aligned(16))) unsigned short tile[64][72];
    const ConvertEntry e = table[owningTensor(table, numEntries, blockIdx.x)];
    const unsigned local = blockIdx.x - e.firstBlock;
    const unsigned ty = local / e.tilesX, tx = local - ty * e.tilesX;
    convertTransposeTile(e.x, e.out, e.rows, e.cols, e.rowsPad, e.vec, e.plain, e.ldPlain, size_t(ty) * 64, size_t(tx) * 64, tile);
}

// ---- the GEMM ----------------------------------------------------------------------------------
// C[M,N] = A[M,K] * Bt[N,K]^T on 32x32x16 bf16 MFMAs.  Two kernels share the operand layout: LDS rows of
// 64 bf16 (one 128-byte line of the operand) padded by 16 bytes, so that the 16-byte fragment reads of a
// wavefront touch every bank once.  Rows past the end of an operand are clamped to its last row (their
// products are never stored) and chunks past the end of the K range read as zero, so neither kernel has
// a branch around a load.
thread_local int g_ntRoute = BF_GEMM_ROUTE_AUTO;   // per host thread
constexpr int BKK = 64;
constexpr int LDS_ROW = BKK + 8;

// A 16-byte chunk of an operand row at column k, or of column 0 when k is past the end of the K range: the
// caller replaces such a chunk by zeros when it consumes the register (zeroPast), not here, so that the load
// stays in flight across the phases in between.
__device__ __forceinline__ uint4v loadChunk(const unsigned short* __restrict__ row, int k, int kEnd) {
    return *reinterpret_cast<const uint4v*>(row + (k < kEnd ? k : 0));
}
__device__ __forceinline__ uint4v zeroPast(uint4v v, int k, int kEnd) {
    const uint4v z = {0u, 0u, 0u, 0u};
    return k < kEnd ? v : z;
}

// Walks tile rows in groups of 8, column-first inside a group, so tiles in flight share operand panels.
__device__ __forceinline__ void tileIndexGrouped(int id, int tilesM, int tilesN, int& tm, int& tn) {
    constexpr int GROUP = 8;
    const int perGroup = GROUP * tilesN;
    const int g = id / perGroup, rem = id - g * perGroup;
    const int rowsInGroup = min(GROUP, tilesM - g * GROUP);
    tm = g * GROUP + rem % rowsInGroup;
    tn = rem / rowsInGroup;
}

// Workgroups go round-robin to the 8 XCDs (id % 8), each with its own L2.  Here every XCD walks whole
// blocks of 2^gmLog x 2^gnLog = 32 tiles, one per CU, so the 32 tiles an XCD works on at a time share
// 2^gmLog + 2^gnLog operand panels in its L2 instead of 33.
__device__ __forceinline__ bool tileIndexXcd(int id, int tilesM, int tilesN, int gmLog, int gnLog, int& tm, int& tn) {
    const int x = id & 7, j = id >> 3;
    const int blocksN = (tilesN + (1 << gnLog) - 1) >> gnLog, blocksM = (tilesM + (1 << gmLog) - 1) >> gmLog;
    const int b = (j >> 5) * 8 + x, q = j & 31;
    if (b >= blocksM * blocksN) return false;
    const int bm = b / blocksN, bn = b - bm * blocksN;
    tm = (bm << gmLog) + (q & ((1 << gmLog) - 1));
    tn = (bn << gnLog) + (q >> gmLog);
    return tm < tilesM && tn < tilesN;
}

// Where a product goes.  The N columns are cut into runs of `splitN` that land in up to three separate
// [M, splitN] outputs (one GEMM for several projections of the same input; splitN is a multiple of the tile
// width, so a tile belongs to one output); a single output has splitN == N.  `bias` ([N]) and `residual`
// ([M, N], single output only) are added to the accumulator in that order before the store, the order in
// which the separate add kernels would have done it.
//
// A feed-forward block's activation fused into the store (`fuse`, single output, everything 16-byte aligned, N a
// multiple of 8; only the one-tile-per-workgroup wide-wave and ping-pong kernels take it):
//   fuse 1 (forward):  c[0] = acc + bias as usual, and image[row, col] = bf16(act(c[0][row, col])) beside it;
//   fuse 2 (backward): image[row, col] = bf16(acc * act'(actZ[row, col])) and nothing else: the fp32 product is never
//                      stored; colPartial[row / 32, col] = the sum of those products, before rounding, over the rows of
//                      a 32-row block (the bias gradient is the sum of these partial rows, in order).
struct Epilogue {
    float* c[3];
    int splitN;
    const float* bias;
    const float* residual;
    int fuse, act;
    unsigned short* image;   // [M, N]
    const float* actZ;       // [M, N]
    float* colPartial;       // [ceil(M / 32), N]
    // products of at most eight rows only (gemmBf16FewRowsKernel), A == NULL: the rows of A are those of rmsnorm(normInput)
    // ([M, K] fp32, dense) rounded to bf16, made while the kernel stages them
    const float* normInput;
    // the same kernel only: outputs c[1] and c[2] are written *rowShift rows further down, as long as the row stays below
    // rowLimit (a decoding step's new keys and values, placed at the cache's device-side length)
    const int* rowShift;
    int rowLimit;
};

// An accumulator tile of the 32x32 MFMA gives lane (li, half) column li of rows 8g + 4 half + 0..3 (g = 0..3).  Stored
// as they lie, the 64 lanes of a store instruction cover two rows of 128 bytes, 4 bytes a lane: a 256 x 256 tile takes
// 128 such instructions per lane, which costs a 768-long product a third of its time.  When everything is 16-byte aligned
// each quad of lanes first transposes its 4 x 4 blocks, so that a lane holds four consecutive columns of ONE row and stores
// them as 16 bytes: a quarter of the instructions, still whole 128-byte lines per row.
template <int TM, int TN>
__device__ __forceinline__ void storeAccumulators(float16v (&acc)[TM][TN], const Epilogue& e, int M, int N, int row0,
                                                  int col0, int li, int half) {
    const int which = col0 / e.splitN;              // uniform over the tile
    float* __restrict__ C = which == 0 ? e.c[0] : which == 1 ? e.c[1] : e.c[2];   // no indexed access: the struct stays in registers
    const int shift = which * e.splitN, ld = e.splitN;
    const bool wide = ((N | ld) & 3) == 0 &&
                      ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(e.bias) | reinterpret_cast<uintptr_t>(e.residual)) & 15u) == 0;
    if (wide) {
        const int t = li & 3, colq = 4 * (li >> 2);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int col = col0 + j * 32 + colq;
                float4v b = {0.0f, 0.0f, 0.0f, 0.0f};
                if (e.bias && col < N) b = loadf4(e.bias + col);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    float v0 = acc[i][j][4 * g], v1 = acc[i][j][4 * g + 1], v2 = acc[i][j][4 * g + 2], v3 = acc[i][j][4 * g + 3];
                    quadTranspose(v0, v1, v2, v3, t);
                    const int row = row0 + i * 32 + 8 * g + 4 * half + t;
                    if (row < M && col < N) {
                        float4v v = {v0, v1, v2, v3};
                        if (e.bias) v = v + b;
                        if (e.residual) v = v + loadf4(e.residual + size_t(row) * N + col);
                        storef4(C + size_t(row) * ld + (col - shift), v);
                    }
                }
            }
        return;
    }
    // One output of any width and alignment (an odd vocabulary): the same transposition, and the four columns of a lane as
    // one 16-byte access from whatever 4-byte boundary they start on (global memory serves those); the last group of a
    // row, which may hold fewer than four columns, goes element by element.
    if (ld == N && shift == 0) {
        const int t = li & 3, colq = 4 * (li >> 2);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int col = col0 + j * 32 + colq;
                const bool whole = col + 4 <= N;
                float b[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                if (e.bias) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) b[c] = col + c < N ? e.bias[col + c] : 0.0f;
                }
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    float v[4] = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    quadTranspose(v[0], v[1], v[2], v[3], t);
                    const int row = row0 + i * 32 + 8 * g + 4 * half + t;
                    if (row < M && col < N) {
                        float* dst = C + size_t(row) * N + col;
                        const float* res = e.residual ? e.residual + size_t(row) * N + col : nullptr;
                        if (e.bias) {   // the same additions, in the same order, as the other two forms
#pragma unroll
                            for (int c = 0; c < 4; ++c) v[c] += b[c];
                        }
                        if (whole) {
                            float4u out = {v[0], v[1], v[2], v[3]};
                            if (res) out = out + *reinterpret_cast<const float4u*>(res);
                            *reinterpret_cast<float4u*>(dst) = out;
                        } else {
#pragma unroll
                            for (int c = 0; c < 4; ++c)
                                if (col + c < N) dst[c] = res ? v[c] + res[c] : v[c];
                        }
                    }
                }
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = col0 + j * 32 + li;
            if (col < N) {
                const float b = e.bias ? e.bias[col] : 0.0f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = row0 + i * 32 + 8 * (r / 4) + 4 * half + (r % 4);
                    if (row < M) {
                        float v = acc[i][j][r];
                        if (e.bias) v += b;
                        if (e.residual) v += e.residual[size_t(row) * N + col];
                        C[size_t(row) * ld + (col - shift)] = v;
                    }
                }
            }
        }
}

__device__ __forceinline__ float4v actF4(int act, float4v v) {
    if (act == BF_ACT_SILU) return float4v{siluF(v.x), siluF(v.y), siluF(v.z), siluF(v.w)};
    if (act == BF_ACT_GELU) return float4v{geluF(v.x), geluF(v.y), geluF(v.z), geluF(v.w)};
    return float4v{reluF(v.x), reluF(v.y), reluF(v.z), reluF(v.w)};
}
__device__ __forceinline__ float4v actD4(int act, float4v v) {
    if (act == BF_ACT_SILU) return float4v{siluD(v.x), siluD(v.y), siluD(v.z), siluD(v.w)};
    if (act == BF_ACT_GELU) return float4v{geluD(v.x), geluD(v.y), geluD(v.z), geluD(v.w)};
    return float4v{reluD(v.x), reluD(v.y), reluD(v.z), reluD(v.w)};
}
__device__ __forceinline__ uint2v packBf16x4(float4v v) {
    return uint2v{unsigned(toBf16Bits(v.x)) | unsigned(toBf16Bits(v.y)) << 16, unsigned(toBf16Bits(v.z)) | unsigned(toBf16Bits(v.w)) << 16};
}

// The store with a fused activation (Epilogue::fuse = FUSE): the 16-byte form of storeAccumulators, a lane holding four
// consecutive columns of one row.  The values written are bit for bit those of the separate passes (the fp32 sum or
// product is the one they would have read back); the column sums of fuse 2 add the rows of a 32-row block in the order
// rows 8g (in the lane), then the four lanes of a quad, then the two halves of the wavefront.
// The image goes out in whole 128-byte lines: a wavefront's share is 64 columns wide (two accumulator blocks side by
// side), and neighbouring lanes (column groups q and q^1) trade one of their two packed groups, so that an even lane
// holds eight consecutive columns of the left block and an odd lane eight of the right one: one 16-byte store per lane
// and row instead of two 8-byte ones that each leave half a line to be merged (measured on 8192 x 3072: 16 us for the
// image stored in halves, as much as the fp32 tensor of twice its size).
template <int TM, int TN, int FUSE>
__device__ __forceinline__ void storeAccumulatorsFused(float16v (&acc)[TM][TN], const Epilogue& e, int M, int N, int row0, int col0,
                                                       int li, int half) {
    static_assert(TN == 2, "the image store pairs the two accumulator blocks of a 64-column share");
    const int t = li & 3, q = li >> 2, colq = 4 * q;
    const bool odd = (q & 1) != 0;
    // fuse 2 reads z where it writes the image: the 16-byte loads of a 32-row strip are issued one strip ahead of their
    // use (the image stores in between may alias them for all the compiler knows, so it would not move them itself)
    float4v zAhead[TM > 1 ? 2 : 1][2][4];
    auto fetchZ = [&](int i, float4v (&z)[2][4]) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int colIn = min(col0 + j * 32 + colq, N - 4);   // columns past the edge read the last ones: no branch around a load
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int row = min(row0 + i * 32 + 8 * g + 4 * half + t, M - 1);
                z[j][g] = __builtin_nontemporal_load(reinterpret_cast<const float4v*>(e.actZ + size_t(row) * N + colIn));
            }
        }
    };
    if constexpr (FUSE == 2) fetchZ(0, zAhead[0]);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        if constexpr (FUSE == 2 && TM > 1) {
            if (i + 1 < TM) fetchZ(i + 1, zAhead[(i + 1) & 1]);
        }
        float4v b[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
        if (FUSE == 1 && e.bias) {
            b[0] = loadf4(e.bias + min(col0 + colq, N - 4));
            b[1] = loadf4(e.bias + min(col0 + 32 + colq, N - 4));
        }
        float4v sums[2] = {{0.0f, 0.0f, 0.0f, 0.0f}, {0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int row = row0 + i * 32 + 8 * g + 4 * half + t;
            uint2v packed[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                float v0 = acc[i][j][4 * g], v1 = acc[i][j][4 * g + 1], v2 = acc[i][j][4 * g + 2], v3 = acc[i][j][4 * g + 3];
                quadTranspose(v0, v1, v2, v3, t);
                const int col = col0 + j * 32 + colq;
                const bool inside = row < M && col < N;
                float4v v = {v0, v1, v2, v3};
                if constexpr (FUSE == 1) {
                    if (e.bias) v = v + b[j];
                    if (inside) storef4(e.c[0] + size_t(row) * N + col, v);
                    packed[j] = packBf16x4(actF4(e.act, v));
                } else {
                    v = v * actD4(e.act, zAhead[TM > 1 ? (i & 1) : 0][j][g]);
                    if (inside) sums[j] = sums[j] + v;
                    packed[j] = packBf16x4(v);
                }
            }
            // an even lane sends its right-block group and receives the left-block group of the odd lane beside it
            const uint2v send = odd ? packed[0] : packed[1];
            const uint2v recv = {unsigned(__shfl_xor(int(send.x), 4, 64)), unsigned(__shfl_xor(int(send.y), 4, 64))};
            const uint4v line = odd ? uint4v{recv.x, recv.y, packed[1].x, packed[1].y} : uint4v{packed[0].x, packed[0].y, recv.x, recv.y};
            const int ocol = odd ? col0 + 32 + colq - 4 : col0 + colq;   // a multiple of 8, like N: the eight columns are inside or outside together
            if (row < M && ocol < N) *reinterpret_cast<uint4v*>(e.image + size_t(row) * N + ocol) = line;
        }
        if constexpr (FUSE == 2) {
            if (e.colPartial) {
                const int blockRow = row0 + i * 32;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        float x = sums[j][c];
                        x += quadXor1(x);
                        x += quadXor2(x);
                        x += __shfl_xor(x, 32, 64);
                        sums[j][c] = x;
                    }
                    const int col = col0 + j * 32 + colq;
                    if (t == 0 && half == 0 && blockRow < M && col < N) storef4(e.colPartial + size_t(blockRow >> 5) * N + col, sums[j]);
                }
            }
        }
    }
}

// Kernel for small tile counts: a workgroup of WAVES_M x WAVES_N wavefronts owns a BM x BN tile, K advances
// in steps of 64 through a double-buffered LDS stage with one barrier per step (while step t is multiplied
// out of buffer t&1, the registers holding step t+1 go to the other buffer and the loads of step t+2 are
// issued).  Several workgroups fit on a CU and cover each other's barriers and epilogues.
// blockIdx.y selects a slice of K (split-K): slice s covers [s*kPerSplit, (s+1)*kPerSplit) and writes its
// partial product to C + s*sliceStride.
template <int BM, int BN, int WAVES_M, int WAVES_N>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64) gemmBf16NtKernel(const unsigned short* __restrict__ A,
                                                                            const unsigned short* __restrict__ Bt,
                                                                            Epilogue epi, int M, int N, int K, int lda,
                                                                            int ldb, int kPerSplit, size_t sliceStride) {
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
    int tm, tn;
    tileIndexGrouped(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int kBegin = blockIdx.y * kPerSplit, kEnd = min(K, kBegin + kPerSplit);
    epi.c[0] += size_t(blockIdx.y) * sliceStride;   // slices are only used with a single plain output

    const int lr = tid >> 3, lc = (tid & 7) * 8;
    const unsigned short* aRow[A_PASSES];
    const unsigned short* bRow[B_PASSES];
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) aRow[i] = A + size_t(min(m0 + lr + ROWS_PER_PASS * i, M - 1)) * lda;
#pragma unroll
    for (int i = 0; i < B_PASSES; ++i) bRow[i] = Bt + size_t(min(n0 + lr + ROWS_PER_PASS * i, N - 1)) * ldb;
    uint4v aReg[A_PASSES], bReg[B_PASSES];
    auto loadGlobal = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i) aReg[i] = loadChunk(aRow[i], k0 + lc, kEnd);
#pragma unroll
        for (int i = 0; i < B_PASSES; ++i) bReg[i] = loadChunk(bRow[i], k0 + lc, kEnd);
    };
    auto storeLds = [&](int buf, int k0) {   // k0: K offset of the step held in the registers
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i)
            *reinterpret_cast<uint4v*>(as + (buf * BM + lr + ROWS_PER_PASS * i) * LDS_ROW + lc) = zeroPast(aReg[i], k0 + lc, kEnd);
#pragma unroll
        for (int i = 0; i < B_PASSES; ++i)
            *reinterpret_cast<uint4v*>(bs + (buf * BN + lr + ROWS_PER_PASS * i) * LDS_ROW + lc) = zeroPast(bReg[i], k0 + lc, kEnd);
    };

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    const int steps = (kEnd - kBegin + BKK - 1) / BKK;   // <= 0 for an empty slice: stores zeros
    if (steps > 0) {
        loadGlobal(kBegin);
        storeLds(0, kBegin);
        if (steps > 1) loadGlobal(kBegin + BKK);
    }
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
            storeLds((t + 1) & 1, kBegin + (t + 1) * BKK);
            if (t + 2 < steps) loadGlobal(kBegin + (t + 2) * BKK);
        }
        __syncthreads();
    }
    storeAccumulators<TM, TN>(acc, epi, M, N, m0 + wm0, n0 + wn0, li, half);
}

// Kernel for large products: 256 x 256 tile, 8 wavefronts in two groups of four.  Wavefronts w and w+4 of
// a workgroup share a SIMD, so each SIMD holds one wavefront of either group.  A K step of 64 is worked
// in two halves; each half has a memory phase (read the 12 operand fragments of the half step from LDS,
// write one staged operand of the next step to the other LDS buffer, issue that operand's global loads for
// the step after) and a compute phase (16 MFMAs out of registers).  A barrier ends every phase and group 1
// runs one phase behind group 0: on every SIMD one wavefront multiplies while the other moves data.
//   phase of group 0:  M(T,0) C(T,0) M(T,1) C(T,1) M(T+1,0) ...
//   phase of group 1:     -   M(T,0) C(T,0) M(T,1) C(T,1)   ...
// Buffer (T+1)&1 is written during the four phases after its last reader (group 1's M(T-1,1)) has passed a
// barrier and before its first reader (group 0's M(T+1,0)) starts, and a global load has four phases to land.
// Operand A is staged in the first half step and Bt in the second, so every load instruction still fetches
// whole 128-byte lines.
// BM = 256, or 128 for products whose 256-row tiles would leave compute units without one (or with a nearly empty
// second round): half the rows per workgroup, the same eight wavefronts, each with a 64 x 64 share instead of 128 x 64.
// The memory phase then moves 8 fragments for 8 MFMAs instead of 12 for 16, so a tile costs more than half of a full
// one; it pays when it fills the chip.
template <int XCD_ORDER, int BM, int FUSE = 0>
__global__ void __launch_bounds__(512, 2) gemmBf16PingPongKernel(const unsigned short* __restrict__ A,
                                                                 const unsigned short* __restrict__ Bt, Epilogue epi,
                                                                 int M, int N, int K, int lda, int ldb, int gmLog, int gnLog,
                                                                 int kPerSplit, size_t sliceStride) {
    constexpr int BN = 256, TM = BM / 64, TN = 2, A_PASSES = BM / 64;
    extern __shared__ __attribute__((aligned(16))) unsigned short lds[];
    unsigned short* as = lds;                        // [2][BM][LDS_ROW]
    unsigned short* bs = lds + 2 * BM * LDS_ROW;     // [2][256][LDS_ROW]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    const int group = wave >> 2;
    int tm, tn;
    if (XCD_ORDER) {
        if (!tileIndexXcd(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, gmLog, gnLog, tm, tn)) return;
    } else {
        tileIndexGrouped(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, tm, tn);
    }
    const int m0 = tm * BM, n0 = tn * BN;
    const int wm0 = group * (BM / 2), wn0 = (wave & 3) * 64;
    const int lr = tid >> 3, lc = (tid & 7) * 8;     // 64 rows x 128 bytes per pass
    const unsigned short* aRow[A_PASSES];
    const unsigned short* bRow[4];
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) aRow[i] = A + size_t(min(m0 + lr + 64 * i, M - 1)) * lda;
#pragma unroll
    for (int i = 0; i < 4; ++i) bRow[i] = Bt + size_t(min(n0 + lr + 64 * i, N - 1)) * ldb;
    uint4v stageA[A_PASSES], stageB[4];
    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    // blockIdx.y selects a slice of K, as in the small-tile kernel: partial products go to C + slice * sliceStride
    const int kBegin = blockIdx.y * kPerSplit, kEnd = min(K, kBegin + kPerSplit);
    epi.c[0] += size_t(blockIdx.y) * sliceStride;
    const int steps = max((kEnd - kBegin + BKK - 1) / BKK, 1);   // an empty slice runs one step of zeros
    const int ldsW = lr * LDS_ROW + lc;
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) stageA[i] = loadChunk(aRow[i], kBegin + lc, kEnd);
#pragma unroll
    for (int i = 0; i < 4; ++i) stageB[i] = loadChunk(bRow[i], kBegin + lc, kEnd);
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) *reinterpret_cast<uint4v*>(as + ldsW + 64 * i * LDS_ROW) = zeroPast(stageA[i], kBegin + lc, kEnd);
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4v*>(bs + ldsW + 64 * i * LDS_ROW) = zeroPast(stageB[i], kBegin + lc, kEnd);
    if (steps > 1) {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i) stageA[i] = loadChunk(aRow[i], kBegin + BKK + lc, kEnd);
#pragma unroll
        for (int i = 0; i < 4; ++i) stageB[i] = loadChunk(bRow[i], kBegin + BKK + lc, kEnd);
    }
    __syncthreads();
    if (group == 1) __builtin_amdgcn_s_barrier();    // group 1 starts one phase late
    bf16x8 a[2][TM], b[2][TN];
    for (int T = 0; T < steps; ++T) {
        const int par = T & 1;
        const unsigned short* ac = as + (par * BM + wm0 + li) * LDS_ROW + 8 * half;
        const unsigned short* bc = bs + (par * BN + wn0 + li) * LDS_ROW + 8 * half;
        unsigned short* aw = as + (par ^ 1) * BM * LDS_ROW + ldsW;
        unsigned short* bw = bs + (par ^ 1) * BN * LDS_ROW + ldsW;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            // ---- memory phase
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
                for (int i = 0; i < TM; ++i) a[kk][i] = *reinterpret_cast<const bf16x8*>(ac + i * 32 * LDS_ROW + h * 32 + kk * 16);
#pragma unroll
                for (int j = 0; j < TN; ++j) b[kk][j] = *reinterpret_cast<const bf16x8*>(bc + j * 32 * LDS_ROW + h * 32 + kk * 16);
            }
            if (T + 1 < steps) {
                if (h == 0) {
#pragma unroll
                    for (int i = 0; i < A_PASSES; ++i) *reinterpret_cast<uint4v*>(aw + 64 * i * LDS_ROW) = zeroPast(stageA[i], kBegin + (T + 1) * BKK + lc, kEnd);
                    if (T + 2 < steps) {
#pragma unroll
                        for (int i = 0; i < A_PASSES; ++i) stageA[i] = loadChunk(aRow[i], kBegin + (T + 2) * BKK + lc, kEnd);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4v*>(bw + 64 * i * LDS_ROW) = zeroPast(stageB[i], kBegin + (T + 1) * BKK + lc, kEnd);
                    if (T + 2 < steps) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) stageB[i] = loadChunk(bRow[i], kBegin + (T + 2) * BKK + lc, kEnd);
                    }
                }
            }
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            // ---- compute phase
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kk][i], b[kk][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
        }
    }
    if (group == 0) __builtin_amdgcn_s_barrier();    // pairs with group 1's last barrier
    if constexpr (FUSE != 0) storeAccumulatorsFused<TM, TN, FUSE>(acc, epi, M, N, m0 + wm0, n0 + wn0, li, half);
    else storeAccumulators<TM, TN>(acc, epi, M, N, m0 + wm0, n0 + wn0, li, half);
}

// 128-row tiles on twelve or sixteen wavefronts (three or four per SIMD, each with a 32 x 64 share: tiles 192 or 256
// wide), one barrier per K step: while step T is multiplied out of LDS buffer T&1 (fragments of the next 16-deep slice are
// read while the current one is multiplied), the registers holding step T+1 go to the other buffer and the loads of step
// T+2 are issued.  The K loop costs what the eight-wavefront ping-pong costs for a tile of this size (the LDS pipe bounds
// both), but filling and draining it does not: all wavefronts fetch the first step and store the tile together, and no
// group waits a phase for the other.  Products with a short contraction, whose tiles live for twenty microseconds, are
// several microseconds faster per round of tiles; long contractions stay on the 256-row ping-pong kernel, which moves
// fewer operand bytes per MFMA.  The 192-wide form is for widths that 256 does not divide into whole rounds of tiles:
// 768 columns are 3 tiles of 256 (192 tiles for 8192 rows, three quarters of the compute units) or 4 of 192 (256 tiles).
// The 128 + BN operand rows of a K step are staged as one run of rows, 32 * WAVES_N per pass, A first.
template <int XCD_ORDER, int WAVES_N, int FUSE = 0>
__global__ void __launch_bounds__(256 * WAVES_N, WAVES_N) gemmBf16WideWaveKernel(const unsigned short* __restrict__ A,
                                                                                 const unsigned short* __restrict__ Bt, Epilogue epi,
                                                                                 int M, int N, int K, int lda, int ldb, int gmLog,
                                                                                 int gnLog) {
    constexpr int BM = 128, BN = 64 * WAVES_N, TM = 1, TN = 2;
    constexpr int ROWS = BM + BN, ROWS_PER_PASS = 32 * WAVES_N, PASSES = (ROWS + ROWS_PER_PASS - 1) / ROWS_PER_PASS;
    constexpr int LAST_ROWS = ROWS - (PASSES - 1) * ROWS_PER_PASS;   // rows of the last pass (the pass is whole waves: 32 rows = 4 waves)
    static_assert(LAST_ROWS % 8 == 0, "the threads of the last pass must be whole wavefronts");
    extern __shared__ __attribute__((aligned(16))) unsigned short lds[];   // [2][ROWS][LDS_ROW]: A rows, then Bt rows
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    int tm, tn;
    if (XCD_ORDER) {
        if (!tileIndexXcd(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, gmLog, gnLog, tm, tn)) return;
    } else {
        tileIndexGrouped(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, tm, tn);
    }
    const int m0 = tm * BM, n0 = tn * BN;
    const int wm0 = (wave & 3) * 32, wn0 = (wave >> 2) * 64;
    const int lr = tid >> 3, lc = (tid & 7) * 8;     // ROWS_PER_PASS rows x 128 bytes per pass
    const bool lastPass = LAST_ROWS == ROWS_PER_PASS || lr < LAST_ROWS;   // uniform over a wavefront
    const unsigned short* src[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const int row = min(lr + ROWS_PER_PASS * p, ROWS - 1);
        src[p] = row < BM ? A + size_t(min(m0 + row, M - 1)) * lda : Bt + size_t(min(n0 + row - BM, N - 1)) * ldb;
    }
    float16v acc[TM][TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[0][j][r] = 0.0f;
    const int steps = max((K + BKK - 1) / BKK, 1);
    const int ldsW = lr * LDS_ROW + lc;
    uint4v stage[PASSES];
    auto loadStep = [&](int k) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            if (p + 1 < PASSES || lastPass) stage[p] = loadChunk(src[p], k, K);
    };
    auto storeStep = [&](int buf, int k) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            if (p + 1 < PASSES || lastPass)
                *reinterpret_cast<uint4v*>(lds + (buf * ROWS + ROWS_PER_PASS * p) * LDS_ROW + ldsW) = zeroPast(stage[p], k, K);
    };
    loadStep(lc);
    storeStep(0, lc);
    if (steps > 1) loadStep(BKK + lc);
    __syncthreads();
    bf16x8 a[2], b[2][TN];
    for (int T = 0; T < steps; ++T) {
        const int par = T & 1;
        const unsigned short* ac = lds + (par * ROWS + wm0 + li) * LDS_ROW + 8 * half;
        const unsigned short* bc = lds + (par * ROWS + BM + wn0 + li) * LDS_ROW + 8 * half;
        if (T + 1 < steps) {
            const int kNext = (T + 1) * BKK + lc;
            storeStep(par ^ 1, kNext);
            if (T + 2 < steps) loadStep(kNext + BKK);
        }
        a[0] = *reinterpret_cast<const bf16x8*>(ac);
#pragma unroll
        for (int j = 0; j < TN; ++j) b[0][j] = *reinterpret_cast<const bf16x8*>(bc + j * 32 * LDS_ROW);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            if (kk < 3) {
                a[(kk + 1) & 1] = *reinterpret_cast<const bf16x8*>(ac + (kk + 1) * 16);
#pragma unroll
                for (int j = 0; j < TN; ++j) b[(kk + 1) & 1][j] = *reinterpret_cast<const bf16x8*>(bc + j * 32 * LDS_ROW + (kk + 1) * 16);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kk & 1], b[kk & 1][j], acc[0][j], 0, 0, 0);
        }
        __syncthreads();
    }
    if constexpr (FUSE != 0) storeAccumulatorsFused<TM, TN, FUSE>(acc, epi, M, N, m0 + wm0, n0 + wn0, li, half);
    else storeAccumulators<TM, TN>(acc, epi, M, N, m0 + wm0, n0 + wn0, li, half);
}

// The next tile this workgroup owns at or after `id`, walking in steps of `stride`; -1 past the end.  With the XCD order
// some ids name no tile (the padding of a block of 32) and are skipped.
template <int XCD_ORDER>
__device__ __forceinline__ int seekTile(int id, int stride, int idEnd, int tilesM, int tilesN, int gmLog, int gnLog, int& tm, int& tn) {
    for (; id < idEnd; id += stride) {
        if (XCD_ORDER) {
            if (tileIndexXcd(id, tilesM, tilesN, gmLog, gnLog, tm, tn)) return id;
        } else {
            tileIndexGrouped(id, tilesM, tilesN, tm, tn);
            return id;
        }
    }
    return -1;
}

// One eighth of a 32 x 64 accumulator share (chunk C = registers 4*(C&3).. of acc[C>>2]: rows 8*(C&3) + 4*half + 0..3),
// stored the way storeAccumulators stores 16-byte aligned outputs.  `adds` holds this lane's four bias and residual values
// of the chunk, loaded by the caller ahead of time.
struct ChunkAdds { float4v b, res; };
template <int C>
__device__ __forceinline__ void loadChunkAdds(ChunkAdds& adds, const Epilogue& e, int M, int N, int row0, int col0, int li, int half) {
    const int t = li & 3, col = col0 + (C >> 2) * 32 + 4 * (li >> 2), row = row0 + 8 * (C & 3) + 4 * half + t;
    // rows and columns past the edge read the last ones (their sums are never stored): no branch around a load
    const int rowIn = min(row, M - 1), colIn = min(col, N - 4);
    if (e.bias) adds.b = loadf4(e.bias + colIn);
    if (e.residual) adds.res = loadf4(e.residual + size_t(rowIn) * N + colIn);
}
// Cout / shift: the output the tile's columns belong to and the column where that output starts (uniform over a tile).
template <int C, bool ADDS>
__device__ __forceinline__ void storeChunk(const float16v (&acc)[2], const ChunkAdds& adds, const Epilogue& e, float* __restrict__ Cout,
                                           int shift, int M, int N, int row0, int col0, int li, int half) {
    constexpr int j = C >> 2, g = C & 3;
    const int ld = e.splitN;
    const int t = li & 3, colq = 4 * (li >> 2);
    float v0 = acc[j][4 * g], v1 = acc[j][4 * g + 1], v2 = acc[j][4 * g + 2], v3 = acc[j][4 * g + 3];
    quadTranspose(v0, v1, v2, v3, t);
    const int row = row0 + 8 * g + 4 * half + t, col = col0 + j * 32 + colq;
    float4v v = {v0, v1, v2, v3};
    if constexpr (ADDS) {
        if (e.bias) v = v + adds.b;
        if (e.residual) v = v + adds.res;
    }
    // Everything but the store itself sits outside the condition: a one-instruction body is predicated, not branched
    // around, and a store that every path issues lets the compiler count it when it waits for the loads around it
    // (a store on one path only would make it wait for ALL outstanding memory operations, this store included).
    float* dst = Cout + size_t(min(row, M - 1)) * ld + (min(col, N - 4) - shift);
    if (row < M && col < N) storef4(dst, v);
}

// The sixteen- (twelve-) wavefront kernel as ONE workgroup per compute unit that walks a list of tiles (ids blockIdx.x,
// blockIdx.x + gridDim.x, ...).  The K steps of all its tiles form one pipeline: while step g is multiplied, step g+1
// is written to the other LDS buffer and step g+2 is loaded, whichever tile those belong to, so a tile's first steps are
// already in flight while the tile before is still being multiplied.  A wavefront's share is only 32 registers of
// accumulators, so it keeps the finished tile's share in a second set and stores it one eighth per K step of the next
// tile, between the MFMAs; bias and residual values of an eighth (ADDS) are fetched at the start of the K step that
// stores it.  Nothing of a tile's fill, drain or store is left outside the MFMA stream except for the first and the last
// tile of a workgroup.  Outputs must be 16-byte aligned with widths that are multiples of 4 (the launcher checks).
// Every output element sees the same MFMAs in the same order as in gemmBf16WideWaveKernel: the same bits.
template <int XCD_ORDER, int WAVES_N, bool ADDS>
__global__ void __launch_bounds__(256 * WAVES_N, WAVES_N) gemmBf16WidePersistentKernel(const unsigned short* __restrict__ A,
                                                                                       const unsigned short* __restrict__ Bt, Epilogue epi,
                                                                                       int M, int N, int K, int lda, int ldb, int gmLog,
                                                                                       int gnLog, int idEnd) {
    constexpr int BM = 128, BN = 64 * WAVES_N, TN = 2;
    constexpr int ROWS = BM + BN, ROWS_PER_PASS = 32 * WAVES_N, PASSES = (ROWS + ROWS_PER_PASS - 1) / ROWS_PER_PASS;
    constexpr int LAST_ROWS = ROWS - (PASSES - 1) * ROWS_PER_PASS;
    static_assert(LAST_ROWS % 8 == 0, "the threads of the last pass must be whole wavefronts");
    extern __shared__ __attribute__((aligned(16))) unsigned short lds[];   // [2][ROWS][LDS_ROW]: A rows, then Bt rows
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    const int tilesM = (M + BM - 1) / BM, tilesN = (N + BN - 1) / BN, stride = gridDim.x;
    const int wm0 = (wave & 3) * 32, wn0 = (wave >> 2) * 64;
    const int lr = tid >> 3, lc = (tid & 7) * 8;
    const bool lastPass = LAST_ROWS == ROWS_PER_PASS || lr < LAST_ROWS;   // uniform over a wavefront
    const int steps = max((K + BKK - 1) / BKK, 1);
    int myTiles = 0;
    {
        int tm, tn;
        for (int id = seekTile<XCD_ORDER>(blockIdx.x, stride, idEnd, tilesM, tilesN, gmLog, gnLog, tm, tn); id >= 0;
             id = seekTile<XCD_ORDER>(id + stride, stride, idEnd, tilesM, tilesN, gmLog, gnLog, tm, tn))
            ++myTiles;
    }
    if (myTiles == 0) return;
    const int total = myTiles * steps;   // K steps of all this workgroup's tiles

    // the load side of the pipeline: (tile, K step) of the next loads, two steps ahead of the MFMAs
    int ldTm, ldTn, ldT = 0;
    int ldId = seekTile<XCD_ORDER>(blockIdx.x, stride, idEnd, tilesM, tilesN, gmLog, gnLog, ldTm, ldTn);
    const unsigned short* src[PASSES];
    auto setSources = [&]() {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int row = min(lr + ROWS_PER_PASS * p, ROWS - 1);
            src[p] = row < BM ? A + size_t(min(ldTm * BM + row, M - 1)) * lda : Bt + size_t(min(ldTn * BN + row - BM, N - 1)) * ldb;
        }
    };
    setSources();
    uint4v stage[PASSES];
    int kStaged = 0;   // K offset (this thread's chunk) of the step the stage registers hold
    auto loadStep = [&]() {
        kStaged = ldT * BKK + lc;
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            if (p + 1 < PASSES || lastPass) stage[p] = loadChunk(src[p], kStaged, K);
        if (++ldT == steps) {
            ldT = 0;
            ldId = seekTile<XCD_ORDER>(ldId + stride, stride, idEnd, tilesM, tilesN, gmLog, gnLog, ldTm, ldTn);
            if (ldId >= 0) setSources();
        }
    };
    const int ldsW = lr * LDS_ROW + lc;
    auto storeStep = [&](int buf) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            if (p + 1 < PASSES || lastPass)
                *reinterpret_cast<uint4v*>(lds + (buf * ROWS + ROWS_PER_PASS * p) * LDS_ROW + ldsW) = zeroPast(stage[p], kStaged, K);
    };

    float16v acc[TN], done[TN];   // the tile being multiplied; the finished tile whose store is in progress
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) { acc[j][r] = 0.0f; done[j][r] = 0.0f; }
    int doneRow0 = 0, doneCol0 = 0, doneShift = 0;
    float* doneOut = epi.c[0];
    ChunkAdds adds;
    adds.b = float4v{0.0f, 0.0f, 0.0f, 0.0f};
    adds.res = adds.b;
    bf16x8 a[2], b[2][TN];
    int g = 0;
    // one K step: C >= 0 also stores chunk C of the finished tile
    auto step = [&](auto chunkTag) {
        constexpr int C = decltype(chunkTag)::value;
        const int par = g & 1;
        const unsigned short* ac = lds + (par * ROWS + wm0 + li) * LDS_ROW + 8 * half;
        const unsigned short* bc = lds + (par * ROWS + BM + wn0 + li) * LDS_ROW + 8 * half;
        if constexpr (C >= 0 && ADDS) {
            loadChunkAdds<C>(adds, epi, M, N, doneRow0, doneCol0, li, half);
            __builtin_amdgcn_sched_barrier(0);   // the chunk's loads stay ahead of the step's: its wait leaves those in flight
        }
        if (g + 1 < total) {
            storeStep(par ^ 1);
            if (g + 2 < total) loadStep();
        }
        a[0] = *reinterpret_cast<const bf16x8*>(ac);
#pragma unroll
        for (int j = 0; j < TN; ++j) b[0][j] = *reinterpret_cast<const bf16x8*>(bc + j * 32 * LDS_ROW);
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            if (kk < 3) {
                a[(kk + 1) & 1] = *reinterpret_cast<const bf16x8*>(ac + (kk + 1) * 16);
#pragma unroll
                for (int j = 0; j < TN; ++j) b[(kk + 1) & 1][j] = *reinterpret_cast<const bf16x8*>(bc + j * 32 * LDS_ROW + (kk + 1) * 16);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kk & 1], b[kk & 1][j], acc[j], 0, 0, 0);
        }
        if constexpr (C >= 0) storeChunk<C, ADDS>(done, adds, epi, doneOut, doneShift, M, N, doneRow0, doneCol0, li, half);
        __syncthreads();
        ++g;
    };
    auto chunkAlone = [&](auto chunkTag) {
        constexpr int C = decltype(chunkTag)::value;
        if constexpr (ADDS) loadChunkAdds<C>(adds, epi, M, N, doneRow0, doneCol0, li, half);
        storeChunk<C, ADDS>(done, adds, epi, doneOut, doneShift, M, N, doneRow0, doneCol0, li, half);
    };
    // the first eight K steps of a tile carry the eight chunks of the tile before (a shorter contraction stores the rest at once)
    auto stepsWithChunks = [&](int& T) {
#define BF_CHUNK_STEP(C)                                              \
        if (T < steps) { step(std::integral_constant<int, C>{}); ++T; } \
        else chunkAlone(std::integral_constant<int, C>{});
        BF_CHUNK_STEP(0) BF_CHUNK_STEP(1) BF_CHUNK_STEP(2) BF_CHUNK_STEP(3)
        BF_CHUNK_STEP(4) BF_CHUNK_STEP(5) BF_CHUNK_STEP(6) BF_CHUNK_STEP(7)
#undef BF_CHUNK_STEP
    };

    loadStep();
    storeStep(0);
    if (total > 1) loadStep();
    __syncthreads();
    int curTm, curTn;
    int curId = seekTile<XCD_ORDER>(blockIdx.x, stride, idEnd, tilesM, tilesN, gmLog, gnLog, curTm, curTn);
    for (int tile = 0; tile < myTiles; ++tile) {
        int T = 0;
        if (tile > 0) stepsWithChunks(T);
        for (; T < steps; ++T) step(std::integral_constant<int, -1>{});
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            done[j] = acc[j];
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[j][r] = 0.0f;
        }
        doneRow0 = curTm * BM + wm0;
        doneCol0 = curTn * BN + wn0;
        {
            const int which = (curTn * BN) / epi.splitN;   // a tile lies in one output
            doneOut = which == 0 ? epi.c[0] : which == 1 ? epi.c[1] : epi.c[2];
            doneShift = which * epi.splitN;
        }
        curId = seekTile<XCD_ORDER>(curId + stride, stride, idEnd, tilesM, tilesN, gmLog, gnLog, curTm, curTn);
    }
    chunkAlone(std::integral_constant<int, 0>{}); chunkAlone(std::integral_constant<int, 1>{});
    chunkAlone(std::integral_constant<int, 2>{}); chunkAlone(std::integral_constant<int, 3>{});
    chunkAlone(std::integral_constant<int, 4>{}); chunkAlone(std::integral_constant<int, 5>{});
    chunkAlone(std::integral_constant<int, 6>{}); chunkAlone(std::integral_constant<int, 7>{});
}

// storeAccumulators for 16-byte aligned outputs with no branch around a memory instruction (clamped addresses, the
// store alone under its condition): inside a kernel that keeps loads in flight across the store, the compiler can then
// count every store when it waits for those loads instead of waiting for all memory operations.  Same values, same order
// of additions.
template <int TM, int TN>
__device__ __forceinline__ void storeAccumulatorsFlat(float16v (&acc)[TM][TN], const Epilogue& e, float* __restrict__ C, int shift,
                                                      int M, int N, int row0, int col0, int li, int half) {
    const int ld = e.splitN;
    const int t = li & 3, colq = 4 * (li >> 2);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = col0 + j * 32 + colq, colIn = min(col, N - 4);
            float4v b = {0.0f, 0.0f, 0.0f, 0.0f};
            if (e.bias) b = loadf4(e.bias + colIn);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float v0 = acc[i][j][4 * g], v1 = acc[i][j][4 * g + 1], v2 = acc[i][j][4 * g + 2], v3 = acc[i][j][4 * g + 3];
                quadTranspose(v0, v1, v2, v3, t);
                const int row = row0 + i * 32 + 8 * g + 4 * half + t, rowIn = min(row, M - 1);
                float4v v = {v0, v1, v2, v3};
                if (e.bias) v = v + b;
                if (e.residual) v = v + loadf4(e.residual + size_t(rowIn) * N + colIn);
                float* dst = C + size_t(rowIn) * ld + (colIn - shift);
                if (row < M && col < N) storef4(dst, v);
            }
        }
}

// The ping-pong kernel as one workgroup per compute unit walking a list of tiles, with the K steps of all its tiles as ONE
// pipeline: the loads of a tile's first two K steps are issued, and its first step written to LDS, while the tile
// before is still being multiplied, and the two groups of wavefronts keep their one-phase offset across tile boundaries,
// so a group stores its accumulators while the other group multiplies.  A tile costs its K loop plus the store's issue
// time; the workgroup launch, the first loads' latency and the pipeline's fill and drain are paid once per workgroup.
// Same MFMAs in the same order per output element as gemmBf16PingPongKernel: the same bits.
template <int XCD_ORDER, int BM>
__global__ void __launch_bounds__(512, 2) gemmBf16PingPongPersistentKernel(const unsigned short* __restrict__ A,
                                                                           const unsigned short* __restrict__ Bt, Epilogue epi,
                                                                           int M, int N, int K, int lda, int ldb, int gmLog, int gnLog,
                                                                           int idEnd) {
    constexpr int BN = 256, TM = BM / 64, TN = 2, A_PASSES = BM / 64;
    extern __shared__ __attribute__((aligned(16))) unsigned short lds[];
    unsigned short* as = lds;                        // [2][BM][LDS_ROW]
    unsigned short* bs = lds + 2 * BM * LDS_ROW;     // [2][256][LDS_ROW]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    const int group = wave >> 2;
    const int tilesM = (M + BM - 1) / BM, tilesN = (N + BN - 1) / BN, stride = gridDim.x;
    const int wm0 = group * (BM / 2), wn0 = (wave & 3) * 64;
    const int lr = tid >> 3, lc = (tid & 7) * 8;     // 64 rows x 128 bytes per pass
    const int steps = max((K + BKK - 1) / BKK, 1);
    int myTiles = 0;
    {
        int tm, tn;
        for (int id = seekTile<XCD_ORDER>(blockIdx.x, stride, idEnd, tilesM, tilesN, gmLog, gnLog, tm, tn); id >= 0;
             id = seekTile<XCD_ORDER>(id + stride, stride, idEnd, tilesM, tilesN, gmLog, gnLog, tm, tn))
            ++myTiles;
    }
    if (myTiles == 0) return;
    const int total = myTiles * steps;
    const bool wideStores = ((N | epi.splitN) & 3) == 0 &&
                            ((reinterpret_cast<uintptr_t>(epi.c[0]) | reinterpret_cast<uintptr_t>(epi.c[1]) | reinterpret_cast<uintptr_t>(epi.c[2]) |
                              reinterpret_cast<uintptr_t>(epi.bias) | reinterpret_cast<uintptr_t>(epi.residual)) & 15u) == 0;

    int ldTm, ldTn, ldT = 0;
    int ldId = seekTile<XCD_ORDER>(blockIdx.x, stride, idEnd, tilesM, tilesN, gmLog, gnLog, ldTm, ldTn);
    const unsigned short* aRow[A_PASSES];
    const unsigned short* bRow[4];
    auto setSources = [&]() {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i) aRow[i] = A + size_t(min(ldTm * BM + lr + 64 * i, M - 1)) * lda;
#pragma unroll
        for (int i = 0; i < 4; ++i) bRow[i] = Bt + size_t(min(ldTn * BN + lr + 64 * i, N - 1)) * ldb;
    };
    setSources();
    uint4v stageA[A_PASSES], stageB[4];
    int kA = 0, kB = 0;   // K offsets (this thread's chunk) of the steps the stage registers hold
    auto loadA = [&]() {
        kA = ldT * BKK + lc;
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i) stageA[i] = loadChunk(aRow[i], kA, K);
    };
    auto loadB = [&]() {   // the second operand of a step: the load side then moves on to the next step
        kB = ldT * BKK + lc;
#pragma unroll
        for (int i = 0; i < 4; ++i) stageB[i] = loadChunk(bRow[i], kB, K);
        if (++ldT == steps) {
            ldT = 0;
            ldId = seekTile<XCD_ORDER>(ldId + stride, stride, idEnd, tilesM, tilesN, gmLog, gnLog, ldTm, ldTn);
            if (ldId >= 0) setSources();
        }
    };
    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    const int ldsW = lr * LDS_ROW + lc;
    loadA();
    loadB();
#pragma unroll
    for (int i = 0; i < A_PASSES; ++i) *reinterpret_cast<uint4v*>(as + ldsW + 64 * i * LDS_ROW) = zeroPast(stageA[i], kA, K);
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4v*>(bs + ldsW + 64 * i * LDS_ROW) = zeroPast(stageB[i], kB, K);
    if (total > 1) {
        loadA();
        loadB();
    }
    __syncthreads();
    if (group == 1) __builtin_amdgcn_s_barrier();    // group 1 runs one phase late from here to the end
    int curTm, curTn;
    int curId = seekTile<XCD_ORDER>(blockIdx.x, stride, idEnd, tilesM, tilesN, gmLog, gnLog, curTm, curTn);
    bf16x8 a[2][TM], b[2][TN];
    int g = 0;
    for (int tile = 0; tile < myTiles; ++tile) {
        for (int T = 0; T < steps; ++T, ++g) {
            const int par = g & 1;
            const unsigned short* ac = as + (par * BM + wm0 + li) * LDS_ROW + 8 * half;
            const unsigned short* bc = bs + (par * BN + wn0 + li) * LDS_ROW + 8 * half;
            unsigned short* aw = as + (par ^ 1) * BM * LDS_ROW + ldsW;
            unsigned short* bw = bs + (par ^ 1) * BN * LDS_ROW + ldsW;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                // ---- memory phase
#pragma unroll
                for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
                    for (int i = 0; i < TM; ++i) a[kk][i] = *reinterpret_cast<const bf16x8*>(ac + i * 32 * LDS_ROW + h * 32 + kk * 16);
#pragma unroll
                    for (int j = 0; j < TN; ++j) b[kk][j] = *reinterpret_cast<const bf16x8*>(bc + j * 32 * LDS_ROW + h * 32 + kk * 16);
                }
                if (g + 1 < total) {
                    if (h == 0) {
#pragma unroll
                        for (int i = 0; i < A_PASSES; ++i) *reinterpret_cast<uint4v*>(aw + 64 * i * LDS_ROW) = zeroPast(stageA[i], kA, K);
                        if (g + 2 < total) loadA();
                    } else {
#pragma unroll
                        for (int i = 0; i < 4; ++i) *reinterpret_cast<uint4v*>(bw + 64 * i * LDS_ROW) = zeroPast(stageB[i], kB, K);
                        if (g + 2 < total) loadB();
                    }
                }
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
                // ---- compute phase
#pragma unroll
                for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kk][i], b[kk][j], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
            }
        }
        if (wideStores) {
            const int which = (curTn * BN) / epi.splitN;   // a tile lies in one output
            float* out = which == 0 ? epi.c[0] : which == 1 ? epi.c[1] : epi.c[2];
            storeAccumulatorsFlat<TM, TN>(acc, epi, out, which * epi.splitN, M, N, curTm * BM + wm0, curTn * BN + wn0, li, half);
        } else {
            storeAccumulators<TM, TN>(acc, epi, M, N, curTm * BM + wm0, curTn * BN + wn0, li, half);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        curId = seekTile<XCD_ORDER>(curId + stride, stride, idEnd, tilesM, tilesN, gmLog, gnLog, curTm, curTn);
    }
    if (group == 0) __builtin_amdgcn_s_barrier();    // pairs with group 1's last barrier
}

// out = sum over slices of partial[s*sliceStride + i] (+ bias[i % N] + residual[i]), slices added in index order
// (deterministic), written through the epilogue's output split.  sliceStride is a multiple of 4; `vec` says
// that every pointer is 16-byte aligned and N and splitN are multiples of 4.
__global__ void __launch_bounds__(kBlock) splitReduceKernel(const float* __restrict__ partial, Epilogue e, size_t count,
                                                            size_t sliceStride, int slices, int vec, size_t N) {
    const size_t stride = size_t(gridDim.x) * blockDim.x;
    const size_t first = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t count4 = vec ? count / 4 : 0;
    const size_t splitN = size_t(e.splitN);
    for (size_t i = first; i < count4; i += stride) {
        float4v sum = loadf4(partial + 4 * i);
        for (int s = 1; s < slices; ++s) {
            float4v p = loadf4(partial + size_t(s) * sliceStride + 4 * i);
            sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
        }
        const size_t row = (4 * i) / N, col = (4 * i) - row * N, which = col / splitN;
        if (e.bias) sum = sum + loadf4(e.bias + col);
        if (e.residual) sum = sum + loadf4(e.residual + 4 * i);
        storef4((which == 0 ? e.c[0] : which == 1 ? e.c[1] : e.c[2]) + row * splitN + (col - which * splitN), sum);
    }
    for (size_t i = 4 * count4 + first; i < count; i += stride) {
        float sum = partial[i];
        for (int s = 1; s < slices; ++s) sum += partial[size_t(s) * sliceStride + i];
        const size_t row = i / N, col = i - row * N, which = col / splitN;
        if (e.bias) sum += e.bias[col];
        if (e.residual) sum += e.residual[i];
        (which == 0 ? e.c[0] : which == 1 ? e.c[1] : e.c[2])[row * splitN + (col - which * splitN)] = sum;
    }
}

// Products of at most eight rows (a step of incremental decoding: one new token per sequence).  A 128 x 128 tile would
// be all padding and six workgroups would walk a 768-wide weight alone; here the product is what it is by nature, a walk
// over the weights: a wavefront owns COLS output columns (rows of Bt), each lane takes 16 bytes (eight bf16) of every
// column per step, U steps loaded before any is used (a weight of a few MB is in flight all at once, which is what the
// memory's latency asks for), and multiplies them with the same eight elements of the M rows of A (one or two rows: held
// in LDS by the workgroup; more: read where they lie).  The lanes' sums are added by a butterfly and lane r * COLS + j stores element (r, n0 + j) through the
// epilogue (fuse 1 included: z and the image of act(z)).  Products in fp32 of the bf16 values, as on the MFMA; the order of
// additions is fixed (even and odd elements of a lane's eight apart, then the butterfly), so results repeat bit for bit.
// K, lda and ldb multiples of 8, operands 16-byte aligned, staged rows within the LDS.
__device__ __forceinline__ void dot8(const uint4v& a, const uint4v& b, float& even, float& odd) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        even = fmaf(__uint_as_float(a[i] << 16), __uint_as_float(b[i] << 16), even);
        odd = fmaf(__uint_as_float(a[i] & 0xffff0000u), __uint_as_float(b[i] & 0xffff0000u), odd);
    }
}
__device__ __forceinline__ float actF1(int act, float v) { return act == BF_ACT_SILU ? siluF(v) : act == BF_ACT_GELU ? geluF(v) : reluF(v); }
template <int MR, int COLS, int U>
__global__ void __launch_bounds__(256) gemmBf16FewRowsKernel(const unsigned short* __restrict__ A, const unsigned short* __restrict__ Bt,
                                                             Epilogue e, int M, int N, int K, int lda, int ldb) {
    extern __shared__ __attribute__((aligned(16))) unsigned short aRows[];   // [M][K]
    const int lane = threadIdx.x & 63;
    const int n0 = (int(blockIdx.x) * 4 + int(threadIdx.x >> 6)) * COLS;
    const bool owner = n0 < N;                               // a wavefront past the last column only helps to stage A
    // lane r * COLS + j stores element (r, n0 + j): what the epilogue adds there is fetched now, not after the sums
    const int storeRow = lane / COLS, storeCol = n0 + lane % COLS;
    const bool stores = owner && lane < MR * COLS && storeRow < M && storeCol < N;
    const float biasHere = stores && e.bias ? e.bias[storeCol] : 0.0f;
    const float residualHere = stores && e.residual ? e.residual[size_t(storeRow) * N + storeCol] : 0.0f;
    float even[MR][COLS], odd[MR][COLS];
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
        for (int j = 0; j < COLS; ++j) even[r][j] = odd[r][j] = 0.0f;
    const unsigned short* bRow[COLS];
#pragma unroll
    for (int j = 0; j < COLS; ++j) bRow[j] = Bt + size_t(min(n0 + j, N - 1)) * ldb;   // a column past the end repeats the last one, unstored
    uint4v b[U][COLS];
    const uint4v none = {0u, 0u, 0u, 0u};
    auto loadSteps = [&](int k0) {
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int j = 0; j < COLS; ++j)
                b[u][j] = owner && k0 + u * 512 < K ? __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(bRow[j] + k0 + u * 512)) : none;
    };
    int k0 = lane * 8;
    loadSteps(k0);                                           // in flight while A is staged
    // One or two rows are staged in LDS (and normalised on the way, if asked).  More rows are read where they lie: every
    // wavefront reads the same few KB, which the caches serve, while staging them would cost each workgroup M * K * 2
    // bytes of copying for the four columns it computes (eight rows of 3072: 48 KB of LDS, three workgroups a compute
    // unit).  Four columns a wavefront instead of one, to read A less often, measured half again as slow at 4 and 8 rows.
    constexpr bool STAGED = MR <= 2;
    if constexpr (!STAGED) {
    } else if (e.normInput == nullptr) {
        for (int at = int(threadIdx.x) * 8; at < M * K; at += 2048) {
            const int r = at / K, k = at - r * K;            // K is a multiple of 8: a group of eight lies in one row
            *reinterpret_cast<uint4v*>(aRows + at) = *reinterpret_cast<const uint4v*>(A + size_t(r) * lda + k);
        }
    } else {
        // x / sqrt(mean(x^2) + eps) with the sum of squares in double and the division in float, as the row kernel that
        // this replaces forms it (ops.cpp:264-275), rounded to bf16; every workgroup normalises all M rows for itself, all
        // rows in one pass (one barrier whatever M)
        __shared__ double squares[4][MR];
        double ss[MR];
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            ss[r] = 0.0;
            if (r < M)
                for (int k = int(threadIdx.x); k < K; k += 256) {
                    const double v = double(e.normInput[size_t(r) * K + k]);
                    ss[r] += v * v;
                }
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) ss[r] += __shfl_xor(ss[r], o, 64);
            if (lane == 0) squares[threadIdx.x >> 6][r] = ss[r];
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < MR; ++r) {
            if (r < M) {
                const float rms = float(sqrt(((squares[0][r] + squares[1][r]) + (squares[2][r] + squares[3][r])) / double(K) + double(kRmsNormEps)));
                for (int k = int(threadIdx.x); k < K; k += 256) aRows[r * K + k] = toBf16Bits(e.normInput[size_t(r) * K + k] / rms);
            }
        }
    }
    if constexpr (STAGED) __syncthreads();
    if (!owner) return;
    while (k0 < K) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = k0 + u * 512;
            if (k < K) {
#pragma unroll
                for (int r = 0; r < MR; ++r) {
                    if (r < M) {
                        const uint4v a = STAGED ? *reinterpret_cast<const uint4v*>(aRows + r * K + k)
                                                : *reinterpret_cast<const uint4v*>(A + size_t(r) * lda + k);
#pragma unroll
                        for (int j = 0; j < COLS; ++j) dot8(a, b[u][j], even[r][j], odd[r][j]);
                    }
                }
            }
        }
        k0 += 512 * U;
        if (k0 < K) loadSteps(k0);
    }
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
        for (int j = 0; j < COLS; ++j) {
            float v = even[r][j] + odd[r][j];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            const int col = n0 + j;
            if (lane == r * COLS + j && r < M && col < N) {
                const int which = col / e.splitN;
                float* C = which == 0 ? e.c[0] : which == 1 ? e.c[1] : e.c[2];
                if (e.bias) v += biasHere;
                if (e.residual) v += residualHere;
                size_t row = size_t(r);
                if (e.rowShift != nullptr && which >= 1) row += size_t(*e.rowShift);
                if (e.rowShift == nullptr || which == 0 || row < size_t(e.rowLimit)) C[row * e.splitN + (col - which * e.splitN)] = v;
                if (e.fuse == 1) e.image[size_t(r) * N + col] = toBf16Bits(actF1(e.act, v));
            }
        }
}
template <int MR>
int launchFewRows(const unsigned short* A, const unsigned short* Bt, const Epilogue& epi, size_t M, size_t N, size_t K, size_t lda, size_t ldb,
                  hipStream_t s) {
    const size_t smem = MR <= 2 ? M * K * sizeof(unsigned short) : 0;   // rows of A in LDS: one or two rows only
    // one column a wavefront until that gives every SIMD several wavefronts; four from there on (fewer butterflies per byte)
    if (N <= 8192) {
        auto kernel = gemmBf16FewRowsKernel<MR, 1, 8>;
        int st = allowDynamicSharedMemory(reinterpret_cast<const void*>(kernel), smem);
        if (st != BF_OK) return st;
        kernel<<<unsigned((N + 3) / 4), 256, smem, s>>>(A, Bt, epi, int(M), int(N), int(K), int(lda), int(ldb));
    } else {
        auto kernel = gemmBf16FewRowsKernel<MR, 4, 2>;
        int st = allowDynamicSharedMemory(reinterpret_cast<const void*>(kernel), smem);
        if (st != BF_OK) return st;
        kernel<<<unsigned((N + 15) / 16), 256, smem, s>>>(A, Bt, epi, int(M), int(N), int(K), int(lda), int(ldb));
    }
    BF_LAUNCH_CHECK();
    return BF_OK;
}
constexpr size_t kFewRowsLds = 128 * 1024;   // what the rows of A may take of a compute unit's 160 KB

// Products of 5 to 128 rows (a decoding step of several sequences, a short prompt, a small batch): 32 x 32 output tiles on the MFMA
// without LDS staging.  A workgroup owns one tile (blockIdx.x: 32 columns, blockIdx.y: 32 rows) and its eight wavefronts
// share out the contraction: wavefront w takes K steps w, w + 8, ... of sixteen, and loads its operand fragments
// straight from memory, which is how they lie there: lane (li, half) needs eight consecutive k of row li of A and of row
// li of Bt, 16 bytes each.  Twelve steps are loaded before the first is multiplied (a wavefront's share of K = 1536),
// longer contractions go round again.  The eight partial tiles are added in wavefront order through LDS and stored through
// the epilogue (bias, residual, split outputs, fuse 1).  K, lda, ldb multiples of 8, operands 16-byte aligned.
constexpr int kSkinnyWaves = 8, kSkinnyDepth = 12;
__global__ void __launch_bounds__(64 * kSkinnyWaves) gemmBf16SkinnyKernel(const unsigned short* __restrict__ A, const unsigned short* __restrict__ Bt,
                                                                          Epilogue e, int M, int N, int K, int lda, int ldb, int kPer,
                                                                          size_t sliceStride) {
    __shared__ float partial[kSkinnyWaves][32][33];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, li = lane & 31, half = lane >> 5;
    const int col0 = int(blockIdx.x) * 32, row0 = int(blockIdx.y) * 32;
    const bool rowLive = row0 + li < M, colLive = col0 + li < N;
    const unsigned short* aRow = A + size_t(rowLive ? row0 + li : 0) * lda + 8 * half;
    const unsigned short* bRow = Bt + size_t(colLive ? col0 + li : 0) * ldb + 8 * half;
    const uint4v none = {0u, 0u, 0u, 0u};
    float16v acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    // blockIdx.z: the slice of K (kPer, a multiple of 16, each) when few tiles share a long contraction; slice z writes its
    // sums sliceStride floats after the slice before it and splitReduceKernel adds them, with the epilogue's adds
    const int kBegin = int(blockIdx.z) * kPer;
    K = min(K, kBegin + kPer);
    if (gridDim.z > 1) e.c[0] += size_t(blockIdx.z) * sliceStride;
    for (int k0 = kBegin + wave * 16; k0 < K; k0 += 16 * kSkinnyWaves * kSkinnyDepth) {   // the same for all lanes of a wavefront
        uint4v a[kSkinnyDepth], b[kSkinnyDepth];
#pragma unroll
        for (int u = 0; u < kSkinnyDepth; ++u) {
            const int k = k0 + u * 16 * kSkinnyWaves;
            const bool in = k + 8 * half < K;            // K is a multiple of 8: the second half of the last step may be past the end
            b[u] = in && colLive ? __builtin_nontemporal_load(reinterpret_cast<const uint4v*>(bRow + k)) : none;
            a[u] = in && rowLive ? *reinterpret_cast<const uint4v*>(aRow + k) : none;
        }
#pragma unroll
        for (int u = 0; u < kSkinnyDepth; ++u)
            if (k0 + u * 16 * kSkinnyWaves < K)
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[u]), __builtin_bit_cast(bf16x8, b[u]), acc, 0, 0, 0);
    }
    // lane (li, half) holds column li of rows 8 g + 4 half + i
#pragma unroll
    for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) partial[wave][8 * g + 4 * half + i][li] = acc[4 * g + i];
    __syncthreads();
    for (int at = t; at < 32 * 32; at += 64 * kSkinnyWaves) {
        const int r = at >> 5, c = at & 31, row = row0 + r, col = col0 + c;
        if (row < M && col < N) {
            float v = partial[0][r][c];
#pragma unroll
            for (int w = 1; w < kSkinnyWaves; ++w) v += partial[w][r][c];
            const int which = col / e.splitN;
            float* C = which == 0 ? e.c[0] : which == 1 ? e.c[1] : e.c[2];
            if (e.bias) v += e.bias[col];
            if (e.residual) v += e.residual[size_t(row) * N + col];
            C[size_t(row) * e.splitN + (col - which * e.splitN)] = v;
            if (e.fuse == 1) e.image[size_t(row) * N + col] = toBf16Bits(actF1(e.act, v));
        }
    }
}
int launchSkinny(const unsigned short* A, const unsigned short* Bt, const Epilogue& epi, size_t M, size_t N, size_t K, size_t lda, size_t ldb,
                 hipStream_t s) {
    const size_t tiles = ((N + 31) / 32) * ((M + 31) / 32);
    // few tiles and a long contraction (a feed-forward block's second product): K in slices over more workgroups, at least
    // four steps a wavefront each, summed in slice order by a second kernel
    size_t slices = 1;
    if (tiles < 64 && K >= 2048 && epi.fuse == 0) slices = std::min<size_t>(std::min<size_t>(8, K / 512), 128 / tiles);
    if (slices > 1) {
        const size_t kPer = ((K + slices - 1) / slices + 127) / 128 * 128;
        slices = (K + kPer - 1) / kPer;
        const size_t count = M * N, sliceStride = (count + 3) / 4 * 4;
        Scratch partial(slices * sliceStride * sizeof(float));
        if (partial.status != BF_OK) return partial.status;
        Epilogue plain{{partial.as<float>(), nullptr, nullptr}, int(N), nullptr, nullptr};
        const dim3 grid{unsigned((N + 31) / 32), unsigned((M + 31) / 32), unsigned(slices)};
        gemmBf16SkinnyKernel<<<grid, 64 * kSkinnyWaves, 0, s>>>(A, Bt, plain, int(M), int(N), int(K), int(lda), int(ldb), int(kPer), sliceStride);
        BF_LAUNCH_CHECK();
        const int vec = ((reinterpret_cast<uintptr_t>(epi.c[0]) | reinterpret_cast<uintptr_t>(epi.c[1]) | reinterpret_cast<uintptr_t>(epi.c[2]) |
                          reinterpret_cast<uintptr_t>(epi.residual) | reinterpret_cast<uintptr_t>(epi.bias)) & 15u) == 0 && N % 4 == 0 && epi.splitN % 4 == 0;
        splitReduceKernel<<<gridFor(count / 4 + 1, kBlock), kBlock, 0, s>>>(partial.as<float>(), epi, count, sliceStride, int(slices), vec, N);
        BF_LAUNCH_CHECK();
        return BF_OK;
    }
    const dim3 grid{unsigned((N + 31) / 32), unsigned((M + 31) / 32), 1u};
    gemmBf16SkinnyKernel<<<grid, 64 * kSkinnyWaves, 0, s>>>(A, Bt, epi, int(M), int(N), int(K), int(lda), int(ldb), int((K + 15) / 16 * 16), size_t(0));
    BF_LAUNCH_CHECK();
    return BF_OK;
}

// The same kernel for operands that lie the other way round: C[M,N] = A^T * B with A [K, lda] and B [K, ldb], the
// contraction index K running over ROWS (a weight gradient dW = X^T * G: both the activations X and the gradient G have
// one row per token).  A K step is 64 rows of either operand, staged in LDS as they lie in memory ([k][m], rows padded
// to pitch = width + 32 elements); the MFMA fragments, which want eight consecutive k per lane, are gathered by the LDS
// transposing read (ds_read_b64_tr_b16: within 16 lanes, lane j receives element j%4 of the 8-byte pieces addressed by
// lanes j/4, j/4 + 4, j/4 + 8, j/4 + 12; with lane i addressing row i/4, columns 4*(i%4).. of a 4 x 16 block, lane j
// ends up with the four rows of column j).  No transposed operand image is ever written to HBM.  The pitch is 64 bytes
// more than a multiple of 256, which spreads the 4 rows x 2 column blocks that half a wavefront reads over all banks.
typedef short short4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bf16x8 readTransposed8(const unsigned short* p, int rowPitch) {
    typedef __attribute__((address_space(3))) short4v* LdsPtr;
    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(p));
    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsPtr)(p + 4 * rowPitch));
    typedef short short8v __attribute__((ext_vector_type(8)));
    const short8v both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8, both);
}

template <int XCD_ORDER, int BM>
__global__ void __launch_bounds__(512, 2) gemmBf16TnPingPongKernel(const unsigned short* __restrict__ A,
                                                                   const unsigned short* __restrict__ B, Epilogue epi,
                                                                   int M, int N, int K, int lda, int ldb, int gmLog, int gnLog,
                                                                   int kPerSplit, size_t sliceStride) {
    constexpr int BN = 256, TM = BM / 64, TN = 2, A_PASSES = BM / 64;
    constexpr int PITCH_A = BM + 32, PITCH_B = BN + 32;           // elements
    constexpr int A_THREADS_PER_ROW = BM / 8, A_ROWS_PER_PASS = 512 / A_THREADS_PER_ROW;   // 16-byte pieces
    constexpr int B_THREADS_PER_ROW = BN / 8, B_ROWS_PER_PASS = 512 / B_THREADS_PER_ROW;
    static_assert(A_ROWS_PER_PASS * A_PASSES == 64 && B_ROWS_PER_PASS * 4 == 64, "a K step is 64 rows");
    extern __shared__ __attribute__((aligned(16))) unsigned short lds[];
    unsigned short* as = lds;                             // [2][64][PITCH_A]
    unsigned short* bs = lds + 2 * 64 * PITCH_A;          // [2][64][PITCH_B]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, li = lane & 31;
    const int group = wave >> 2;
    int tm, tn;
    if (XCD_ORDER) {
        if (!tileIndexXcd(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, gmLog, gnLog, tm, tn)) return;
    } else {
        tileIndexGrouped(blockIdx.x, (M + BM - 1) / BM, (N + BN - 1) / BN, tm, tn);
    }
    const int m0 = tm * BM, n0 = tn * BN;
    const int wm0 = group * (BM / 2), wn0 = (wave & 3) * 64;
    const int kBegin = blockIdx.y * kPerSplit, kEnd = min(K, kBegin + kPerSplit);
    epi.c[0] += size_t(blockIdx.y) * sliceStride;
    const int steps = max((kEnd - kBegin + BKK - 1) / BKK, 1);

    // staging: thread -> (row of the K step, 16-byte piece of that row); columns past the operand's width are clamped
    // into it (their products are never stored), rows past kEnd are clamped to the last row and stored as zeros
    const int aRow = tid / A_THREADS_PER_ROW, aCol = (tid % A_THREADS_PER_ROW) * 8;
    const int bRow = tid / B_THREADS_PER_ROW, bCol = (tid % B_THREADS_PER_ROW) * 8;
    const unsigned short* aSrc = A + min(m0 + aCol, lda - 8);
    const unsigned short* bSrc = B + min(n0 + bCol, ldb - 8);
    uint4v stageA[A_PASSES], stageB[4];
    auto loadA = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i)
            stageA[i] = *reinterpret_cast<const uint4v*>(aSrc + size_t(min(k0 + aRow + A_ROWS_PER_PASS * i, K - 1)) * lda);
    };
    auto loadB = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            stageB[i] = *reinterpret_cast<const uint4v*>(bSrc + size_t(min(k0 + bRow + B_ROWS_PER_PASS * i, K - 1)) * ldb);
    };
    auto storeA = [&](int buf, int k0) {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i)
            *reinterpret_cast<uint4v*>(as + (buf * 64 + aRow + A_ROWS_PER_PASS * i) * PITCH_A + aCol) =
                zeroPast(stageA[i], k0 + aRow + A_ROWS_PER_PASS * i, kEnd);
    };
    auto storeB = [&](int buf, int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<uint4v*>(bs + (buf * 64 + bRow + B_ROWS_PER_PASS * i) * PITCH_B + bCol) =
                zeroPast(stageB[i], k0 + bRow + B_ROWS_PER_PASS * i, kEnd);
    };

    float16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    loadA(kBegin);
    loadB(kBegin);
    storeA(0, kBegin);
    storeB(0, kBegin);
    if (steps > 1) {
        loadA(kBegin + BKK);
        loadB(kBegin + BKK);
    }
    __syncthreads();
    if (group == 1) __builtin_amdgcn_s_barrier();    // group 1 starts one phase late
    // this lane's corner of a fragment's 16-row x 32-column block: lanes 0-15 and 16-31 take the two 16-column halves,
    // lanes 32-63 the rows eight further down; inside 16 lanes, lane i addresses row i/4, columns 4*(i%4)..
    const int fragRow = (lane >> 5) * 8 + ((lane & 15) >> 2), fragCol = ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    bf16x8 a[2][TM], b[2][TN];
    for (int T = 0; T < steps; ++T) {
        const int par = T & 1;
        const unsigned short* ac = as + (par * 64 + fragRow) * PITCH_A + wm0 + fragCol;
        const unsigned short* bc = bs + (par * 64 + fragRow) * PITCH_B + wn0 + fragCol;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            // ---- memory phase
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
                for (int i = 0; i < TM; ++i) a[kk][i] = readTransposed8(ac + (h * 32 + kk * 16) * PITCH_A + i * 32, PITCH_A);
#pragma unroll
                for (int j = 0; j < TN; ++j) b[kk][j] = readTransposed8(bc + (h * 32 + kk * 16) * PITCH_B + j * 32, PITCH_B);
            }
            if (T + 1 < steps) {
                if (h == 0) {
                    storeA(par ^ 1, kBegin + (T + 1) * BKK);
                    if (T + 2 < steps) loadA(kBegin + (T + 2) * BKK);
                } else {
                    storeB(par ^ 1, kBegin + (T + 1) * BKK);
                    if (T + 2 < steps) loadB(kBegin + (T + 2) * BKK);
                }
            }
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            // ---- compute phase
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[kk][i], b[kk][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
        }
    }
    if (group == 0) __builtin_amdgcn_s_barrier();    // pairs with group 1's last barrier
    storeAccumulators<TM, TN>(acc, epi, M, N, m0 + wm0, n0 + wn0, li, half);
}

// What the matrix pipes deliver when nothing else runs: the K loop of the 256 x 256 ping-pong tile (eight wavefronts of a
// 128 x 64 share each, two per SIMD) with every memory instruction removed.  The operand fragments of one 64-deep K step
// are read once from `operands` and stay in registers; `steps` K steps are then multiplied out of them.  SHAPE 0: 32 MFMAs
// 32x32x16 per step and wavefront; SHAPE 1: 64 MFMAs 16x16x32.  One workgroup per compute unit; the accumulators' sums go
// to `out` so that the loop cannot be removed.
template <int SHAPE>
__global__ void __launch_bounds__(512, 2) mfmaOnlyKernel(const uint4v* __restrict__ operands, float* __restrict__ out, int steps) {
    const int tid = threadIdx.x;
    bf16x8 fa[16], fb[8];
#pragma unroll
    for (int i = 0; i < 16; ++i) fa[i] = __builtin_bit_cast(bf16x8, operands[(tid * 24 + i) & 4095]);
#pragma unroll
    for (int i = 0; i < 8; ++i) fb[i] = __builtin_bit_cast(bf16x8, operands[(tid * 24 + 16 + i) & 4095]);
    float sum = 0.0f;
    if constexpr (SHAPE == 0) {
        float16v acc[4][2];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        for (int t = 0; t < steps; ++t) {
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[kk * 4 + i], fb[kk * 2 + j], acc[i][j], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
    } else {
        float4v acc[8][4];
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = float4v{0.0f, 0.0f, 0.0f, 0.0f};
        for (int t = 0; t < steps; ++t) {
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                for (int i = 0; i < 8; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[kk * 8 + i], fb[kk * 4 + j], acc[i][j], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) sum += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    }
    out[size_t(blockIdx.x) * 512 + tid] = sum;
}

template <typename Kernel>
int allowSharedMemory(Kernel kernel, size_t smem) {
    return allowDynamicSharedMemory(reinterpret_cast<const void*>(kernel), smem);
}

// slices > 1: K is cut into `slices` ranges of kPer (a multiple of 64) and range i writes to epi.c[0] + i * sliceStride
template <int BM>
int launchPingPong(const unsigned short* A, const unsigned short* Bt, const Epilogue& epi, size_t M, size_t N, size_t K,
                   size_t lda, size_t ldb, hipStream_t s, size_t slices = 1, size_t kPer = 0, size_t sliceStride = 0, bool persistent = true) {
    if (slices <= 1) { slices = 1; kPer = K; sliceStride = 0; }
    const size_t tilesM = (M + BM - 1) / BM, tilesN = (N + 255) / 256;
    constexpr size_t smem = size_t(2) * (BM + 256) * LDS_ROW * sizeof(unsigned short);
    // XCD block shape: the 2^g x 2^(5-g) block that pads the tile grid least, squarest on ties
    int gmLog = 2, gnLog = 3;
    size_t bestCost = 0, blocks = 0;
    for (int g = 0; g <= 5; ++g) {
        size_t gm = size_t(1) << g, gn = size_t(32) >> g;
        size_t nb = ((tilesM + gm - 1) / gm) * ((tilesN + gn - 1) / gn);
        size_t cost = nb * 1000 + gm + gn;
        if (g == 0 || cost < bestCost) { bestCost = cost; gmLog = g; gnLog = 5 - g; blocks = nb; }
    }
    // blocks are dealt to XCDs eight at a time: only worth it when that deal is (nearly) even
    const bool xcdOrder = blocks * 32 <= (tilesM * tilesN) * 5 / 4 && (blocks % 8 == 0 || blocks >= 64);
    const size_t cus = size_t(computeUnits());
    if (epi.fuse != 0 && slices != 1) return failInvalid("gemm_bf16", "a fused activation does not go with K slices");
    if (persistent && epi.fuse == 0 && slices == 1 && tilesM * tilesN > cus) {
        // one workgroup per compute unit walks ids blockIdx.x + r * cus (see launchWideWave)
        const bool xcd = xcdOrder && cus % 8 == 0;
        const size_t idEnd = xcd ? (blocks + 7) / 8 * 8 * 32 : tilesM * tilesN;
        if (idEnd >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
        auto kernel = xcd ? gemmBf16PingPongPersistentKernel<1, BM> : gemmBf16PingPongPersistentKernel<0, BM>;
        int st = allowSharedMemory(kernel, smem);
        if (st != BF_OK) return st;
        kernel<<<dim3(unsigned(cus)), 512, smem, s>>>(A, Bt, epi, int(M), int(N), int(K), int(lda), int(ldb), xcd ? gmLog : 0, xcd ? gnLog : 0,
                                                      int(idEnd));
        BF_LAUNCH_CHECK();
        return BF_OK;
    }
    if (xcdOrder) {
        size_t grid = (blocks + 7) / 8 * 8 * 32;
        if (grid >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
        auto kernel = epi.fuse == 1 ? gemmBf16PingPongKernel<1, BM, 1> : epi.fuse == 2 ? gemmBf16PingPongKernel<1, BM, 2> : gemmBf16PingPongKernel<1, BM>;
        int st = allowSharedMemory(kernel, smem);
        if (st != BF_OK) return st;
        kernel<<<dim3(unsigned(grid), unsigned(slices)), 512, smem, s>>>(A, Bt, epi, int(M), int(N), int(K), int(lda), int(ldb), gmLog, gnLog,
                                                                         int(kPer), sliceStride);
    } else {
        size_t grid = tilesM * tilesN;
        if (grid >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
        auto kernel = epi.fuse == 1 ? gemmBf16PingPongKernel<0, BM, 1> : epi.fuse == 2 ? gemmBf16PingPongKernel<0, BM, 2> : gemmBf16PingPongKernel<0, BM>;
        int st = allowSharedMemory(kernel, smem);
        if (st != BF_OK) return st;
        kernel<<<dim3(unsigned(grid), unsigned(slices)), 512, smem, s>>>(A, Bt, epi, int(M), int(N), int(K), int(lda), int(ldb), 0, 0,
                                                                         int(kPer), sliceStride);
    }
    BF_LAUNCH_CHECK();
    return BF_OK;
}

template <int WAVES_N>
int launchWideWave(const unsigned short* A, const unsigned short* Bt, const Epilogue& epi, size_t M, size_t N, size_t K,
                   size_t lda, size_t ldb, hipStream_t s, bool persistent = true) {
    constexpr size_t BN = 64 * WAVES_N;
    const size_t tilesM = (M + 127) / 128, tilesN = (N + BN - 1) / BN;
    constexpr size_t smem = size_t(2) * (128 + BN) * LDS_ROW * sizeof(unsigned short);
    int gmLog = 2, gnLog = 3;
    size_t bestCost = 0, blocks = 0;
    for (int g = 0; g <= 5; ++g) {
        size_t gm = size_t(1) << g, gn = size_t(32) >> g;
        size_t nb = ((tilesM + gm - 1) / gm) * ((tilesN + gn - 1) / gn);
        size_t cost = nb * 1000 + gm + gn;
        if (g == 0 || cost < bestCost) { bestCost = cost; gmLog = g; gnLog = 5 - g; blocks = nb; }
    }
    const bool xcdOrder = blocks * 32 <= (tilesM * tilesN) * 5 / 4 && (blocks % 8 == 0 || blocks >= 64);
    const size_t grid = xcdOrder ? (blocks + 7) / 8 * 8 * 32 : tilesM * tilesN;
    if (grid >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
    const size_t cus = size_t(computeUnits());
    const bool wideStores = ((N | size_t(epi.splitN)) & 3) == 0 &&
                            ((reinterpret_cast<uintptr_t>(epi.c[0]) | reinterpret_cast<uintptr_t>(epi.c[1]) | reinterpret_cast<uintptr_t>(epi.c[2]) |
                              reinterpret_cast<uintptr_t>(epi.bias) | reinterpret_cast<uintptr_t>(epi.residual)) & 15u) == 0;
    // With sixteen wavefronts (128 registers each) the second accumulator set leaves no room for the bias and residual
    // values fetched ahead: such products keep the one-tile-per-workgroup form.
    const bool adds = epi.bias || epi.residual;
    constexpr bool kAddsFit = WAVES_N < 4;
    if (persistent && epi.fuse == 0 && wideStores && tilesM * tilesN > cus && (!adds || kAddsFit)) {
        // one workgroup per compute unit walks ids blockIdx.x + r * cus; with a CU count that is a multiple of 8 a workgroup
        // stays on its XCD and round r of the XCD order is one block of 32 tiles per XCD, as in the one-tile-per-workgroup launch
        const bool xcd = xcdOrder && cus % 8 == 0;
        auto kernel = xcd ? (adds ? gemmBf16WidePersistentKernel<1, WAVES_N, kAddsFit> : gemmBf16WidePersistentKernel<1, WAVES_N, false>)
                          : (adds ? gemmBf16WidePersistentKernel<0, WAVES_N, kAddsFit> : gemmBf16WidePersistentKernel<0, WAVES_N, false>);
        int st = allowSharedMemory(kernel, smem);
        if (st != BF_OK) return st;
        kernel<<<dim3(unsigned(cus)), 256 * WAVES_N, smem, s>>>(A, Bt, epi, int(M), int(N), int(K), int(lda), int(ldb), xcd ? gmLog : 0,
                                                                 xcd ? gnLog : 0, int(xcd ? grid : tilesM * tilesN));
        BF_LAUNCH_CHECK();
        return BF_OK;
    }
    auto kernel = epi.fuse == 1 ? (xcdOrder ? gemmBf16WideWaveKernel<1, WAVES_N, 1> : gemmBf16WideWaveKernel<0, WAVES_N, 1>)
                : epi.fuse == 2 ? (xcdOrder ? gemmBf16WideWaveKernel<1, WAVES_N, 2> : gemmBf16WideWaveKernel<0, WAVES_N, 2>)
                                : (xcdOrder ? gemmBf16WideWaveKernel<1, WAVES_N> : gemmBf16WideWaveKernel<0, WAVES_N>);
    int st = allowSharedMemory(kernel, smem);
    if (st != BF_OK) return st;
    kernel<<<dim3(unsigned(grid)), 256 * WAVES_N, smem, s>>>(A, Bt, epi, int(M), int(N), int(K), int(lda), int(ldb), xcdOrder ? gmLog : 0,
                                                             xcdOrder ? gnLog : 0);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

template <int BM>
int launchPingPongTn(const unsigned short* A, const unsigned short* B, const Epilogue& epi, size_t M, size_t N, size_t K,
                     size_t lda, size_t ldb, hipStream_t s, size_t slices, size_t kPer, size_t sliceStride) {
    const size_t tilesM = (M + BM - 1) / BM, tilesN = (N + 255) / 256;
    constexpr size_t smem = size_t(2) * 64 * ((BM + 32) + (256 + 32)) * sizeof(unsigned short);
    int gmLog = 2, gnLog = 3;
    size_t bestCost = 0, blocks = 0;
    for (int g = 0; g <= 5; ++g) {
        size_t gm = size_t(1) << g, gn = size_t(32) >> g;
        size_t nb = ((tilesM + gm - 1) / gm) * ((tilesN + gn - 1) / gn);
        size_t cost = nb * 1000 + gm + gn;
        if (g == 0 || cost < bestCost) { bestCost = cost; gmLog = g; gnLog = 5 - g; blocks = nb; }
    }
    const bool xcdOrder = blocks * 32 <= (tilesM * tilesN) * 5 / 4 && (blocks % 8 == 0 || blocks >= 64);
    if (xcdOrder) {
        size_t grid = (blocks + 7) / 8 * 8 * 32;
        if (grid >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
        auto kernel = gemmBf16TnPingPongKernel<1, BM>;
        int st = allowSharedMemory(kernel, smem);
        if (st != BF_OK) return st;
        kernel<<<dim3(unsigned(grid), unsigned(slices)), 512, smem, s>>>(A, B, epi, int(M), int(N), int(K), int(lda), int(ldb), gmLog, gnLog,
                                                                         int(kPer), sliceStride);
    } else {
        size_t grid = tilesM * tilesN;
        if (grid >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
        auto kernel = gemmBf16TnPingPongKernel<0, BM>;
        int st = allowSharedMemory(kernel, smem);
        if (st != BF_OK) return st;
        kernel<<<dim3(unsigned(grid), unsigned(slices)), 512, smem, s>>>(A, B, epi, int(M), int(N), int(K), int(lda), int(ldb), 0, 0,
                                                                         int(kPer), sliceStride);
    }
    BF_LAUNCH_CHECK();
    return BF_OK;
}

// C = A^T B for products too small for the tile kernel to matter: one thread per output element.
__global__ void __launch_bounds__(kBlock) gemmBf16TnSmallKernel(const unsigned short* __restrict__ A, const unsigned short* __restrict__ B,
                                                                float* __restrict__ C, size_t M, size_t N, size_t K, size_t lda, size_t ldb) {
    const size_t idx = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= M * N) return;
    const size_t i = idx / N, j = idx - i * N;
    float acc = 0.0f;
    for (size_t k = 0; k < K; ++k)
        acc += __uint_as_float(unsigned(A[k * lda + i]) << 16) * __uint_as_float(unsigned(B[k * ldb + j]) << 16);
    C[idx] = acc;
}

// Form (256- or 128-row tiles) and number of K slices for a product on the large-tile kernels, by the estimate
// described at launchGemmNt; false when even the best plan leaves more than half of the CUs without a workgroup.
bool planLargeTiles(size_t M, size_t N, size_t K, int* form, size_t* slices) {
    const size_t cus = size_t(computeUnits());
    const size_t bigTiles = ((M + 255) / 256) * ((N + 255) / 256), halfTiles = ((M + 127) / 128) * ((N + 255) / 256);
    const size_t stepsAll = (K + BKK - 1) / BKK;
    constexpr double kHalfTileCost = 0.78;
    double best = 1e30;
    for (int f = 0; f < 2; ++f) {
        const size_t t = f == 0 ? bigTiles : halfTiles;
        for (size_t sl = 1; sl <= 16 && (sl == 1 || sl * 8 <= stepsAll); ++sl) {
            if (t * sl < cus / 2) continue;
            const size_t rounds = (t * sl + cus - 1) / cus;
            const double gemmUs = double(rounds) * double((stepsAll + sl - 1) / sl) * 1.4 * (f == 0 ? 1.0 : kHalfTileCost);
            const double reduceUs = sl == 1 ? 0.0 : double(sl + 1) * double(M * N) * 2.0 * sizeof(float) / 4e6;
            if (gemmUs + reduceUs < best) { best = gemmUs + reduceUs; *form = f; *slices = sl; }
        }
    }
    return best < 1e30;
}

// C[M,N] = A^T B for A [K, lda], B [K, ldb] (see gemmBf16TnPingPongKernel).  *done = false, and nothing launched, when the
// product is too small for the large-tile kernel (the caller then builds transposed images and uses launchGemmNt).
int launchGemmTn(const unsigned short* A, const unsigned short* B, const Epilogue& epi, size_t M, size_t N, size_t K, size_t lda,
                 size_t ldb, hipStream_t s, bool* done) {
    *done = false;
    if (M >= (size_t(1) << 31) || N >= (size_t(1) << 31) || K >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
    int form = 0;
    size_t slices = 1;
    if (lda < 8 || ldb < 8 || !planLargeTiles(M, N, K, &form, &slices)) return BF_OK;
    const size_t stepsAll = (K + BKK - 1) / BKK;
    const size_t kPer = (stepsAll + slices - 1) / slices * BKK;
    slices = (K + kPer - 1) / kPer;
    *done = true;
    if (slices <= 1) {
        return form == 0 ? launchPingPongTn<256>(A, B, epi, M, N, K, lda, ldb, s, 1, K, 0)
                         : launchPingPongTn<128>(A, B, epi, M, N, K, lda, ldb, s, 1, K, 0);
    }
    const size_t count = M * N, sliceStride = (count + 3) / 4 * 4;
    Scratch partial(slices * sliceStride * sizeof(float));
    if (partial.status != BF_OK) return partial.status;
    Epilogue plain{{partial.as<float>(), nullptr, nullptr}, int(N), nullptr, nullptr};
    int st = form == 0 ? launchPingPongTn<256>(A, B, plain, M, N, K, lda, ldb, s, slices, kPer, sliceStride)
                       : launchPingPongTn<128>(A, B, plain, M, N, K, lda, ldb, s, slices, kPer, sliceStride);
    if (st != BF_OK) return st;
    const int vec = ((reinterpret_cast<uintptr_t>(epi.c[0]) | reinterpret_cast<uintptr_t>(epi.c[1]) |
                      reinterpret_cast<uintptr_t>(epi.c[2]) | reinterpret_cast<uintptr_t>(epi.residual) |
                      reinterpret_cast<uintptr_t>(epi.bias)) & 15u) == 0 && N % 4 == 0 && epi.splitN % 4 == 0;
    splitReduceKernel<<<gridFor(count / 4 + 1, kBlock), kBlock, 0, s>>>(partial.as<float>(), epi, count, sliceStride, int(slices), vec, N);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

// Whether launchGemmNt takes a product of this shape with Epilogue::fuse set: a kernel chosen by the caller (tests and
// tuning) never does, so that the separate passes stay reachable, and neither do products too small for the
// one-tile-per-workgroup kernels.
// what the walk over the weights (gemmBf16FewRowsKernel) asks for; launchGemmNt sends every such product there
bool fewRowsServe(const void* A, const void* Bt, int fuse, size_t M, size_t K, size_t lda, size_t ldb) {
    return g_ntRoute == BF_GEMM_ROUTE_AUTO && M <= 8 && fuse != 2 && K % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 &&
           (M > 2 || M * K * sizeof(unsigned short) <= kFewRowsLds) && ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(Bt)) & 15u) == 0;
}
// what the 32 x 32 tiles without LDS staging (gemmBf16SkinnyKernel) ask for: the products between the walk and the big tiles
bool skinnyServes(const void* A, const void* Bt, int fuse, size_t M, size_t K, size_t lda, size_t ldb) {
    // five rows and up: below, the walk measures the same or better; to 128 rows: a 128-token prompt of GPT-small takes 1.26 ms on the
    // 128-row tiles and 1.06 here, at 256 rows the tiles are ahead (1.35 against 1.40) and at 512 far ahead
    return g_ntRoute == BF_GEMM_ROUTE_AUTO && M >= 5 && M <= 128 && fuse != 2 && K % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 &&
           ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(Bt)) & 15u) == 0;
}
// ... and with the rows of A made from fp32 rows by rmsnorm while they are staged (Epilogue::normInput): staged rows only
bool fewRowsNormalise(size_t M, size_t K) { return M <= 2 && fewRowsServe(nullptr, nullptr, 0, M, K, K, K); }
bool fusedActivationFits(size_t M, size_t N, size_t K, int fuse) {
    if (g_ntRoute != BF_GEMM_ROUTE_AUTO || N % 8 != 0) return false;
    const size_t cus = size_t(computeUnits());
    if (skinnyServes(nullptr, nullptr, fuse, M, K, K, K)) return fuse == 1;
    if (M <= 8) return fuse == 1 && fewRowsServe(nullptr, nullptr, 1, M, K, K, K);   // the walk over the weights
    const size_t halfTiles = ((M + 127) / 128) * ((N + 255) / 256);   // the 256-row form needs no fewer
    return halfTiles >= cus * 3 / 4 || (N % 192 == 0 && ((M + 127) / 128) * (N / 192) >= cus * 3 / 4);
}

// epi.splitN must be N (one output) or a multiple of 256 (several outputs: a tile must lie in one of them).
int launchGemmNt(const unsigned short* A, const unsigned short* Bt, const Epilogue& epi, size_t M, size_t N, size_t K,
                 size_t lda, size_t ldb, hipStream_t s) {
    if (M >= (size_t(1) << 31) || N >= (size_t(1) << 31) || K >= (size_t(1) << 31)) return failInvalid("gemm_bf16", "shape too large");
    if (epi.fuse != 0) {   // what the fused stores assume (storeAccumulatorsFused); callers ask fusedActivationFits() first
        const uintptr_t bits = reinterpret_cast<uintptr_t>(epi.c[0]) | reinterpret_cast<uintptr_t>(epi.bias) | reinterpret_cast<uintptr_t>(epi.image) |
                               reinterpret_cast<uintptr_t>(epi.actZ) | reinterpret_cast<uintptr_t>(epi.colPartial);
        const bool operands = epi.fuse == 1 ? (epi.c[0] && epi.image) : (epi.fuse == 2 && epi.image && epi.actZ && !epi.bias);
        if (!operands || epi.residual || size_t(epi.splitN) != N || N % 8 != 0 || (bits & 15u) != 0 || g_ntRoute != BF_GEMM_ROUTE_AUTO)
            return failInvalid("gemm_bf16", "fused activation: one 16-byte aligned output of a width that is a multiple of 8, no residual");
    }
    const size_t cus = size_t(computeUnits());
    switch (g_ntRoute) {   // a kernel named by the caller (tests and tuning); BF_GEMM_ROUTE_AUTO otherwise
        case BF_GEMM_ROUTE_PINGPONG_256: return launchPingPong<256>(A, Bt, epi, M, N, K, lda, ldb, s, 1, 0, 0, false);
        case BF_GEMM_ROUTE_PINGPONG_128: return launchPingPong<128>(A, Bt, epi, M, N, K, lda, ldb, s, 1, 0, 0, false);
        case BF_GEMM_ROUTE_PINGPONG_256_PERSISTENT: return launchPingPong<256>(A, Bt, epi, M, N, K, lda, ldb, s);
        case BF_GEMM_ROUTE_PINGPONG_128_PERSISTENT: return launchPingPong<128>(A, Bt, epi, M, N, K, lda, ldb, s);
        case BF_GEMM_ROUTE_WIDE_256: return launchWideWave<4>(A, Bt, epi, M, N, K, lda, ldb, s, false);
        case BF_GEMM_ROUTE_WIDE_256_PERSISTENT: return launchWideWave<4>(A, Bt, epi, M, N, K, lda, ldb, s, true);
        case BF_GEMM_ROUTE_WIDE_192:
        case BF_GEMM_ROUTE_WIDE_192_PERSISTENT:
            if (size_t(epi.splitN) != N && epi.splitN % 192 != 0) return failInvalid("gemm_bf16", "192-wide tiles need outputs whose width is a multiple of 192");
            return launchWideWave<3>(A, Bt, epi, M, N, K, lda, ldb, s, g_ntRoute == BF_GEMM_ROUTE_WIDE_192_PERSISTENT);
        default: break;
    }
    if (skinnyServes(A, Bt, epi.fuse, M, K, lda, ldb)) return N == 0 ? BF_OK : launchSkinny(A, Bt, epi, M, N, K, lda, ldb, s);
    if (fewRowsServe(A, Bt, epi.fuse, M, K, lda, ldb)) {   // a walk over the weights, no tiles
        if (M == 0 || N == 0) return BF_OK;
        return M == 1 ? launchFewRows<1>(A, Bt, epi, M, N, K, lda, ldb, s) : M == 2 ? launchFewRows<2>(A, Bt, epi, M, N, K, lda, ldb, s)
             : M <= 4 ? launchFewRows<4>(A, Bt, epi, M, N, K, lda, ldb, s) : launchFewRows<8>(A, Bt, epi, M, N, K, lda, ldb, s);
    }
    // 256x256 ping-pong tiles once they give three quarters of the CUs a tile; otherwise 128x128 tiles,
    // with K cut into slices when even those leave CUs idle and K is long enough to share out.
    // A workgroup per CU at a time, so a product takes ceil(tiles / CUs) rounds; a 128-row tile costs kHalfTileCost of a
    // 256-row one (measured).  Either form is used only if its first round covers most of the chip.
    const size_t bigTiles = ((M + 255) / 256) * ((N + 255) / 256), halfTiles = ((M + 127) / 128) * ((N + 255) / 256);
    constexpr double kHalfTileCost = 0.78;
    const double bigTime = bigTiles >= cus * 3 / 4 ? double((bigTiles + cus - 1) / cus) : 1e30;
    const double halfTime = halfTiles >= cus * 3 / 4 ? double((halfTiles + cus - 1) / cus) * kHalfTileCost : 1e30;
    {
        // measured per round of tiles, in microseconds: the 256-row ping-pong 8 + 1.56 per K step, sixteen wavefronts on
        // 128 x 256 tiles 5 + 0.95 per K step, twelve on 128 x 192 tiles 5 + kNarrowStep per K step
        constexpr double kNarrowStep = 0.86;
        const double stepsAll = double((K + BKK - 1) / BKK);
        const size_t narrowTiles = ((M + 127) / 128) * ((N + 191) / 192);
        const bool narrowFits = size_t(epi.splitN) == N || epi.splitN % 192 == 0;   // a tile must lie in one output
        const double big = bigTiles >= cus * 3 / 4 ? double((bigTiles + cus - 1) / cus) * (8.0 + 1.56 * stepsAll) : 1e30;
        const double wide = halfTiles >= cus * 3 / 4 ? double((halfTiles + cus - 1) / cus) * (5.0 + 0.95 * stepsAll) : 1e30;
        const double narrow = narrowFits && narrowTiles >= cus * 3 / 4 ? double((narrowTiles + cus - 1) / cus) * (5.0 + kNarrowStep * stepsAll) : 1e30;
        if (narrow < wide && narrow < big) return launchWideWave<3>(A, Bt, epi, M, N, K, lda, ldb, s);
        if (wide < big) return launchWideWave<4>(A, Bt, epi, M, N, K, lda, ldb, s);
    }
    // (the ping-pong kernel keeps one tile per workgroup: its tile-walking form measured no faster, see below)
    if (bigTime <= halfTime && bigTime < 1e30) return launchPingPong<256>(A, Bt, epi, M, N, K, lda, ldb, s, 1, 0, 0, false);
    if (halfTime < 1e30) return launchPingPong<128>(A, Bt, epi, M, N, K, lda, ldb, s, 1, 0, 0, false);
    if (epi.fuse != 0) return failInvalid("gemm_bf16", "a fused activation needs a product of at least three quarters of a round of tiles");
    // Few tiles but a long contraction (the weight-gradient products, K = all tokens): the same kernel with K cut into
    // slices, one workgroup per (tile, slice), partial products summed in slice order by a second kernel.  More slices
    // fill more CUs but write and re-read more partial sums; the estimate below (K steps at the measured ~1.4 us per
    // step of a full tile, partial sums at ~4 TB/s) picks the form and the slice count.
    if (K >= 4096) {
        const size_t stepsAll = (K + BKK - 1) / BKK;
        double best = 1e30;
        size_t bestSlices = 0, bestTiles = 0;
        int bestForm = 0;
        for (int form = 0; form < 2; ++form) {
            const size_t t = form == 0 ? bigTiles : halfTiles;
            for (size_t sl = 2; sl <= 16 && sl * 8 <= stepsAll; ++sl) {
                const size_t rounds = (t * sl + cus - 1) / cus;
                const double gemmUs = double(rounds) * double((stepsAll + sl - 1) / sl) * 1.4 * (form == 0 ? 1.0 : kHalfTileCost);
                const double reduceUs = double(sl + 1) * double(M * N) * 2.0 * sizeof(float) / 4e6;
                if (gemmUs + reduceUs < best) { best = gemmUs + reduceUs; bestSlices = sl; bestTiles = t; bestForm = form; }
            }
        }
        if (bestSlices > 1 && bestTiles * bestSlices >= cus / 2) {
            const size_t kPer = (stepsAll + bestSlices - 1) / bestSlices * BKK;
            const size_t sl = (K + kPer - 1) / kPer;
            const size_t count = M * N, sliceStride = (count + 3) / 4 * 4;
            Scratch partial(sl * sliceStride * sizeof(float));
            if (partial.status != BF_OK) return partial.status;
            Epilogue plain{{partial.as<float>(), nullptr, nullptr}, int(N), nullptr, nullptr};
            int st = bestForm == 0 ? launchPingPong<256>(A, Bt, plain, M, N, K, lda, ldb, s, sl, kPer, sliceStride, false)
                                   : launchPingPong<128>(A, Bt, plain, M, N, K, lda, ldb, s, sl, kPer, sliceStride, false);
            if (st != BF_OK) return st;
            const int vec = ((reinterpret_cast<uintptr_t>(epi.c[0]) | reinterpret_cast<uintptr_t>(epi.c[1]) |
                              reinterpret_cast<uintptr_t>(epi.c[2]) | reinterpret_cast<uintptr_t>(epi.residual) |
                              reinterpret_cast<uintptr_t>(epi.bias)) & 15u) == 0 && N % 4 == 0 && epi.splitN % 4 == 0;
            splitReduceKernel<<<gridFor(count / 4 + 1, kBlock), kBlock, 0, s>>>(partial.as<float>(), epi, count, sliceStride, int(sl), vec, N);
            BF_LAUNCH_CHECK();
            return BF_OK;
        }
    }
    const size_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    constexpr size_t smem = size_t(2) * (128 + 128) * LDS_ROW * sizeof(unsigned short);
    auto kernel = gemmBf16NtKernel<128, 128, 2, 2>;
    int st = allowSharedMemory(kernel, smem);
    if (st != BF_OK) return st;
    size_t slices = 1;
    if (tiles < cus && K >= 2048) slices = std::min<size_t>(std::min<size_t>(8, (2 * cus) / tiles), K / 1024);
    if (slices > 1) {
        const size_t steps = (K + BKK - 1) / BKK;
        const size_t kPer = (steps + slices - 1) / slices * BKK;
        slices = (K + kPer - 1) / kPer;
        const size_t count = M * N, sliceStride = (count + 3) / 4 * 4;
        Scratch partial(slices * sliceStride * sizeof(float));
        if (partial.status != BF_OK) return partial.status;
        Epilogue plain{{partial.as<float>(), nullptr, nullptr}, int(N), nullptr, nullptr};
        kernel<<<dim3(unsigned(tiles), unsigned(slices)), 256, smem, s>>>(A, Bt, plain, int(M), int(N), int(K), int(lda), int(ldb),
                                                                         int(kPer), sliceStride);
        BF_LAUNCH_CHECK();
        const int vec = ((reinterpret_cast<uintptr_t>(epi.c[0]) | reinterpret_cast<uintptr_t>(epi.c[1]) |
                          reinterpret_cast<uintptr_t>(epi.c[2]) | reinterpret_cast<uintptr_t>(epi.residual) |
                          reinterpret_cast<uintptr_t>(epi.bias)) & 15u) == 0 && N % 4 == 0 && epi.splitN % 4 == 0;
        splitReduceKernel<<<gridFor(count / 4 + 1, kBlock), kBlock, 0, s>>>(partial.as<float>(), epi, count, sliceStride, int(slices),
                                                                          vec, N);
        BF_LAUNCH_CHECK();
        return BF_OK;
    }
    kernel<<<dim3(unsigned(tiles), 1), 256, smem, s>>>(A, Bt, epi, int(M), int(N), int(K), int(lda), int(ldb), int(K), size_t(0));
    BF_LAUNCH_CHECK();
    return BF_OK;
}
int launchGemmNt(const unsigned short* A, const unsigned short* Bt, float* C, size_t M, size_t N, size_t K, size_t lda,
                 size_t ldb, hipStream_t s) {
    return launchGemmNt(A, Bt, Epilogue{{C, nullptr, nullptr}, int(N), nullptr, nullptr}, M, N, K, lda, ldb, s);
}

// ld: elements between rows of `out` (0 = pad8(cols), a dense image); with ld > pad8(cols) the image is a column
// slice of a wider one.
int convertPlain(const float* x, unsigned short* out, size_t rows, size_t cols, hipStream_t s, size_t ld = 0) {
    size_t colsPad = pad8(cols);
    size_t groups = rows * (colsPad / 8);
    if (groups == 0) return BF_OK;
    if (streamsPastCache(rows * cols * 6)) convertKernel<true><<<gridFor(groups, kBlock), kBlock, 0, s>>>(x, out, rows, cols, colsPad, ld ? ld : colsPad);
    else convertKernel<false><<<gridFor(groups, kBlock), kBlock, 0, s>>>(x, out, rows, cols, colsPad, ld ? ld : colsPad);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

// plain / ldPlain: optional second output, the untransposed image with row stride ldPlain (a multiple of 8).
// `count` matrices (at most three) of one shape in one launch: matrix i goes to out + i * outStep and plain + i * plainStep.
int convertTransposedGroup(const float* const* x, size_t count, unsigned short* out, size_t outStep, size_t rows, size_t cols, hipStream_t s,
                           bool padRows, unsigned short* plain, size_t ldPlain, size_t plainStep) {
    if (rows == 0 || cols == 0 || count == 0) return BF_OK;
    size_t rowsPad = padRows ? pad8(rows) : rows;   // length of an output row
    // the grid covers pad8(cols) columns so that the plain image's zero padding is written too
    dim3 grid(unsigned(((plain ? pad8(cols) : cols) + 63) / 64), unsigned((rowsPad + 63) / 64), unsigned(count));
    if (grid.y > 65535) return failInvalid("cvt_f32_bf16_transpose", "too many rows");
    ConvertSources xs{{x[0], count > 1 ? x[1] : nullptr, count > 2 ? x[2] : nullptr}};
    // the sources need no alignment beyond a float's and rows of any length do (16-byte loads from any 4-byte boundary)
    uintptr_t outBits = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(plain) | (outStep * 2) | (plainStep * 2);
    const int vec = (outBits & 15u) == 0 && rowsPad % 8 == 0 && ldPlain % 8 == 0;
    convertTransposeKernel<<<grid, kBlock, 0, s>>>(xs, out, rows, cols, rowsPad, vec, plain, ldPlain, outStep, plainStep);
    BF_LAUNCH_CHECK();
    return BF_OK;
}
int convertTransposed(const float* x, unsigned short* out, size_t rows, size_t cols, hipStream_t s, bool padRows = true,
                      unsigned short* plain = nullptr, size_t ldPlain = 0) {
    return convertTransposedGroup(&x, 1, out, 0, rows, cols, s, padRows, plain, ldPlain, 0);
}

// out[c, r] = in[r, c] for a bf16 image `in` [rows, ldIn] (cols columns used); `out` is [cols, ldOut] with ldOut >= rows,
// columns rows..ldOut-1 zero.
__global__ void __launch_bounds__(kBlock) transposeBf16Kernel(const unsigned short* __restrict__ in, unsigned short* __restrict__ out,
                                                              size_t rows, size_t cols, size_t ldIn, size_t ldOut) {
    __shared__ unsigned short tile[64][66];
    const size_t r0 = size_t(blockIdx.y) * 64, c0 = size_t(blockIdx.x) * 64;
    for (int i = threadIdx.x; i < 4096; i += kBlock) {
        const int r = i >> 6, c = i & 63;
        tile[r][c] = (r0 + r < rows && c0 + c < cols) ? in[(r0 + r) * ldIn + c0 + c] : static_cast<unsigned short>(0);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 4096; i += kBlock) {
        const int c = i >> 6, r = i & 63;
        if (c0 + c < cols && r0 + r < ldOut) out[(c0 + c) * ldOut + r0 + r] = tile[r][c];
    }
}
int transposeImage(const unsigned short* in, unsigned short* out, size_t rows, size_t cols, size_t ldIn, size_t ldOut, hipStream_t s) {
    dim3 grid(unsigned((cols + 63) / 64), unsigned((ldOut + 63) / 64));
    if (grid.y > 65535) return failInvalid("feedforward_bf16", "too many rows");
    transposeBf16Kernel<<<grid, kBlock, 0, s>>>(in, out, rows, cols, ldIn, ldOut);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

// ---- bf16 images of weights, kept per (device, pointers, layout) until invalidated ------------------
// Layouts: 0 plain [rows, pad8(cols)]; 1 transposed [cols, pad8(rows)]; for a group of up to three weights of one
// shape, 2 = their transposed images stacked row-wise ([count*cols, pad8(rows)], the Bt operand of one GEMM that
// produces all their products) and 3 = their plain images side by side ([rows, count*cols], the Bt operand of
// the one GEMM that sums their input gradients).
struct CachedWeight {
    size_t generation;   // the generation whose weights the image holds; 0 = never filled
    void* buffer;
    size_t bytes;
    size_t count, rows, cols;   // the weights behind the image: `count` matrices [rows, cols]
};
// One generation per cache: an invalidation recorded into a graph must not mark the eager images stale, and the eager
// generation also advances whenever a recorded graph is launched (its kernels may step an optimizer over the weights
// whose images the eager cache holds: noteGraphLaunched).
size_t g_generationEager = 1, g_generationCaptured = 1;
size_t& generation() { return capturing() ? g_generationCaptured : g_generationEager; }
using WeightKey = std::tuple<int, const float*, const float*, const float*, int>;
// While a graph is being captured the images live in a cache of their own, filled and emptied inside the capture: the
// recorded conversions and products address arena blocks that no later eager call can be handed.
std::map<WeightKey, CachedWeight>& weightCache() {
    static std::map<WeightKey, CachedWeight> eager, captured;
    return capturing() ? captured : eager;
}

// `plain`: for the transposed layouts (1, 2) the plain counterpart (0, 3) written in the same pass, or NULL.
int fillWeightImage(const float* const* w, size_t count, size_t rows, size_t cols, int layout, unsigned short* image, unsigned short* plain,
                    hipStream_t s) {
    if (layout == 2 && count <= 3)   // the stacked transposed images of a group (and their plain ones side by side) in one launch
        return convertTransposedGroup(w, count, image, cols * pad8(rows), rows, cols, s, true, plain, count * cols, cols);
    int st = BF_OK;
    for (size_t i = 0; i < count && st == BF_OK; ++i) {
        if (layout == 0) st = convertPlain(w[i], image, rows, cols, s);
        else if (layout == 1) st = convertTransposed(w[i], image, rows, cols, s, true, plain, pad8(cols));
        else if (layout == 2) st = convertTransposed(w[i], image + i * cols * pad8(rows), rows, cols, s, true, plain ? plain + i * cols : nullptr, count * cols);
        else st = convertPlain(w[i], image + i * cols, rows, cols, s, count * cols);   // cols % 8 == 0 checked by the caller
    }
    return st;
}

size_t weightImageBytes(size_t count, size_t rows, size_t cols, int layout) {
    return ((layout == 0 || layout == 3) ? rows * pad8(cols) * count : count * cols * pad8(rows)) * sizeof(unsigned short);
}

// The cache entry of `key` with a buffer of `bytes` (acquired, or re-acquired when the size changed); its generation
// says whether the buffer's contents are current.  Entries stay where they are in the map, so the pointer holds.
int cacheSlot(const WeightKey& key, size_t count, size_t rows, size_t cols, CachedWeight** slot) {
    const size_t bytes = weightImageBytes(count, rows, cols, std::get<4>(key));
    auto& cache = weightCache();
    auto it = cache.find(key);
    if (it != cache.end() && it->second.bytes != bytes) {
        bf_hip_pool_release(it->second.buffer, it->second.bytes);
        cache.erase(it);
        it = cache.end();
    }
    if (it == cache.end()) {
        void* buf = nullptr;
        int st = bf_hip_pool_acquire(bytes, &buf);
        if (st != BF_OK) return st;
        it = cache.emplace(key, CachedWeight{0, buf, bytes, count, rows, cols}).first;
    }
    it->second.count = count;   // (equal bytes do not pin the shape)
    it->second.rows = rows;
    it->second.cols = cols;
    *slot = &it->second;
    return BF_OK;
}

// Returns the bf16 image of `count` weights w[i][rows, cols] in `layout`.  With `cache` the image is kept;
// otherwise it is a scratch buffer the caller releases with bf_hip_pool_release(image, bytes).  A cached transposed
// image (the forward operand) is filled together with its plain counterpart (the operand of the input-gradient
// product of the same weights), one pass over the fp32 weights for both.  An entry is marked current only once its
// conversion has been launched, so a failed launch is never served as an image.
int weightImage(const float* const* w, size_t count, size_t rows, size_t cols, int layout, bool cache, hipStream_t s,
                unsigned short** image, size_t* imageBytes) {
    const size_t bytes = weightImageBytes(count, rows, cols, layout);
    *imageBytes = bytes;
    if (!cache) {
        void* buf = nullptr;
        int st = bf_hip_pool_acquire(bytes, &buf);
        if (st != BF_OK) return st;
        st = fillWeightImage(w, count, rows, cols, layout, static_cast<unsigned short*>(buf), nullptr, s);
        if (st != BF_OK) {
            bf_hip_pool_release(buf, bytes);
            return st;
        }
        *image = static_cast<unsigned short*>(buf);
        return BF_OK;
    }
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    const float* w1 = count > 1 ? w[1] : nullptr;
    const float* w2 = count > 2 ? w[2] : nullptr;
    CachedWeight* slot = nullptr;
    int st = cacheSlot(WeightKey{dev, w[0], w1, w2, layout}, count, rows, cols, &slot);
    if (st != BF_OK) return st;
    *image = static_cast<unsigned short*>(slot->buffer);
    if (slot->generation == generation()) return BF_OK;
    CachedWeight* mate = nullptr;
    if (layout == 1 || (layout == 2 && cols % 8 == 0)) {
        const int mateLayout = layout == 1 ? 0 : 3;
        st = cacheSlot(WeightKey{dev, w[0], w1, w2, mateLayout}, count, rows, cols, &mate);
        if (st != BF_OK) return st;
        if (mate->generation == generation()) mate = nullptr;   // already current
    }
    st = fillWeightImage(w, count, rows, cols, layout, *image, mate ? static_cast<unsigned short*>(mate->buffer) : nullptr, s);
    if (st != BF_OK) return st;
    slot->generation = generation();
    if (mate) mate->generation = generation();
    return BF_OK;
}
int weightImage(const float* w, size_t rows, size_t cols, bool transposed, bool cache, hipStream_t s, unsigned short** image,
                size_t* imageBytes) {
    return weightImage(&w, 1, rows, cols, transposed ? 1 : 0, cache, s, image, imageBytes);
}


// After an optimizer step over `changed`: every transposed image (with its plain mate) that was in use during the
// generation that just ended and whose weights are all among `changed` is made again, all of them in one launch, and
// is current in the new generation.  The caller has already advanced the generation.
int refreshImagesOf(const float* const* changed, size_t count, size_t ending, hipStream_t s) {
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    const std::set<const float*> touched(changed, changed + count);
    auto& cache = weightCache();
    std::vector<ConvertEntry> table;
    std::vector<CachedWeight*> made;
    size_t blocks = 0;
    for (auto& [key, slot] : cache) {
        const int layout = std::get<4>(key);
        if (std::get<0>(key) != dev || (layout != 1 && layout != 2) || slot.generation != ending) continue;
        const float* w[3] = {std::get<1>(key), std::get<2>(key), std::get<3>(key)};
        bool all = slot.count >= 1 && slot.count <= 3;
        for (size_t i = 0; i < slot.count && all; ++i) all = w[i] != nullptr && touched.count(w[i]) != 0;
        if (!all || slot.rows >= (size_t(1) << 31) || slot.cols >= (size_t(1) << 31)) continue;
        CachedWeight* mate = nullptr;
        if (layout == 1 || slot.cols % 8 == 0) {
            auto it = cache.find(WeightKey{dev, w[0], w[1], w[2], layout == 1 ? 0 : 3});
            if (it != cache.end() && it->second.generation == ending && it->second.rows == slot.rows && it->second.cols == slot.cols &&
                it->second.count == slot.count)
                mate = &it->second;
        }
        const size_t rowsPad = pad8(slot.rows);
        const size_t ldPlain = layout == 1 ? pad8(slot.cols) : slot.count * slot.cols;
        for (size_t i = 0; i < slot.count; ++i) {
            unsigned short* out = static_cast<unsigned short*>(slot.buffer) + i * slot.cols * rowsPad;
            unsigned short* plain = mate ? static_cast<unsigned short*>(mate->buffer) + i * slot.cols : nullptr;
            const size_t tilesX = ((plain ? pad8(slot.cols) : slot.cols) + 63) / 64, tilesY = (rowsPad + 63) / 64;
            const int vec = ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(plain)) & 15u) == 0 && ldPlain % 8 == 0;
            table.push_back(ConvertEntry{w[i], out, plain, unsigned(slot.rows), unsigned(slot.cols), unsigned(rowsPad), unsigned(ldPlain),
                                         unsigned(blocks), unsigned(tilesX), vec, 0});
            blocks += tilesX * tilesY;
            if (blocks >= (size_t(1) << 31)) return failInvalid("bf16_weight_cache_refresh", "too many elements for one launch");
        }
        made.push_back(&slot);
        if (mate) made.push_back(mate);
    }
    // plain images in use without a transposed one (the input-gradient product of weights whose forward pass took
    // another form): the same kernel, writing the plain image only
    for (auto& [key, slot] : cache) {
        const int layout = std::get<4>(key);
        if (std::get<0>(key) != dev || (layout != 0 && layout != 3) || slot.generation != ending) continue;
        if (std::find(made.begin(), made.end(), &slot) != made.end()) continue;
        const float* w[3] = {std::get<1>(key), std::get<2>(key), std::get<3>(key)};
        bool all = slot.count >= 1 && slot.count <= 3;
        for (size_t i = 0; i < slot.count && all; ++i) all = w[i] != nullptr && touched.count(w[i]) != 0;
        if (!all || slot.rows >= (size_t(1) << 31) || slot.cols >= (size_t(1) << 31)) continue;
        const size_t ldPlain = layout == 0 ? pad8(slot.cols) : slot.count * slot.cols;
        for (size_t i = 0; i < slot.count; ++i) {
            unsigned short* plain = static_cast<unsigned short*>(slot.buffer) + i * slot.cols;
            const size_t tilesX = (pad8(slot.cols) + 63) / 64, tilesY = (slot.rows + 63) / 64;
            const int vec = (reinterpret_cast<uintptr_t>(plain) & 15u) == 0 && ldPlain % 8 == 0;
            table.push_back(ConvertEntry{w[i], nullptr, plain, unsigned(slot.rows), unsigned(slot.cols), unsigned(pad8(slot.rows)),
                                         unsigned(ldPlain), unsigned(blocks), unsigned(tilesX), vec, 0});
            blocks += tilesX * tilesY;
            if (blocks >= (size_t(1) << 31)) return failInvalid("bf16_weight_cache_refresh", "too many elements for one launch");
        }
        made.push_back(&slot);
    }
    if (blocks == 0) return BF_OK;
    const void* device = nullptr;
    int st = uploadDescriptorTable(kSlotConvert, table.data(), table.size() * sizeof(ConvertEntry), s, &device);
    if (st != BF_OK) return st;
    convertTransposeMultiKernel<<<unsigned(blocks), kBlock, 0, s>>>(static_cast<const ConvertEntry*>(device), int(table.size()));
    BF_LAUNCH_CHECK();
    for (CachedWeight* slot : made) slot->generation = generation();
    return BF_OK;
}

}  // namespace

void noteGraphLaunched() { ++g_generationEager; }

void dropCaptureWeightImages() {
    if (!capturing()) return;
    auto& cache = weightCache();
    for (auto& entry : cache) bf_hip_pool_release(entry.second.buffer, entry.second.bytes);
    cache.clear();
}
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

int bf_hip_gemm_bf16_tn(const uint16_t* A, const uint16_t* B, float* C, size_t M, size_t N, size_t K, bf_stream_t stream) {
    if (M == 0 || N == 0) return BF_OK;
    BF_REQUIRE(C != nullptr, "NULL output");
    if (K == 0) return bf_hip_fill_zero(C, M * N * sizeof(float), stream);
    BF_REQUIRE(A && B, "NULL operand");
    BF_REQUIRE(M % 8 == 0 && N % 8 == 0, "M and N must be multiples of 8 (16-byte operand rows)");
    BF_REQUIRE(((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15u) == 0, "operands must be 16-byte aligned");
    bool done = false;
    int st = launchGemmTn(A, B, Epilogue{{C, nullptr, nullptr}, int(N), nullptr, nullptr}, M, N, K, M, N, asStream(stream), &done);
    if (st != BF_OK || done) return st;
    gemmBf16TnSmallKernel<<<gridFor(M * N, kBlock, 1u << 30), kBlock, 0, asStream(stream)>>>(A, B, C, M, N, K, M, N);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_matmul_bf16(const float* a, const float* b, float* c, size_t m, size_t k, size_t n, int cacheWeight,
                       bf_stream_t stream) {
    return bf_hip_linear_bf16_img(a, nullptr, b, nullptr, nullptr, c, m, k, n, cacheWeight, stream);
}

int bf_hip_matmul_bf16_backward_img(const float* a, const uint16_t* aImage, const float* b, const float* g, const uint16_t* gImage,
                                    float* dA, float* dB, size_t m, size_t k, size_t n, int cacheWeight, bf_stream_t stream) {
    hipStream_t s = asStream(stream);
    if (m == 0 || k == 0 || n == 0) {   // degenerate: gradients are zero (ops_tensorcore.cu:412-415)
        int st = BF_OK;
        if (dA && m * k) st = bf_hip_fill_zero(dA, m * k * sizeof(float), stream);
        if (st == BF_OK && dB && k * n) st = bf_hip_fill_zero(dB, k * n * sizeof(float), stream);
        return st;
    }
    BF_REQUIRE((a || aImage || !dB) && b && (g || gImage), "NULL operand");
    BF_REQUIRE(((reinterpret_cast<uintptr_t>(aImage) | reinterpret_cast<uintptr_t>(gImage)) & 15u) == 0, "operand images must be 16-byte aligned");
    int st = BF_OK;
    const size_t mp = pad8(m), np = pad8(n), kp = pad8(k);
    // dB = a^T g contracts over the rows of both operands.  When the product is big enough for the large-tile kernel
    // that transposes fragments on their way out of LDS, both operands are used as they lie (g's plain image also
    // serves dA); otherwise transposed images are built and the row-by-row kernel is used.
    int form = 0;
    size_t slices = 1;
    const bool transposeInLds = dB != nullptr && planLargeTiles(k, n, m, &form, &slices);
    const bool needPlainG = dA || transposeInLds || (dB && !g);   // without the fp32 gradient its transposed image comes from the plain one
    Scratch gT(dB && !transposeInLds ? n * mp * sizeof(unsigned short) : 0);
    if (gT.status != BF_OK) return gT.status;
    Scratch gImg(needPlainG && !gImage ? m * np * sizeof(unsigned short) : 0);
    if (gImg.status != BF_OK) return gImg.status;
    bool gTransposed = false;
    if (needPlainG && !gImage) {
        // with both gradients wanted on the transposed-image route, one pass over g writes the plain and the transposed image
        if (dB && !transposeInLds) { st = convertTransposed(g, gT.as<unsigned short>(), m, n, s, true, gImg.as<unsigned short>(), np); gTransposed = true; }
        else st = convertPlain(g, gImg.as<unsigned short>(), m, n, s);
        if (st != BF_OK) return st;
        gImage = gImg.as<unsigned short>();
    }
    if (dA) {   // dA[m,k] = g[m,n] * b[k,n]^T : contraction over n
        unsigned short* bImg = nullptr;
        size_t bBytes = 0;
        st = weightImage(b, k, n, /*transposed=*/false, cacheWeight != 0, s, &bImg, &bBytes);
        if (st != BF_OK) return st;
        st = launchGemmNt(gImage, bImg, dA, m, k, np, np, np, s);
        if (!cacheWeight) bf_hip_pool_release(bImg, bBytes);
        if (st != BF_OK) return st;
    }
    if (dB && transposeInLds) {
        Scratch aImg(aImage ? 0 : m * kp * sizeof(unsigned short));
        if (aImg.status != BF_OK) return aImg.status;
        if (!aImage) {
            st = convertPlain(a, aImg.as<unsigned short>(), m, k, s);
            if (st != BF_OK) return st;
            aImage = aImg.as<unsigned short>();
        }
        bool done = false;
        return launchGemmTn(aImage, gImage, Epilogue{{dB, nullptr, nullptr}, int(n), nullptr, nullptr}, k, n, m, kp, np, s, &done);
    }
    if (dB) {   // dB[k,n] = a[m,k]^T * g[m,n] : contraction over m
        Scratch aT(k * mp * sizeof(unsigned short));
        if (aT.status != BF_OK) return aT.status;
        st = a ? convertTransposed(a, aT.as<unsigned short>(), m, k, s) : transposeImage(aImage, aT.as<unsigned short>(), m, k, kp, mp, s);
        if (st != BF_OK) return st;
        if (!gTransposed) st = g ? convertTransposed(g, gT.as<unsigned short>(), m, n, s) : transposeImage(gImage, gT.as<unsigned short>(), m, n, np, mp, s);
        if (st != BF_OK) return st;
        st = launchGemmNt(aT.as<unsigned short>(), gT.as<unsigned short>(), dB, k, n, mp, mp, mp, s);
    }
    return st;
}

int bf_hip_matmul_bf16_backward(const float* a, const float* b, const float* g, float* dA, float* dB, size_t m,
                                size_t k, size_t n, int cacheWeight, bf_stream_t stream) {
    if (m != 0 && k != 0 && n != 0) BF_REQUIRE(a && g, "NULL operand");
    return bf_hip_matmul_bf16_backward_img(a, nullptr, b, g, nullptr, dA, dB, m, k, n, cacheWeight, stream);
}

int bf_hip_linear_bf16_img(const float* a, const uint16_t* aImage, const float* w, const float* bias, const float* residual, float* out,
                           size_t m, size_t k, size_t n, int cacheWeight, bf_stream_t stream) {
    if (m == 0 || n == 0) return BF_OK;
    BF_REQUIRE(out != nullptr, "NULL output");
    int st = BF_OK;
    if (k == 0) {   // empty contraction: out = bias + residual
        st = bf_hip_fill_zero(out, m * n * sizeof(float), stream);
        if (st == BF_OK && bias) st = bf_hip_add_bias(out, bias, out, m, n, stream);
        if (st == BF_OK && residual) st = bf_hip_accumulate(out, residual, m * n, stream);
        return st;
    }
    BF_REQUIRE((a || aImage) && w, "NULL operand");
    BF_REQUIRE((reinterpret_cast<uintptr_t>(aImage) & 15u) == 0, "operand images must be 16-byte aligned");
    hipStream_t s = asStream(stream);
    const size_t kp = pad8(k);
    Scratch aImg(aImage ? 0 : m * kp * sizeof(unsigned short));
    if (aImg.status != BF_OK) return aImg.status;
    unsigned short* wImg = nullptr;
    size_t wBytes = 0;
    if (!aImage) {
        st = convertPlain(a, aImg.as<unsigned short>(), m, k, s);
        if (st != BF_OK) return st;
        aImage = aImg.as<unsigned short>();
    }
    st = weightImage(w, k, n, /*transposed=*/true, cacheWeight != 0, s, &wImg, &wBytes);
    if (st != BF_OK) return st;
    st = launchGemmNt(aImage, wImg, Epilogue{{out, nullptr, nullptr}, int(n), bias, residual}, m, n, kp, kp, kp, s);
    if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
    return st;
}

int bf_hip_linear_bf16(const float* a, const float* w, const float* bias, const float* residual, float* out, size_t m, size_t k,
                       size_t n, int cacheWeight, bf_stream_t stream) {
    if (m != 0 && n != 0 && k != 0) BF_REQUIRE(a != nullptr, "NULL operand");
    return bf_hip_linear_bf16_img(a, nullptr, w, bias, residual, out, m, k, n, cacheWeight, stream);
}

int bf_hip_matmul_bf16_shared_input(const float* a, const float* const* b, float* const* c, size_t count, size_t m, size_t k,
                                    size_t n, int cacheWeight, bf_stream_t stream) {
    if (m != 0 && n != 0 && k != 0) BF_REQUIRE(a != nullptr, "NULL operand");
    return bf_hip_matmul_bf16_shared_input_img(a, nullptr, b, c, count, m, k, n, cacheWeight, stream);
}

int bf_hip_matmul_bf16_shared_input_img(const float* a, const uint16_t* aImage, const float* const* b, float* const* c, size_t count,
                                        size_t m, size_t k, size_t n, int cacheWeight, bf_stream_t stream) {
    BF_REQUIRE(count >= 1 && count <= 3, "count must be 1, 2 or 3");
    BF_REQUIRE(b && c, "NULL pointer array");
    if (m == 0 || n == 0) return BF_OK;
    for (size_t i = 0; i < count; ++i) BF_REQUIRE(c[i] != nullptr, "NULL output");
    if (k == 0) {
        for (size_t i = 0; i < count; ++i) {
            int st = bf_hip_fill_zero(c[i], m * n * sizeof(float), stream);
            if (st != BF_OK) return st;
        }
        return BF_OK;
    }
    BF_REQUIRE(a != nullptr || aImage != nullptr, "NULL operand");
    BF_REQUIRE((reinterpret_cast<uintptr_t>(aImage) & 15u) == 0, "operand images must be 16-byte aligned");
    for (size_t i = 0; i < count; ++i) BF_REQUIRE(b[i] != nullptr, "NULL operand");
    hipStream_t s = asStream(stream);
    const size_t kp = pad8(k);
    Scratch aImg(aImage ? 0 : m * kp * sizeof(unsigned short));
    if (aImg.status != BF_OK) return aImg.status;
    int st = BF_OK;
    if (!aImage) {
        st = convertPlain(a, aImg.as<unsigned short>(), m, k, s);
        if (st != BF_OK) return st;
        aImage = aImg.as<unsigned short>();
    }
    unsigned short* wImg = nullptr;
    size_t wBytes = 0;
    if (count > 1 && n % 256 == 0) {   // one GEMM over the stacked weight images, tiles routed to their output
        st = weightImage(b, count, k, n, 2, cacheWeight != 0, s, &wImg, &wBytes);
        if (st != BF_OK) return st;
        Epilogue epi{{c[0], count > 1 ? c[1] : nullptr, count > 2 ? c[2] : nullptr}, int(n), nullptr, nullptr};
        st = launchGemmNt(aImage, wImg, epi, m, count * n, kp, kp, kp, s);
        if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
        return st;
    }
    for (size_t i = 0; i < count; ++i) {
        st = weightImage(b[i], k, n, /*transposed=*/true, cacheWeight != 0, s, &wImg, &wBytes);
        if (st != BF_OK) return st;
        st = launchGemmNt(aImage, wImg, c[i], m, n, kp, kp, kp, s);
        if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
        if (st != BF_OK) return st;
    }
    return BF_OK;
}

// c[i] = bf16(rmsnorm(x)) b[i]: the projections of an attention block's normalised input (ops_transformer.cu:217-232) for
// a caller that keeps nothing for a backward pass.  One or two rows: the normalisation is made by the product's own
// kernel while it stages the rows (one launch); otherwise the row kernel writes the image and the products follow.
int bf_hip_rmsnorm_matmul_bf16_shared_input(const float* x, const float* const* b, float* const* c, size_t count, size_t m, size_t k, size_t n,
                                            int cacheWeight, bf_stream_t stream) {
    BF_REQUIRE(count >= 1 && count <= 3, "count must be 1, 2 or 3");
    BF_REQUIRE(b && c, "NULL pointer array");
    if (m == 0 || n == 0) return BF_OK;
    BF_REQUIRE(k > 0 && x != nullptr, "NULL or empty input");
    for (size_t i = 0; i < count; ++i) BF_REQUIRE(b[i] != nullptr && c[i] != nullptr, "NULL operand");
    hipStream_t s = asStream(stream);
    const bool stacked = count == 1 || n % 256 == 0;
    if (stacked && fewRowsNormalise(m, k)) {
        unsigned short* wImg = nullptr;
        size_t wBytes = 0;
        int st = count > 1 ? weightImage(b, count, k, n, 2, cacheWeight != 0, s, &wImg, &wBytes)
                           : weightImage(b[0], k, n, /*transposed=*/true, cacheWeight != 0, s, &wImg, &wBytes);
        if (st != BF_OK) return st;
        Epilogue epi{{c[0], count > 1 ? c[1] : nullptr, count > 2 ? c[2] : nullptr}, int(n), nullptr, nullptr};
        epi.normInput = x;
        st = fewRowsServe(nullptr, wImg, 0, m, k, k, k) ? launchGemmNt(nullptr, wImg, epi, m, count * n, k, k, k, s)
                                                        : failInvalid(__func__, "unaligned weight image");
        if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
        return st;
    }
    const size_t kp = pad8(k);
    Scratch image(m * kp * sizeof(unsigned short));
    if (image.status != BF_OK) return image.status;
    int st = bf_hip_rmsnorm_img(x, nullptr, image.as<uint16_t>(), m, k, stream);
    if (st != BF_OK) return st;
    return bf_hip_matmul_bf16_shared_input_img(nullptr, image.as<uint16_t>(), b, c, count, m, k, n, cacheWeight, stream);
}

// The projections of a decoding step whose position lives on the device: q = bf16(rmsnorm(x)) wq, and the rows of
// bf16(rmsnorm(x)) wk and ... wv appended to caches of `capacity` rows a sequence at row *position.  One sequence of one or
// two new rows, width a multiple of 256: one launch (the few-row kernel normalises, multiplies and stores the keys and
// values where they belong); anything else: the products into scratch rows, then bf_hip_kv_append_indirect.
int bf_hip_decode_projections_bf16(const float* x, const float* wq, const float* wk, const float* wv, float* q, float* kCache, float* vCache,
                                   size_t batch, size_t newLen, size_t dim, size_t capacity, const int* position, int cacheWeight,
                                   bf_stream_t stream) {
    if (batch == 0 || newLen == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(x && wq && wk && wv && q && kCache && vCache && position, "NULL pointer");
    BF_REQUIRE(newLen <= capacity && capacity < (size_t(1) << 31), "more new rows than the cache holds");
    hipStream_t s = asStream(stream);
    const size_t rows = batch * newLen;
    const float* weights[3] = {wq, wk, wv};
    if (batch == 1 && dim % 256 == 0 && fewRowsNormalise(rows, dim)) {
        unsigned short* wImg = nullptr;
        size_t wBytes = 0;
        int st = weightImage(weights, 3, dim, dim, 2, cacheWeight != 0, s, &wImg, &wBytes);
        if (st != BF_OK) return st;
        Epilogue epi{{q, kCache, vCache}, int(dim), nullptr, nullptr};
        epi.normInput = x;
        epi.rowShift = position;
        epi.rowLimit = int(capacity);
        st = fewRowsServe(nullptr, wImg, 0, rows, dim, dim, dim) ? launchGemmNt(nullptr, wImg, epi, rows, 3 * dim, dim, dim, dim, s)
                                                                 : failInvalid(__func__, "unaligned weight image");
        if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
        return st;
    }
    Scratch fresh(2 * rows * dim * sizeof(float));
    if (fresh.status != BF_OK) return fresh.status;
    float* outs[3] = {q, fresh.as<float>(), fresh.as<float>() + rows * dim};
    int st = bf_hip_rmsnorm_matmul_bf16_shared_input(x, weights, outs, 3, rows, dim, dim, cacheWeight, stream);
    if (st != BF_OK) return st;
    return bf_hip_kv_append_indirect(kCache, vCache, outs[1], outs[2], batch, newLen, dim, capacity, position, stream);
}

// out = input + act(bf16(rmsnorm(input)) w1 + b1) w2 + b2: the feed-forward block (ops_transformer.cu:182-215) for a
// caller that keeps nothing for a backward pass (incremental decoding).  One or two rows: two launches, the
// normalisation made while the first product stages its rows and the activation in its store.
int bf_hip_rmsnorm_feedforward_bf16(const float* input, const float* w1, const float* b1, const float* w2, const float* b2, int act, float* out,
                                    size_t m, size_t d, size_t hidden, int cacheWeight, bf_stream_t stream) {
    if (m == 0) return BF_OK;
    BF_REQUIRE(d > 0 && hidden > 0 && d % 8 == 0 && hidden % 8 == 0, "d and hidden must be positive multiples of 8");
    BF_REQUIRE(act == BF_ACT_SILU || act == BF_ACT_GELU || act == BF_ACT_RELU, "unknown activation");
    BF_REQUIRE(input && w1 && w2 && out, "NULL pointer");
    hipStream_t s = asStream(stream);
    Scratch z(m * hidden * sizeof(float)), hImage(m * hidden * sizeof(unsigned short));
    if (z.status != BF_OK) return z.status;
    if (hImage.status != BF_OK) return hImage.status;
    if (fewRowsNormalise(m, d) && fewRowsServe(nullptr, nullptr, 0, m, hidden, hidden, hidden) && (reinterpret_cast<uintptr_t>(b1) & 15u) == 0) {
        unsigned short* wImg = nullptr;
        size_t wBytes = 0;
        int st = weightImage(w1, d, hidden, /*transposed=*/true, cacheWeight != 0, s, &wImg, &wBytes);
        if (st != BF_OK) return st;
        Epilogue first{{z.as<float>(), nullptr, nullptr}, int(hidden), b1, nullptr};
        first.fuse = 1; first.act = act; first.image = hImage.as<unsigned short>();
        first.normInput = input;
        st = launchGemmNt(nullptr, wImg, first, m, hidden, d, d, d, s);
        if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
        if (st != BF_OK) return st;
        st = weightImage(w2, hidden, d, /*transposed=*/true, cacheWeight != 0, s, &wImg, &wBytes);
        if (st != BF_OK) return st;
        st = launchGemmNt(hImage.as<unsigned short>(), wImg, Epilogue{{out, nullptr, nullptr}, int(d), b2, input}, m, d, hidden, hidden, hidden, s);
        if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
        return st;
    }
    Scratch xImage(m * d * sizeof(unsigned short));
    if (xImage.status != BF_OK) return xImage.status;
    int st = bf_hip_rmsnorm_img(input, nullptr, xImage.as<uint16_t>(), m, d, stream);
    if (st != BF_OK) return st;
    return bf_hip_feedforward_bf16(nullptr, w1, b1, w2, b2, input, act, z.as<float>(), hImage.as<uint16_t>(), xImage.as<uint16_t>(), out, m, d, hidden,
                                   cacheWeight, stream);
}

int bf_hip_matmul_bf16_shared_input_backward(const float* a, const float* const* b, const float* const* g, float* dA,
                                             float* const* dB, size_t count, size_t m, size_t k, size_t n, int cacheWeight,
                                             bf_stream_t stream) {
    BF_REQUIRE(g != nullptr, "NULL pointer array");
    if (m != 0 && k != 0 && n != 0) {
        BF_REQUIRE(a != nullptr, "NULL operand");
        for (size_t i = 0; i < count && i < 3; ++i) BF_REQUIRE(g[i] != nullptr, "NULL operand");
    }
    return bf_hip_matmul_bf16_shared_input_backward_img(a, nullptr, b, g, nullptr, dA, dB, count, m, k, n, cacheWeight, stream);
}

int bf_hip_matmul_bf16_shared_input_backward_img(const float* a, const uint16_t* aImage, const float* const* b, const float* const* g,
                                                 const uint16_t* gImage, float* dA, float* const* dB, size_t count, size_t m, size_t k,
                                                 size_t n, int cacheWeight, bf_stream_t stream) {
    BF_REQUIRE(count >= 1 && count <= 3, "count must be 1, 2 or 3");
    BF_REQUIRE(b && (g || gImage), "NULL pointer array");
    hipStream_t s = asStream(stream);
    if (m == 0 || k == 0 || n == 0) {   // degenerate: gradients are zero
        int st = BF_OK;
        if (dA && m * k) st = bf_hip_fill_zero(dA, m * k * sizeof(float), stream);
        for (size_t i = 0; dB && i < count && st == BF_OK; ++i)
            if (dB[i] && k * n) st = bf_hip_fill_zero(dB[i], k * n * sizeof(float), stream);
        return st;
    }
    BF_REQUIRE(a != nullptr || aImage != nullptr, "NULL operand");
    for (size_t i = 0; i < count; ++i) BF_REQUIRE(b[i] && (gImage || g[i]), "NULL operand");
    BF_REQUIRE(gImage == nullptr || n % 8 == 0, "a side-by-side gradient image needs a width that is a multiple of 8");
    BF_REQUIRE(((reinterpret_cast<uintptr_t>(aImage) | reinterpret_cast<uintptr_t>(gImage)) & 15u) == 0, "operand images must be 16-byte aligned");
    int st = BF_OK;
    bool anyDb = false, allDb = dB != nullptr;
    for (size_t i = 0; dB && i < count; ++i) anyDb = anyDb || dB[i] != nullptr;
    for (size_t i = 0; dB && i < count; ++i) allDb = allDb && dB[i] != nullptr;
    {
        // Every gradient wanted and the weight-gradient product big enough for the kernel that transposes fragments in
        // LDS: the gradients are converted once, side by side and as they lie; that image is the A operand of the
        // input-gradient product and the B operand of the weight-gradient product, whose other operand is the plain
        // image of `a`.  No transposed image is built.
        int form = 0;
        size_t slices = 1;
        const size_t nn = count * n;
        if (dA && allDb && count > 1 && n % 256 == 0 && planLargeTiles(k, nn, m, &form, &slices)) {
            const size_t kp = pad8(k);
            Scratch gImg(gImage ? 0 : m * nn * sizeof(unsigned short));
            if (gImg.status != BF_OK) return gImg.status;
            if (!gImage) {
                for (size_t i = 0; i < count; ++i) {
                    st = convertPlain(g[i], gImg.as<unsigned short>() + i * n, m, n, s, nn);
                    if (st != BF_OK) return st;
                }
                gImage = gImg.as<unsigned short>();
            }
            unsigned short* wImg = nullptr;
            size_t wBytes = 0;
            st = weightImage(b, count, k, n, 3, cacheWeight != 0, s, &wImg, &wBytes);
            if (st != BF_OK) return st;
            st = launchGemmNt(gImage, wImg, dA, m, k, nn, nn, nn, s);
            if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
            if (st != BF_OK) return st;
            Scratch aImg(aImage ? 0 : m * kp * sizeof(unsigned short));
            if (aImg.status != BF_OK) return aImg.status;
            if (!aImage) {
                st = convertPlain(a, aImg.as<unsigned short>(), m, k, s);
                if (st != BF_OK) return st;
                aImage = aImg.as<unsigned short>();
            }
            Epilogue epi{{dB[0], count > 1 ? dB[1] : nullptr, count > 2 ? dB[2] : nullptr}, int(n), nullptr, nullptr};
            bool done = false;
            return launchGemmTn(aImage, gImage, epi, k, nn, m, kp, nn, s, &done);
        }
    }
    const size_t mp = pad8(m);
    Scratch gT(anyDb ? count * n * mp * sizeof(unsigned short) : 0);   // transposed gradient images, stacked
    if (gT.status != BF_OK) return gT.status;
    bool transposedDone[3] = {false, false, false};
    if (dA) {
        if (count > 1 && n % 8 == 0) {
            // dA = sum_i g_i b_i^T = [g_0 | g_1 | g_2] [b_0 | b_1 | b_2]^T: one GEMM whose contraction runs over all of them
            const size_t nn = count * n;
            Scratch gImg(gImage ? 0 : m * nn * sizeof(unsigned short));
            if (gImg.status != BF_OK) return gImg.status;
            for (size_t i = 0; i < count && !gImage; ++i) {
                if (dB && dB[i]) {   // one pass over g_i writes its column slice of the plain image and its transposed image
                    st = convertTransposed(g[i], gT.as<unsigned short>() + i * n * mp, m, n, s, true, gImg.as<unsigned short>() + i * n, nn);
                    transposedDone[i] = true;
                } else {
                    st = convertPlain(g[i], gImg.as<unsigned short>() + i * n, m, n, s, nn);
                }
                if (st != BF_OK) return st;
            }
            unsigned short* wImg = nullptr;
            size_t wBytes = 0;
            st = weightImage(b, count, k, n, 3, cacheWeight != 0, s, &wImg, &wBytes);
            if (st != BF_OK) return st;
            st = launchGemmNt(gImage ? gImage : gImg.as<unsigned short>(), wImg, dA, m, k, nn, nn, nn, s);
            if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
            if (st != BF_OK) return st;
        } else {
            Scratch extra(count > 1 ? m * k * sizeof(float) : 0);
            if (extra.status != BF_OK) return extra.status;
            for (size_t i = 0; i < count; ++i) {
                float* target = i == 0 ? dA : extra.as<float>();
                // a side-by-side image exists only for widths that are multiples of 8, which the branch above takes unless count == 1
                st = bf_hip_matmul_bf16_backward_img(a, aImage, b[i], g ? g[i] : nullptr, count == 1 ? gImage : nullptr, target, nullptr, m, k, n,
                                                     cacheWeight, stream);
                if (st != BF_OK) return st;
                if (i > 0) st = bf_hip_accumulate(dA, target, m * k, stream);
                if (st != BF_OK) return st;
            }
        }
    }
    if (anyDb) {
        Scratch aT(k * mp * sizeof(unsigned short));
        if (aT.status != BF_OK) return aT.status;
        st = a ? convertTransposed(a, aT.as<unsigned short>(), m, k, s) : transposeImage(aImage, aT.as<unsigned short>(), m, k, pad8(k), mp, s);
        if (st != BF_OK) return st;
        bool all = true;
        for (size_t i = 0; i < count; ++i) all = all && dB[i] != nullptr;
        for (size_t i = 0; i < count; ++i) {
            if (!dB[i] || transposedDone[i]) continue;
            st = (g && g[i]) ? convertTransposed(g[i], gT.as<unsigned short>() + i * n * mp, m, n, s)
                             : transposeImage(gImage + i * n, gT.as<unsigned short>() + i * n * mp, m, n, count * n, mp, s);
            if (st != BF_OK) return st;
        }
        if (all && count > 1 && n % 256 == 0) {
            Epilogue epi{{dB[0], count > 1 ? dB[1] : nullptr, count > 2 ? dB[2] : nullptr}, int(n), nullptr, nullptr};
            st = launchGemmNt(aT.as<unsigned short>(), gT.as<unsigned short>(), epi, k, count * n, mp, mp, mp, s);
            if (st != BF_OK) return st;
        } else {
            for (size_t i = 0; i < count; ++i) {
                if (!dB[i]) continue;
                st = launchGemmNt(aT.as<unsigned short>(), gT.as<unsigned short>() + i * n * mp, dB[i], k, n, mp, mp, mp, s);
                if (st != BF_OK) return st;
            }
        }
    }
    return st;
}

int bf_hip_feedforward_bf16(const float* x, const float* w1, const float* b1, const float* w2, const float* b2, const float* residual,
                            int act, float* z, uint16_t* hImage, uint16_t* xImage, float* out, size_t m, size_t d, size_t hidden,
                            int cacheWeight, bf_stream_t stream) {
    if (m == 0) return BF_OK;
    BF_REQUIRE(d > 0 && hidden > 0 && d % 8 == 0 && hidden % 8 == 0, "d and hidden must be positive multiples of 8");
    BF_REQUIRE(act == BF_ACT_SILU || act == BF_ACT_GELU || act == BF_ACT_RELU, "unknown activation");
    BF_REQUIRE((x || xImage) && w1 && w2 && z && hImage && out, "NULL pointer");
    BF_REQUIRE(((reinterpret_cast<uintptr_t>(xImage) | reinterpret_cast<uintptr_t>(hImage)) & 15u) == 0, "operand images must be 16-byte aligned");
    hipStream_t s = asStream(stream);
    Scratch xScratch(xImage ? 0 : m * d * sizeof(unsigned short));
    if (xScratch.status != BF_OK) return xScratch.status;
    unsigned short* xImg = xImage ? xImage : xScratch.as<unsigned short>();
    int st = BF_OK;
    if (x) {   // x == NULL: xImage already holds bf16(x)
        st = convertPlain(x, xImg, m, d, s);
        if (st != BF_OK) return st;
    }
    unsigned short* wImg = nullptr;
    size_t wBytes = 0;
    st = weightImage(w1, d, hidden, /*transposed=*/true, cacheWeight != 0, s, &wImg, &wBytes);
    if (st != BF_OK) return st;
    // the activation's image is written by the product's own store when the product is large enough for the kernels
    // that can do it (the same bits as the separate pass over z)
    const bool fused = fusedActivationFits(m, hidden, d, 1) && ((reinterpret_cast<uintptr_t>(z) | reinterpret_cast<uintptr_t>(b1)) & 15u) == 0;
    Epilogue first{{z, nullptr, nullptr}, int(hidden), b1, nullptr};
    if (fused) { first.fuse = 1; first.act = act; first.image = hImage; }
    st = launchGemmNt(xImg, wImg, first, m, hidden, d, d, d, s);
    if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
    if (st != BF_OK) return st;
    if (!fused) {
        st = actToBf16Image(z, hImage, m * hidden, act, s);
        if (st != BF_OK) return st;
    }
    st = weightImage(w2, hidden, d, /*transposed=*/true, cacheWeight != 0, s, &wImg, &wBytes);
    if (st != BF_OK) return st;
    st = launchGemmNt(hImage, wImg, Epilogue{{out, nullptr, nullptr}, int(d), b2, residual}, m, d, hidden, hidden, hidden, s);
    if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
    return st;
}

int bf_hip_feedforward_bf16_backward(const float* x, const uint16_t* xImage, const float* w1, const float* w2, const float* z,
                                     const uint16_t* hImage, const float* g, int act, float* dX, float* dW1, float* dB1, float* dW2,
                                     float* dB2, size_t m, size_t d, size_t hidden, int cacheWeight, bf_stream_t stream) {
    return bf_hip_feedforward_bf16_backward_img(x, xImage, w1, w2, z, hImage, g, nullptr, act, dX, dW1, dB1, dW2, dB2, m, d, hidden,
                                                cacheWeight, stream);
}

int bf_hip_feedforward_bf16_backward_img(const float* x, const uint16_t* xImage, const float* w1, const float* w2, const float* z,
                                         const uint16_t* hImage, const float* g, const uint16_t* gImage, int act, float* dX, float* dW1,
                                         float* dB1, float* dW2, float* dB2, size_t m, size_t d, size_t hidden, int cacheWeight,
                                         bf_stream_t stream) {
    BF_REQUIRE(d > 0 && hidden > 0 && d % 8 == 0 && hidden % 8 == 0, "d and hidden must be positive multiples of 8");
    BF_REQUIRE(act == BF_ACT_SILU || act == BF_ACT_GELU || act == BF_ACT_RELU, "unknown activation");
    hipStream_t s = asStream(stream);
    int st = BF_OK;
    if (m == 0) {   // no rows: parameter gradients are zero
        if (dW1) st = bf_hip_fill_zero(dW1, d * hidden * sizeof(float), stream);
        if (st == BF_OK && dW2) st = bf_hip_fill_zero(dW2, d * hidden * sizeof(float), stream);
        if (st == BF_OK && dB1) st = bf_hip_fill_zero(dB1, hidden * sizeof(float), stream);
        if (st == BF_OK && dB2) st = bf_hip_fill_zero(dB2, d * sizeof(float), stream);
        return st;
    }
    BF_REQUIRE((x || xImage) && w1 && w2 && z && hImage && (g || gImage), "NULL operand");
    BF_REQUIRE(g != nullptr || dB2 == nullptr, "the bias gradient dB2 is taken from the fp32 gradient");
    BF_REQUIRE(((reinterpret_cast<uintptr_t>(xImage) | reinterpret_cast<uintptr_t>(hImage) | reinterpret_cast<uintptr_t>(gImage)) & 15u) == 0,
               "operand images must be 16-byte aligned");
    const size_t mp = pad8(m);
    Scratch gImg(gImage ? 0 : m * d * sizeof(unsigned short));
    if (gImg.status != BF_OK) return gImg.status;
    if (!gImage) {   // gImage: bf16(g) made by whoever produced g
        st = convertPlain(g, gImg.as<unsigned short>(), m, d, s);
        if (st != BF_OK) return st;
        gImage = gImg.as<unsigned short>();
    }
    if (dB2) {
        st = bf_hip_bias_grad(g, dB2, m, d, stream);
        if (st != BF_OK) return st;
    }
    if (dW2) {   // dW2[hidden, d] = h^T g, contraction over the m rows
        bool done = false;
        st = launchGemmTn(hImage, gImage, Epilogue{{dW2, nullptr, nullptr}, int(d), nullptr, nullptr}, hidden, d, m,
                          hidden, d, s, &done);
        if (st != BF_OK) return st;
        if (!done) {
            Scratch hT(hidden * mp * sizeof(unsigned short)), gT(d * mp * sizeof(unsigned short));
            if (hT.status != BF_OK) return hT.status;
            if (gT.status != BF_OK) return gT.status;
            st = transposeImage(hImage, hT.as<unsigned short>(), m, hidden, hidden, mp, s);
            if (st == BF_OK) st = g ? convertTransposed(g, gT.as<unsigned short>(), m, d, s) : transposeImage(gImage, gT.as<unsigned short>(), m, d, d, mp, s);
            if (st == BF_OK) st = launchGemmNt(hT.as<unsigned short>(), gT.as<unsigned short>(), dW2, hidden, d, mp, mp, mp, s);
            if (st != BF_OK) return st;
        }
    }
    if (!dX && !dW1 && !dB1) return BF_OK;
    // dH = g w2^T; one pass over it writes bf16(dz), dz = act'(z) . dH, and dz's column sums: dz is never stored in fp32
    // When the product is large enough for the kernels that can do it, its store multiplies by act'(z) and writes the image
    // itself (dH never exists in memory; the same bits as the separate pass), with dz's column sums per 32-row block, which
    // a bias-gradient pass over those few rows finishes.
    const bool fused = fusedActivationFits(m, hidden, d, 2) && ((reinterpret_cast<uintptr_t>(z) | reinterpret_cast<uintptr_t>(dB1)) & 15u) == 0;
    const size_t rowBlocks = (m + 31) / 32;
    Scratch dH(fused ? 0 : m * hidden * sizeof(float)), dzImg(m * hidden * sizeof(unsigned short));
    Scratch partial(fused && dB1 ? rowBlocks * hidden * sizeof(float) : 0);
    if (dH.status != BF_OK) return dH.status;
    if (dzImg.status != BF_OK) return dzImg.status;
    if (partial.status != BF_OK) return partial.status;
    unsigned short* wImg = nullptr;
    size_t wBytes = 0;
    st = weightImage(w2, hidden, d, /*transposed=*/false, cacheWeight != 0, s, &wImg, &wBytes);
    if (st != BF_OK) return st;
    Epilogue toDz{{dH.as<float>(), nullptr, nullptr}, int(hidden), nullptr, nullptr};
    if (fused) {
        toDz.fuse = 2;
        toDz.act = act;
        toDz.image = dzImg.as<unsigned short>();
        toDz.actZ = z;
        toDz.colPartial = dB1 ? partial.as<float>() : nullptr;
    }
    st = launchGemmNt(gImage, wImg, toDz, m, hidden, d, d, d, s);
    if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
    if (st != BF_OK) return st;
    if (!fused) st = actBackwardToBf16Image(z, dH.as<float>(), dzImg.as<unsigned short>(), dB1, m, hidden, act, s);
    else if (dB1) st = bf_hip_bias_grad(partial.as<float>(), dB1, rowBlocks, hidden, stream);
    if (st != BF_OK) return st;
    if (dW1) {   // dW1[d, hidden] = x^T dz
        Scratch xScratch(xImage ? 0 : m * d * sizeof(unsigned short));
        if (xScratch.status != BF_OK) return xScratch.status;
        const unsigned short* xImg = xImage;
        if (!xImg) {
            st = convertPlain(x, xScratch.as<unsigned short>(), m, d, s);
            if (st != BF_OK) return st;
            xImg = xScratch.as<unsigned short>();
        }
        bool done = false;
        st = launchGemmTn(xImg, dzImg.as<unsigned short>(), Epilogue{{dW1, nullptr, nullptr}, int(hidden), nullptr, nullptr}, d, hidden, m,
                          d, hidden, s, &done);
        if (st != BF_OK) return st;
        if (!done) {
            Scratch xT(d * mp * sizeof(unsigned short)), dzT(hidden * mp * sizeof(unsigned short));
            if (xT.status != BF_OK) return xT.status;
            if (dzT.status != BF_OK) return dzT.status;
            st = transposeImage(xImg, xT.as<unsigned short>(), m, d, d, mp, s);
            if (st == BF_OK) st = transposeImage(dzImg.as<unsigned short>(), dzT.as<unsigned short>(), m, hidden, hidden, mp, s);
            if (st == BF_OK) st = launchGemmNt(xT.as<unsigned short>(), dzT.as<unsigned short>(), dW1, d, hidden, mp, mp, mp, s);
            if (st != BF_OK) return st;
        }
    }
    if (dX) {   // dX[m, d] = dz w1^T
        st = weightImage(w1, d, hidden, /*transposed=*/false, cacheWeight != 0, s, &wImg, &wBytes);
        if (st != BF_OK) return st;
        st = launchGemmNt(dzImg.as<unsigned short>(), wImg, dX, m, d, hidden, hidden, hidden, s);
        if (!cacheWeight) bf_hip_pool_release(wImg, wBytes);
    }
    return st;
}

int bf_hip_mfma_only_loop(const uint16_t* operands, float* out, int shape, int workgroups, int kSteps, bf_stream_t stream) {
    BF_REQUIRE(operands && out, "NULL pointer");
    BF_REQUIRE((reinterpret_cast<uintptr_t>(operands) & 15u) == 0, "operands must be 16-byte aligned");
    BF_REQUIRE(shape == 0 || shape == 1, "shape: 0 (32x32x16) or 1 (16x16x32)");
    BF_REQUIRE(workgroups > 0 && workgroups <= 65536 && kSteps > 0, "workgroups in 1..65536, kSteps > 0");
    hipStream_t s = asStream(stream);
    if (shape == 0) bf::mfmaOnlyKernel<0><<<dim3(unsigned(workgroups)), 512, 0, s>>>(reinterpret_cast<const uint4v*>(operands), out, kSteps);
    else bf::mfmaOnlyKernel<1><<<dim3(unsigned(workgroups)), 512, 0, s>>>(reinterpret_cast<const uint4v*>(operands), out, kSteps);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_gemm_bf16_set_route(int route) {
    BF_REQUIRE(route >= BF_GEMM_ROUTE_AUTO && route <= BF_GEMM_ROUTE_PINGPONG_128_PERSISTENT, "unknown route");
    bf::g_ntRoute = route;
    return BF_OK;
}

int bf_hip_invalidate_bf16_weight_cache(void) {
    // Images that nobody asked for during the generation that ends here belong to weights that are gone (a destroyed
    // model) or idle: their buffers go back to the pool.  An idle weight that is used again just converts once more.
    auto& cache = bf::weightCache();
    for (auto it = cache.begin(); it != cache.end();) {
        if (it->second.generation != bf::generation()) {
            bf_hip_pool_release(it->second.buffer, it->second.bytes);
            it = cache.erase(it);
        } else {
            ++it;
        }
    }
    ++bf::generation();
    return BF_OK;
}

int bf_hip_bf16_weight_cache_refresh(const float* const* changed, size_t count, bf_stream_t stream) {
    BF_REQUIRE(changed || count == 0, "NULL pointer");
    const size_t ending = bf::generation();
    int st = bf_hip_invalidate_bf16_weight_cache();
    // (a recording makes its images where its products need them: a refresh recorded at the end of a step would only
    // be repeated by the conversions recorded at its beginning)
    if (st != BF_OK || count == 0 || bf::capturing()) return st;
    return bf::refreshImagesOf(changed, count, ending, bf::asStream(stream));
}

}  // extern "C"
