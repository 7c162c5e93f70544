// Gather / scatter ops: embedding lookup and its scatter-add gradient, positional embedding,
// KV-cache concatenation, token-id range check and last-position argmax.
//
// All HBM-bound.  The embedding gradient avoids both the memset and the per-element global atomics of
// the usual scatter-add: tokens are bucketed by id with a counting sort (integer work only), then one
// wavefront per vocabulary row adds that row's tokens in token order and writes the row once (rows
// nobody used are written as zeros).  The result is deterministic and equals a sequential
// token-order sum in fp32.
#include "common.hpp"

namespace bf {
namespace {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

__device__ __forceinline__ long long roundId(float v) { return (long long)lroundf(v); }

__global__ void __launch_bounds__(kBlock) countOutOfRangeKernel(const float* __restrict__ ids, size_t count, long long limit,
                                                                unsigned long long* __restrict__ result) {
    // result[0] = number of bad ids, result[1] = one bad value (any)
    size_t stride = size_t(gridDim.x) * blockDim.x;
    unsigned long long bad = 0;
    long long sample = 0;
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride) {
        long long id = roundId(ids[i]);
        if (id < 0 || id >= limit) { ++bad; sample = id; }
    }
    if (bad) {
        atomicAdd(&result[0], bad);
        atomicExch(&result[1], (unsigned long long)sample);
    }
}

// One row of `dim` floats per (token); 2-D layout as in the bias kernels: no division on the memory path.
template <int VEC>
__global__ void __launch_bounds__(256) embeddingForwardKernel(const float* __restrict__ ids, const float* __restrict__ table,
                                                              float* __restrict__ out, size_t tokens, size_t dim) {
    size_t col = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
    if (col >= dim) return;
    size_t step = size_t(gridDim.y) * blockDim.y;
    for (size_t t = size_t(blockIdx.y) * blockDim.y + threadIdx.y; t < tokens; t += step) {
        size_t id = size_t(roundId(ids[t]));
        if constexpr (VEC == 4) storef4(out + t * dim + col, loadf4(table + id * dim + col));
        else out[t * dim + col] = table[id * dim + col];
    }
}

// ---- embedding backward: counting sort by id ---------------------------------------------------
__global__ void __launch_bounds__(kBlock) histogramKernel(const float* __restrict__ ids, size_t tokens, unsigned* __restrict__ counts) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < tokens) atomicAdd(&counts[size_t(roundId(ids[i]))], 1u);
}

// Exclusive scan of counts[0..vocab) into offsets[0..vocab], single block of 1024 threads, four consecutive
// entries per thread and pass (integer sums: any order gives the same result).
__global__ void __launch_bounds__(1024) exclusiveScanKernel(const unsigned* __restrict__ counts, unsigned* __restrict__ offsets, size_t vocab) {
    __shared__ unsigned waveTotals[16];
    __shared__ unsigned carry;
    if (threadIdx.x == 0) carry = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (size_t base = 0; base < vocab; base += 4096) {
        const size_t i = base + size_t(threadIdx.x) * 4;
        unsigned v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = i + j < vocab ? counts[i + j] : 0u;
        const unsigned mine = v[0] + v[1] + v[2] + v[3];
        unsigned incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            unsigned n = __shfl_up(incl, off, 64);
            if (lane >= off) incl += n;
        }
        if (lane == 63) waveTotals[wave] = incl;
        __syncthreads();
        unsigned before = carry;
        for (int w = 0; w < wave; ++w) before += waveTotals[w];
        unsigned run = before + incl - mine;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (i + j < vocab) offsets[i + j] = run;
            run += v[j];
        }
        __syncthreads();
        if (threadIdx.x == 1023) carry = before + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) offsets[vocab] = carry;
}

// Tokens are first dropped into their id's segment in whatever order the atomics resolve
// (slot = offsets[id] + one of counts[id]-1 .. 0), then every token finds its rank among the tokens of its
// segment (how many of them are smaller) and moves to order[offsets[id] + rank]: segments end up sorted by
// token index whatever the atomics did, so the sums below run in token order.  The rank loop is as long as
// the segment (the number of tokens that share the id).
__global__ void __launch_bounds__(kBlock) scatterTokensKernel(const float* __restrict__ ids, size_t tokens,
                                                              const unsigned* __restrict__ offsets, unsigned* __restrict__ counts,
                                                              unsigned* __restrict__ unordered) {
    size_t t = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    size_t id = size_t(roundId(ids[t]));
    unsigned left = atomicSub(&counts[id], 1u);   // value before the decrement: counts[id] .. 1
    unordered[offsets[id] + left - 1u] = unsigned(t);
}
__global__ void __launch_bounds__(kBlock) rankTokensKernel(const float* __restrict__ ids, size_t tokens,
                                                           const unsigned* __restrict__ offsets,
                                                           const unsigned* __restrict__ unordered, unsigned* __restrict__ order) {
    size_t t = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    size_t id = size_t(roundId(ids[t]));
    unsigned begin = offsets[id], end = offsets[id + 1], rank = 0;
    for (unsigned j = begin; j < end; ++j) rank += unordered[j] < unsigned(t) ? 1u : 0u;
    order[begin + rank] = unsigned(t);
}

// One wavefront per vocabulary row.
template <int VEC>
__global__ void __launch_bounds__(kBlock) embeddingBackwardKernel(const float* __restrict__ g, float* __restrict__ dTable,
                                                                  const unsigned* __restrict__ offsets, const unsigned* __restrict__ order,
                                                                  size_t vocab, size_t dim) {
    const int lane = threadIdx.x & 63;
    const size_t wavesPerBlock = blockDim.x / 64;
    const size_t step = size_t(gridDim.x) * wavesPerBlock;
    for (size_t row = size_t(blockIdx.x) * wavesPerBlock + threadIdx.x / 64; row < vocab; row += step) {
        unsigned begin = offsets[row], end = offsets[row + 1];
        for (size_t col = size_t(lane) * VEC; col < dim; col += 64 * VEC) {
            if constexpr (VEC == 4) {
                float4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
                for (unsigned j = begin; j < end; ++j) acc = acc + loadf4(g + size_t(order[j]) * dim + col);
                storef4(dTable + row * dim + col, acc);
            } else {
                float acc = 0.0f;
                for (unsigned j = begin; j < end; ++j) acc += g[size_t(order[j]) * dim + col];
                dTable[row * dim + col] = acc;
            }
        }
    }
}

template <int VEC>
__global__ void __launch_bounds__(256) positionalForwardKernel(const float* __restrict__ x, const float* __restrict__ table,
                                                               float* __restrict__ out, size_t batch, size_t seq, size_t dim,
                                                               size_t offset) {
    size_t col = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
    if (col >= dim) return;
    size_t step = size_t(gridDim.y) * blockDim.y;
    for (size_t s = size_t(blockIdx.y) * blockDim.y + threadIdx.y; s < seq; s += step) {
        if constexpr (VEC == 4) {
            float4v tv = loadf4(table + (offset + s) * dim + col);
            for (size_t b = 0; b < batch; ++b) {
                size_t idx = (b * seq + s) * dim + col;
                storef4(out + idx, loadf4(x + idx) + tv);
            }
        } else {
            float tv = table[(offset + s) * dim + col];
            for (size_t b = 0; b < batch; ++b) {
                size_t idx = (b * seq + s) * dim + col;
                out[idx] = x[idx] + tv;
            }
        }
    }
}

// dTable[s,:] = sum over batch in batch order; rows s >= seq are zero.
template <int VEC>
__global__ void __launch_bounds__(256) positionalBackwardKernel(const float* __restrict__ g, float* __restrict__ dTable,
                                                                size_t batch, size_t seq, size_t dim, size_t maxSeq) {
    size_t col = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
    if (col >= dim) return;
    size_t step = size_t(gridDim.y) * blockDim.y;
    for (size_t s = size_t(blockIdx.y) * blockDim.y + threadIdx.y; s < maxSeq; s += step) {
        if constexpr (VEC == 4) {
            float4v acc = {0.0f, 0.0f, 0.0f, 0.0f};
            if (s < seq)
                for (size_t b = 0; b < batch; ++b) acc = acc + loadf4(g + (b * seq + s) * dim + col);
            storef4(dTable + s * dim + col, acc);
        } else {
            float acc = 0.0f;
            if (s < seq)
                for (size_t b = 0; b < batch; ++b) acc += g[(b * seq + s) * dim + col];
            dTable[s * dim + col] = acc;
        }
    }
}

// out[b, s, :] = s < seqA ? a[b, s, :] : b_[b, s - seqA, :]; rows of `out` walked by threadIdx.y
template <int VEC>
__global__ void __launch_bounds__(256) concatSeqKernel(const float* __restrict__ a, const float* __restrict__ b,
                                                       float* __restrict__ out, size_t batch, size_t seqA, size_t seqB,
                                                       size_t dim) {
    size_t col = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
    if (col >= dim) return;
    size_t total = seqA + seqB;
    size_t rows = batch * total;
    size_t step = size_t(gridDim.y) * blockDim.y;
    for (size_t r = size_t(blockIdx.y) * blockDim.y + threadIdx.y; r < rows; r += step) {
        size_t bi = r / total, s = r - bi * total;
        const float* src = s < seqA ? a + (bi * seqA + s) * dim + col : b + (bi * seqB + (s - seqA)) * dim + col;
        if constexpr (VEC == 4) storef4(out + r * dim + col, loadf4(src));
        else out[r * dim + col] = *src;
    }
}

// Lowest index of the maximum of one row: the result of the host loop "best = 0; if (row[c] > row[best])
// best = c" it replaces.  A NaN never wins a strict '>' and, at index 0, is never beaten; the key
// below encodes exactly that.
__device__ __forceinline__ float argmaxKey(float v, size_t i) {
    if (v != v) return i == 0 ? INFINITY : -INFINITY;
    return v;
}
__global__ void __launch_bounds__(1024) argmaxRowKernel(const float* __restrict__ row, size_t n, long long* __restrict__ result) {
    __shared__ float vals[16];
    __shared__ unsigned long long idxs[16];
    float best = -INFINITY;
    unsigned long long bestIdx = ~0ull;  // "no candidate": loses against everything
    for (size_t i = threadIdx.x; i < n; i += blockDim.x) {
        float k = argmaxKey(row[i], i);
        if (bestIdx == ~0ull || k > best) { best = k; bestIdx = i; }
    }
    // (value, index) pairs: larger value wins, equal values go to the lower index
    auto takeOther = [](float v, unsigned long long i, float ov, unsigned long long oi) {
        return oi != ~0ull && (i == ~0ull || ov > v || (ov == v && oi < i));
    };
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        float ov = __shfl_xor(best, off, 64);
        unsigned long long oi = __shfl_xor(bestIdx, off, 64);
        if (takeOther(best, bestIdx, ov, oi)) { best = ov; bestIdx = oi; }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { vals[wave] = best; idxs[wave] = bestIdx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (unsigned w = 1; w < (blockDim.x >> 6); ++w)
            if (takeOther(best, bestIdx, vals[w], idxs[w])) { best = vals[w]; bestIdx = idxs[w]; }
        result[0] = (long long)bestIdx;
    }
}

struct Geom2D {
    dim3 grid, block;
    int vec;
};
Geom2D geometry2D(size_t rows, size_t cols, bool canVectorise) {
    Geom2D g;
    g.vec = (canVectorise && cols % 4 == 0) ? 4 : 1;
    size_t groups = cols / g.vec;
    unsigned bx = 1;
    while (bx < 256 && bx < groups) bx <<= 1;
    unsigned by = 256 / bx;
    unsigned gx = unsigned((groups + bx - 1) / bx);
    size_t gy = (rows + by - 1) / by;
    if (gy > 65535) gy = 65535;   // every row block once, in address order
    if (gy < 1) gy = 1;
    g.block = dim3(bx, by);
    g.grid = dim3(gx, unsigned(gy));
    return g;
}

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" {

int bf_hip_count_out_of_range(const float* ids, size_t count, size_t limit, size_t* numBad, long long* firstBad,
                              bf_stream_t stream) {
    BF_REQUIRE(numBad != nullptr, "numBad is NULL");
    *numBad = 0;
    if (firstBad) *firstBad = 0;
    if (count == 0) return BF_OK;
    BF_REQUIRE(ids != nullptr, "NULL pointer");
    hipStream_t s = asStream(stream);
    Scratch result(2 * sizeof(unsigned long long));
    if (result.status != BF_OK) return result.status;
    int st = bf_hip_fill_zero(result.ptr, 2 * sizeof(unsigned long long), stream);
    if (st != BF_OK) return st;
    countOutOfRangeKernel<<<gridFor(count, kBlock, unsigned(computeUnits()) * 8), kBlock, 0, s>>>(
        ids, count, (long long)limit, result.as<unsigned long long>());
    BF_LAUNCH_CHECK();
    unsigned long long host[2] = {0, 0};
    BF_HIP_TRY(hipMemcpyAsync(host, result.ptr, sizeof(host), hipMemcpyDeviceToHost, s));
    BF_HIP_TRY(hipStreamSynchronize(s));
    *numBad = size_t(host[0]);
    if (firstBad) *firstBad = (long long)host[1];
    return BF_OK;
}

int bf_hip_embedding_forward(const float* ids, const float* table, float* out, size_t tokens, size_t vocab, size_t dim,
                             bf_stream_t stream) {
    (void)vocab;
    if (tokens == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(ids && table && out, "NULL pointer");
    Geom2D g = geometry2D(tokens, dim, aligned16(table) && aligned16(out));
    if (g.vec == 4) embeddingForwardKernel<4><<<g.grid, g.block, 0, asStream(stream)>>>(ids, table, out, tokens, dim);
    else embeddingForwardKernel<1><<<g.grid, g.block, 0, asStream(stream)>>>(ids, table, out, tokens, dim);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_embedding_backward(const float* ids, const float* g, float* dTable, size_t tokens, size_t vocab, size_t dim,
                              bf_stream_t stream) {
    if (vocab == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(dTable != nullptr, "NULL pointer");
    BF_REQUIRE(tokens < (size_t(1) << 32), "too many tokens");
    hipStream_t s = asStream(stream);
    if (tokens == 0) return bf_hip_fill_zero(dTable, vocab * dim * sizeof(float), stream);
    BF_REQUIRE(ids && g, "NULL pointer");
    // counts[vocab] | offsets[vocab+1] | unordered[tokens] | order[tokens]
    size_t words = vocab + (vocab + 1) + 2 * tokens;
    Scratch work(words * sizeof(unsigned));
    if (work.status != BF_OK) return work.status;
    unsigned* counts = work.as<unsigned>();
    unsigned* offsets = counts + vocab;
    unsigned* unordered = offsets + vocab + 1;
    unsigned* order = unordered + tokens;
    int st = bf_hip_fill_zero(counts, vocab * sizeof(unsigned), stream);
    if (st != BF_OK) return st;
    histogramKernel<<<gridFor(tokens, kBlock), kBlock, 0, s>>>(ids, tokens, counts);
    BF_LAUNCH_CHECK();
    exclusiveScanKernel<<<1, 1024, 0, s>>>(counts, offsets, vocab);
    BF_LAUNCH_CHECK();
    scatterTokensKernel<<<gridFor(tokens, kBlock), kBlock, 0, s>>>(ids, tokens, offsets, counts, unordered);
    BF_LAUNCH_CHECK();
    rankTokensKernel<<<gridFor(tokens, kBlock), kBlock, 0, s>>>(ids, tokens, offsets, unordered, order);
    BF_LAUNCH_CHECK();
    unsigned grid = gridFor(vocab, kBlock / 64);
    if (aligned16(g) && aligned16(dTable) && dim % 4 == 0)
        embeddingBackwardKernel<4><<<grid, kBlock, 0, s>>>(g, dTable, offsets, order, vocab, dim);
    else
        embeddingBackwardKernel<1><<<grid, kBlock, 0, s>>>(g, dTable, offsets, order, vocab, dim);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_positional_forward(const float* x, const float* table, float* out, size_t batch, size_t seq, size_t dim,
                              size_t maxSeq, size_t offset, bf_stream_t stream) {
    BF_REQUIRE(offset + seq <= maxSeq, "absolute position " + std::to_string(offset + seq) + " exceeds maxSeqLen " +
                                           std::to_string(maxSeq));
    if (batch == 0 || seq == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(x && table && out, "NULL pointer");
    Geom2D g = geometry2D(seq, dim, aligned16(x) && aligned16(table) && aligned16(out));
    if (g.vec == 4) positionalForwardKernel<4><<<g.grid, g.block, 0, asStream(stream)>>>(x, table, out, batch, seq, dim, offset);
    else positionalForwardKernel<1><<<g.grid, g.block, 0, asStream(stream)>>>(x, table, out, batch, seq, dim, offset);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_positional_backward(const float* g, float* dTable, size_t batch, size_t seq, size_t dim, size_t maxSeq,
                               bf_stream_t stream) {
    BF_REQUIRE(seq <= maxSeq, "sequence " + std::to_string(seq) + " exceeds maxSeqLen " + std::to_string(maxSeq));
    if (maxSeq == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(dTable && (g || batch * seq == 0), "NULL pointer");
    Geom2D geo = geometry2D(maxSeq, dim, aligned16(g) && aligned16(dTable));
    if (geo.vec == 4) positionalBackwardKernel<4><<<geo.grid, geo.block, 0, asStream(stream)>>>(g, dTable, batch, seq, dim, maxSeq);
    else positionalBackwardKernel<1><<<geo.grid, geo.block, 0, asStream(stream)>>>(g, dTable, batch, seq, dim, maxSeq);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_concat_seq(const float* a, const float* b, float* out, size_t batch, size_t seqA, size_t seqB, size_t dim,
                      bf_stream_t stream) {
    if (batch == 0 || dim == 0 || seqA + seqB == 0) return BF_OK;
    BF_REQUIRE(out && (a || seqA == 0) && (b || seqB == 0), "NULL pointer");
    Geom2D g = geometry2D(batch * (seqA + seqB), dim, aligned16(a) && aligned16(b) && aligned16(out));
    if (g.vec == 4) concatSeqKernel<4><<<g.grid, g.block, 0, asStream(stream)>>>(a, b, out, batch, seqA, seqB, dim);
    else concatSeqKernel<1><<<g.grid, g.block, 0, asStream(stream)>>>(a, b, out, batch, seqA, seqB, dim);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_argmax_last_position(const float* logits, size_t seq, size_t vocab, long long* index, bf_stream_t stream) {
    BF_REQUIRE(index != nullptr, "index is NULL");
    BF_REQUIRE(seq > 0 && vocab > 0, "empty logits");
    BF_REQUIRE(logits != nullptr, "NULL pointer");
    hipStream_t s = asStream(stream);
    Scratch result(sizeof(long long));
    if (result.status != BF_OK) return result.status;
    argmaxRowKernel<<<1, 1024, 0, s>>>(logits + (seq - 1) * vocab, vocab, result.as<long long>());
    BF_LAUNCH_CHECK();
    BF_HIP_TRY(hipMemcpyAsync(index, result.ptr, sizeof(long long), hipMemcpyDeviceToHost, s));
    BF_HIP_TRY(hipStreamSynchronize(s));
    return BF_OK;
}

}  // extern "C"
