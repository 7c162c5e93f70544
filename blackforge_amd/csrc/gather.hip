// Gather / scatter ops: embedding lookup and its scatter-add gradient, positional embedding,
// KV-cache concatenation, token-id range check and last-position argmax.
//
// All HBM-bound.  The embedding gradient avoids both the memset and the per-element global atomics of
// the usual scatter-add.  A training batch (up to 16384 tokens) runs as ONE launch in which a wavefront per
// token finds the other tokens with its id through bitmaps in LDS and the workgroups share out the rows
// that stay zero; longer token lists are bucketed by id with a counting sort (integer work only), then one
// wavefront per vocabulary row adds that row's tokens.  Either way a row's tokens are added in token order
// and every row is written once: the result is deterministic and equals the CPU loop's sum bit for bit.
#include "common.hpp"

#include <algorithm>
#include <type_traits>

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
                                                              float* __restrict__ out, size_t tokens, size_t dim, long long vocab) {
    size_t col = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
    if (col >= dim) return;
    size_t step = size_t(gridDim.y) * blockDim.y;
    for (size_t t = size_t(blockIdx.y) * blockDim.y + threadIdx.y; t < tokens; t += step) {
        // an id outside the table (the validating variant rejects those before the launch) reads nothing: zeros
        const long long id = roundId(ids[t]);
        const bool inside = id >= 0 && id < vocab;
        if constexpr (VEC == 4) storef4(out + t * dim + col, inside ? loadf4(table + size_t(id) * dim + col) : float4v{0.0f, 0.0f, 0.0f, 0.0f});
        else out[t * dim + col] = inside ? table[size_t(id) * dim + col] : 0.0f;
    }
}

// ---- embedding backward: counting sort by id ---------------------------------------------------
// Ids outside [0, vocab) take no part in any of the kernels below (no count, no slot, no sum).
__device__ __forceinline__ bool idInside(long long id, size_t vocab) { return id >= 0 && (unsigned long long)id < vocab; }

__global__ void __launch_bounds__(kBlock) histogramKernel(const float* __restrict__ ids, size_t tokens, unsigned* __restrict__ counts, size_t vocab) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= tokens) return;
    const long long id = roundId(ids[i]);
    if (idInside(id, vocab)) atomicAdd(&counts[size_t(id)], 1u);
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
                                                              unsigned* __restrict__ unordered, size_t vocab) {
    size_t t = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    if (!idInside(roundId(ids[t]), vocab)) return;
    size_t id = size_t(roundId(ids[t]));
    unsigned left = atomicSub(&counts[id], 1u);   // value before the decrement: counts[id] .. 1
    unordered[offsets[id] + left - 1u] = unsigned(t);
}
__global__ void __launch_bounds__(kBlock) rankTokensKernel(const float* __restrict__ ids, size_t tokens,
                                                           const unsigned* __restrict__ offsets,
                                                           const unsigned* __restrict__ unordered, unsigned* __restrict__ order, size_t vocab) {
    size_t t = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= tokens) return;
    if (!idInside(roundId(ids[t]), vocab)) return;
    size_t id = size_t(roundId(ids[t]));
    unsigned begin = offsets[id], end = offsets[id + 1], rank = 0;
    for (unsigned j = begin; j < end; ++j) rank += unordered[j] < unsigned(t) ? 1u : 0u;
    order[begin + rank] = unsigned(t);
}

// Few tokens (at most kByTokenMax: a training batch) against a large table: no sort, ONE launch.  A workgroup takes 16
// tokens, one per wavefront, and a share of consecutive table rows.  All 1024 threads together look at every token's id
// once: they compare it with the workgroup's 16 ids (a register compare away) and mark the matches in 16 bitmaps in LDS,
// one bit per token, and they mark the rows of the workgroup's share that some token uses.  The rows of the share that
// no token uses are then written as zeros.  A wavefront whose token is not the first with its id (a bit below its own
// is set) has nothing more to do; otherwise it walks its bitmap upwards, adds the rows of the tokens it finds, in token
// order, and writes the table row.  Every table row is written exactly once, by whoever knows its value, with no chain
// of small dependent launches in front of the 98 MB that the gradient of a 32000 x 768 table has to move (the counting
// sort below spends more time in its five small launches than in that write).
constexpr size_t kByTokenMax = 16384;
constexpr int kTokensPerGroup = 16;
template <int VEC>
__global__ void __launch_bounds__(1024) embeddingBackwardByTokenKernel(const float* __restrict__ ids, const float* __restrict__ g,
                                                                       float* __restrict__ dTable, unsigned tokens, size_t vocab,
                                                                       size_t dim) {
    extern __shared__ unsigned bitmaps[];   // [16][words]: bit j of bitmaps[s] = token j has the id of the group's token s
    __shared__ int groupId[kTokensPerGroup];
    const unsigned words = (tokens + 31) / 32;
    // this workgroup's share of the table rows, and (after the 16 bitmaps) one bit per row of it: some token uses the row
    const unsigned share = unsigned((vocab + gridDim.x - 1) / gridDim.x);
    const long long rowLo = (long long)blockIdx.x * share, rowHi = rowLo + share < (long long)vocab ? rowLo + share : (long long)vocab;
    unsigned* used = bitmaps + words * kTokensPerGroup;
    const unsigned usedWords = (share + 31) / 32;
    const unsigned lane = threadIdx.x & 63, slot = threadIdx.x >> 6, t0 = blockIdx.x * kTokensPerGroup;
    auto toId = [&](float v) { const long long id = roundId(v); return idInside(id, vocab) ? int(id) : -2; };   // -2: matches nothing
    for (unsigned w = threadIdx.x; w < words * kTokensPerGroup + usedWords; w += 1024) bitmaps[w] = 0u;
    if (threadIdx.x < kTokensPerGroup) {
        const unsigned t = t0 + threadIdx.x;
        const int id = t < tokens ? toId(ids[t]) : -2;
        groupId[threadIdx.x] = id == -2 ? -1 : id;   // -1: no row to write; never equal to a token's -2
    }
    __syncthreads();
    int mine[kTokensPerGroup];
#pragma unroll
    for (int s = 0; s < kTokensPerGroup; ++s) mine[s] = groupId[s];
    auto mark = [&](unsigned j, int id) {
#pragma unroll
        for (int s = 0; s < kTokensPerGroup; ++s)
            if (id == mine[s]) atomicOr(&bitmaps[s * words + (j >> 5)], 1u << (j & 31u));
        if (id >= rowLo && id < rowHi) atomicOr(&used[unsigned(id - rowLo) >> 5], 1u << (unsigned(id - rowLo) & 31u));
    };
    if ((reinterpret_cast<uintptr_t>(ids) & 15u) == 0) {
        // four ids per load and every load of a thread issued before the first is used: one memory latency, not one per id
        constexpr int PER = int(kByTokenMax / 4 / 1024);
        float4v v[PER];
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const unsigned i4 = threadIdx.x + 1024u * u;
            v[u] = 4 * i4 + 4 <= tokens ? loadf4(ids + 4 * i4) : float4v{-1.0f, -1.0f, -1.0f, -1.0f};
        }
#pragma unroll
        for (int u = 0; u < PER; ++u) {
            const unsigned j = 4 * (threadIdx.x + 1024u * u);
            if (j + 4 <= tokens) { mark(j, toId(v[u].x)); mark(j + 1, toId(v[u].y)); mark(j + 2, toId(v[u].z)); mark(j + 3, toId(v[u].w)); }
        }
        for (unsigned j = (tokens & ~3u) + threadIdx.x; j < tokens; j += 1024) mark(j, toId(ids[j]));
    } else {
        for (unsigned j = threadIdx.x; j < tokens; j += 1024) mark(j, toId(ids[j]));
    }
    __syncthreads();
    // zeros for the rows of the share that no token uses: a wavefront per row, 64 * VEC columns per store
    for (long long row = rowLo + slot; row < rowHi; row += kTokensPerGroup) {
        const unsigned r = unsigned(row - rowLo);
        if ((used[r >> 5] >> (r & 31u)) & 1u) continue;
        float* out = dTable + size_t(row) * dim;
        for (size_t col = size_t(lane) * VEC; col < dim; col += size_t(64) * VEC) {
            if constexpr (VEC == 4) storef4(out + col, float4v{0.0f, 0.0f, 0.0f, 0.0f});
            else out[col] = 0.0f;
        }
    }
    const unsigned t = t0 + slot;
    if (t >= tokens) return;
    const int id = groupId[slot];
    if (id < 0) return;
    const unsigned* bits = bitmaps + slot * words;
    // wave-uniform: a set bit below this token's own means an earlier token owns the id's row
    for (unsigned base = 0; base <= (t >> 5); base += 64) {
        const unsigned w = base + lane;
        unsigned word = w <= (t >> 5) ? bits[w] : 0u;
        if (w == (t >> 5)) word &= (1u << (t & 31u)) - 1u;
        if (__ballot(word != 0u) != 0) return;
    }
    constexpr int CHUNKS = 4;   // column groups of 64 * VEC held in registers per pass over the bitmap
    typedef typename std::conditional<VEC == 4, float4v, float>::type V;
    for (size_t col0 = 0; col0 < dim; col0 += size_t(64) * VEC * CHUNKS) {
        V acc[CHUNKS];
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) acc[c] = V{};
        for (unsigned base = (t >> 5) & ~63u; base < words; base += 64) {
            const unsigned w = base + lane;
            const unsigned word = w < words ? bits[w] : 0u;
            unsigned long long lanes = __ballot(word != 0u);
            while (lanes != 0) {   // words in ascending order, bits of a word in ascending order: token order
                const int src = __ffsll((long long)lanes) - 1;
                lanes &= lanes - 1;
                unsigned pending = unsigned(__builtin_amdgcn_readlane(int(word), src));
                while (pending != 0) {
                    const unsigned k = (base + unsigned(src)) * 32u + unsigned(__ffs(int(pending))) - 1u;   // >= t: lower bits were ruled out above
                    pending &= pending - 1;
                    const float* row = g + size_t(k) * dim;
#pragma unroll
                    for (int c = 0; c < CHUNKS; ++c) {
                        const size_t col = col0 + (size_t(c) * 64 + lane) * VEC;
                        if (col < dim) {
                            if constexpr (VEC == 4) acc[c] = acc[c] + loadf4(row + col);
                            else acc[c] += row[col];
                        }
                    }
                }
            }
        }
        float* out = dTable + size_t(id) * dim;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const size_t col = col0 + (size_t(c) * 64 + lane) * VEC;
            if (col < dim) {
                if constexpr (VEC == 4) storef4(out + col, acc[c]);
                else out[col] = acc[c];
            }
        }
    }
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
                                                               size_t offset, const int* __restrict__ offsetOnDevice, size_t maxSeq) {
    size_t col = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
    if (col >= dim) return;
    if (offsetOnDevice) {                      // launched ahead of the device: the position is whatever the device-side counter says by then
        offset = size_t(*offsetOnDevice);
        if (offset + seq > maxSeq) return;     // the caller's promise, broken: nothing is written rather than read out of bounds
    }
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

// dst[r * dstPitch + c] = src[r * srcPitch + c] for c < width: blocks of `width` floats that lie `pitch` floats apart
// (the rows of a sequence in a key/value cache that has room to grow); rows walked by threadIdx.y
template <int VEC>
__global__ void __launch_bounds__(256) copyPitchedKernel(float* __restrict__ dst, size_t dstPitch, const float* __restrict__ src,
                                                         size_t srcPitch, size_t width, size_t rows) {
    size_t col = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
    if (col >= width) return;
    size_t step = size_t(gridDim.y) * blockDim.y;
    for (size_t r = size_t(blockIdx.y) * blockDim.y + threadIdx.y; r < rows; r += step) {
        if constexpr (VEC == 4) storef4(dst + r * dstPitch + col, loadf4(src + r * srcPitch + col));
        else dst[r * dstPitch + col] = src[r * srcPitch + col];
    }
}

// New keys and values, [batch, newLen, dim] each, to rows *position .. of every sequence of caches with `capacity` rows a
// sequence: the append of a step launched before the position is known to the host.  blockIdx.z picks
// the cache; nothing is written when the rows would not fit.
template <int VEC>
__global__ void __launch_bounds__(256) kvAppendKernel(float* __restrict__ kCache, float* __restrict__ vCache, const float* __restrict__ kNew,
                                                      const float* __restrict__ vNew, size_t batch, size_t newLen, size_t dim, size_t capacity,
                                                      const int* __restrict__ position, size_t hostPosition) {
    const size_t at = position ? size_t(*position) : hostPosition;   // the caller's position when it knows it
    if (at + newLen > capacity) return;
    float* cache = blockIdx.z == 0 ? kCache : vCache;
    const float* rows = blockIdx.z == 0 ? kNew : vNew;
    size_t col = (size_t(blockIdx.x) * blockDim.x + threadIdx.x) * VEC;
    if (col >= dim) return;
    size_t step = size_t(gridDim.y) * blockDim.y;
    for (size_t r = size_t(blockIdx.y) * blockDim.y + threadIdx.y; r < batch * newLen; r += step) {
        const size_t b = r / newLen, i = r - b * newLen;
        float* dst = cache + (b * capacity + at + i) * dim + col;
        if constexpr (VEC == 4) storef4(dst, loadf4(rows + r * dim + col));
        else *dst = rows[r * dim + col];
    }
}

__global__ void addToCounterKernel(int* counter, int by) { *counter += by; }

// Lowest index of the maximum of one row: the result of the host loop "best = 0; if (row[c] > row[best])
// best = c" it replaces.  A NaN never wins a strict '>' and, at index 0, is never beaten; the key
// below encodes exactly that.
__device__ __forceinline__ float argmaxKey(float v, size_t i) {
    if (v != v) return i == 0 ? INFINITY : -INFINITY;
    return v;
}
// thread 0 returns the index; every thread of the 1024 takes part
__device__ __forceinline__ unsigned long long argmaxOfRow(const float* __restrict__ row, size_t n) {
    __shared__ float vals[16];
    __shared__ unsigned long long idxs[16];
    float best = -INFINITY;
    unsigned long long bestIdx = ~0ull;  // "no candidate": loses against everything
    for (size_t i0 = threadIdx.x; i0 < n; i0 += size_t(8) * blockDim.x) {   // eight loads in flight, compared in index order
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const size_t i = i0 + size_t(u) * blockDim.x;
            v[u] = i < n ? row[i] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const size_t i = i0 + size_t(u) * blockDim.x;
            if (i < n) {
                const float k = argmaxKey(v[u], i);
                if (bestIdx == ~0ull || k > best) { best = k; bestIdx = i; }
            }
        }
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
    }
    return bestIdx;
}
__global__ void __launch_bounds__(1024) argmaxRowKernel(const float* __restrict__ row, size_t n, long long* __restrict__ result) {
    const unsigned long long best = argmaxOfRow(row, n);
    if (threadIdx.x == 0) result[0] = (long long)best;
}
// The same index left on the device: as a float token id in token[0] (the next step's input) and, when `history` is
// given, in history[*position + historyOffset] if that lies within historyLen; *position is advanced by `advance` first
// (the step that produced the logits has consumed that many positions).
__global__ void __launch_bounds__(1024) argmaxToTokenKernel(const float* __restrict__ row, size_t n, float* __restrict__ token,
                                                            float* __restrict__ history, size_t historyLen, int* __restrict__ position,
                                                            int advance, long long historyOffset) {
    const unsigned long long best = argmaxOfRow(row, n);
    if (threadIdx.x == 0) {
        token[0] = float(best);
        long long at = 0;
        if (position) {
            at = (long long)(*position) + advance;
            if (advance != 0) *position = int(at);
        }
        if (history) {
            const long long slot = at + historyOffset;
            if (slot >= 0 && size_t(slot) < historyLen) history[slot] = float(best);
        }
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
    if (tokens == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(ids && table && out, "NULL pointer");
    Geom2D g = geometry2D(tokens, dim, aligned16(table) && aligned16(out));
    if (g.vec == 4) embeddingForwardKernel<4><<<g.grid, g.block, 0, asStream(stream)>>>(ids, table, out, tokens, dim, (long long)vocab);
    else embeddingForwardKernel<1><<<g.grid, g.block, 0, asStream(stream)>>>(ids, table, out, tokens, dim, (long long)vocab);
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
    if (tokens <= kByTokenMax && vocab * 2 >= tokens && vocab < (size_t(1) << 31)) {   // a batch of tokens against a table at least half as large
        const bool vec = aligned16(g) && aligned16(dTable) && dim % 4 == 0;
        // a workgroup per 16 tokens, and never fewer than two per compute unit: they also share out the rows to zero
        const unsigned grid = std::max(unsigned((tokens + kTokensPerGroup - 1) / kTokensPerGroup), unsigned(computeUnits()) * 2u);
        const size_t share = (vocab + grid - 1) / grid;
        const size_t lds = ((tokens + 31) / 32 * kTokensPerGroup + (share + 31) / 32) * sizeof(unsigned);
        const void* kernel = vec ? reinterpret_cast<const void*>(embeddingBackwardByTokenKernel<4>)
                                 : reinterpret_cast<const void*>(embeddingBackwardByTokenKernel<1>);
        int st = allowDynamicSharedMemory(kernel, lds);
        if (st != BF_OK) return st;
        if (vec) embeddingBackwardByTokenKernel<4><<<grid, 1024, lds, s>>>(ids, g, dTable, unsigned(tokens), vocab, dim);
        else embeddingBackwardByTokenKernel<1><<<grid, 1024, lds, s>>>(ids, g, dTable, unsigned(tokens), vocab, dim);
        BF_LAUNCH_CHECK();
        return BF_OK;
    }
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
    histogramKernel<<<gridFor(tokens, kBlock), kBlock, 0, s>>>(ids, tokens, counts, vocab);
    BF_LAUNCH_CHECK();
    exclusiveScanKernel<<<1, 1024, 0, s>>>(counts, offsets, vocab);
    BF_LAUNCH_CHECK();
    scatterTokensKernel<<<gridFor(tokens, kBlock), kBlock, 0, s>>>(ids, tokens, offsets, counts, unordered, vocab);
    BF_LAUNCH_CHECK();
    rankTokensKernel<<<gridFor(tokens, kBlock), kBlock, 0, s>>>(ids, tokens, offsets, unordered, order, vocab);
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
    if (g.vec == 4) positionalForwardKernel<4><<<g.grid, g.block, 0, asStream(stream)>>>(x, table, out, batch, seq, dim, offset, nullptr, maxSeq);
    else positionalForwardKernel<1><<<g.grid, g.block, 0, asStream(stream)>>>(x, table, out, batch, seq, dim, offset, nullptr, maxSeq);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_positional_forward_indirect(const float* x, const float* table, float* out, size_t batch, size_t seq, size_t dim, size_t maxSeq,
                                       const int* offset, bf_stream_t stream) {
    BF_REQUIRE(seq <= maxSeq, "sequence " + std::to_string(seq) + " exceeds maxSeqLen " + std::to_string(maxSeq));
    if (batch == 0 || seq == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(x && table && out && offset, "NULL pointer");
    Geom2D g = geometry2D(seq, dim, aligned16(x) && aligned16(table) && aligned16(out));
    if (g.vec == 4) positionalForwardKernel<4><<<g.grid, g.block, 0, asStream(stream)>>>(x, table, out, batch, seq, dim, 0, offset, maxSeq);
    else positionalForwardKernel<1><<<g.grid, g.block, 0, asStream(stream)>>>(x, table, out, batch, seq, dim, 0, offset, maxSeq);
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

int bf_hip_copy_pitched(float* dst, size_t dstPitch, const float* src, size_t srcPitch, size_t width, size_t rows, bf_stream_t stream) {
    if (width == 0 || rows == 0) return BF_OK;
    BF_REQUIRE(dst && src, "NULL pointer");
    BF_REQUIRE(dstPitch >= width && srcPitch >= width, "a pitch must be at least the width");
    Geom2D g = geometry2D(rows, width, aligned16(dst) && aligned16(src) && dstPitch % 4 == 0 && srcPitch % 4 == 0);
    if (g.vec == 4) copyPitchedKernel<4><<<g.grid, g.block, 0, asStream(stream)>>>(dst, dstPitch, src, srcPitch, width, rows);
    else copyPitchedKernel<1><<<g.grid, g.block, 0, asStream(stream)>>>(dst, dstPitch, src, srcPitch, width, rows);
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

int bf_hip_argmax_last_position_device(const float* logits, size_t seq, size_t vocab, float* token, float* history, size_t historyLen,
                                       int* position, int advance, long long historyOffset, bf_stream_t stream) {
    BF_REQUIRE(seq > 0 && vocab > 0, "empty logits");
    BF_REQUIRE(vocab <= (size_t(1) << 24), "a token id beyond 2^24 has no exact float");
    BF_REQUIRE(logits && token, "NULL pointer");
    argmaxToTokenKernel<<<1, 1024, 0, asStream(stream)>>>(logits + (seq - 1) * vocab, vocab, token, history, historyLen, position, advance, historyOffset);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_kv_append_indirect(float* kCache, float* vCache, const float* kNew, const float* vNew, size_t batch, size_t newLen, size_t dim,
                              size_t capacity, const int* position, bf_stream_t stream) {
    if (batch == 0 || newLen == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(kCache && vCache && kNew && vNew && position, "NULL pointer");
    BF_REQUIRE(newLen <= capacity, "more new rows than the cache holds");
    Geom2D g = geometry2D(batch * newLen, dim, aligned16(kCache) && aligned16(vCache) && aligned16(kNew) && aligned16(vNew));
    g.grid.z = 2;
    if (g.vec == 4) kvAppendKernel<4><<<g.grid, g.block, 0, asStream(stream)>>>(kCache, vCache, kNew, vNew, batch, newLen, dim, capacity, position, 0);
    else kvAppendKernel<1><<<g.grid, g.block, 0, asStream(stream)>>>(kCache, vCache, kNew, vNew, batch, newLen, dim, capacity, position, 0);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_kv_append(float* kCache, float* vCache, const float* kNew, const float* vNew, size_t batch, size_t newLen, size_t dim, size_t capacity,
                     size_t position, bf_stream_t stream) {
    if (batch == 0 || newLen == 0 || dim == 0) return BF_OK;
    BF_REQUIRE(kCache && vCache && kNew && vNew, "NULL pointer");
    BF_REQUIRE(position + newLen <= capacity, "the new rows do not fit the cache");
    Geom2D g = geometry2D(batch * newLen, dim, aligned16(kCache) && aligned16(vCache) && aligned16(kNew) && aligned16(vNew));
    g.grid.z = 2;
    if (g.vec == 4) kvAppendKernel<4><<<g.grid, g.block, 0, asStream(stream)>>>(kCache, vCache, kNew, vNew, batch, newLen, dim, capacity, nullptr, position);
    else kvAppendKernel<1><<<g.grid, g.block, 0, asStream(stream)>>>(kCache, vCache, kNew, vNew, batch, newLen, dim, capacity, nullptr, position);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

int bf_hip_counter_add(int* counter, int by, bf_stream_t stream) {
    BF_REQUIRE(counter != nullptr, "NULL pointer");
    addToCounterKernel<<<1, 1, 0, asStream(stream)>>>(counter, by);
    BF_LAUNCH_CHECK();
    return BF_OK;
}

}  // extern "C"
