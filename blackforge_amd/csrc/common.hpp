// Shared host/device helpers for the gfx950 operator library (internal; not part of the C ABI).
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <string>

#include "bf_hip.h"

namespace bf {

// ---- error reporting ---------------------------------------------------------------------------
void setLastError(const std::string& message);
int failInvalid(const char* function, const std::string& message);
int failRuntime(const char* function, hipError_t error, const char* file, int line);

#define BF_REQUIRE(cond, msg)                                       \
    do {                                                            \
        if (!(cond)) return ::bf::failInvalid(__func__, (msg));     \
    } while (0)

#define BF_HIP_TRY(expr)                                                            \
    do {                                                                            \
        hipError_t bf_err_ = (expr);                                                \
        if (bf_err_ != hipSuccess) return ::bf::failRuntime(__func__, bf_err_, __FILE__, __LINE__); \
    } while (0)

#define BF_LAUNCH_CHECK() BF_HIP_TRY(hipGetLastError())

// The stream a NULL bf_stream_t stands for: the device's default stream, or, between bf_hip_capture_begin and
// bf_hip_capture_end, the stream that is being captured (so that code written against the default stream, like the
// C++ operator layer, records into the graph unchanged).
extern hipStream_t g_defaultStream;
// The stream the library last enqueued work on (per process; NULL = the default stream) and whether one is known.
extern hipStream_t g_currentStream;
extern bool g_currentStreamKnown;
// Orders `next` behind everything enqueued on the current stream (an event recorded there, waited for on `next`) and
// makes it the current stream.  Pool blocks, cached weight images and descriptor tables return to their registries at
// host-call exit while kernels using them may still be queued; their next user is then ordered behind those kernels
// whichever stream it runs on, because every change of stream passes through here.  Nothing happens while a graph is
// being captured (a capture uses one stream).
void switchStream(hipStream_t next);
inline hipStream_t asStream(bf_stream_t s) {
    hipStream_t r = s ? static_cast<hipStream_t>(s) : g_defaultStream;
    if (r != g_currentStream || !g_currentStreamKnown) switchStream(r);
    return r;
}
// True between bf_hip_capture_begin and bf_hip_capture_end.  While it holds, pool blocks come from and return to the
// capture's own arena, descriptor tables are private copies, and weight images are cached per capture: nothing the
// recorded kernels address can be handed to anyone else while the graph lives.
bool capturing();
// gemm_bf16.hip: returns the weight images cached during the capture to the pool (the arena, at that point).
void dropCaptureWeightImages();
// gemm_bf16.hip: a recorded graph is about to run; whatever weights it updates, the eager weight images are stale after it.
void noteGraphLaunched();

// ---- launch geometry ---------------------------------------------------------------------------
constexpr int kWave = 64;            // CDNA wavefront
constexpr int kBlock = 256;          // 4 waves: one per SIMD of a CU
constexpr unsigned kMaxGridX = 1u << 20;

inline unsigned gridFor(size_t work, size_t perBlock, unsigned cap = kMaxGridX) {
    size_t blocks = (work + perBlock - 1) / perBlock;
    if (blocks < 1) blocks = 1;
    if (blocks > cap) blocks = cap;
    return static_cast<unsigned>(blocks);
}

// True when a launch moves more bytes than the device's last-level cache holds (256 MB on MI355X): such streams are
// read and written with the non-temporal hint (ldf4<true> / stf4<true>).
constexpr size_t kLastLevelCacheBytes = size_t(256) << 20;
inline bool streamsPastCache(size_t bytes) { return bytes > kLastLevelCacheBytes; }

// Number of compute units of the current device (cached); used to size persistent grids.
int computeUnits();
// Total memory of the current device in bytes (cached per device; 0 if it cannot be read).
size_t deviceMemoryBytes();

// Raises a kernel's dynamic shared-memory limit to `bytes` on the current device (needed above 48 KiB).  The
// setting is per (kernel, device) and sticks, so it is made once and remembered.
int allowDynamicSharedMemory(const void* kernel, size_t bytes);

// Scratch memory from the per-device pool, returned on scope exit.  The release only puts the block
// back on the pool's free list; kernels already enqueued on a stream keep using it safely because
// every later user of the block is enqueued behind them on the same stream or is ordered by the
// caller (single host thread, one stream at a time per device, like the reference).
struct Scratch {
    void* ptr = nullptr;
    size_t bytes = 0;
    int status = BF_OK;
    explicit Scratch(size_t n) : bytes(n) { status = bf_hip_pool_acquire(n, &ptr); }
    ~Scratch() { if (ptr) bf_hip_pool_release(ptr, bytes); }
    Scratch(const Scratch&) = delete;
    Scratch& operator=(const Scratch&) = delete;
    template <typename T> T* as() const { return static_cast<T*>(ptr); }
};

// A small table of descriptors (pointers, counts, chunk lists) that a multi-tensor kernel reads from
// device memory.  The same table is needed step after step, so the device copy is kept per (device,
// slot) and re-uploaded only when the host bytes change; an unchanged table costs no copy and no
// host synchronisation.  `slot` separates users (zero, sgd, adamw, the weight-image refresh).
constexpr float kRmsNormEps = 1e-6f;   // rmsnorm: x / sqrt(mean(x^2) + eps), ops.cpp:250-275

enum { kSlotZero = 0, kSlotSgd = 1, kSlotAdamW = 2, kSlotConvert = 3, kSlotCount = 4 };
int uploadDescriptorTable(int slot, const void* hostBytes, size_t bytes, hipStream_t stream, const void** devicePtr);

// ---- device helpers ----------------------------------------------------------------------------
#if defined(__HIPCC__)

typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef float float16v __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float waveSum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ double waveSumD(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float waveMax(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Block-wide reductions for blocks of up to 1024 threads (16 waves).  `scratch` must hold 16 values.
template <typename T, typename Op>
__device__ __forceinline__ T blockReduce(T v, T identity, Op op, T* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = op(v, __shfl_xor(v, off, 64));
    __syncthreads();  // protect scratch from a previous reduction still being read
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    T r = identity;
    for (int w = 0; w < waves; ++w) r = op(r, scratch[w]);  // same order in every thread
    return r;
}
struct OpSum { template <typename T> __device__ T operator()(T a, T b) const { return a + b; } };
struct OpMaxF { __device__ float operator()(float a, float b) const { return fmaxf(a, b); } };

// For the flat multi-tensor kernels: tensors are laid end to end in units of blocks and entry i of `table`
// (any struct with a `firstBlock` member) starts at block table[i].firstBlock.  Returns the entry that owns
// `block`: the last one whose firstBlock is <= block (empty tensors share their successor's firstBlock and
// are skipped by that rule).  The wavefront tests 64 entries per step, so a typical parameter list takes one
// round of loads instead of a chain of dependent ones.
template <typename T>
__device__ __forceinline__ int owningTensor(const T* __restrict__ table, int numTensors, unsigned block) {
    const int lane = threadIdx.x & 63;
    int notAfter = 0;
    for (int base = 0; base < numTensors; base += 64) {
        const int i = base + lane;
        const bool le = i < numTensors && table[i].firstBlock <= block;
        notAfter += __popcll(__ballot(le));
    }
    return notAfter - 1;
}

typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float4v loadf4(const float* p) { return *reinterpret_cast<const float4v*>(p); }
__device__ __forceinline__ void storef4(float* p, float4v v) { *reinterpret_cast<float4v*>(p) = v; }
// The same accesses with the non-temporal hint (NT = true): the data is streamed past the last-level cache instead of
// being kept there.  Measured on MI355X, a kernel whose loads AND stores both carry the hint moves 6.6-6.7 TB/s on
// streams longer than the 256 MB last-level cache, against 6.0-6.2 TB/s without it (either hint alone changes nothing);
// on tensors that fit, the cache is worth more than the hint (a consumer finds its producer's output there), so the
// launchers choose by the bytes a launch moves (streamsPastCache).
template <bool NT> __device__ __forceinline__ float4v ldf4(const float* p) {
    if constexpr (NT) return __builtin_nontemporal_load(reinterpret_cast<const float4v*>(p));
    else return *reinterpret_cast<const float4v*>(p);
}
template <bool NT> __device__ __forceinline__ void stf4(float* p, float4v v) {
    if constexpr (NT) __builtin_nontemporal_store(v, reinterpret_cast<float4v*>(p));
    else *reinterpret_cast<float4v*>(p) = v;
}
template <bool NT> __device__ __forceinline__ float ldf1(const float* p) {
    if constexpr (NT) return __builtin_nontemporal_load(p);
    else return *p;
}
template <bool NT> __device__ __forceinline__ void stf1(float* p, float v) {
    if constexpr (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}
template <bool NT> __device__ __forceinline__ void stu4(void* p, uint4v v) {
    if constexpr (NT) __builtin_nontemporal_store(v, reinterpret_cast<uint4v*>(p));
    else *reinterpret_cast<uint4v*>(p) = v;
}
template <bool NT> __device__ __forceinline__ void stu2(void* p, uint2v v) {
    if constexpr (NT) __builtin_nontemporal_store(v, reinterpret_cast<uint2v*>(p));
    else *reinterpret_cast<uint2v*>(p) = v;
}

// Activations: the functions of the reference CPU backend (ops.cpp: silu x / (1 + e^-x), gelu 0.5 x (1 + tanh u) with
// u = 0.79788456 (x + 0.044715 x^3)), written through the logistic function s(y) = 1 / (1 + e^-y), which both reduce to
// without a subtraction of nearly equal numbers: silu = x s(x); 0.5 (1 + tanh u) = s(2u), so gelu = x s(2u) and
// 1 - tanh^2 u = 4 s (1 - s).  s is one hardware exponential and one hardware reciprocal (each within one unit in the
// last place), so a value costs about ten instructions instead of the forty of tanhf and an IEEE division, and is
// within 1e-6 of the exact function relative to max(|x|, 1): these kernels move 8 to 12 bytes per element and were bound
// by their arithmetic as much as by memory.
__device__ __forceinline__ float logisticF(float y) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * y)); }
__device__ __forceinline__ float siluF(float x) { return x * logisticF(x); }
__device__ __forceinline__ float reluF(float x) { return x > 0.0f ? x : 0.0f; }
// gelu's logistic argument 2u = 1.5957691216 x + 0.0713548163 x^3 goes to the hardware exponential as
// -log2(e) * 2u = x (kGeluC1 + kGeluC3 x^2): the constants multiplied out once, four operations instead of eight
constexpr float kGeluC1 = -2.3022081947f, kGeluC3 = -0.1029432389f;
__device__ __forceinline__ float geluGate(float x) {   // s(2u) = 0.5 (1 + tanh u)
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * (kGeluC1 + kGeluC3 * (x * x))));
}
__device__ __forceinline__ float geluF(float x) { return x * geluGate(x); }
__device__ __forceinline__ float siluD(float x) {
    float s = logisticF(x);
    return s * (1.0f + x * (1.0f - s));
}
__device__ __forceinline__ float reluD(float x) { return x > 0.0f ? 1.0f : 0.0f; }
__device__ __forceinline__ float geluD(float x) {
    // s + 0.5 x (1 - tanh^2 u) u' = s + x s (1 - s) 2u', 2u' = 1.5957691216 + 0.2140644488 x^2
    const float s = geluGate(x);
    return s + x * (s * (1.0f - s)) * (1.5957691216f + 0.2140644488f * (x * x));
}
template <int ACT> __device__ __forceinline__ float actF(float x) {
    if constexpr (ACT == BF_ACT_SILU) return siluF(x);
    else if constexpr (ACT == BF_ACT_GELU) return geluF(x);
    else return reluF(x);
}
template <int ACT> __device__ __forceinline__ float actD(float x) {
    if constexpr (ACT == BF_ACT_SILU) return siluD(x);
    else if constexpr (ACT == BF_ACT_GELU) return geluD(x);
    else return reluD(x);
}
// 4 x 4 transposition among the four lanes of a quad: lane t comes in holding one column of a 4 x 4 block (v_k = element
// (k, t)) and leaves holding one row (v_c = element (t, c)).  Two exchange steps (with lane t^1, then lane t^2), each a
// data-parallel move between neighbouring lanes, no LDS.
__device__ __forceinline__ float quadXor1(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
}
__device__ __forceinline__ float quadXor2(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
}
__device__ __forceinline__ void quadTranspose(float& v0, float& v1, float& v2, float& v3, int t) {
    const bool odd = (t & 1) != 0;
    const float r01 = quadXor1(odd ? v0 : v1), r23 = quadXor1(odd ? v2 : v3);
    if (odd) { v0 = r01; v2 = r23; } else { v1 = r01; v3 = r23; }
    const bool upper = (t & 2) != 0;
    const float r02 = quadXor2(upper ? v0 : v2), r13 = quadXor2(upper ? v1 : v3);
    if (upper) { v0 = r02; v1 = r13; } else { v2 = r02; v3 = r13; }
}

// fp32 -> bf16 bits, round to nearest even, NaN preserved (floatToBf16, ops_tensorcore.cu:21-26)
__device__ __forceinline__ unsigned short toBf16Bits(float x) {
    __bf16 h = static_cast<__bf16>(x);
    return __builtin_bit_cast(unsigned short, h);
}

#endif  // __HIPCC__

// Feed-forward helpers defined with the elementwise kernels and used by the bf16 GEMM entry points (features % 8 == 0,
// 16-byte aligned pointers): image[i] = bf16(act(z[i])), and dzImage = bf16(dHidden * act'(z)) with the column sums of
// that product before rounding in dBias (may be NULL).
int actToBf16Image(const float* z, unsigned short* image, size_t n, int act, hipStream_t stream);
int actBackwardToBf16Image(const float* z, const float* dHidden, unsigned short* dzImage, float* dBias, size_t rows,
                           size_t features, int act, hipStream_t stream);

}  // namespace bf
