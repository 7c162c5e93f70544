/*
 * bf_hip.h -- C ABI of the MI355X (gfx950) operator backend for BlackForge.
 *
 * This is the drop-in boundary: plain pointers and sizes, no C++ types.  Each entry point is what
 * the host-side operator of the reference GPU backend (namespace blackforge::backend::cuda, headers
 * under include/blackforge/backend/cuda/ of the reference) would call instead of launching its own
 * kernels; the reference declaration each one serves is cited beside it.  The C++ operator layer with
 * the reference's signatures (blackforge::backend::hip, include/blackforge/backend/hip/) is written
 * on top of these functions only.
 *
 * Conventions
 *   - Every tensor is dense row-major float32 in device memory (reference: device_tensor.hpp:19-75).
 *     Token ids and class indices are floats holding integers, rounded to nearest (lroundf), as in the
 *     reference (ops_elementwise.cu:305-326, loss.cu:134-192).
 *   - Every function returns BF_OK or an error code; bf_hip_last_error() gives the message of the last
 *     failure on the calling thread.  BF_ERR_INVALID_ARGUMENT corresponds to the reference throwing
 *     std::invalid_argument, BF_ERR_RUNTIME to std::runtime_error from its CUDA check macros
 *     (cuda_check.hpp:14-53).
 *   - `stream` is a hipStream_t passed as void*; NULL is the default stream.  Kernels are enqueued
 *     and not waited for, as in the reference; only the *_h2d / *_d2h copies and the functions
 *     documented as synchronous block the host.
 *   - Outputs never alias inputs unless a parameter says "in/out".  Zero-sized tensors are accepted
 *     and launch nothing (reference: device_pool.cu:30-32).
 *   - One host thread at a time per PROCESS, like the reference (device_pool.hpp:39-40): the pool, the cached bf16
 *     weight images and the descriptor tables are unguarded registries.
 *   - Streams: workspace and result blocks return to the pool when the host call returns, while the kernels using
 *     them may still be queued, and the cached weight images and descriptor tables are shared by all streams.  The
 *     library therefore orders streams itself: whenever a call names another stream than the call before it (on the
 *     same device), the new stream first waits for everything enqueued on the old one (an event recorded there).
 *     Calls on different streams are correct in any interleaving; they do not overlap on the device.  Devices are
 *     selected with bf_hip_set_device (the stream last used is remembered per device).
 *   - The tuning switches (bf_hip_gemm_bf16_set_route, bf_hip_attention_set_route, bf_hip_attention_set_workspace_limit)
 *     are per host thread: a thread that names a kernel for a test does not change what another thread's calls run.
 */
#ifndef BF_HIP_H
#define BF_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BF_OK 0
#define BF_ERR_INVALID_ARGUMENT 1
#define BF_ERR_RUNTIME 2
#define BF_ERR_UNSUPPORTED 3

typedef void* bf_stream_t;
typedef void* bf_event_t;

/* Activation selector for the fused bias+activation entry points. */
enum { BF_ACT_SILU = 0, BF_ACT_GELU = 1, BF_ACT_RELU = 2 };

const char* bf_hip_last_error(void);
const char* bf_hip_version(void);

/* ---------------------------------------------------------------------------------------------
 * Devices, streams, events          (reference: device_query.hpp:21,33; device_query.cu:9-40)
 * ------------------------------------------------------------------------------------------- */
typedef struct {
    char name[128];
    char arch[32];            /* e.g. "gfx950" */
    int compute_units;
    int clock_khz;            /* peak engine clock */
    int wavefront_size;
    int lds_bytes_per_block;  /* max LDS a workgroup may use */
    size_t total_memory;      /* bytes of HBM */
} bf_device_props;

int bf_hip_device_count(int* count);                 /* enumerateDevices(): 0 devices is not an error */
int bf_hip_device_props(int index, bf_device_props* props);
int bf_hip_set_device(int index);                    /* setActiveDevice() */
int bf_hip_get_device(int* index);
int bf_hip_synchronize(void);                        /* hipDeviceSynchronize */

int bf_hip_stream_create(bf_stream_t* stream);       /* default priority; ordered with the default stream */
int bf_hip_stream_destroy(bf_stream_t stream);
int bf_hip_stream_synchronize(bf_stream_t stream);
int bf_hip_event_create(bf_event_t* event);
int bf_hip_event_destroy(bf_event_t event);
int bf_hip_event_record(bf_event_t event, bf_stream_t stream);
int bf_hip_event_synchronize(bf_event_t event);
int bf_hip_event_elapsed_ms(bf_event_t start, bf_event_t stop, float* ms);

/* ---------------------------------------------------------------------------------------------
 * Device memory: per-device size-class pool over hipMalloc   (reference: device_pool.hpp:47-54,
 * device_pool.cu:29-65; DeviceTensor::fromHost/toHost/zeros/clone device_tensor.cu:68-117)
 * ------------------------------------------------------------------------------------------- */
int bf_hip_pool_acquire(size_t bytes, void** ptr);   /* devicePoolAcquire; bytes == 0 -> *ptr = NULL */
int bf_hip_pool_release(void* ptr, size_t bytes);    /* devicePoolRelease; same `bytes` as acquired */
typedef struct {
    size_t bytes_from_driver;   /* total hipMalloc'd by the pool on the current device */
    size_t bytes_in_use;        /* handed out and not yet released */
    size_t driver_allocations;  /* number of hipMalloc calls */
    size_t acquires;            /* number of acquire calls served */
} bf_pool_stats;
int bf_hip_pool_stats(bf_pool_stats* stats);
int bf_hip_pool_trim(void);                          /* hipFree every cached block of the current device */

/* ---------------------------------------------------------------------------------------------
 * Recording a sequence of calls once and replaying it (HIP graphs).  No counterpart in the reference, which launches
 * every kernel of every step from the host; for small models a step is bounded by those launches.
 *
 * Between capture_begin(stream) and capture_end every call of this library that takes a stream records its kernels
 * instead of running them; a NULL stream argument stands for `stream` while the capture lasts, so code written against
 * the default stream records unchanged.  Memory the calls take from the pool during the capture belongs to the graph
 * until bf_hip_graph_destroy: a replay never shares a buffer with anyone else, and pool_trim cannot free it.
 * Rules for the recorded region: no call that copies to or from the host or waits for the device (memcpy_h2d/d2h,
 * synchronize, the validating embedding entry points, argmax read-backs); tensors that the region reads without writing
 * them first (parameters, optimizer state, inputs) must exist before capture_begin and stay where they are; values
 * passed BY VALUE (learning rate, AdamW step) are frozen into the graph: use the *_indirect optimizer entry points,
 * which read them from device memory.  capture_end(NULL) abandons the recording.  Replays are asynchronous on the
 * stream they are launched on; one capture at a time per process.
 * ------------------------------------------------------------------------------------------- */
typedef void* bf_graph_t;
int bf_hip_capture_begin(bf_stream_t stream);
int bf_hip_capture_end(bf_graph_t* graph);
int bf_hip_graph_launch(bf_graph_t graph, bf_stream_t stream);
int bf_hip_graph_destroy(bf_graph_t graph);

int bf_hip_memcpy_h2d(void* dst, const void* src, size_t bytes);   /* synchronous (fromHost) */
int bf_hip_memcpy_d2h(void* dst, const void* src, size_t bytes);   /* synchronous (toHost)   */
int bf_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, bf_stream_t stream);  /* clone() */
int bf_hip_fill_zero(void* dst, size_t bytes, bf_stream_t stream); /* zeros(); a fill kernel, not a memset node */

/* ---------------------------------------------------------------------------------------------
 * Elementwise family                                             (reference: ops_elementwise.cu)
 * ------------------------------------------------------------------------------------------- */
/* add: ops.hpp:8 */
int bf_hip_add(const float* a, const float* b, float* out, size_t n, bf_stream_t stream);
/* scale(x, factor): backend::cpu::scale, used by the reference's gradient averaging
 * (multi_gpu_train_runner.cu:282-297) */
int bf_hip_scale(const float* x, float factor, float* out, size_t n, bf_stream_t stream);
/* addBias: ops.hpp:14   out[r,c] = x[r,c] + bias[c] */
int bf_hip_add_bias(const float* x, const float* bias, float* out, size_t rows, size_t features,
                    bf_stream_t stream);
/* addBiasSilu: ops.hpp:23 (act = BF_ACT_SILU); BF_ACT_GELU / BF_ACT_RELU give the same fusion with
 * the reference's gelu / relu formulas.  out = act(gemm + bias) */
int bf_hip_add_bias_act(const float* gemm, const float* bias, float* out, size_t rows, size_t features, int act,
                        bf_stream_t stream);
/* addBiasResidual: ops.hpp:30   out = gemm + bias + residual */
int bf_hip_add_bias_residual(const float* gemm, const float* bias, const float* residual, float* out, size_t rows,
                             size_t features, bf_stream_t stream);
/* silu / relu / gelu: ops.hpp:82-84 */
int bf_hip_act_forward(const float* x, float* out, size_t n, int act, bf_stream_t stream);
/* siluBackward / reluBackward / geluBackward: autodiff.hpp:74-76   out = g * act'(x) */
int bf_hip_act_backward(const float* x, const float* g, float* out, size_t n, int act, bf_stream_t stream);
/* addBiasSiluBackward: autodiff.hpp:71.  dGemm = dHidden * act'(gemm + bias); dBias = column sums of
 * dGemm (dBias may be NULL to skip it). */
int bf_hip_add_bias_act_backward(const float* gemm, const float* bias, const float* dHidden, float* dGemm,
                                 float* dBias, size_t rows, size_t features, int act, bf_stream_t stream);
/* accumulate: model.cu:40-46   target += delta (in/out) */
int bf_hip_accumulate(float* target, const float* delta, size_t n, bf_stream_t stream);
/* zeroFused: model.cu:84-105.  `ptrs`/`counts` are HOST arrays of numTensors device pointers / element
 * counts; one launch zeroes them all. */
int bf_hip_zero_multi(float* const* ptrs, const size_t* counts, size_t numTensors, bf_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Row-wise ops                                     (reference: ops_elementwise.cu, autodiff.cu)
 * ------------------------------------------------------------------------------------------- */
/* rmsnorm: ops.hpp:92   y = x / sqrt(mean(x^2) + 1e-6), no gain */
int bf_hip_rmsnorm(const float* x, float* out, size_t rows, size_t features, bf_stream_t stream);
/* rmsnormBackward: autodiff.hpp:79 */
int bf_hip_rmsnorm_backward(const float* x, const float* g, float* out, size_t rows, size_t features,
                            bf_stream_t stream);
/* The same with the gradient that bypassed the normalisation added in: out = addend + rmsnormBackward(x, g), the
 * `add(gradOutput, rmsnormBackward(...))` that ends both composite blocks' backward passes (autodiff.cu:746,794).
 * addend may be NULL; out must not be addend. */
int bf_hip_rmsnorm_backward_add(const float* x, const float* g, const float* addend, float* out, size_t rows,
                                size_t features, bf_stream_t stream);
/* rmsnorm / rmsnorm_backward_add that also (or only) write the bf16 image of their result (round to nearest even,
 * [rows, features], features a multiple of 8): a result whose consumers are bf16 GEMMs needs no conversion pass, and
 * rmsnorm's fp32 output may be NULL when nothing else reads it.  No counterpart in the reference, whose cuBLASLt
 * operands are converted by floatToBf16Kernel (ops_tensorcore.cu:21-26,80-87) on every call. */
int bf_hip_rmsnorm_img(const float* x, float* out, uint16_t* image, size_t rows, size_t features, bf_stream_t stream);
int bf_hip_rmsnorm_backward_add_img(const float* x, const float* g, const float* addend, float* out, uint16_t* outImage, size_t rows,
                                    size_t features, bf_stream_t stream);
/* softmax: ops.hpp:98 */
int bf_hip_softmax(const float* x, float* out, size_t rows, size_t features, bf_stream_t stream);
/* softmaxBackward: autodiff.hpp:84 (takes the forward INPUT, recomputes y) */
int bf_hip_softmax_backward(const float* x, const float* g, float* out, size_t rows, size_t features,
                            bf_stream_t stream);
/* biasGradientOnly / addBiasBackward's dBias: autodiff.hpp:52,59   dBias[c] = sum_r g[r,c] */
int bf_hip_bias_grad(const float* g, float* dBias, size_t rows, size_t features, bf_stream_t stream);
/* bf_hip_bias_grad for callers that cannot allocate device memory (code under HIP graph capture, serving loops that
 * forbid hipMalloc): no counterpart in the reference.  Same kernels and same results as bf_hip_bias_grad, but the
 * partial sums go to an 8 MiB array that is part of the library's code object (one copy per device, held until the
 * process ends) instead of a pool block; the call makes no hipMalloc/hipFree and takes nothing from the pool.
 * Limit: min(256, ceil(rows / (4 * r))) * features <= 2^21, with r = 256 / min(256, 2^ceil(log2(features / 4))) rows
 * per workgroup: any row count up to 8192 features, fewer rows above that; BF_ERR_INVALID_ARGUMENT beyond it.
 * Calls on one device share the array, so two of them in flight at once (on different streams) race. */
int bf_hip_bias_grad_static(const float* g, float* dBias, size_t rows, size_t features, bf_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Gather / scatter                                 (reference: ops_elementwise.cu, autodiff.cu)
 * ------------------------------------------------------------------------------------------- */
/* Range check used by the validating variants (embeddingLookup ops.hpp:104,
 * embeddingLookupBackward autodiff.hpp:90, softmaxCrossEntropySparse loss.hpp:37): counts entries of
 * `ids` whose rounded value is outside [0, limit).  Synchronous; *firstBad receives one offending
 * rounded value when the count is non-zero. */
int bf_hip_count_out_of_range(const float* ids, size_t count, size_t limit, size_t* numBad, long long* firstBad,
                              bf_stream_t stream);
/* embeddingLookupPreValidated: ops.hpp:110   out[t,:] = table[lround(ids[t]),:]  (bit-exact copy) */
int bf_hip_embedding_forward(const float* ids, const float* table, float* out, size_t tokens, size_t vocab,
                             size_t dim, bf_stream_t stream);
/* embeddingLookupBackwardPreValidated: autodiff.hpp:98.  Writes every element of dTable[vocab,dim]
 * once: rows are summed over their tokens in token order (deterministic, no atomics). */
int bf_hip_embedding_backward(const float* ids, const float* g, float* dTable, size_t tokens, size_t vocab,
                              size_t dim, bf_stream_t stream);
/* addPositionalEmbedding / addPositionalEmbeddingAt: ops.hpp:115,122   out[b,s,:] = x[b,s,:] + table[offset+s,:] */
int bf_hip_positional_forward(const float* x, const float* table, float* out, size_t batch, size_t seq, size_t dim,
                              size_t maxSeq, size_t offset, bf_stream_t stream);
/* addPositionalEmbeddingBackward: autodiff.hpp:106   dTable[s,:] = sum_b g[b,s,:]; rows >= seq are zero */
int bf_hip_positional_backward(const float* g, float* dTable, size_t batch, size_t seq, size_t dim, size_t maxSeq,
                               bf_stream_t stream);
/* concatSeq (KV-cache growth): ops_transformer.cu:22-58   [batch,seqA,dim] ++ [batch,seqB,dim] */
int bf_hip_concat_seq(const float* a, const float* b, float* out, size_t batch, size_t seqA, size_t seqB, size_t dim,
                      bf_stream_t stream);
/* dst[r * dstPitch + c] = src[r * srcPitch + c], c < width, r < rows (floats; pitches >= width): the copy that appends
 * new keys and values to a cache with room to grow (hip::KVCache), where the reference concatenates into a new tensor at
 * every step (ops_transformer.cu:22-58). */
int bf_hip_copy_pitched(float* dst, size_t dstPitch, const float* src, size_t srcPitch, size_t width, size_t rows, bf_stream_t stream);
/* New keys and values, [batch, newLen, dim] each, to rows position.. of every sequence of caches with `capacity` rows a
 * sequence, both in one launch: the append of selfAttentionIncremental for several sequences (ops_transformer.cu:147-160,
 * where the reference concatenates). */
int bf_hip_kv_append(float* kCache, float* vCache, const float* kNew, const float* vNew, size_t batch, size_t newLen, size_t dim, size_t capacity,
                     size_t position, bf_stream_t stream);
/* argmaxLastPosition: main.cpp:504-518, moved to the device.  logits: [seq, vocab]; *index (HOST) gets
 * the lowest index of the maximum of the last row.  Synchronous. */
int bf_hip_argmax_last_position(const float* logits, size_t seq, size_t vocab, long long* index, bf_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * GEMM                                      (reference: ops_gemm.cu, ops_tensorcore.cu, autodiff.cu)
 * ------------------------------------------------------------------------------------------- */
/* C[M,N] = op(A) * op(B) in fp32 on fp32 MFMA.  op(A) is M x K: A is [M,K] (transA = 0) or [K,M]
 * (transA = 1); op(B) is K x N: B is [K,N] (transB = 0) or [N,K] (transB = 1).
 * matmul ops.hpp:35 (0,0); matmulTransposeB ops.hpp:40 (0,1); matmulBackward autodiff.hpp:23 (dA: 0,1 on
 * G,B; dB: 1,0 on A,G); matmulTransposeBBackward autodiff.hpp:44 (dA: 0,0 on G,B; dB: 1,0 on G,A). */
int bf_hip_gemm_f32(int transA, int transB, const float* A, const float* B, float* C, size_t M, size_t N, size_t K,
                    bf_stream_t stream);
/* The same product with the adds that follow it done where the product is stored: C = op(A) op(B) + bias (a row of N,
 * optional) + residual ([M,N], optional, may be C itself: C += op(A) op(B)), in that order, bit-identical to the
 * product followed by addBias / addBiasResidual / add.  linear ops.hpp:46 (ops_gemm.cu:112-132: cublasSgemm, then the
 * addBias kernel); the fp32 attention block's output projection + residual and the feed-forward block's second
 * projection + bias + residual (ops_transformer.cu:121-130,207-214); the sum of the Q, K and V input gradients
 * (autodiff.cu:693-699). */
int bf_hip_gemm_f32_adds(int transA, int transB, const float* A, const float* B, const float* bias, const float* residual,
                         float* C, size_t M, size_t N, size_t K, bf_stream_t stream);
/* Several independent fp32 products at once (`problems` is a HOST array): each is what bf_hip_gemm_f32_adds computes,
 * bit for bit.  Small products (the ones a model a few hundred wide consists of) share ONE launch; anything else is
 * launched product by product.  The outputs must not overlap each other or another product's operands.  Serves the two
 * gradient products of matmulBackward (autodiff.cu:294-322: two kernels, one after the other) and the three
 * projections of one input in the attention block (ops_transformer.cu:107-111) and their gradients. */
typedef struct {
    const float* A;
    const float* B;
    float* C;
    const float* bias;      /* [N] or NULL */
    const float* residual;  /* [M,N] or NULL; may be C */
    size_t M, N, K;
    int transA, transB;
} bf_gemm_f32_problem;
int bf_hip_gemm_f32_group(const bf_gemm_f32_problem* problems, size_t count, bf_stream_t stream);
/* floatToBf16 (round to nearest even): ops_tensorcore.cu:21-26,80-87.  `out` holds n bf16 values. */
int bf_hip_cvt_f32_bf16(const float* x, uint16_t* out, size_t n, bf_stream_t stream);
/* Same rounding, writing out[c,r] = bf16(x[r,c]) for x:[rows,cols]. */
int bf_hip_cvt_f32_bf16_transpose(const float* x, uint16_t* out, size_t rows, size_t cols, bf_stream_t stream);
/* C[M,N] (fp32) = A[M,K] * Bt[N,K]^T with bf16 operands, fp32 accumulate, on bf16 MFMA
 * (the cublasLtMatmul call, ops_tensorcore.cu:293-304). */
int bf_hip_gemm_bf16_nt(const uint16_t* A, const uint16_t* Bt, float* C, size_t M, size_t N, size_t K,
                        bf_stream_t stream);
/* C[M,N] (fp32) = A^T * B for bf16 A[K,M] and B[K,N] (M, N multiples of 8): the contraction runs over rows, the
 * form of a weight gradient dB = a^T g (the CUBLAS_OP_T product of matmulBf16Backward, ops_tensorcore.cu:409-411).
 * Operand fragments are transposed on their way out of LDS; no transposed image is built. */
int bf_hip_gemm_bf16_tn(const uint16_t* A, const uint16_t* B, float* C, size_t M, size_t N, size_t K,
                        bf_stream_t stream);
/* matmulBf16 ops.hpp:53 (cacheWeight = 0) / matmulBf16CachedWeight ops.hpp:72 (cacheWeight = 1):
 * c[m,n] = bf16(a[m,k]) * bf16(b[k,n]), fp32 accumulate.  With cacheWeight the bf16 image of `b` is kept
 * per (device, pointer) until bf_hip_invalidate_bf16_weight_cache(). */
int bf_hip_matmul_bf16(const float* a, const float* b, float* c, size_t m, size_t k, size_t n, int cacheWeight,
                       bf_stream_t stream);
/* matmulBf16Backward autodiff.hpp:29 / matmulBf16BackwardCachedWeight autodiff.hpp:36:
 * dA[m,k] = bf16(g) * bf16(b)^T, dB[k,n] = bf16(a)^T * bf16(g).  Either output may be NULL. */
int bf_hip_matmul_bf16_backward(const float* a, const float* b, const float* g, float* dA, float* dB, size_t m,
                                size_t k, size_t n, int cacheWeight, bf_stream_t stream);
/* linearBf16 ops.hpp:253 / linearBf16CachedWeight ops.hpp:258, with the adds that follow a projection in the
 * composite blocks folded into the GEMM's store: out[m,n] = bf16(a[m,k]) * bf16(w[k,n]) + bias[n] + residual[m,n].
 * `bias` and `residual` may each be NULL (both NULL = matmulBf16).  The sum is formed in the order the separate
 * kernels would use (addBias ops.hpp:14, addBiasResidual ops.hpp:30, add ops.hpp:8): product, then bias, then residual. */
int bf_hip_linear_bf16(const float* a, const float* w, const float* bias, const float* residual, float* out, size_t m,
                       size_t k, size_t n, int cacheWeight, bf_stream_t stream);
/* The Q, K and V projections of selfAttentionForwardCached (ops_transformer.cu:217-257: three matmulBf16 calls on
 * the same normalised input): c[i][m,n] = bf16(a[m,k]) * bf16(b[i][k,n]) for i < count (count <= 3; `b` and `c` are
 * HOST arrays of device pointers).  The input is converted once; when n is a multiple of 256 the products run as
 * one GEMM over the stacked weight images, each tile stored to its own output. */
int bf_hip_matmul_bf16_shared_input(const float* a, const float* const* b, float* const* c, size_t count, size_t m,
                                    size_t k, size_t n, int cacheWeight, bf_stream_t stream);
/* Their gradients in selfAttentionBackwardCached (autodiff.cu:756-798: three matmulBf16Backward calls and two adds):
 * dA[m,k] = sum_i bf16(g[i][m,n]) * bf16(b[i][k,n])^T (one GEMM whose contraction runs over all outputs when n is a
 * multiple of 8), dB[i][k,n] = bf16(a)^T * bf16(g[i]).  dA, dB and any dB[i] may be NULL. */
int bf_hip_matmul_bf16_shared_input_backward(const float* a, const float* const* b, const float* const* g, float* dA,
                                             float* const* dB, size_t count, size_t m, size_t k, size_t n,
                                             int cacheWeight, bf_stream_t stream);
/* The feed-forward block between its normalisation and its output in the bf16 mode (feedForwardForwardCached,
 * ops_transformer.cu:182-215: linearBf16CachedWeight, activation, linearBf16CachedWeight, residual add) with the adds
 * done by the GEMMs' stores and the activation by one pass that writes only what the second GEMM reads:
 *   z[m,hidden]      = bf16(x[m,d]) * bf16(w1[d,hidden]) + b1       fp32, kept for the backward pass
 *   hImage[m,hidden] = bf16(act(z))                                 the second GEMM's operand; no fp32 copy is written
 *   out[m,d]         = hImage * bf16(w2[hidden,d]) + b2 + residual
 * d and hidden must be multiples of 8; b1, b2 and residual may be NULL; xImage, if not NULL, receives bf16(x) ([m,d]) for
 * the backward call -- or, with x == NULL, already holds it.  Results equal those of bf_hip_matmul_bf16 + bf_hip_add_bias_act + bf_hip_linear_bf16. */
int bf_hip_feedforward_bf16(const float* x, const float* w1, const float* b1, const float* w2, const float* b2,
                            const float* residual, int act, float* z, uint16_t* hImage, uint16_t* xImage, float* out, size_t m,
                            size_t d, size_t hidden, int cacheWeight, bf_stream_t stream);
/* Its gradients (feedForwardBackwardCached, autodiff.cu:719-750, between the output gradient g[m,d] and the
 * normalisation's backward): dB2 = column sums of g; dW2 = hImage^T * bf16(g); dz = act'(z) . (bf16(g) * bf16(w2)^T),
 * of which one pass keeps the bf16 image and the column sums dB1 (taken before the rounding) and nothing else;
 * dW1 = bf16(x)^T * bf16(dz); dX = bf16(dz) * bf16(w1)^T.  One of x and xImage may be NULL; any output may be NULL. */
int bf_hip_feedforward_bf16_backward(const float* x, const uint16_t* xImage, const float* w1, const float* w2, const float* z,
                                     const uint16_t* hImage, const float* g, int act, float* dX, float* dW1, float* dB1,
                                     float* dW2, float* dB2, size_t m, size_t d, size_t hidden, int cacheWeight,
                                     bf_stream_t stream);
/* The projection entry points above with operands that already exist as bf16 images (made by the *_img producers, or
 * kept from the forward pass): wherever a fp32 operand `a` / `g` / `x` is paired with an image pointer, a non-NULL image
 * ([rows, pad8(width)] bf16, 16-byte aligned) is used as it is and the fp32 pointer may be NULL.  For the shared-input
 * backward the image holds the `count` gradients side by side: gImage[m, count * n], gradient i in columns i*n .. (n a
 * multiple of 8).  Results are those of the fp32-operand entry points, bit for bit: the images hold the same roundings. */
int bf_hip_linear_bf16_img(const float* a, const uint16_t* aImage, const float* w, const float* bias, const float* residual, float* out,
                           size_t m, size_t k, size_t n, int cacheWeight, bf_stream_t stream);
int bf_hip_matmul_bf16_backward_img(const float* a, const uint16_t* aImage, const float* b, const float* g, const uint16_t* gImage,
                                    float* dA, float* dB, size_t m, size_t k, size_t n, int cacheWeight, bf_stream_t stream);
int bf_hip_matmul_bf16_shared_input_img(const float* a, const uint16_t* aImage, const float* const* b, float* const* c, size_t count,
                                        size_t m, size_t k, size_t n, int cacheWeight, bf_stream_t stream);
int bf_hip_matmul_bf16_shared_input_backward_img(const float* a, const uint16_t* aImage, const float* const* b, const float* const* g,
                                                 const uint16_t* gImage, float* dA, float* const* dB, size_t count, size_t m, size_t k,
                                                 size_t n, int cacheWeight, bf_stream_t stream);
/* bf_hip_feedforward_bf16 itself accepts x == NULL with xImage holding bf16(x) on entry; the backward pass takes the
 * image of g beside g (g is still read for dB2; with dB2 == NULL it may be NULL). */
int bf_hip_feedforward_bf16_backward_img(const float* x, const uint16_t* xImage, const float* w1, const float* w2, const float* z,
                                         const uint16_t* hImage, const float* g, const uint16_t* gImage, int act, float* dX, float* dW1,
                                         float* dB1, float* dW2, float* dB2, size_t m, size_t d, size_t hidden, int cacheWeight,
                                         bf_stream_t stream);
/* Which kernel bf_hip_gemm_bf16_nt and the projections built on it use for C = A * Bt^T.  AUTO (the default) picks by
 * a cost estimate from the shape; the others name one tile form whatever the shape, for tests that must reach every
 * kernel with the same operands and for tuning the estimate.  Every form gives the same bits (each output element is
 * accumulated in the same order of k).  No counterpart in the reference. */
enum {
    BF_GEMM_ROUTE_AUTO = 0,
    BF_GEMM_ROUTE_PINGPONG_256 = 1,   /* 256 x 256 tiles, eight wavefronts in two alternating groups */
    BF_GEMM_ROUTE_PINGPONG_128 = 2,   /* 128 x 256 tiles, same schedule */
    BF_GEMM_ROUTE_WIDE_256 = 3,       /* 128 x 256 tiles, sixteen wavefronts */
    BF_GEMM_ROUTE_WIDE_192 = 4,       /* 128 x 192 tiles, twelve wavefronts */
    /* one workgroup per compute unit walking a list of tiles, K steps pipelined across tile boundaries (products of
     * more tiles than compute units; with fewer they fall back to the form of the same tile shape above) */
    BF_GEMM_ROUTE_WIDE_256_PERSISTENT = 5,
    BF_GEMM_ROUTE_WIDE_192_PERSISTENT = 6,
    BF_GEMM_ROUTE_PINGPONG_256_PERSISTENT = 7,
    BF_GEMM_ROUTE_PINGPONG_128_PERSISTENT = 8
};
int bf_hip_gemm_bf16_set_route(int route);
/* A measurement aid with no counterpart in the reference: the K loop of the 256 x 256 bf16 GEMM tile with every memory
 * instruction removed (operand fragments held in registers), `workgroups` workgroups of eight wavefronts, `kSteps`
 * 64-deep K steps each = 2*256*256*64 flops per step and workgroup.  shape 0 issues v_mfma_f32_32x32x16_bf16, shape 1
 * v_mfma_f32_16x16x32_bf16.  `operands`: 32768 bf16 values the fragments are drawn from (16-byte aligned);
 * `out`: workgroups*512 floats (sums of the accumulators, so the loop has a result).  What this loop reaches on a box
 * is the ceiling of any bf16 GEMM there: the matrix pipes' rate at the clock the chip holds under that load. */
int bf_hip_mfma_only_loop(const uint16_t* operands, float* out, int shape, int workgroups, int kSteps, bf_stream_t stream);
/* invalidateBf16WeightCache: ops.hpp:80 */
int bf_hip_invalidate_bf16_weight_cache(void);
/* For the caller that has just changed `count` weights in place (an optimizer step over changed[0..count)): the same
 * as bf_hip_invalidate_bf16_weight_cache(), and then every cached transposed image (with the plain image of the same
 * weights) that was used since the previous invalidation and whose weights are all among `changed` is made again from
 * the new values, all of them in ONE launch, and counts as current.  The reference converts each weight again inside
 * the next forward pass (ops_tensorcore.cu:117-131 after :448); the images and the products are the same, only the
 * dozens of small conversion launches of a step become one.  Inside a recording it only invalidates. */
int bf_hip_bf16_weight_cache_refresh(const float* const* changed, size_t count, bf_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Fused causal attention                                  (reference: fused_attention.hpp:55,73)
 * q:[batch,newLen,dim]  k,v:[batch,totalLen,dim]  heads contiguous in dim, headDim = dim/heads <= 256.
 * Query row i (absolute position oldLen+i) attends to keys j <= oldLen+i.
 * Tuned head dims are 32, 64 and 128 (forward and backward 110-175 TFLOP/s of fp32 work at 1024-4096 positions).  Head
 * dims above 128 are accepted, like the reference accepts them, and run on the fp32-MFMA kernels padded to 192 or 256:
 * measured at batch 4, 8 heads, 2048 positions, headDim 192: forward 100, dK/dV 96, dQ 96 TFLOP/s = 0.61 of the fp32
 * MFMA peak for forward + backward; headDim 256: 100 / 92 / 97 = 0.60 (headDim 224, an eighth of it padding: 90 / 81 /
 * 85).  When the dS hand-over buffer is refused (bf_hip_attention_set_workspace_limit) the dK/dV pass of such heads
 * falls to about half of that.
 * A forward pass of few queries against many keys (a step of incremental decoding: batch * heads * ceil(newLen / 128)
 * workgroups would be fewer than half the compute units, 1024 keys or more) takes the keys in chunks, a workgroup per
 * (head, chunk), and puts the chunks together in a second kernel: batch 1, 12 heads of 64, 4096 cached positions 244 ->
 * 38 us; the results are the unchunked ones up to the order of the additions.  So does a causal pass from position 0
 * (oldLen = 0, newLen = totalLen >= 1024) over so few (batch, head) pairs that the last query tile's row of key tiles is
 * at least two and a half times an even share of the work (a prompt: batch 1, 12 heads, 1024 positions 158 -> 42 us
 * inside the model's pass).
 * ------------------------------------------------------------------------------------------- */
/* fusedAttentionForward: out:[batch,newLen,dim]; m,l:[batch,heads,newLen] = row max of the scaled
 * scores and sum of exp(score - m) (the statistics the backward reuses). */
int bf_hip_attention_forward(const float* q, const float* k, const float* v, float* out, float* m, float* l,
                             size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim, float scale,
                             size_t oldLen, bf_stream_t stream);
/* The same with the bf16 image of the output written as well (outImage[batch*newLen, imageLd], imageLd >= dim, both
 * multiples of 8), for the output projection that consumes it; `out` is still needed by the backward pass. */
int bf_hip_attention_forward_img(const float* q, const float* k, const float* v, float* out, uint16_t* outImage, size_t imageLd, float* m,
                                 float* l, size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim, float scale,
                                 size_t oldLen, bf_stream_t stream);
/* The same with the keys and values of a sequence `kvRows` >= totalLen rows apart (k, v: [batch, kvRows, dim], the first
 * totalLen rows of each sequence used): attention over a cache with room to grow.  bf_hip_attention_forward_img is this
 * with kvRows = totalLen.  (No counterpart in the reference, whose cache is exactly totalLen rows long.)
 * At most eight queries per sequence with 16-byte aligned operands and a head dim that is a multiple of 4 (a step of
 * incremental decoding) are served without tiles, as a walk over the cache: the lanes that share a key hold four of the
 * head's columns each, the keys go to the workgroups in chunks of 128 or more so that about four workgroups per compute
 * unit run, and the chunks are joined by a second kernel when there are several. */
int bf_hip_attention_forward_rows(const float* q, const float* k, const float* v, float* out, uint16_t* outImage, size_t imageLd, float* m,
                                  float* l, size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t kvRows, size_t dim, float scale,
                                  size_t oldLen, bf_stream_t stream);
/* Blocks of an incremental decoding step, which keeps nothing for a backward pass (no counterparts in the reference,
 * which runs the training-time operators: ops_transformer.cu:133-180, 182-215).
 * rmsnorm_matmul_bf16_shared_input: c[i] = bf16(rmsnorm(x)) b[i] for up to three weights [k, n] (an attention block's Q, K
 * and V projections of its normalised input).  rmsnorm_feedforward_bf16: out = input + act(bf16(rmsnorm(input)) w1 + b1) w2
 * + b2 (d and hidden multiples of 8).  For one or two rows the normalisation is made by the first product's kernel
 * while it stages its rows (double sum of squares, float division, as bf_hip_rmsnorm) and the activation in its store: one
 * launch for the projections, two for the block; more rows run the row kernel and the products one after the other. */
/* The same two blocks in fp32 (products by bf_hip_gemm_f32's kernels): the normalisation inside the first product for one
 * or two rows, the feed-forward's activation where that product's K slices are summed. */
int bf_hip_rmsnorm_matmul_f32_shared_input(const float* x, const float* const* b, float* const* c, size_t count, size_t m, size_t k, size_t n,
                                           bf_stream_t stream);
int bf_hip_rmsnorm_feedforward_f32(const float* input, const float* w1, const float* b1, const float* w2, const float* b2, int act, float* out,
                                   size_t m, size_t d, size_t hidden, bf_stream_t stream);
int bf_hip_rmsnorm_matmul_bf16_shared_input(const float* x, const float* const* b, float* const* c, size_t count, size_t m, size_t k, size_t n,
                                            int cacheWeight, bf_stream_t stream);
int bf_hip_rmsnorm_feedforward_bf16(const float* input, const float* w1, const float* b1, const float* w2, const float* b2, int act, float* out,
                                    size_t m, size_t d, size_t hidden, int cacheWeight, bf_stream_t stream);
/* ---- A decoding step whose position lives on the device (no counterparts in the reference, whose generation loop
 * reads the next token back and passes the position from the host at every step, main.cpp:594-617).  These entry points
 * read the number of cached positions from device memory instead, so that the host can launch step after step without
 * waiting for the one before: positional_forward_indirect adds the table rows *offset.., kv_append_indirect copies the new
 * keys and values to rows *position.. of caches with `capacity` rows a sequence, attention_forward_rows_indirect attends
 * to the first *oldLen + newLen rows of k and v (the walk over the cache of bf_hip_attention_forward_rows, at most eight
 * queries per sequence; its chunks cover all kvRows and those past the current length do nothing),
 * argmax_last_position_device first advances *position by `advance` (the positions the step that made the logits has
 * consumed), then leaves the index on the device as a float token id (and in history[*position + historyOffset] when that
 * lies within historyLen), counter_add advances a counter on its own.  The caller promises that the
 * positions fit (table rows, cache capacity): a kernel that finds otherwise writes nothing.  (They may also be recorded
 * in a graph, whose arguments are frozen; replaying a whole decoding step that way measured slower than launching it.) */
/* decode_projections_{bf16,f32}: the attention block's three projections in that form: q = rmsnorm(x) wq (bf16: of the rows
 * rounded to bf16), the rows of rmsnorm(x) wk and rmsnorm(x) wv appended to the caches at row *position.  One sequence of
 * one or two new rows (bf16: width a multiple of 256) is one launch that stores the keys and values where they belong;
 * anything else computes them into scratch rows and appends. */
int bf_hip_decode_projections_bf16(const float* x, const float* wq, const float* wk, const float* wv, float* q, float* kCache, float* vCache,
                                   size_t batch, size_t newLen, size_t dim, size_t capacity, const int* position, int cacheWeight,
                                   bf_stream_t stream);
int bf_hip_decode_projections_f32(const float* x, const float* wq, const float* wk, const float* wv, float* q, float* kCache, float* vCache,
                                  size_t batch, size_t newLen, size_t dim, size_t capacity, const int* position, bf_stream_t stream);
int bf_hip_positional_forward_indirect(const float* x, const float* table, float* out, size_t batch, size_t seq, size_t dim, size_t maxSeq,
                                       const int* offset, bf_stream_t stream);
int bf_hip_kv_append_indirect(float* kCache, float* vCache, const float* kNew, const float* vNew, size_t batch, size_t newLen, size_t dim,
                              size_t capacity, const int* position, bf_stream_t stream);
int bf_hip_attention_forward_rows_indirect(const float* q, const float* k, const float* v, float* out, uint16_t* outImage, size_t imageLd,
                                           float* m, float* l, size_t batch, size_t heads, size_t newLen, size_t kvRows, size_t dim, float scale,
                                           const int* oldLen, bf_stream_t stream);
int bf_hip_argmax_last_position_device(const float* logits, size_t seq, size_t vocab, float* token, float* history, size_t historyLen,
                                       int* position, int advance, long long historyOffset, bf_stream_t stream);
int bf_hip_counter_add(int* counter, int by, bf_stream_t stream);
/* computeDKernel: fused_attention.cu:166-190   D[b,h,i] = dot(out[b,i,h,:], dOut[b,i,h,:]) */
int bf_hip_attention_dot_o_do(const float* out, const float* dOut, float* D, size_t batch, size_t heads,
                              size_t newLen, size_t dim, bf_stream_t stream);
/* fusedAttentionBackward: dQ:[batch,newLen,dim], dK,dV:[batch,totalLen,dim].  dK/dV are accumulated
 * by the workgroup that owns a key tile and written once; dQ by the workgroup that owns a query
 * tile.  No atomics: results are bit-reproducible run to run. */
int bf_hip_attention_backward(const float* dOut, const float* q, const float* k, const float* v, const float* out,
                              const float* m, const float* l, float* dQ, float* dK, float* dV, size_t batch,
                              size_t heads, size_t newLen, size_t totalLen, size_t dim, float scale, size_t oldLen,
                              bf_stream_t stream);

/* fusedAttentionBackward whose gradients go to bf16 images (row r of a gradient at image + r * imageLd; the three images
 * may be column slices of one [rows, 3 * dim] image, the operand layout of bf_hip_matmul_bf16_shared_input_backward_img).
 * Any image may be NULL; a gradient with an image may have a NULL fp32 tensor, which then is not written at all. */
int bf_hip_attention_backward_img(const float* dOut, const float* q, const float* k, const float* v, const float* out, const float* m,
                                  const float* l, float* dQ, float* dK, float* dV, uint16_t* dQImage, uint16_t* dKImage,
                                  uint16_t* dVImage, size_t imageLd, size_t batch, size_t heads, size_t newLen, size_t totalLen,
                                  size_t dim, float scale, size_t oldLen, bf_stream_t stream);

/* The three stages of bf_hip_attention_backward, for callers that need only one of the gradients
 * (frozen keys/values, or a query-only probe) or want to time the stages; same kernels, same results.
 * prepare: lse2[b,h,i] = m*log2(e) + log2(l) and D[b,h,i] = dot(out, dOut) (computeDKernel plus the
 * statistics fold); dkv: dK, dV from a key-tile owner; dq: dQ from a query-tile owner
 * (tiledFusedAttentionBackwardKernel, fused_attention.cu:201-303, split by which gradient is owned). */
int bf_hip_attention_backward_prepare(const float* out, const float* dOut, const float* m, const float* l, float* lse2,
                                      float* D, size_t batch, size_t heads, size_t newLen, size_t dim,
                                      bf_stream_t stream);
int bf_hip_attention_backward_dkv(const float* dOut, const float* q, const float* k, const float* v, const float* lse2,
                                  const float* D, float* dK, float* dV, size_t batch, size_t heads, size_t newLen,
                                  size_t totalLen, size_t dim, float scale, size_t oldLen, bf_stream_t stream);
int bf_hip_attention_backward_dq(const float* dOut, const float* q, const float* k, const float* v, const float* lse2,
                                 const float* D, float* dQ, size_t batch, size_t heads, size_t newLen, size_t totalLen,
                                 size_t dim, float scale, size_t oldLen, bf_stream_t stream);

/* The same backward pass with dS handed from the key-tile owner to the query-tile owner through HBM instead of
 * being recomputed: dkv_ds also writes dS = P * (dP - D) (without the scale factor) as 32x32 fp32 sub-blocks,
 * dS[((bh * ceil(newLen/32) + queryBlock) * ceil(totalLen/32) + keyBlock) * 1024 + query%32 * 32 + key%32], at least
 * every sub-block whose first key is not after its last query (the others hold no visible pair and are not read);
 * dq_from_ds contracts those sub-blocks with K (dQ = scale *
 * dS * K), so the pass runs the five matrix products of tiledFusedAttentionBackwardKernel (fused_attention.cu:201-303)
 * once each.  ds_bytes gives the size of that buffer (16-byte aligned device memory).  bf_hip_attention_backward
 * takes this route by itself when the buffer fits under the workspace limit (default: an eighth of the device's
 * memory; 0 = always recompute); the limit has no counterpart in the reference, whose kernel holds dS in registers. */
int bf_hip_attention_ds_bytes(size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t* bytes);
int bf_hip_attention_set_workspace_limit(size_t bytes);
/* Which matrix instruction the attention products use (a tuning and test switch; no counterpart in the reference, whose
 * kernel has one form).  The SPLIT bits put a kernel's products on the bf16 matrix pipe at fp32 accuracy: each fp32
 * operand is the exact sum of three bf16 terms and each product six bf16 MFMAs (everything above 2^-24 of the product),
 * accumulated in fp32 in the order of the terms' sizes; head dims up to 128, larger ones stay on the fp32 MFMA
 * (v_mfma_f32_32x32x2_f32), which route 0 uses throughout.  The default is all three bits: the forward and dK/dV
 * kernels then recompute the same scores S, and the results are as close to a float64 evaluation as route 0's (the
 * forward output closer).  With the forward or the dK/dV bit alone the forward statistics (m, l) and the backward
 * pass's S differ in the last bits, which a row whose maximum drifts by hundreds shows as an error about 1.2 times
 * route 0's.  The DQ bit covers the kernel that forms dQ from the stored dS; the dQ kernel that recomputes S and dP
 * (taken when the dS buffer would exceed the workspace limit) runs on the fp32 MFMA on every route. */
enum { BF_ATTN_ROUTE_FP32_MFMA = 0, BF_ATTN_ROUTE_SPLIT_FORWARD = 1, BF_ATTN_ROUTE_SPLIT_DKV = 2, BF_ATTN_ROUTE_SPLIT_DQ = 4,
       BF_ATTN_ROUTE_SPLIT = 7,
       BF_ATTN_ROUTE_TILES_ONLY = 8 /* added to any of the above: forward passes of few queries stay on the tile kernels */ };
int bf_hip_attention_set_route(int route);
int bf_hip_attention_backward_dkv_ds(const float* dOut, const float* q, const float* k, const float* v, const float* lse2,
                                     const float* D, float* dK, float* dV, float* dS, size_t batch, size_t heads,
                                     size_t newLen, size_t totalLen, size_t dim, float scale, size_t oldLen,
                                     bf_stream_t stream);
int bf_hip_attention_backward_dq_from_ds(const float* dS, const float* k, float* dQ, size_t batch, size_t heads, size_t newLen,
                                         size_t totalLen, size_t dim, float scale, size_t oldLen, bf_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Losses                                                      (reference: loss.hpp:20-70, loss.cu)
 * Each writes grad (same shape as the prediction) and the SUM over the batch of the per-row (per-
 * element for MSE) loss terms into lossSum[0] (device): overwritten when accumulate == 0, added to when
 * accumulate != 0 (the *Accumulate variants, loss.hpp:54-70).  The mean is lossSum / rows (/ n).
 * ------------------------------------------------------------------------------------------- */
/* meanSquaredError[Accumulate]: grad = 2 (p - t) / n, lossSum = sum (p - t)^2 */
int bf_hip_mse(const float* pred, const float* target, float* grad, float* lossSum, size_t n, int accumulate,
               bf_stream_t stream);
/* The same with the gradient's bf16 image written too (gradImage[n], round to nearest even; needs 16-byte aligned
 * tensors): the gradient products of a bf16 model's last linear layer read it in place of a conversion pass. */
int bf_hip_mse_img(const float* pred, const float* target, float* grad, uint16_t* gradImage, float* lossSum, size_t n, int accumulate,
                   bf_stream_t stream);
/* softmaxCrossEntropy[Accumulate]: dense targets */
int bf_hip_cross_entropy(const float* logits, const float* target, float* grad, float* lossSum, size_t rows,
                         size_t classes, int accumulate, bf_stream_t stream);
/* softmaxCrossEntropySparse[Accumulate]: target class index per row; indices must already be in range */
int bf_hip_cross_entropy_sparse(const float* logits, const float* targetIdx, float* grad, float* lossSum,
                                size_t rows, size_t classes, int accumulate, bf_stream_t stream);
/* The same with the gradient's bf16 image written too (gradImage[rows, classes], classes a multiple of 8, 16-byte
 * aligned tensors), for the language-model head's backward GEMMs. */
int bf_hip_cross_entropy_sparse_img(const float* logits, const float* targetIdx, float* grad, uint16_t* gradImage, float* lossSum,
                                    size_t rows, size_t classes, int accumulate, bf_stream_t stream);
/* The loss of a language-model head whose gradient is read by nothing but the head's own gradient products
 * (softmaxCrossEntropySparseAccumulate followed by the backward pass of the last linear layer, loss.cu:381-411 and
 * model.cu:278-284 in one pass over the logits): gradImage receives the gradient rounded to bf16 (the operand of
 * bf_hip_matmul_bf16_backward_img: rows of classes rounded up to 8 elements, the extra columns zero), biasGrad[classes]
 * the bias gradient, and no fp32 gradient is written.  16-byte aligned tensors with classes a multiple of 8 between
 * 4096 and 32768 take one pass: same loss and same image as bf_hip_cross_entropy_sparse_img, the column sums taken in fp32
 * before the rounding, added in another (fixed) order than bf_hip_bias_grad adds them.  Other class counts from 4096 to
 * 2^20 (an odd vocabulary such as 50257: rows on any 4-byte boundary; 128256 or 256000 words: rows walked twice, the
 * second time out of the cache) and unaligned logits take two: the loss with the image (an element may differ from the
 * other kernels' image by one bf16 step: the row sums add in another order), then the image's column sums, i.e. the
 * bias gradient of the rounded gradient values that the head's products use.  Anything else (fewer than 4096 or more
 * than 2^20 classes, an image that is not 16-byte aligned) returns BF_ERR_UNSUPPORTED and launches nothing. */
int bf_hip_cross_entropy_sparse_head(const float* logits, const float* targetIdx, uint16_t* gradImage, float* biasGrad, float* lossSum,
                                     size_t rows, size_t classes, int accumulate, bf_stream_t stream);
/* softmaxCrossEntropyMasked (the CPU backend's loss for masked-language-model training, src/backend/cpu/loss.cpp:149-215;
 * the CUDA backend has no counterpart): as the sparse form, except that a row whose index rounds to -1 is ignored (zero
 * gradient, no loss term) and gradient and loss are averaged over the n rows that are not: grad = (p - onehot) / n, and
 * lossMean[0] receives (or, with accumulate != 0, is increased by) the MEAN over those n rows, 0 when n == 0.  n is
 * counted on the device.  Every other index must already be in [0, classes). */
int bf_hip_cross_entropy_masked(const float* logits, const float* targetIdx, float* grad, float* lossMean, size_t rows,
                                size_t classes, int accumulate, bf_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Optimizers                                              (reference: optimizer.hpp:28-66, optimizer.cu)
 * `params`, `grads`, `m`, `v`, `counts` are HOST arrays with one entry per tensor; one launch updates
 * every tensor in place.
 * ------------------------------------------------------------------------------------------- */
/* SGD::step: p -= lr * g */
int bf_hip_sgd_multi(float* const* params, const float* const* grads, const size_t* counts, size_t numTensors,
                     float lr, bf_stream_t stream);
/* AdamW::step with `step` the 1-based count after increment (optimizer.cu:103-107):
 * m = b1 m + (1-b1) g; v = b2 v + (1-b2) g^2; p -= lr (m/(1-b1^t) / (sqrt(v/(1-b2^t)) + eps) + wd p) */
int bf_hip_adamw_multi(float* const* params, const float* const* grads, float* const* m, float* const* v,
                       const size_t* counts, size_t numTensors, long long step, float lr, float beta1, float beta2,
                       float eps, float weightDecay, bf_stream_t stream);
/* The same steps with what changes from step to step read from DEVICE memory, for launches that are recorded in a
 * graph (a value passed by value would be frozen into it).  bf_hip_adamw_publish / bf_hip_sgd_publish write the block
 * for one step (a one-thread kernel on `stream`, bias corrections computed on the host exactly as bf_hip_adamw_multi
 * does): call it before each replay.  No counterpart in the reference. */
typedef struct {
    float lr, beta1, beta2, eps, weight_decay, bias1, bias2;   /* bias1 = 1 - beta1^t, bias2 = 1 - beta2^t */
} bf_adamw_hyper;
int bf_hip_adamw_publish(bf_adamw_hyper* hyperDevice, long long step, float lr, float beta1, float beta2, float eps,
                         float weightDecay, bf_stream_t stream);
int bf_hip_adamw_multi_indirect(float* const* params, const float* const* grads, float* const* m, float* const* v,
                                const size_t* counts, size_t numTensors, const bf_adamw_hyper* hyperDevice, bf_stream_t stream);
int bf_hip_sgd_publish(float* lrDevice, float lr, bf_stream_t stream);
int bf_hip_sgd_multi_indirect(float* const* params, const float* const* grads, const size_t* counts, size_t numTensors,
                              const float* lrDevice, bf_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* BF_HIP_H */
