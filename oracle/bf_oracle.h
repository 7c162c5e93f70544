/*
 * CPU oracle for the BlackForge operator layer -- TEST INFRASTRUCTURE ONLY.
 *
 * This header is implemented twice with identical symbols:
 *   - oracle/bf_oracle.c      : a plain-C restatement of the reference CPU backend
 *                               (blackforge::backend::cpu), built into oracle/libbf_oracle.so;
 *   - oracle/ref_shim.cpp     : a thin wrapper that calls the real reference functions, compiled
 *                               together with the reference's own sources (where they are present)
 *                               into oracle/_ref/libbf_ref.so.
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may load either library.  The
 * shipped library (libbf_hip.so) never links, loads or calls anything declared here.
 *
 * Conventions: dense row-major float32 everywhere (the reference's runtime::Tensor); token ids and
 * class indices are floats holding integers (rounded with lround, as the reference does).  Every
 * function returns 0 on success and BFO_INVALID_ARGUMENT where the reference throws
 * std::invalid_argument.
 */
#ifndef BF_ORACLE_H
#define BF_ORACLE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BFO_OK 0
#define BFO_INVALID_ARGUMENT 1

/* 0 = the restatement, 1 = the real reference build. */
int bfo_is_reference(void);

/* ---- forward ops: src/backend/cpu/ops.cpp ---- */
int bfo_add(const float* a, const float* b, float* out, size_t n);                               /* ops.cpp:113 */
int bfo_scale(const float* x, float factor, float* out, size_t n);                               /* ops.cpp:122 */
int bfo_add_bias(const float* x, const float* bias, float* out, size_t rows, size_t features);   /* ops.cpp:130 */
int bfo_matmul(const float* a, const float* b, float* c, size_t m, size_t k, size_t n);          /* ops.cpp:161 */
int bfo_matmul_transpose_b(const float* a, const float* b, float* c, size_t m, size_t k, size_t n); /* ops.cpp:183 */
int bfo_silu(const float* x, float* out, size_t n);                                              /* ops.cpp:211 */
int bfo_relu(const float* x, float* out, size_t n);                                              /* ops.cpp:215 */
int bfo_gelu(const float* x, float* out, size_t n);                                              /* ops.cpp:219 */
int bfo_linear(const float* x, const float* w, const float* bias, float* out, size_t rows, size_t inF,
               size_t outF);                                                                     /* ops.cpp:226 */
int bfo_rmsnorm(const float* x, float* out, size_t rows, size_t features);                       /* ops.cpp:250 */
int bfo_softmax(const float* x, float* out, size_t rows, size_t features);                       /* ops.cpp:280 */
int bfo_embedding_lookup(const float* ids, const float* table, float* out, size_t batch, size_t seq,
                         size_t vocab, size_t dim);                                              /* ops.cpp:317 */
int bfo_add_positional_embedding_at(const float* x, const float* table, float* out, size_t batch, size_t seq,
                                    size_t dim, size_t maxSeq, size_t offset);                   /* ops.cpp:352,391 */
/* act: 0 = SiLU (the reference's feedForward), 1 = GELU (same block with gelu substituted; a
 * composition of reference primitives, not a reference function). */
int bfo_feed_forward(const float* x, const float* w1, const float* b1, const float* w2, const float* b2,
                     float* out, size_t rows, size_t dim, size_t hidden, int act);               /* ops.cpp:427 */
int bfo_self_attention(const float* x, const float* wq, const float* wk, const float* wv, const float* wout,
                       float* out, size_t batch, size_t seq, size_t dim, size_t heads, int causal); /* ops.cpp:444-495 */
/* kCache/vCache: [batch, oldLen, dim] on entry (ignored when oldLen == 0); kOut/vOut receive
 * [batch, oldLen+newLen, dim]. */
int bfo_self_attention_incremental(const float* xNew, const float* wq, const float* wk, const float* wv,
                                   const float* wout, float* out, const float* kCache, const float* vCache,
                                   float* kOut, float* vOut, size_t batch, size_t newLen, size_t oldLen,
                                   size_t dim, size_t heads);                                    /* ops.cpp:509-566 */

/* The attention core the GPU op `fusedAttentionForward` replaces: the per-(batch, head) body of
 * selfAttention (ops.cpp:476-485) generalised to oldLen as in selfAttentionIncremental
 * (ops.cpp:553-558).  q:[batch,newLen,dim] k,v:[batch,totalLen,dim]; out:[batch,newLen,dim];
 * m,l:[batch,heads,newLen] = row max of the masked scaled scores and sum of exp(score-m). */
int bfo_attention_core_forward(const float* q, const float* k, const float* v, float* out, float* m, float* l,
                               size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim,
                               float scale, size_t oldLen);
/* Gradients of the core: autodiff.cpp:444-462 per (batch, head). */
int bfo_attention_core_backward(const float* dOut, const float* q, const float* k, const float* v, float* dQ,
                                float* dK, float* dV, size_t batch, size_t heads, size_t newLen,
                                size_t totalLen, size_t dim, float scale, size_t oldLen);

/* ---- backward ops: src/backend/cpu/autodiff.cpp ---- */
int bfo_matmul_backward(const float* a, const float* b, const float* g, float* dA, float* dB, size_t m, size_t k,
                        size_t n);                                                               /* autodiff.cpp:78 */
int bfo_matmul_transpose_b_backward(const float* a, const float* b, const float* g, float* dA, float* dB,
                                    size_t m, size_t k, size_t n);                               /* autodiff.cpp:136 */
int bfo_add_bias_backward(const float* g, float* dBias, size_t rows, size_t features);           /* autodiff.cpp:114 */
int bfo_silu_backward(const float* x, const float* g, float* out, size_t n);                     /* autodiff.cpp:175 */
int bfo_relu_backward(const float* x, const float* g, float* out, size_t n);                     /* autodiff.cpp:182 */
int bfo_gelu_backward(const float* x, const float* g, float* out, size_t n);                     /* autodiff.cpp:186 */
int bfo_rmsnorm_backward(const float* x, const float* g, float* out, size_t rows, size_t features); /* autodiff.cpp:195 */
int bfo_softmax_backward(const float* x, const float* g, float* out, size_t rows, size_t features); /* autodiff.cpp:236 */
int bfo_embedding_lookup_backward(const float* ids, const float* g, float* dTable, size_t batch, size_t seq,
                                  size_t vocab, size_t dim);                                     /* autodiff.cpp:271 */
int bfo_add_positional_embedding_backward(const float* g, float* dTable, size_t batch, size_t seq, size_t dim,
                                          size_t maxSeq);                                        /* autodiff.cpp:302 */
int bfo_feed_forward_backward(const float* x, const float* w1, const float* b1, const float* w2, const float* b2,
                              const float* g, float* dX, float* dW1, float* dB1, float* dW2, float* dB2,
                              size_t rows, size_t dim, size_t hidden, int act);                  /* autodiff.cpp:335 */
int bfo_self_attention_backward(const float* x, const float* wq, const float* wk, const float* wv,
                                const float* wout, const float* g, float* dX, float* dWq, float* dWk, float* dWv,
                                float* dWout, size_t batch, size_t seq, size_t dim, size_t heads,
                                int causal);                                                     /* autodiff.cpp:382-483 */

/* ---- losses: src/backend/cpu/loss.cpp ---- */
int bfo_mean_squared_error(const float* pred, const float* target, float* grad, float* value, size_t n); /* loss.cpp:9 */
int bfo_softmax_cross_entropy(const float* logits, const float* target, float* grad, float* value, size_t rows,
                              size_t classes);                                                   /* loss.cpp:30 */
int bfo_softmax_cross_entropy_sparse(const float* logits, const float* targetIdx, float* grad, float* value,
                                     size_t rows, size_t classes);                               /* loss.cpp:84 */
/* Index -1 = row ignored; loss and gradient are means over the other rows (0 when there is none). */
int bfo_softmax_cross_entropy_masked(const float* logits, const float* targetIdx, float* grad, float* value,
                                     size_t rows, size_t classes);                               /* loss.cpp:149 */

/* ---- optimizers: src/backend/cpu/optimizer.cpp ---- */
int bfo_sgd_step(float* param, const float* grad, size_t n, float lr);                           /* optimizer.cpp:7 */
/* `step` is the 1-based step count after the increment at optimizer.cpp:19. */
int bfo_adamw_step(float* param, const float* grad, float* m, float* v, size_t n, long long step, float lr,
                   float beta1, float beta2, float eps, float weightDecay);                      /* optimizer.cpp:18-46 */

/* ---- misc ---- */
int bfo_round_to_bf16(const float* x, float* out, size_t n);                                     /* quantize.cpp:16-31 */
/* logits: [seq, vocab]; first-max index over the last position (src/main.cpp:504-518). */
int bfo_argmax_last_position(const float* logits, size_t seq, size_t vocab, long long* index);

/* ---- trainable pipeline: src/backend/cpu/model.cpp (forward :174-239, backward :241-342) ---- */
enum {
    BFO_LINEAR = 0,      /* arg0 = out features */
    BFO_SILU = 1,
    BFO_RELU = 2,
    BFO_GELU = 3,
    BFO_RMSNORM = 4,
    BFO_SOFTMAX = 5,
    BFO_EMBEDDING = 6,   /* arg0 = vocab, arg1 = dim */
    BFO_POSITIONAL = 7,  /* arg0 = max sequence length */
    BFO_ATTENTION = 8,   /* arg0 = heads */
    BFO_FEEDFORWARD = 9, /* arg0 = hidden, arg1 = activation (0 SiLU, 1 GELU) */
    BFO_BIDIRECTIONAL_ATTENTION = 10   /* arg0 = heads; the attention block without the causal mask (ops.cpp:504) */
};
typedef struct bfo_model bfo_model;
/* inputFeatures: last dimension of the model input (ignored when the first layer is an embedding). */
bfo_model* bfo_model_create(int numLayers, const int* kinds, const long long* arg0, const long long* arg1,
                            size_t inputFeatures);
void bfo_model_destroy(bfo_model* model);
int bfo_model_num_params(const bfo_model* model);
/* Parameter order and names follow cpu::Model::parameters() (model.cpp:421-446). */
int bfo_model_param_info(const bfo_model* model, int index, char* name, size_t nameCapacity, size_t* count);
float* bfo_model_param_value(bfo_model* model, int index);
float* bfo_model_param_grad(bfo_model* model, int index);
/* input: rank-2 [batch, seq] ids or [batch, features], or rank-3 [batch, seq, features];
 * output written to `out` (capacity outCapacity floats); *outCount receives the element count. */
int bfo_model_forward(bfo_model* model, const float* input, int rank, const size_t* shape, float* out,
                      size_t outCapacity, size_t* outCount);
int bfo_model_backward(bfo_model* model, const float* outputGrad, size_t count);
int bfo_model_zero_grad(bfo_model* model);
/* One AdamW step over parameters() with per-model moment state (optimizer.cpp:18-46). */
int bfo_model_adamw_step(bfo_model* model, float lr, float beta1, float beta2, float eps, float weightDecay);


/* ---- training run (cpu/train_runner.cpp, data/dataset.cpp, cpu/checkpoint.cpp, backend/lr_schedule.hpp) ---- */
/* The permutation of data::Dataset::shuffle(seed) (dataset.cpp:102-131): order[i] = example that moves to position i. */
int bfo_shuffle_order(size_t numExamples, unsigned seed, size_t* order);
/* cosineAnnealingLearningRate (lr_schedule.hpp:7-15). */
float bfo_cosine_learning_rate(long long epoch, long long totalEpochs, float base);
/* saveCheckpoint / loadCheckpoint in the BFCKPT1 format (cpu/checkpoint.cpp:58-135). */
int bfo_model_save_checkpoint(const bfo_model* model, const char* path);
int bfo_model_load_checkpoint(bfo_model* model, const char* path);
/* cpu::runTraining (train_runner.cpp:38-211) over a BFDATA1 dataset file (dataset.cpp:133-184).  lossKind: 0 mse,
 * 1 cross_entropy, 2 cross_entropy_sparse, 3 cross_entropy_masked; optimizerKind: 0 sgd, 1 adamw; cosineSchedule: 0/1.  The run starts from
 * `fromCheckpoint` (required: the reference's random initialisation is not restated) and writes `saveCheckpoint`
 * when that is a non-empty path.  epochLosses receives `epochs` values. */
int bfo_model_run_training(bfo_model* model, const char* datasetPath, int lossKind, int optimizerKind, long long epochs,
                           size_t batchSize, float learningRate, int cosineSchedule, const char* fromCheckpoint,
                           const char* saveCheckpoint, double* epochLosses);
/* Reference build only (returns BFO_INVALID_ARGUMENT in the restatement): writes the checkpoint of a model of this
 * layer list as cpu::Model(modelIR, seed 42) initialises it (model.cpp, random_init.cpp), for use as `fromCheckpoint`. */
int bfo_model_write_initial_checkpoint(bfo_model* model, const char* path);
/* data::saveDataset (dataset.cpp:133-152). */
int bfo_save_dataset(const char* path, int inputRank, const size_t* inputShape, int targetRank, const size_t* targetShape,
                     const float* inputs, const float* targets, size_t numExamples);

#ifdef __cplusplus
}
#endif

#endif /* BF_ORACLE_H */
