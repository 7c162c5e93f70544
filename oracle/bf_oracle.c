/*
 * CPU oracle (restatement) of the BlackForge reference CPU backend -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain C99.  Every function follows the loop nest, accumulation order and precision (float vs
 * double) of the reference function cited beside its declaration in bf_oracle.h, so that on the
 * same inputs it reproduces the reference bit for bit wherever the C and C++ math libraries agree
 * (expf/tanhf/exp/log/sqrt/powf are the same libm entry points).  It is pinned by
 * tests/test_oracle_*.py against the literal vectors held in the reference's own tests, against
 * fixtures written by the real reference build (tests/golden/), against oracle/_ref where that is
 * built, and against closed forms; see the header of each test for what it fixes.
 *
 * Not part of the shipped library.  Only tests, the smoke check and the benchmark's cpu_baseline
 * leg load libbf_oracle.so.
 *
 * Parity status: every function below is pinned (none is "parity unpinned"); the GELU variant of
 * the feed-forward block (act = 1) has no reference function and is pinned as the composition of
 * the reference primitives rmsnorm / linear / gelu / add and their backwards.
 */
#include "bf_oracle.h"

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

int bfo_is_reference(void) { return 0; }

static float* alloc_floats(size_t n) { return (float*)malloc((n ? n : 1) * sizeof(float)); }
static float* calloc_floats(size_t n) { return (float*)calloc(n ? n : 1, sizeof(float)); }

/* ------------------------------------------------------------------------------------------- */
/* forward ops                                                                                   */
/* ------------------------------------------------------------------------------------------- */

int bfo_add(const float* a, const float* b, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
    return BFO_OK;
}

int bfo_scale(const float* x, float factor, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = x[i] * factor;
    return BFO_OK;
}

int bfo_add_bias(const float* x, const float* bias, float* out, size_t rows, size_t features) {
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < features; ++c) out[r * features + c] = x[r * features + c] + bias[c];
    return BFO_OK;
}

/* i-p-j order with a float accumulator living in the output row (ops.cpp:170-178). */
int bfo_matmul(const float* a, const float* b, float* c, size_t m, size_t k, size_t n) {
    for (size_t i = 0; i < m * n; ++i) c[i] = 0.0f;
    for (size_t i = 0; i < m; ++i) {
        for (size_t p = 0; p < k; ++p) {
            float av = a[i * k + p];
            for (size_t j = 0; j < n; ++j) c[i * n + j] += av * b[p * n + j];
        }
    }
    return BFO_OK;
}

/* a:[m,k] b:[n,k] -> a b^T; one float dot product per output (ops.cpp:197-206). */
int bfo_matmul_transpose_b(const float* a, const float* b, float* c, size_t m, size_t k, size_t n) {
    for (size_t i = 0; i < m; ++i) {
        for (size_t j = 0; j < n; ++j) {
            float sum = 0.0f;
            for (size_t p = 0; p < k; ++p) sum += a[i * k + p] * b[j * k + p];
            c[i * n + j] = sum;
        }
    }
    return BFO_OK;
}

static float silu_scalar(float x) { return x / (1.0f + expf(-x)); }
static float relu_scalar(float x) { return x > 0.0f ? x : 0.0f; }
static const float kGeluCoeff = 0.044715f;
static const float kSqrt2OverPi = 0.7978845608f;
static float gelu_scalar(float x) {
    float inner = kSqrt2OverPi * (x + kGeluCoeff * x * x * x);
    return 0.5f * x * (1.0f + tanhf(inner));
}

int bfo_silu(const float* x, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = silu_scalar(x[i]);
    return BFO_OK;
}
int bfo_relu(const float* x, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = relu_scalar(x[i]);
    return BFO_OK;
}
int bfo_gelu(const float* x, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = gelu_scalar(x[i]);
    return BFO_OK;
}

int bfo_linear(const float* x, const float* w, const float* bias, float* out, size_t rows, size_t inF,
               size_t outF) {
    float* prod = alloc_floats(rows * outF);
    bfo_matmul(x, w, prod, rows, inF, outF);
    bfo_add_bias(prod, bias, out, rows, outF);
    free(prod);
    return BFO_OK;
}

static const float kRmsNormEps = 1e-6f;

int bfo_rmsnorm(const float* x, float* out, size_t rows, size_t features) {
    for (size_t r = 0; r < rows; ++r) {
        const float* row = x + r * features;
        double sumSquares = 0.0;
        for (size_t c = 0; c < features; ++c) sumSquares += (double)row[c] * (double)row[c];
        double meanSquare = sumSquares / (double)features;
        float rms = (float)sqrt(meanSquare + (double)kRmsNormEps);
        for (size_t c = 0; c < features; ++c) out[r * features + c] = row[c] / rms;
    }
    return BFO_OK;
}

int bfo_softmax(const float* x, float* out, size_t rows, size_t features) {
    for (size_t r = 0; r < rows; ++r) {
        const float* row = x + r * features;
        float* o = out + r * features;
        float maxVal = row[0];
        for (size_t c = 1; c < features; ++c) maxVal = row[c] > maxVal ? row[c] : maxVal;
        double sumExp = 0.0;
        for (size_t c = 0; c < features; ++c) {
            double e = exp((double)(row[c] - maxVal));
            o[c] = (float)e;
            sumExp += e;
        }
        for (size_t c = 0; c < features; ++c) o[c] = (float)((double)o[c] / sumExp);
    }
    return BFO_OK;
}

int bfo_embedding_lookup(const float* ids, const float* table, float* out, size_t batch, size_t seq,
                         size_t vocab, size_t dim) {
    for (size_t i = 0; i < batch * seq; ++i) {
        long long id = (long long)lroundf(ids[i]);
        if (id < 0 || (size_t)id >= vocab) return BFO_INVALID_ARGUMENT;
        memcpy(out + i * dim, table + (size_t)id * dim, dim * sizeof(float));
    }
    return BFO_OK;
}

int bfo_add_positional_embedding_at(const float* x, const float* table, float* out, size_t batch, size_t seq,
                                    size_t dim, size_t maxSeq, size_t offset) {
    if (offset + seq > maxSeq) return BFO_INVALID_ARGUMENT;
    for (size_t b = 0; b < batch; ++b)
        for (size_t s = 0; s < seq; ++s)
            for (size_t d = 0; d < dim; ++d)
                out[(b * seq + s) * dim + d] = x[(b * seq + s) * dim + d] + table[(offset + s) * dim + d];
    return BFO_OK;
}

static void activation_forward(const float* x, float* out, size_t n, int act) {
    if (act == 1) bfo_gelu(x, out, n);
    else bfo_silu(x, out, n);
}

int bfo_feed_forward(const float* x, const float* w1, const float* b1, const float* w2, const float* b2,
                     float* out, size_t rows, size_t dim, size_t hidden, int act) {
    float* normed = alloc_floats(rows * dim);
    float* pre = alloc_floats(rows * hidden);
    float* hid = alloc_floats(rows * hidden);
    float* proj = alloc_floats(rows * dim);
    bfo_rmsnorm(x, normed, rows, dim);
    bfo_linear(normed, w1, b1, pre, rows, dim, hidden);
    activation_forward(pre, hid, rows * hidden, act);
    bfo_linear(hid, w2, b2, proj, rows, hidden, dim);
    bfo_add(x, proj, out, rows * dim);
    free(normed); free(pre); free(hid); free(proj);
    return BFO_OK;
}

/* Copy head h of example b out of / into a [batch, seq, dim] buffer (ops.cpp:26-48). */
static void extract_head(const float* full, float* head, size_t b, size_t h, size_t seq, size_t dim, size_t hd) {
    for (size_t s = 0; s < seq; ++s) memcpy(head + s * hd, full + (b * seq + s) * dim + h * hd, hd * sizeof(float));
}
static void scatter_head(float* full, const float* head, size_t b, size_t h, size_t seq, size_t dim, size_t hd) {
    for (size_t s = 0; s < seq; ++s) memcpy(full + (b * seq + s) * dim + h * hd, head + s * hd, hd * sizeof(float));
}

/* Query row i (absolute position oldLen+i) sees keys j <= oldLen+i (ops.cpp:55-65,96-107). */
static void apply_causal_mask(float* scores, size_t newLen, size_t totalLen, size_t oldLen) {
    for (size_t i = 0; i < newLen; ++i)
        for (size_t j = oldLen + i + 1; j < totalLen; ++j) scores[i * totalLen + j] = -INFINITY;
}

/* One (batch, head): scores -> mask -> softmax -> probs @ v (ops.cpp:476-485).  `masked` keeps
 * the masked scaled scores for the caller (may be NULL). */
static void head_forward(const float* qh, const float* kh, const float* vh, float* oh, float* masked,
                         size_t newLen, size_t totalLen, size_t hd, float scale, size_t oldLen, int causal) {
    float* raw = alloc_floats(newLen * totalLen);
    float* scores = masked ? masked : alloc_floats(newLen * totalLen);
    float* probs = alloc_floats(newLen * totalLen);
    bfo_matmul_transpose_b(qh, kh, raw, newLen, hd, totalLen);
    bfo_scale(raw, scale, scores, newLen * totalLen);
    if (causal) apply_causal_mask(scores, newLen, totalLen, oldLen);
    bfo_softmax(scores, probs, newLen, totalLen);
    bfo_matmul(probs, vh, oh, newLen, totalLen, hd);
    free(raw); free(probs);
    if (!masked) free(scores);
}

int bfo_attention_core_forward(const float* q, const float* k, const float* v, float* out, float* m, float* l,
                               size_t batch, size_t heads, size_t newLen, size_t totalLen, size_t dim,
                               float scale, size_t oldLen) {
    if (heads == 0 || dim % heads != 0) return BFO_INVALID_ARGUMENT;
    size_t hd = dim / heads;
    float* qh = alloc_floats(newLen * hd);
    float* kh = alloc_floats(totalLen * hd);
    float* vh = alloc_floats(totalLen * hd);
    float* oh = alloc_floats(newLen * hd);
    float* masked = alloc_floats(newLen * totalLen);
    for (size_t b = 0; b < batch; ++b) {
        for (size_t h = 0; h < heads; ++h) {
            extract_head(q, qh, b, h, newLen, dim, hd);
            extract_head(k, kh, b, h, totalLen, dim, hd);
            extract_head(v, vh, b, h, totalLen, dim, hd);
            head_forward(qh, kh, vh, oh, masked, newLen, totalLen, hd, scale, oldLen, 1);
            scatter_head(out, oh, b, h, newLen, dim, hd);
            if (m || l) {
                for (size_t i = 0; i < newLen; ++i) {
                    const float* row = masked + i * totalLen;
                    float mx = row[0];
                    for (size_t j = 1; j < totalLen; ++j) mx = row[j] > mx ? row[j] : mx;
                    double sum = 0.0;
                    for (size_t j = 0; j < totalLen; ++j) sum += exp((double)(row[j] - mx));
                    if (m) m[(b * heads + h) * newLen + i] = mx;
                    if (l) l[(b * heads + h) * newLen + i] = (float)sum;
                }
            }
        }
    }
    free(qh); free(kh); free(vh); free(oh); free(masked);
    return BFO_OK;
}

int bfo_self_attention(const float* x, const float* wq, const float* wk, const float* wv, const float* wout,
                       float* out, size_t batch, size_t seq, size_t dim, size_t heads, int causal) {
    if (heads == 0 || dim % heads != 0) return BFO_INVALID_ARGUMENT;
    size_t hd = dim / heads;
    size_t rows = batch * seq;
    float scale = 1.0f / sqrtf((float)hd);
    float* normed = alloc_floats(rows * dim);
    float* q = alloc_floats(rows * dim);
    float* k = alloc_floats(rows * dim);
    float* v = alloc_floats(rows * dim);
    float* concat = alloc_floats(rows * dim);
    float* proj = alloc_floats(rows * dim);
    float* qh = alloc_floats(seq * hd);
    float* kh = alloc_floats(seq * hd);
    float* vh = alloc_floats(seq * hd);
    float* oh = alloc_floats(seq * hd);
    bfo_rmsnorm(x, normed, rows, dim);
    bfo_matmul(normed, wq, q, rows, dim, dim);
    bfo_matmul(normed, wk, k, rows, dim, dim);
    bfo_matmul(normed, wv, v, rows, dim, dim);
    for (size_t b = 0; b < batch; ++b) {
        for (size_t h = 0; h < heads; ++h) {
            extract_head(q, qh, b, h, seq, dim, hd);
            extract_head(k, kh, b, h, seq, dim, hd);
            extract_head(v, vh, b, h, seq, dim, hd);
            head_forward(qh, kh, vh, oh, NULL, seq, seq, hd, scale, 0, causal);
            scatter_head(concat, oh, b, h, seq, dim, hd);
        }
    }
    bfo_matmul(concat, wout, proj, rows, dim, dim);
    bfo_add(x, proj, out, rows * dim);
    free(normed); free(q); free(k); free(v); free(concat); free(proj);
    free(qh); free(kh); free(vh); free(oh);
    return BFO_OK;
}

/* [batch,seqA,dim] ++ [batch,seqB,dim] along seq (ops.cpp:72-89). */
static void concat_seq(const float* a, const float* b, float* out, size_t batch, size_t seqA, size_t seqB,
                       size_t dim) {
    size_t total = seqA + seqB;
    for (size_t i = 0; i < batch; ++i) {
        if (seqA) memcpy(out + i * total * dim, a + i * seqA * dim, seqA * dim * sizeof(float));
        memcpy(out + i * total * dim + seqA * dim, b + i * seqB * dim, seqB * dim * sizeof(float));
    }
}

int bfo_self_attention_incremental(const float* xNew, const float* wq, const float* wk, const float* wv,
                                   const float* wout, float* out, const float* kCache, const float* vCache,
                                   float* kOut, float* vOut, size_t batch, size_t newLen, size_t oldLen,
                                   size_t dim, size_t heads) {
    if (heads == 0 || dim % heads != 0) return BFO_INVALID_ARGUMENT;
    size_t hd = dim / heads;
    size_t rows = batch * newLen;
    size_t totalLen = oldLen + newLen;
    float scale = 1.0f / sqrtf((float)hd);
    float* normed = alloc_floats(rows * dim);
    float* qNew = alloc_floats(rows * dim);
    float* kNew = alloc_floats(rows * dim);
    float* vNew = alloc_floats(rows * dim);
    float* concat = alloc_floats(rows * dim);
    float* proj = alloc_floats(rows * dim);
    float* qh = alloc_floats(newLen * hd);
    float* kh = alloc_floats(totalLen * hd);
    float* vh = alloc_floats(totalLen * hd);
    float* oh = alloc_floats(newLen * hd);
    bfo_rmsnorm(xNew, normed, rows, dim);
    bfo_matmul(normed, wq, qNew, rows, dim, dim);
    bfo_matmul(normed, wk, kNew, rows, dim, dim);
    bfo_matmul(normed, wv, vNew, rows, dim, dim);
    concat_seq(kCache, kNew, kOut, batch, oldLen, newLen, dim);
    concat_seq(vCache, vNew, vOut, batch, oldLen, newLen, dim);
    for (size_t b = 0; b < batch; ++b) {
        for (size_t h = 0; h < heads; ++h) {
            extract_head(qNew, qh, b, h, newLen, dim, hd);
            extract_head(kOut, kh, b, h, totalLen, dim, hd);
            extract_head(vOut, vh, b, h, totalLen, dim, hd);
            head_forward(qh, kh, vh, oh, NULL, newLen, totalLen, hd, scale, oldLen, 1);
            scatter_head(concat, oh, b, h, newLen, dim, hd);
        }
    }
    bfo_matmul(concat, wout, proj, rows, dim, dim);
    bfo_add(xNew, proj, out, rows * dim);
    free(normed); free(qNew); free(kNew); free(vNew); free(concat); free(proj);
    free(qh); free(kh); free(vh); free(oh);
    return BFO_OK;
}

/* ------------------------------------------------------------------------------------------- */
/* backward ops                                                                                  */
/* ------------------------------------------------------------------------------------------- */

int bfo_matmul_backward(const float* a, const float* b, const float* g, float* dA, float* dB, size_t m, size_t k,
                        size_t n) {
    for (size_t i = 0; i < m; ++i) {
        for (size_t p = 0; p < k; ++p) {
            float sum = 0.0f;
            for (size_t j = 0; j < n; ++j) sum += g[i * n + j] * b[p * n + j];
            dA[i * k + p] = sum;
        }
    }
    for (size_t p = 0; p < k; ++p) {
        for (size_t j = 0; j < n; ++j) {
            float sum = 0.0f;
            for (size_t i = 0; i < m; ++i) sum += a[i * k + p] * g[i * n + j];
            dB[p * n + j] = sum;
        }
    }
    return BFO_OK;
}

/* forward was a:[m,k] b:[n,k] -> [m,n]. */
int bfo_matmul_transpose_b_backward(const float* a, const float* b, const float* g, float* dA, float* dB,
                                    size_t m, size_t k, size_t n) {
    for (size_t i = 0; i < m; ++i) {
        for (size_t p = 0; p < k; ++p) {
            float sum = 0.0f;
            for (size_t j = 0; j < n; ++j) sum += g[i * n + j] * b[j * k + p];
            dA[i * k + p] = sum;
        }
    }
    for (size_t j = 0; j < n; ++j) {
        for (size_t p = 0; p < k; ++p) {
            float sum = 0.0f;
            for (size_t i = 0; i < m; ++i) sum += g[i * n + j] * a[i * k + p];
            dB[j * k + p] = sum;
        }
    }
    return BFO_OK;
}

int bfo_add_bias_backward(const float* g, float* dBias, size_t rows, size_t features) {
    for (size_t c = 0; c < features; ++c) dBias[c] = 0.0f;
    for (size_t r = 0; r < rows; ++r)
        for (size_t c = 0; c < features; ++c) dBias[c] += g[r * features + c];
    return BFO_OK;
}

static float silu_derivative(float x) {
    float sigmoid = 1.0f / (1.0f + expf(-x));
    return sigmoid * (1.0f + x * (1.0f - sigmoid));
}
static float relu_derivative(float x) { return x > 0.0f ? 1.0f : 0.0f; }
static float gelu_derivative(float x) {
    const float coeffDeriv = 3.0f * kGeluCoeff;
    float inner = kSqrt2OverPi * (x + kGeluCoeff * x * x * x);
    float t = tanhf(inner);
    float innerDerivative = kSqrt2OverPi * (1.0f + coeffDeriv * x * x);
    return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * innerDerivative;
}

int bfo_silu_backward(const float* x, const float* g, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = g[i] * silu_derivative(x[i]);
    return BFO_OK;
}
int bfo_relu_backward(const float* x, const float* g, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = g[i] * relu_derivative(x[i]);
    return BFO_OK;
}
int bfo_gelu_backward(const float* x, const float* g, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = g[i] * gelu_derivative(x[i]);
    return BFO_OK;
}

int bfo_rmsnorm_backward(const float* x, const float* g, float* out, size_t rows, size_t features) {
    for (size_t r = 0; r < rows; ++r) {
        const float* xr = x + r * features;
        const float* gr = g + r * features;
        double sumSquares = 0.0, weightedSum = 0.0;
        for (size_t c = 0; c < features; ++c) {
            double xv = (double)xr[c];
            sumSquares += xv * xv;
            weightedSum += (double)gr[c] * xv;
        }
        double meanSquare = sumSquares / (double)features;
        double rr = sqrt(meanSquare + (double)kRmsNormEps);
        for (size_t c = 0; c < features; ++c) {
            double xv = (double)xr[c];
            double gv = (double)gr[c];
            out[r * features + c] = (float)(gv / rr - xv * weightedSum / ((double)features * rr * rr * rr));
        }
    }
    return BFO_OK;
}

int bfo_softmax_backward(const float* x, const float* g, float* out, size_t rows, size_t features) {
    float* y = alloc_floats(rows * features);
    bfo_softmax(x, y, rows, features);
    for (size_t r = 0; r < rows; ++r) {
        const float* yr = y + r * features;
        const float* gr = g + r * features;
        double weightedSum = 0.0;
        for (size_t c = 0; c < features; ++c) weightedSum += (double)gr[c] * (double)yr[c];
        for (size_t c = 0; c < features; ++c)
            out[r * features + c] = (float)((double)yr[c] * ((double)gr[c] - weightedSum));
    }
    free(y);
    return BFO_OK;
}

int bfo_embedding_lookup_backward(const float* ids, const float* g, float* dTable, size_t batch, size_t seq,
                                  size_t vocab, size_t dim) {
    for (size_t i = 0; i < vocab * dim; ++i) dTable[i] = 0.0f;
    for (size_t i = 0; i < batch * seq; ++i) {
        long long id = (long long)lroundf(ids[i]);
        if (id < 0 || (size_t)id >= vocab) return BFO_INVALID_ARGUMENT;
        for (size_t d = 0; d < dim; ++d) dTable[(size_t)id * dim + d] += g[i * dim + d];
    }
    return BFO_OK;
}

int bfo_add_positional_embedding_backward(const float* g, float* dTable, size_t batch, size_t seq, size_t dim,
                                          size_t maxSeq) {
    if (seq > maxSeq) return BFO_INVALID_ARGUMENT;
    for (size_t i = 0; i < maxSeq * dim; ++i) dTable[i] = 0.0f;
    for (size_t b = 0; b < batch; ++b)
        for (size_t s = 0; s < seq; ++s)
            for (size_t d = 0; d < dim; ++d) dTable[s * dim + d] += g[(b * seq + s) * dim + d];
    return BFO_OK;
}

int bfo_feed_forward_backward(const float* x, const float* w1, const float* b1, const float* w2, const float* b2,
                              const float* g, float* dX, float* dW1, float* dB1, float* dW2, float* dB2,
                              size_t rows, size_t dim, size_t hidden, int act) {
    (void)b2;
    float* normed = alloc_floats(rows * dim);
    float* pre = alloc_floats(rows * hidden);
    float* hid = alloc_floats(rows * hidden);
    float* dHid = alloc_floats(rows * hidden);
    float* dPre = alloc_floats(rows * hidden);
    float* dNormed = alloc_floats(rows * dim);
    float* branch = alloc_floats(rows * dim);
    /* the backward recomputes the forward (autodiff.cpp:339-341) */
    bfo_rmsnorm(x, normed, rows, dim);
    bfo_linear(normed, w1, b1, pre, rows, dim, hidden);
    activation_forward(pre, hid, rows * hidden, act);

    bfo_add_bias_backward(g, dB2, rows, dim);
    bfo_matmul_backward(hid, w2, g, dHid, dW2, rows, hidden, dim);
    if (act == 1) bfo_gelu_backward(pre, dHid, dPre, rows * hidden);
    else bfo_silu_backward(pre, dHid, dPre, rows * hidden);
    bfo_add_bias_backward(dPre, dB1, rows, hidden);
    bfo_matmul_backward(normed, w1, dPre, dNormed, dW1, rows, dim, hidden);
    bfo_rmsnorm_backward(x, dNormed, branch, rows, dim);
    bfo_add(g, branch, dX, rows * dim);
    free(normed); free(pre); free(hid); free(dHid); free(dPre); free(dNormed); free(branch);
    return BFO_OK;
}

/* One (batch, head) of the backward (autodiff.cpp:444-462): probs = softmax(masked);
 * (dProbs, dV) = matmulBackward(probs, v, dO); dMasked = softmaxBackward(masked, dProbs);
 * dScores = scale * dMasked; (dQ, dK) = matmulTransposeBBackward(q, k, dScores). */
static void head_backward(const float* qh, const float* kh, const float* vh, const float* masked,
                          const float* dOh, float* dQh, float* dKh, float* dVh, size_t newLen, size_t totalLen,
                          size_t hd, float scale) {
    float* probs = alloc_floats(newLen * totalLen);
    float* dProbs = alloc_floats(newLen * totalLen);
    float* dMasked = alloc_floats(newLen * totalLen);
    float* dScores = alloc_floats(newLen * totalLen);
    bfo_softmax(masked, probs, newLen, totalLen);
    bfo_matmul_backward(probs, vh, dOh, dProbs, dVh, newLen, totalLen, hd);
    bfo_softmax_backward(masked, dProbs, dMasked, newLen, totalLen);
    bfo_scale(dMasked, scale, dScores, newLen * totalLen);
    bfo_matmul_transpose_b_backward(qh, kh, dScores, dQh, dKh, newLen, hd, totalLen);
    free(probs); free(dProbs); free(dMasked); free(dScores);
}

int bfo_attention_core_backward(const float* dOut, const float* q, const float* k, const float* v, float* dQ,
                                float* dK, float* dV, size_t batch, size_t heads, size_t newLen,
                                size_t totalLen, size_t dim, float scale, size_t oldLen) {
    if (heads == 0 || dim % heads != 0) return BFO_INVALID_ARGUMENT;
    size_t hd = dim / heads;
    float* qh = alloc_floats(newLen * hd);
    float* kh = alloc_floats(totalLen * hd);
    float* vh = alloc_floats(totalLen * hd);
    float* oh = alloc_floats(newLen * hd);
    float* dOh = alloc_floats(newLen * hd);
    float* dQh = alloc_floats(newLen * hd);
    float* dKh = alloc_floats(totalLen * hd);
    float* dVh = alloc_floats(totalLen * hd);
    float* masked = alloc_floats(newLen * totalLen);
    for (size_t b = 0; b < batch; ++b) {
        for (size_t h = 0; h < heads; ++h) {
            extract_head(q, qh, b, h, newLen, dim, hd);
            extract_head(k, kh, b, h, totalLen, dim, hd);
            extract_head(v, vh, b, h, totalLen, dim, hd);
            extract_head(dOut, dOh, b, h, newLen, dim, hd);
            head_forward(qh, kh, vh, oh, masked, newLen, totalLen, hd, scale, oldLen, 1);
            head_backward(qh, kh, vh, masked, dOh, dQh, dKh, dVh, newLen, totalLen, hd, scale);
            scatter_head(dQ, dQh, b, h, newLen, dim, hd);
            scatter_head(dK, dKh, b, h, totalLen, dim, hd);
            scatter_head(dV, dVh, b, h, totalLen, dim, hd);
        }
    }
    free(qh); free(kh); free(vh); free(oh); free(dOh); free(dQh); free(dKh); free(dVh); free(masked);
    return BFO_OK;
}

int bfo_self_attention_backward(const float* x, const float* wq, const float* wk, const float* wv,
                                const float* wout, const float* g, float* dX, float* dWq, float* dWk, float* dWv,
                                float* dWout, size_t batch, size_t seq, size_t dim, size_t heads, int causal) {
    if (heads == 0 || dim % heads != 0) return BFO_INVALID_ARGUMENT;
    size_t hd = dim / heads;
    size_t rows = batch * seq;
    float scale = 1.0f / sqrtf((float)hd);
    float* normed = alloc_floats(rows * dim);
    float* q = alloc_floats(rows * dim);
    float* k = alloc_floats(rows * dim);
    float* v = alloc_floats(rows * dim);
    float* concat = alloc_floats(rows * dim);
    float* dConcat = alloc_floats(rows * dim);
    float* dQ = calloc_floats(rows * dim);
    float* dK = calloc_floats(rows * dim);
    float* dV = calloc_floats(rows * dim);
    float* dNq = alloc_floats(rows * dim);
    float* dNk = alloc_floats(rows * dim);
    float* dNv = alloc_floats(rows * dim);
    float* dNormed = alloc_floats(rows * dim);
    float* branch = alloc_floats(rows * dim);
    float* qh = alloc_floats(seq * hd);
    float* kh = alloc_floats(seq * hd);
    float* vh = alloc_floats(seq * hd);
    float* oh = alloc_floats(seq * hd);
    float* dOh = alloc_floats(seq * hd);
    float* dQh = alloc_floats(seq * hd);
    float* dKh = alloc_floats(seq * hd);
    float* dVh = alloc_floats(seq * hd);
    /* the reference keeps every head's masked scores alive between its two loops
     * (autodiff.cpp:403-426); recomputing them per head in the second loop gives the same values */
    float* masked = alloc_floats(seq * seq);

    bfo_rmsnorm(x, normed, rows, dim);
    bfo_matmul(normed, wq, q, rows, dim, dim);
    bfo_matmul(normed, wk, k, rows, dim, dim);
    bfo_matmul(normed, wv, v, rows, dim, dim);
    for (size_t b = 0; b < batch; ++b) {
        for (size_t h = 0; h < heads; ++h) {
            extract_head(q, qh, b, h, seq, dim, hd);
            extract_head(k, kh, b, h, seq, dim, hd);
            extract_head(v, vh, b, h, seq, dim, hd);
            head_forward(qh, kh, vh, oh, NULL, seq, seq, hd, scale, 0, causal);
            scatter_head(concat, oh, b, h, seq, dim, hd);
        }
    }
    bfo_matmul_backward(concat, wout, g, dConcat, dWout, rows, dim, dim);
    for (size_t b = 0; b < batch; ++b) {
        for (size_t h = 0; h < heads; ++h) {
            extract_head(q, qh, b, h, seq, dim, hd);
            extract_head(k, kh, b, h, seq, dim, hd);
            extract_head(v, vh, b, h, seq, dim, hd);
            extract_head(dConcat, dOh, b, h, seq, dim, hd);
            head_forward(qh, kh, vh, oh, masked, seq, seq, hd, scale, 0, causal);
            head_backward(qh, kh, vh, masked, dOh, dQh, dKh, dVh, seq, seq, hd, scale);
            scatter_head(dQ, dQh, b, h, seq, dim, hd);
            scatter_head(dK, dKh, b, h, seq, dim, hd);
            scatter_head(dV, dVh, b, h, seq, dim, hd);
        }
    }
    bfo_matmul_backward(normed, wq, dQ, dNq, dWq, rows, dim, dim);
    bfo_matmul_backward(normed, wk, dK, dNk, dWk, rows, dim, dim);
    bfo_matmul_backward(normed, wv, dV, dNv, dWv, rows, dim, dim);
    bfo_add(dNq, dNk, dNormed, rows * dim);
    bfo_add(dNormed, dNv, dNormed, rows * dim);
    bfo_rmsnorm_backward(x, dNormed, branch, rows, dim);
    bfo_add(g, branch, dX, rows * dim);

    free(normed); free(q); free(k); free(v); free(concat); free(dConcat); free(dQ); free(dK); free(dV);
    free(dNq); free(dNk); free(dNv); free(dNormed); free(branch);
    free(qh); free(kh); free(vh); free(oh); free(dOh); free(dQh); free(dKh); free(dVh); free(masked);
    return BFO_OK;
}

/* ------------------------------------------------------------------------------------------- */
/* losses                                                                                        */
/* ------------------------------------------------------------------------------------------- */

int bfo_mean_squared_error(const float* pred, const float* target, float* grad, float* value, size_t n) {
    double sumSquares = 0.0;
    for (size_t i = 0; i < n; ++i) {
        float diff = pred[i] - target[i];
        sumSquares += (double)diff * (double)diff;
        grad[i] = 2.0f * diff / (float)n;
    }
    *value = (float)(sumSquares / (double)n);
    return BFO_OK;
}

static void row_probabilities(const float* row, double* probs, size_t classes) {
    float maxLogit = row[0];
    for (size_t c = 1; c < classes; ++c) maxLogit = row[c] > maxLogit ? row[c] : maxLogit;
    double sumExp = 0.0;
    for (size_t c = 0; c < classes; ++c) {
        probs[c] = exp((double)(row[c] - maxLogit));
        sumExp += probs[c];
    }
    for (size_t c = 0; c < classes; ++c) probs[c] /= sumExp;
}

int bfo_softmax_cross_entropy(const float* logits, const float* target, float* grad, float* value, size_t rows,
                              size_t classes) {
    double* probs = (double*)malloc((classes ? classes : 1) * sizeof(double));
    double totalLoss = 0.0;
    for (size_t b = 0; b < rows; ++b) {
        row_probabilities(logits + b * classes, probs, classes);
        for (size_t c = 0; c < classes; ++c) {
            float t = target[b * classes + c];
            if (t != 0.0f) {
                double p = probs[c] > 1e-12 ? probs[c] : 1e-12;
                totalLoss += -(double)t * log(p);
            }
            grad[b * classes + c] = (float)((probs[c] - (double)t) / (double)rows);
        }
    }
    *value = (float)(totalLoss / (double)rows);
    free(probs);
    return BFO_OK;
}

int bfo_softmax_cross_entropy_sparse(const float* logits, const float* targetIdx, float* grad, float* value,
                                     size_t rows, size_t classes) {
    double* probs = (double*)malloc((classes ? classes : 1) * sizeof(double));
    double totalLoss = 0.0;
    for (size_t b = 0; b < rows; ++b) {
        long long cls = (long long)lroundf(targetIdx[b]);
        if (cls < 0 || (size_t)cls >= classes) {
            free(probs);
            return BFO_INVALID_ARGUMENT;
        }
        row_probabilities(logits + b * classes, probs, classes);
        for (size_t c = 0; c < classes; ++c) {
            float t = (c == (size_t)cls) ? 1.0f : 0.0f;
            grad[b * classes + c] = (float)((probs[c] - (double)t) / (double)rows);
        }
        double p = probs[cls] > 1e-12 ? probs[cls] : 1e-12;
        totalLoss += -log(p);
    }
    *value = (float)(totalLoss / (double)rows);
    free(probs);
    return BFO_OK;
}

/* loss.cpp:149-215.  A row whose index rounds to -1 is skipped; gradient rows are first written unnormalised
 * (float(prob) - t) and then multiplied by 1.0f / numMaskedRows in float (loss.cpp:194-213). */
int bfo_softmax_cross_entropy_masked(const float* logits, const float* targetIdx, float* grad, float* value,
                                     size_t rows, size_t classes) {
    double* probs = (double*)malloc((classes ? classes : 1) * sizeof(double));
    double totalLoss = 0.0;
    size_t numMaskedRows = 0;
    for (size_t i = 0; i < rows * classes; ++i) grad[i] = 0.0f;
    for (size_t b = 0; b < rows; ++b) {
        long long cls = (long long)lroundf(targetIdx[b]);
        if (cls == -1) continue;
        if (cls < 0 || (size_t)cls >= classes) {
            free(probs);
            return BFO_INVALID_ARGUMENT;
        }
        ++numMaskedRows;
        row_probabilities(logits + b * classes, probs, classes);
        double p = probs[cls] > 1e-12 ? probs[cls] : 1e-12;
        totalLoss += -log(p);
        for (size_t c = 0; c < classes; ++c) {
            float t = (c == (size_t)cls) ? 1.0f : 0.0f;
            grad[b * classes + c] = (float)probs[c] - t;
        }
    }
    *value = 0.0f;
    if (numMaskedRows > 0) {
        *value = (float)(totalLoss / (double)numMaskedRows);
        float invMaskedRows = 1.0f / (float)numMaskedRows;
        for (size_t i = 0; i < rows * classes; ++i) grad[i] *= invMaskedRows;
    }
    free(probs);
    return BFO_OK;
}

/* ------------------------------------------------------------------------------------------- */
/* optimizers, quantisation, argmax                                                              */
/* ------------------------------------------------------------------------------------------- */

int bfo_sgd_step(float* param, const float* grad, size_t n, float lr) {
    for (size_t i = 0; i < n; ++i) param[i] -= lr * grad[i];
    return BFO_OK;
}

int bfo_adamw_step(float* param, const float* grad, float* m, float* v, size_t n, long long step, float lr,
                   float beta1, float beta2, float eps, float weightDecay) {
    float t = (float)step;
    float bias1 = 1.0f - powf(beta1, t);
    float bias2 = 1.0f - powf(beta2, t);
    for (size_t i = 0; i < n; ++i) {
        float g = grad[i];
        m[i] = beta1 * m[i] + (1.0f - beta1) * g;
        v[i] = beta2 * v[i] + (1.0f - beta2) * g * g;
        float mHat = m[i] / bias1;
        float vHat = v[i] / bias2;
        param[i] -= lr * (mHat / (sqrtf(vHat) + eps) + weightDecay * param[i]);
    }
    return BFO_OK;
}

/* Round-to-nearest-even on the upper 16 bits; non-finite values pass through. */
int bfo_round_to_bf16(const float* x, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) {
        float value = x[i];
        if (!isfinite(value)) {
            out[i] = value;
            continue;
        }
        unsigned int bits;
        memcpy(&bits, &value, sizeof(bits));
        unsigned int lsb = (bits >> 16) & 1u;
        bits = (bits + 0x7FFFu + lsb) & 0xFFFF0000u;
        memcpy(&out[i], &bits, sizeof(bits));
    }
    return BFO_OK;
}

/* Strict '>' keeps the lowest index on ties. */
int bfo_argmax_last_position(const float* logits, size_t seq, size_t vocab, long long* index) {
    if (seq == 0 || vocab == 0) return BFO_INVALID_ARGUMENT;
    const float* row = logits + (seq - 1) * vocab;
    size_t best = 0;
    float bestVal = row[0];
    for (size_t c = 1; c < vocab; ++c) {
        if (row[c] > bestVal) {
            bestVal = row[c];
            best = c;
        }
    }
    *index = (long long)best;
    return BFO_OK;
}

/* ------------------------------------------------------------------------------------------- */
/* trainable pipeline                                                                            */
/* ------------------------------------------------------------------------------------------- */

typedef struct {
    char name[64];
    size_t count;
    size_t rows, cols; /* shape: [rows, cols], or [rows] when cols == 0 */
    float* value;
    float* grad;
    float* m; /* AdamW moments, allocated on first step */
    float* v;
} bfo_param;

typedef struct {
    int kind;
    long long arg0, arg1;
    size_t inFeatures;  /* last dim of the layer input (0 for embedding) */
    size_t outFeatures; /* last dim of the layer output */
    int params[6];      /* indices into model->params, -1 = unused */
    float* cachedInput;
    size_t cachedCount;
    size_t cachedShape[3];
    int cachedRank;
} bfo_layer;

struct bfo_model {
    int numLayers;
    bfo_layer* layers;
    int numParams;
    bfo_param* params;
    long long adamStep;
};

static int add_param(bfo_model* model, const char* base, const char* suffix, size_t rows, size_t cols) {
    const size_t count = cols ? rows * cols : rows;
    model->params = (bfo_param*)realloc(model->params, (size_t)(model->numParams + 1) * sizeof(bfo_param));
    bfo_param* p = &model->params[model->numParams];
    snprintf(p->name, sizeof(p->name), "%s.%s", base, suffix);
    p->count = count;
    p->rows = rows;
    p->cols = cols;
    p->value = calloc_floats(count);
    p->grad = calloc_floats(count);
    p->m = NULL;
    p->v = NULL;
    return model->numParams++;
}

bfo_model* bfo_model_create(int numLayers, const int* kinds, const long long* arg0, const long long* arg1,
                            size_t inputFeatures) {
    bfo_model* model = (bfo_model*)calloc(1, sizeof(bfo_model));
    model->numLayers = numLayers;
    model->layers = (bfo_layer*)calloc((size_t)(numLayers > 0 ? numLayers : 1), sizeof(bfo_layer));
    size_t features = inputFeatures;
    for (int i = 0; i < numLayers; ++i) {
        bfo_layer* layer = &model->layers[i];
        layer->kind = kinds[i];
        layer->arg0 = arg0[i];
        layer->arg1 = arg1 ? arg1[i] : 0;
        layer->inFeatures = features;
        for (int s = 0; s < 6; ++s) layer->params[s] = -1;
        char base[48];
        /* value ids: the model input is value 0, layer i writes value i+1 (names as model.cpp:68-156) */
        int outputId = i + 1;
        switch (layer->kind) {
            case BFO_LINEAR: {
                size_t outF = (size_t)layer->arg0;
                snprintf(base, sizeof(base), "linear%d", outputId);
                layer->params[0] = add_param(model, base, "weight", features, outF);
                layer->params[1] = add_param(model, base, "bias", outF, 0);
                features = outF;
                break;
            }
            case BFO_EMBEDDING: {
                snprintf(base, sizeof(base), "embedding%d", outputId);
                layer->params[0] = add_param(model, base, "table", (size_t)layer->arg0, (size_t)layer->arg1);
                features = (size_t)layer->arg1;
                break;
            }
            case BFO_POSITIONAL: {
                snprintf(base, sizeof(base), "positional_embedding%d", outputId);
                layer->params[0] = add_param(model, base, "table", (size_t)layer->arg0, features);
                break;
            }
            case BFO_ATTENTION:
            case BFO_BIDIRECTIONAL_ATTENTION: {   /* model.cpp:124-150: same parameters, named after the op */
                if (layer->arg0 <= 0 || features % (size_t)layer->arg0 != 0) {
                    bfo_model_destroy(model);
                    return NULL;
                }
                snprintf(base, sizeof(base), layer->kind == BFO_ATTENTION ? "attention%d" : "bidirectional_attention%d", outputId);
                layer->params[0] = add_param(model, base, "wq", features, features);
                layer->params[1] = add_param(model, base, "wk", features, features);
                layer->params[2] = add_param(model, base, "wv", features, features);
                layer->params[3] = add_param(model, base, "wout", features, features);
                break;
            }
            case BFO_FEEDFORWARD: {
                size_t hidden = (size_t)layer->arg0;
                snprintf(base, sizeof(base), "feedforward%d", outputId);
                layer->params[0] = add_param(model, base, "w1", features, hidden);
                layer->params[1] = add_param(model, base, "b1", hidden, 0);
                layer->params[2] = add_param(model, base, "w2", hidden, features);
                layer->params[3] = add_param(model, base, "b2", features, 0);
                break;
            }
            default:
                break;
        }
        layer->outFeatures = features;
    }
    return model;
}

void bfo_model_destroy(bfo_model* model) {
    if (!model) return;
    for (int i = 0; i < model->numParams; ++i) {
        free(model->params[i].value);
        free(model->params[i].grad);
        free(model->params[i].m);
        free(model->params[i].v);
    }
    for (int i = 0; i < model->numLayers; ++i) free(model->layers[i].cachedInput);
    free(model->params);
    free(model->layers);
    free(model);
}

int bfo_model_num_params(const bfo_model* model) { return model->numParams; }

int bfo_model_param_info(const bfo_model* model, int index, char* name, size_t nameCapacity, size_t* count) {
    if (index < 0 || index >= model->numParams) return BFO_INVALID_ARGUMENT;
    if (name && nameCapacity) snprintf(name, nameCapacity, "%s", model->params[index].name);
    if (count) *count = model->params[index].count;
    return BFO_OK;
}

float* bfo_model_param_value(bfo_model* model, int index) { return model->params[index].value; }
float* bfo_model_param_grad(bfo_model* model, int index) { return model->params[index].grad; }

static float* pv(bfo_model* model, const bfo_layer* layer, int slot) { return model->params[layer->params[slot]].value; }
static float* pg(bfo_model* model, const bfo_layer* layer, int slot) { return model->params[layer->params[slot]].grad; }

static void accumulate(float* target, const float* delta, size_t n) {
    for (size_t i = 0; i < n; ++i) target[i] += delta[i];
}

int bfo_model_forward(bfo_model* model, const float* input, int rank, const size_t* shape, float* out,
                      size_t outCapacity, size_t* outCount) {
    if (rank < 2 || rank > 3) return BFO_INVALID_ARGUMENT;
    size_t curShape[3] = {shape[0], shape[1], rank == 3 ? shape[2] : 0};
    int curRank = rank;
    size_t count = shape[0] * shape[1] * (rank == 3 ? shape[2] : 1);
    float* current = alloc_floats(count);
    memcpy(current, input, count * sizeof(float));
    int status = BFO_OK;

    for (int li = 0; li < model->numLayers && status == BFO_OK; ++li) {
        bfo_layer* layer = &model->layers[li];
        free(layer->cachedInput);
        layer->cachedInput = alloc_floats(count);
        memcpy(layer->cachedInput, current, count * sizeof(float));
        layer->cachedCount = count;
        layer->cachedRank = curRank;
        memcpy(layer->cachedShape, curShape, sizeof(curShape));

        size_t features = curShape[curRank - 1];
        size_t rows = features ? count / features : 0;
        float* next = NULL;
        size_t nextCount = count;
        switch (layer->kind) {
            case BFO_LINEAR: {
                size_t outF = (size_t)layer->arg0;
                if (features != layer->inFeatures) { status = BFO_INVALID_ARGUMENT; break; }
                nextCount = rows * outF;
                next = alloc_floats(nextCount);
                bfo_linear(current, pv(model, layer, 0), pv(model, layer, 1), next, rows, features, outF);
                curShape[curRank - 1] = outF;
                break;
            }
            case BFO_SILU: next = alloc_floats(count); bfo_silu(current, next, count); break;
            case BFO_RELU: next = alloc_floats(count); bfo_relu(current, next, count); break;
            case BFO_GELU: next = alloc_floats(count); bfo_gelu(current, next, count); break;
            case BFO_RMSNORM: next = alloc_floats(count); bfo_rmsnorm(current, next, rows, features); break;
            case BFO_SOFTMAX: next = alloc_floats(count); bfo_softmax(current, next, rows, features); break;
            case BFO_EMBEDDING: {
                if (curRank != 2) { status = BFO_INVALID_ARGUMENT; break; }
                size_t dim = (size_t)layer->arg1;
                nextCount = count * dim;
                next = alloc_floats(nextCount);
                status = bfo_embedding_lookup(current, pv(model, layer, 0), next, curShape[0], curShape[1],
                                              (size_t)layer->arg0, dim);
                curRank = 3;
                curShape[2] = dim;
                break;
            }
            case BFO_POSITIONAL: {
                if (curRank != 3) { status = BFO_INVALID_ARGUMENT; break; }
                next = alloc_floats(count);
                status = bfo_add_positional_embedding_at(current, pv(model, layer, 0), next, curShape[0], curShape[1],
                                                         curShape[2], (size_t)layer->arg0, 0);
                break;
            }
            case BFO_ATTENTION:
            case BFO_BIDIRECTIONAL_ATTENTION: {   /* model.cpp:218-226 */
                if (curRank != 3) { status = BFO_INVALID_ARGUMENT; break; }
                next = alloc_floats(count);
                status = bfo_self_attention(current, pv(model, layer, 0), pv(model, layer, 1), pv(model, layer, 2),
                                            pv(model, layer, 3), next, curShape[0], curShape[1], curShape[2],
                                            (size_t)layer->arg0, layer->kind == BFO_ATTENTION);
                break;
            }
            case BFO_FEEDFORWARD: {
                next = alloc_floats(count);
                status = bfo_feed_forward(current, pv(model, layer, 0), pv(model, layer, 1), pv(model, layer, 2),
                                          pv(model, layer, 3), next, rows, features, (size_t)layer->arg0,
                                          (int)layer->arg1);
                break;
            }
            default: status = BFO_INVALID_ARGUMENT; break;
        }
        if (next) {
            free(current);
            current = next;
            count = nextCount;
        }
    }
    if (status == BFO_OK) {
        if (outCount) *outCount = count;
        if (count > outCapacity) status = BFO_INVALID_ARGUMENT;
        else memcpy(out, current, count * sizeof(float));
    }
    free(current);
    return status;
}

int bfo_model_backward(bfo_model* model, const float* outputGrad, size_t count) {
    float* grad = alloc_floats(count);
    memcpy(grad, outputGrad, count * sizeof(float));
    int status = BFO_OK;
    for (int li = model->numLayers - 1; li >= 0 && status == BFO_OK; --li) {
        bfo_layer* layer = &model->layers[li];
        if (!layer->cachedInput) { status = BFO_INVALID_ARGUMENT; break; }
        size_t inCount = layer->cachedCount;
        int inRank = layer->cachedRank;
        const size_t* inShape = layer->cachedShape;
        size_t inFeatures = inShape[inRank - 1];
        size_t rows = inFeatures ? inCount / inFeatures : 0;
        float* next = alloc_floats(inCount);
        switch (layer->kind) {
            case BFO_LINEAR: {
                size_t outF = (size_t)layer->arg0;
                float* dBias = alloc_floats(outF);
                float* dW = alloc_floats(inFeatures * outF);
                bfo_add_bias_backward(grad, dBias, rows, outF);
                bfo_matmul_backward(layer->cachedInput, pv(model, layer, 0), grad, next, dW, rows, inFeatures, outF);
                accumulate(pg(model, layer, 0), dW, inFeatures * outF);
                accumulate(pg(model, layer, 1), dBias, outF);
                free(dBias); free(dW);
                break;
            }
            case BFO_SILU: bfo_silu_backward(layer->cachedInput, grad, next, inCount); break;
            case BFO_RELU: bfo_relu_backward(layer->cachedInput, grad, next, inCount); break;
            case BFO_GELU: bfo_gelu_backward(layer->cachedInput, grad, next, inCount); break;
            case BFO_RMSNORM: bfo_rmsnorm_backward(layer->cachedInput, grad, next, rows, inFeatures); break;
            case BFO_SOFTMAX: bfo_softmax_backward(layer->cachedInput, grad, next, rows, inFeatures); break;
            case BFO_EMBEDDING: {
                size_t vocab = (size_t)layer->arg0, dim = (size_t)layer->arg1;
                float* dTable = alloc_floats(vocab * dim);
                status = bfo_embedding_lookup_backward(layer->cachedInput, grad, dTable, inShape[0], inShape[1], vocab, dim);
                if (status == BFO_OK) accumulate(pg(model, layer, 0), dTable, vocab * dim);
                free(dTable);
                /* ids carry no gradient: zeros of the ids' shape flow on (model.cpp:290-299) */
                for (size_t i = 0; i < inCount; ++i) next[i] = 0.0f;
                break;
            }
            case BFO_POSITIONAL: {
                size_t maxSeq = (size_t)layer->arg0;
                float* dTable = alloc_floats(maxSeq * inShape[2]);
                status = bfo_add_positional_embedding_backward(grad, dTable, inShape[0], inShape[1], inShape[2], maxSeq);
                if (status == BFO_OK) accumulate(pg(model, layer, 0), dTable, maxSeq * inShape[2]);
                free(dTable);
                memcpy(next, grad, inCount * sizeof(float));
                break;
            }
            case BFO_ATTENTION:
            case BFO_BIDIRECTIONAL_ATTENTION: {   /* model.cpp:310-325 */
                size_t dim = inShape[2];
                float* dWq = alloc_floats(dim * dim);
                float* dWk = alloc_floats(dim * dim);
                float* dWv = alloc_floats(dim * dim);
                float* dWo = alloc_floats(dim * dim);
                status = bfo_self_attention_backward(layer->cachedInput, pv(model, layer, 0), pv(model, layer, 1),
                                                     pv(model, layer, 2), pv(model, layer, 3), grad, next, dWq, dWk,
                                                     dWv, dWo, inShape[0], inShape[1], dim, (size_t)layer->arg0,
                                                     layer->kind == BFO_ATTENTION);
                accumulate(pg(model, layer, 0), dWq, dim * dim);
                accumulate(pg(model, layer, 1), dWk, dim * dim);
                accumulate(pg(model, layer, 2), dWv, dim * dim);
                accumulate(pg(model, layer, 3), dWo, dim * dim);
                free(dWq); free(dWk); free(dWv); free(dWo);
                break;
            }
            case BFO_FEEDFORWARD: {
                size_t hidden = (size_t)layer->arg0;
                float* dW1 = alloc_floats(inFeatures * hidden);
                float* dB1 = alloc_floats(hidden);
                float* dW2 = alloc_floats(hidden * inFeatures);
                float* dB2 = alloc_floats(inFeatures);
                status = bfo_feed_forward_backward(layer->cachedInput, pv(model, layer, 0), pv(model, layer, 1),
                                                   pv(model, layer, 2), pv(model, layer, 3), grad, next, dW1, dB1,
                                                   dW2, dB2, rows, inFeatures, hidden, (int)layer->arg1);
                accumulate(pg(model, layer, 0), dW1, inFeatures * hidden);
                accumulate(pg(model, layer, 1), dB1, hidden);
                accumulate(pg(model, layer, 2), dW2, hidden * inFeatures);
                accumulate(pg(model, layer, 3), dB2, inFeatures);
                free(dW1); free(dB1); free(dW2); free(dB2);
                break;
            }
            default: status = BFO_INVALID_ARGUMENT; break;
        }
        free(grad);
        grad = next;
    }
    free(grad);
    return status;
}

int bfo_model_zero_grad(bfo_model* model) {
    for (int i = 0; i < model->numParams; ++i) memset(model->params[i].grad, 0, model->params[i].count * sizeof(float));
    return BFO_OK;
}

int bfo_model_adamw_step(bfo_model* model, float lr, float beta1, float beta2, float eps, float weightDecay) {
    ++model->adamStep;
    for (int i = 0; i < model->numParams; ++i) {
        bfo_param* p = &model->params[i];
        if (!p->m) {
            p->m = calloc_floats(p->count);
            p->v = calloc_floats(p->count);
        }
        bfo_adamw_step(p->value, p->grad, p->m, p->v, p->count, model->adamStep, lr, beta1, beta2, eps, weightDecay);
    }
    return BFO_OK;
}

/* ---------------------------------------------------------------------------------------------
 * Training run: dataset file, per-epoch shuffle, learning-rate schedule, checkpoints
 * ------------------------------------------------------------------------------------------- */

/* std::mt19937 (the 32-bit Mersenne twister of the C++ standard: fixed algorithm and constants). */
typedef struct {
    uint32_t state[624];
    int index;
} mt19937;
static void mt_seed(mt19937* g, uint32_t seed) {
    g->state[0] = seed;
    for (int i = 1; i < 624; ++i) g->state[i] = 1812433253u * (g->state[i - 1] ^ (g->state[i - 1] >> 30)) + (uint32_t)i;
    g->index = 624;
}
static uint32_t mt_next(mt19937* g) {
    if (g->index >= 624) {
        for (int i = 0; i < 624; ++i) {
            uint32_t y = (g->state[i] & 0x80000000u) | (g->state[(i + 1) % 624] & 0x7fffffffu);
            g->state[i] = g->state[(i + 397) % 624] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
        }
        g->index = 0;
    }
    uint32_t y = g->state[g->index++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
}
/* std::uniform_int_distribution<size_t>(0, hi) drawing from a 32-bit generator, as libstdc++ (GCC 11 and later)
 * evaluates it for hi < 2^32 - 1: Lemire's nearly divisionless reduction of one 32-bit draw to [0, hi]. */
static uint32_t uniform_below_inclusive(mt19937* g, uint32_t hi) {
    const uint64_t range = (uint64_t)hi + 1u;
    uint64_t product = (uint64_t)mt_next(g) * range;
    uint32_t low = (uint32_t)product;
    if (low < range) {
        const uint32_t threshold = (uint32_t)((0u - (uint32_t)range) % (uint32_t)range);
        while (low < threshold) {
            product = (uint64_t)mt_next(g) * range;
            low = (uint32_t)product;
        }
    }
    return (uint32_t)(product >> 32);
}

/* data::Dataset::shuffle (dataset.cpp:102-131): Fisher-Yates from the last position down, generator seeded with
 * the epoch number; order[i] is the example that moves to position i. */
int bfo_shuffle_order(size_t numExamples, unsigned seed, size_t* order) {
    if (numExamples >= 0xffffffffu) return BFO_INVALID_ARGUMENT;
    for (size_t i = 0; i < numExamples; ++i) order[i] = i;
    if (numExamples <= 1) return BFO_OK;
    mt19937 g;
    mt_seed(&g, seed);
    for (size_t i = numExamples - 1; i > 0; --i) {
        size_t j = uniform_below_inclusive(&g, (uint32_t)i);
        size_t t = order[i];
        order[i] = order[j];
        order[j] = t;
    }
    return BFO_OK;
}

/* cosineAnnealingLearningRate (backend/lr_schedule.hpp:...): double arithmetic, rounded to float once. */
float bfo_cosine_learning_rate(long long epoch, long long totalEpochs, float base) {
    if (totalEpochs <= 1) return base;
    const double kPi = 3.14159265358979323846;
    double progress = (double)(epoch - 1) / (double)(totalEpochs - 1);
    return (float)(base * 0.5 * (1.0 + cos(kPi * progress)));
}

typedef struct {
    uint32_t numExamples;
    size_t inputRank, targetRank;
    size_t inputShape[8], targetShape[8];
    size_t inputSize, targetSize; /* elements per example */
    float* inputs;
    float* targets;
} bfo_dataset;

static int read_shape(FILE* f, size_t* rank, size_t* shape, size_t* product) {
    uint32_t r = 0;
    if (fread(&r, 4, 1, f) != 1 || r > 8) return 0;
    *rank = r;
    *product = 1;
    for (uint32_t i = 0; i < r; ++i) {
        uint64_t d = 0;
        if (fread(&d, 8, 1, f) != 1) return 0;
        shape[i] = (size_t)d;
        *product *= (size_t)d;
    }
    return 1;
}
/* data::loadDataset (dataset.cpp:154-184): "BFDATA1\0", u32 examples, two shapes (u32 rank + u64 dims), inputs, targets. */
static int dataset_load(const char* path, bfo_dataset* d) {
    memset(d, 0, sizeof(*d));
    FILE* f = fopen(path, "rb");
    if (!f) return 0;
    char magic[8];
    int ok = fread(magic, 1, 8, f) == 8 && memcmp(magic, "BFDATA1\0", 8) == 0 && fread(&d->numExamples, 4, 1, f) == 1 &&
             read_shape(f, &d->inputRank, d->inputShape, &d->inputSize) && read_shape(f, &d->targetRank, d->targetShape, &d->targetSize);
    if (ok) {
        d->inputs = calloc_floats((size_t)d->numExamples * d->inputSize);
        d->targets = calloc_floats((size_t)d->numExamples * d->targetSize);
        ok = fread(d->inputs, 4, (size_t)d->numExamples * d->inputSize, f) == (size_t)d->numExamples * d->inputSize &&
             fread(d->targets, 4, (size_t)d->numExamples * d->targetSize, f) == (size_t)d->numExamples * d->targetSize;
    }
    fclose(f);
    return ok;
}
static void dataset_free(bfo_dataset* d) {
    free(d->inputs);
    free(d->targets);
}
static void dataset_shuffle(bfo_dataset* d, unsigned seed) {
    const size_t n = d->numExamples;
    if (n <= 1) return;
    size_t* order = (size_t*)malloc(n * sizeof(size_t));
    bfo_shuffle_order(n, seed, order);
    float* in2 = calloc_floats(n * d->inputSize);
    float* tg2 = calloc_floats(n * d->targetSize);
    for (size_t i = 0; i < n; ++i) {
        memcpy(in2 + i * d->inputSize, d->inputs + order[i] * d->inputSize, d->inputSize * sizeof(float));
        memcpy(tg2 + i * d->targetSize, d->targets + order[i] * d->targetSize, d->targetSize * sizeof(float));
    }
    free(d->inputs);
    free(d->targets);
    free(order);
    d->inputs = in2;
    d->targets = tg2;
}

/* saveCheckpoint (cpu/checkpoint.cpp:58-83): "BFCKPT1\0", u32 count, then per parameter u32 name length, name,
 * u32 rank, u64 dims, fp32 data. */
int bfo_model_save_checkpoint(const bfo_model* model, const char* path) {
    FILE* f = fopen(path, "wb");
    if (!f) return BFO_INVALID_ARGUMENT;
    fwrite("BFCKPT1\0", 1, 8, f);
    uint32_t count = (uint32_t)model->numParams;
    fwrite(&count, 4, 1, f);
    for (int i = 0; i < model->numParams; ++i) {
        const bfo_param* p = &model->params[i];
        uint32_t len = (uint32_t)strlen(p->name), rank = p->cols ? 2u : 1u;
        uint64_t d0 = p->rows, d1 = p->cols;
        fwrite(&len, 4, 1, f);
        fwrite(p->name, 1, len, f);
        fwrite(&rank, 4, 1, f);
        fwrite(&d0, 8, 1, f);
        if (rank == 2) fwrite(&d1, 8, 1, f);
        fwrite(p->value, 4, p->count, f);
    }
    int bad = ferror(f);
    fclose(f);
    return bad ? BFO_INVALID_ARGUMENT : BFO_OK;
}
/* loadCheckpoint (cpu/checkpoint.cpp:85-135): parameters are matched by name; unknown names, shape mismatches and
 * truncated files are errors; parameters the file does not mention keep their values. */
int bfo_model_load_checkpoint(bfo_model* model, const char* path) {
    FILE* f = fopen(path, "rb");
    if (!f) return BFO_INVALID_ARGUMENT;
    char magic[8];
    uint32_t count = 0;
    int status = BFO_OK;
    if (fread(magic, 1, 8, f) != 8 || memcmp(magic, "BFCKPT1\0", 8) != 0 || fread(&count, 4, 1, f) != 1) status = BFO_INVALID_ARGUMENT;
    for (uint32_t i = 0; i < count && status == BFO_OK; ++i) {
        uint32_t len = 0, rank = 0;
        char name[256];
        uint64_t dims[8] = {0};
        if (fread(&len, 4, 1, f) != 1 || len >= sizeof(name) || fread(name, 1, len, f) != len || fread(&rank, 4, 1, f) != 1 || rank > 8 ||
            fread(dims, 8, rank, f) != rank) { status = BFO_INVALID_ARGUMENT; break; }
        name[len] = 0;
        bfo_param* p = NULL;
        for (int j = 0; j < model->numParams; ++j)
            if (strcmp(model->params[j].name, name) == 0) p = &model->params[j];
        const uint32_t wantRank = p && p->cols ? 2u : 1u;
        if (!p || rank != wantRank || dims[0] != p->rows || (rank == 2 && dims[1] != p->cols)) { status = BFO_INVALID_ARGUMENT; break; }
        if (fread(p->value, 4, p->count, f) != p->count) status = BFO_INVALID_ARGUMENT;
    }
    fclose(f);
    return status;
}

/* cpu::runTraining (cpu/train_runner.cpp:38-211) for a model built from a layer list: per epoch, shuffle with the
 * epoch number as seed, optional cosine learning rate, floor(examples / batch) batches of zeroGrad, forward, loss,
 * backward, optimizer step; the epoch loss is the mean of the batch losses (accumulated in double).
 * lossKind: 0 mse, 1 cross_entropy, 2 cross_entropy_sparse, 3 cross_entropy_masked.  optimizerKind: 0 sgd, 1 adamw (reference defaults).
 * The model starts from `fromCheckpoint` when that is a non-empty path, else from its current values. */
int bfo_model_run_training(bfo_model* model, const char* datasetPath, int lossKind, int optimizerKind, long long epochs,
                           size_t batchSize, float learningRate, int cosineSchedule, const char* fromCheckpoint,
                           const char* saveCheckpoint, double* epochLosses) {
    bfo_dataset data;
    if (!dataset_load(datasetPath, &data)) return BFO_INVALID_ARGUMENT;
    int status = BFO_OK;
    if (fromCheckpoint && fromCheckpoint[0]) status = bfo_model_load_checkpoint(model, fromCheckpoint);
    if (status == BFO_OK && (batchSize == 0 || data.numExamples < batchSize)) status = BFO_INVALID_ARGUMENT;
    if (status != BFO_OK) { dataset_free(&data); return status; }
    const size_t batches = data.numExamples / batchSize;
    float* input = calloc_floats(batchSize * data.inputSize);
    float* target = calloc_floats(batchSize * data.targetSize);
    size_t shape[9];
    shape[0] = batchSize;
    for (size_t i = 0; i < data.inputRank; ++i) shape[i + 1] = data.inputShape[i];
    size_t outCapacity = 0;
    float* out = NULL;
    float* grad = NULL;
    float lr = learningRate;
    for (long long epoch = 1; epoch <= epochs && status == BFO_OK; ++epoch) {
        dataset_shuffle(&data, (unsigned)epoch);
        if (cosineSchedule) lr = bfo_cosine_learning_rate(epoch, epochs, learningRate);
        double sum = 0.0;
        for (size_t b = 0; b < batches && status == BFO_OK; ++b) {
            for (size_t i = 0; i < batchSize; ++i) {
                size_t e = (b * batchSize + i) % data.numExamples;
                memcpy(input + i * data.inputSize, data.inputs + e * data.inputSize, data.inputSize * sizeof(float));
                memcpy(target + i * data.targetSize, data.targets + e * data.targetSize, data.targetSize * sizeof(float));
            }
            bfo_model_zero_grad(model);
            size_t outCount = 0;
            status = bfo_model_forward(model, input, (int)data.inputRank + 1, shape, out, outCapacity, &outCount);
            if (status != BFO_OK && outCount > outCapacity) {   /* first batch: size the output buffers and run again */
                free(out);
                free(grad);
                outCapacity = outCount;
                out = calloc_floats(outCapacity);
                grad = calloc_floats(outCapacity);
                status = bfo_model_forward(model, input, (int)data.inputRank + 1, shape, out, outCapacity, &outCount);
            }
            if (status != BFO_OK) break;
            const size_t classes = model->layers[model->numLayers - 1].outFeatures, rows = outCount / classes;
            float value = 0.0f;
            if (lossKind == 0) status = bfo_mean_squared_error(out, target, grad, &value, outCount);
            else if (lossKind == 1) status = bfo_softmax_cross_entropy(out, target, grad, &value, rows, classes);
            else if (lossKind == 2) status = bfo_softmax_cross_entropy_sparse(out, target, grad, &value, rows, classes);
            else status = bfo_softmax_cross_entropy_masked(out, target, grad, &value, rows, classes);
            if (status != BFO_OK) break;
            status = bfo_model_backward(model, grad, outCount);
            if (status != BFO_OK) break;
            if (optimizerKind == 0) {
                for (int i = 0; i < model->numParams; ++i) bfo_sgd_step(model->params[i].value, model->params[i].grad, model->params[i].count, lr);
            } else {
                bfo_model_adamw_step(model, lr, 0.9f, 0.999f, 1e-8f, 0.01f);
            }
            sum += value;
        }
        epochLosses[epoch - 1] = sum / (double)batches;
    }
    if (status == BFO_OK && saveCheckpoint && saveCheckpoint[0]) status = bfo_model_save_checkpoint(model, saveCheckpoint);
    free(input); free(target); free(out); free(grad);
    dataset_free(&data);
    return status;
}

int bfo_model_write_initial_checkpoint(bfo_model* model, const char* path) {
    (void)model;
    (void)path;
    return BFO_INVALID_ARGUMENT; /* the reference's std:: random streams are not restated */
}

int bfo_save_dataset(const char* path, int inputRank, const size_t* inputShape, int targetRank, const size_t* targetShape,
                     const float* inputs, const float* targets, size_t numExamples) {
    FILE* f = fopen(path, "wb");
    if (!f) return BFO_INVALID_ARGUMENT;
    fwrite("BFDATA1\0", 1, 8, f);
    uint32_t n = (uint32_t)numExamples;
    fwrite(&n, 4, 1, f);
    size_t inSize = 1, tgSize = 1;
    for (int pass = 0; pass < 2; ++pass) {
        uint32_t rank = (uint32_t)(pass == 0 ? inputRank : targetRank);
        const size_t* shape = pass == 0 ? inputShape : targetShape;
        fwrite(&rank, 4, 1, f);
        for (uint32_t i = 0; i < rank; ++i) {
            uint64_t d = shape[i];
            fwrite(&d, 8, 1, f);
            if (pass == 0) inSize *= shape[i]; else tgSize *= shape[i];
        }
    }
    fwrite(inputs, 4, numExamples * inSize, f);
    fwrite(targets, 4, numExamples * tgSize, f);
    int bad = ferror(f);
    fclose(f);
    return bad ? BFO_INVALID_ARGUMENT : BFO_OK;
}
