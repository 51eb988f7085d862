/*
 * CPU oracle for the BERT forward pass of zhihu/cuBERT -- TEST INFRASTRUCTURE ONLY.
 * See cubert_oracle.h for what each function restates and what pins it.
 * Build: make -C oracle   (gcc -O2 -fopenmp -ffp-contract=off)
 */
#define _GNU_SOURCE
#include "cubert_oracle.h"

#include <dlfcn.h>
#include <float.h>
#include <math.h>
#include <omp.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ BLAS */

typedef void (*cblas_sgemm_fn)(int order, int transA, int transB, int M, int N, int K, float alpha,
                               const float *A, int lda, const float *B, int ldb, float beta,
                               float *C, int ldc);

static cblas_sgemm_fn g_sgemm = NULL;
static void *g_blas_handle = NULL;
static char g_blas_name[512] = "builtin triple loop";
static void (*g_blas_set_threads)(int) = NULL; /* the loaded BLAS's own thread-count calls, when it has them */
static int (*g_blas_get_threads)(void) = NULL;
static int g_batch_parallel = 1;

/* Wall-clock seconds per part of a forward pass, for the CPU baseline's breakdown (not used by any test). */
static double g_seconds[ORACLE_PROFILE_PARTS];
#define TIMED(part, call)                      \
    do {                                       \
        double t0_ = omp_get_wtime();          \
        call;                                  \
        g_seconds[part] += omp_get_wtime() - t0_; \
    } while (0)

void oracle_profile_reset(void) { memset(g_seconds, 0, sizeof g_seconds); }

void oracle_profile_read(double seconds[ORACLE_PROFILE_PARTS]) { memcpy(seconds, g_seconds, sizeof g_seconds); }

int oracle_use_cblas(const char *path, const char *sym) {
    void *h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    if (!h) return -1;
    void *f = dlsym(h, sym);
    if (!f) {
        dlclose(h);
        return -2;
    }
    g_blas_handle = h;
    g_sgemm = (cblas_sgemm_fn) f;
    g_blas_set_threads = NULL;
    g_blas_get_threads = NULL;
    {
        const char *setters[] = {"scipy_openblas_set_num_threads", "openblas_set_num_threads", "MKL_Set_Num_Threads"};
        const char *getters[] = {"scipy_openblas_get_num_threads", "openblas_get_num_threads", "MKL_Get_Max_Threads"};
        for (int i = 0; i < 3 && !g_blas_set_threads; ++i) {
            void *set = dlsym(h, setters[i]), *get = dlsym(h, getters[i]);
            if (set && get) {
                g_blas_set_threads = (void (*)(int)) set;
                g_blas_get_threads = (int (*)(void)) get;
            }
        }
    }
    snprintf(g_blas_name, sizeof g_blas_name, "%s:%s", path, sym);
    return 0;
}

void oracle_use_builtin_gemm(void) {
    g_sgemm = NULL;
    g_blas_set_threads = NULL;
    g_blas_get_threads = NULL;
    snprintf(g_blas_name, sizeof g_blas_name, "builtin triple loop");
}

const char *oracle_blas_name(void) { return g_blas_name; }

/* Column-major reference loop: one dot product per element of C, k ascending. */
static void builtin_sgemm(int transA, int transB, int M, int N, int K, float alpha, const float *A,
                          int lda, const float *B, int ldb, float beta, float *C, int ldc) {
#pragma omp parallel for schedule(static)
    for (int j = 0; j < N; ++j) {
        for (int i = 0; i < M; ++i) {
            float acc = 0.f;
            for (int k = 0; k < K; ++k) {
                float a = transA ? A[k + (size_t) i * lda] : A[i + (size_t) k * lda];
                float b = transB ? B[j + (size_t) k * ldb] : B[k + (size_t) j * ldb];
                acc += a * b;
            }
            float *c = &C[i + (size_t) j * ldc];
            *c = (beta == 0.f) ? alpha * acc : alpha * acc + beta * (*c);
        }
    }
}

/* reference: common.cpp:247-257 (cblas_sgemm, CblasColMajor) */
void oracle_sgemm(int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda,
                  const float *B, int ldb, float beta, float *C, int ldc) {
    if (g_sgemm) {
        g_sgemm(102 /*CblasColMajor*/, transA ? 112 : 111, transB ? 112 : 111, M, N, K, alpha, A,
                lda, B, ldb, beta, C, ldc);
    } else {
        builtin_sgemm(transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
    }
}

void oracle_set_batch_parallel(int on) { g_batch_parallel = on != 0; }

int oracle_blas_threads(void) { return g_blas_get_threads ? g_blas_get_threads() : 0; }

/* reference: common.cpp:260-298 (blas_gemm_batch<float>, HAVE_MKL branch): one cblas_sgemm_batch group of
 * `count` independent problems of one shape.  MKL spreads the problems of a group over its threads; here
 * the problems are an OpenMP loop around single-threaded sgemm calls when the loaded BLAS lets its thread count
 * be set (oracle_set_batch_parallel(0): one multi-threaded sgemm per problem, in order).  Either way every
 * problem is the same sgemm on the same operands. */
void oracle_sgemm_batch(int transA, int transB, int M, int N, int K, float alpha, const float **A, int lda,
                        const float **B, int ldb, float beta, float **C, int ldc, int count) {
    if (g_sgemm && g_batch_parallel && g_blas_set_threads && count > 1 && omp_get_max_threads() > 1) {
        int before = g_blas_get_threads();
        g_blas_set_threads(1);
#pragma omp parallel for schedule(static)
        for (int i = 0; i < count; ++i) {
            g_sgemm(102, transA ? 112 : 111, transB ? 112 : 111, M, N, K, alpha, A[i], lda, B[i], ldb, beta, C[i], ldc);
        }
        g_blas_set_threads(before);
        return;
    }
    for (int i = 0; i < count; ++i) {
        oracle_sgemm(transA, transB, M, N, K, alpha, A[i], lda, B[i], ldb, beta, C[i], ldc);
    }
}

/* --------------------------------------------------------- primitive ops */

/* reference: op/Embedding.cpp:10-20 -- one row memcpy per id, no bounds check */
void oracle_embedding(const int32_t *ids, int n, const float *table, int width, float *out) {
    for (int i = 0; i < n; ++i) {
        memcpy(out + (size_t) i * width, table + (size_t) width * ids[i], width * sizeof(float));
    }
}

/* reference: op/Embedding.cpp:22-33 */
void oracle_embedding_i8(const int8_t *ids, int n, const float *table, int width, float *out) {
    for (int i = 0; i < n; ++i) {
        memcpy(out + (size_t) i * width, table + (size_t) width * ids[i], width * sizeof(float));
    }
}

/* reference: op/LayerNorm.cpp:20-41 -- sums of t and t*t in one serial pass,
 * biased variance as E[t^2] - mean^2, epsilon 1e-12 inside the square root. */
void oracle_layer_norm_(const float *in, float *inout, int rows, int channels, const float *beta,
                        const float *gamma) {
#pragma omp parallel for
    for (int r = 0; r < rows; ++r) {
        float mean = 0;
        float var = 0;
        for (size_t i = (size_t) r * channels; i < (size_t) (r + 1) * channels; ++i) {
            float t = inout[i] + in[i];
            mean += t;
            var += t * t;
        }
        mean = mean / channels;
        var = var / channels - mean * mean;
        var = 1.f / sqrtf(var + 1e-12f);
        for (int i = 0; i < channels; ++i) {
            size_t j = (size_t) r * channels + i;
            inout[j] = beta[i] + gamma[i] * var * (inout[j] + in[j] - mean);
        }
    }
}

/* reference: op/Softmax.cpp:18-36 */
void oracle_softmax_(const float *in, float *out, int rows, int channel) {
#pragma omp parallel for
    for (int r = 0; r < rows; ++r) {
        const float *x = in + (size_t) r * channel;
        float *y = out + (size_t) r * channel;
        float max = -FLT_MAX;
        for (int i = 0; i < channel; ++i) {
            if (x[i] > max) max = x[i];
        }
        float sum = 0;
        for (int i = 0; i < channel; ++i) {
            y[i] = expf(x[i] - max);
            sum += y[i];
        }
        for (int i = 0; i < channel; ++i) {
            y[i] = y[i] / sum;
        }
    }
}

/* reference: op/GELU.cpp:11-14 */
void oracle_gelu(size_t n, float *inout) {
#pragma omp parallel for
    for (long i = 0; i < (long) n; ++i) {
        inout[i] = inout[i] * 0.5f * (1.0f + erff(inout[i] * sqrtf(0.5f)));
    }
}

/* reference: op_att/AttentionMask.cpp:13-16 */
void oracle_not(const int8_t *in, float *out, int n) {
#pragma omp parallel for
    for (int i = 0; i < n; ++i) {
        out[i] = !in[i];
    }
}

/* reference: op_bert/BertPooler.cpp:11-14 */
void oracle_tanh_(float *inout, int n) {
#pragma omp parallel for
    for (int i = 0; i < n; ++i) {
        inout[i] = tanhf(inout[i]);
    }
}

/* reference: op_bert/BertPooler.cpp:21-31 -- serial sum over the sequence, then / S */
void oracle_reduce_mean_1(const float *in, float *out, int batch, int seq_length, int hidden) {
#pragma omp parallel for
    for (int idx = 0; idx < batch * hidden; ++idx) {
        size_t b = idx / hidden;
        size_t c = idx % hidden;
        float sum = 0;
        for (int s = 0; s < seq_length; ++s) {
            sum += in[c + (size_t) s * hidden + b * seq_length * hidden];
        }
        out[idx] = sum / seq_length;
    }
}

/* --------------------------------------------------------- composite ops */

/* reference: op/Dense.cpp:41-44 (bias rows copied into the output) and
 * :47-57 (column-major gemm N,N m=units n=rows k=inputs, alpha=beta=1). */
void oracle_dense(int rows, int inputs, int units, const float *kernel, const float *bias,
                  const float *in, float *out) {
    for (int r = 0; r < rows; ++r) {
        memcpy(out + (size_t) r * units, bias, units * sizeof(float));
    }
    oracle_sgemm(0, 0, units, rows, inputs, 1.f, kernel, units, in, inputs, 1.f, out, units);
}

/* reference: op_att/AttentionMask.cpp:41-54 -- neg = !mask, then a k=1
 * strided-batched GEMM neg[b] (S x 1) * ones (1 x A*S) writes [b][a*S+q][k]. */
void oracle_attention_mask(int batch, int seq_length, int heads, const int8_t *mask, float *out) {
    int S = seq_length;
    float *neg = (float *) malloc(sizeof(float) * (size_t) batch * S);
    float *ones = (float *) malloc(sizeof(float) * (size_t) heads * S);
    oracle_not(mask, neg, batch * S);
    for (int i = 0; i < heads * S; ++i) ones[i] = 1.f;
    for (int b = 0; b < batch; ++b) {
        oracle_sgemm(0, 0, S, heads * S, 1, 1.f, neg + (size_t) b * S, S, ones, 1, 0.f,
                     out + (size_t) b * S * heads * S, S);
    }
    free(ones);
    free(neg);
}

/* reference: op_att/BatchMatMul.cpp:31-38 (per-(b,h) base pointers) and
 * :57-68 (gemm_batch T,N m=n=S k=d, lda=ldb=H, ldc=S*A). */
void oracle_att_q_k(int batch, int seq_length, int heads, int size_per_head, const float *query,
                    const float *key, float *scores, float alpha, float beta) {
    int S = seq_length, A = heads, d = size_per_head, count = batch * heads;
    const float **q = (const float **) malloc(sizeof(float *) * (size_t) count);
    const float **k = (const float **) malloc(sizeof(float *) * (size_t) count);
    float **out = (float **) malloc(sizeof(float *) * (size_t) count);
    for (int b = 0; b < batch; ++b) {
        for (int h = 0; h < A; ++h) {
            size_t idx = (size_t) b * S * d * A + (size_t) d * h;
            q[b * A + h] = query + idx;
            k[b * A + h] = key + idx;
            out[b * A + h] = scores + (size_t) b * S * S * A + (size_t) S * h;
        }
    }
    oracle_sgemm_batch(1, 0, S, S, d, alpha, k, d * A, q, d * A, beta, out, S * A, count);
    free(out);
    free(k);
    free(q);
}

/* reference: op_att/BatchMatMul.cpp:103-110 and :129-140
 * (gemm_batch N,N m=d n=S k=S, lda=H, ldb=S*A, ldc=H). */
void oracle_att_qk_v(int batch, int seq_length, int heads, int size_per_head, const float *qk,
                     const float *value, float *out, float alpha, float beta) {
    int S = seq_length, A = heads, d = size_per_head, count = batch * heads;
    const float **v = (const float **) malloc(sizeof(float *) * (size_t) count);
    const float **p = (const float **) malloc(sizeof(float *) * (size_t) count);
    float **o = (float **) malloc(sizeof(float *) * (size_t) count);
    for (int b = 0; b < batch; ++b) {
        for (int h = 0; h < A; ++h) {
            size_t idx = (size_t) b * S * d * A + (size_t) d * h;
            v[b * A + h] = value + idx;
            p[b * A + h] = qk + (size_t) b * S * S * A + (size_t) S * h;
            o[b * A + h] = out + idx;
        }
    }
    oracle_sgemm_batch(0, 0, d, S, S, alpha, v, d * A, p, S * A, beta, o, d * A, count);
    free(o);
    free(p);
    free(v);
}

static const float *find_var(const oracle_vars *vars, const char *name) {
    for (int i = 0; i < vars->n; ++i) {
        if (strcmp(vars->names[i], name) == 0) return vars->data[i];
    }
    return NULL;
}

static const float *find_var2(const oracle_vars *vars, const char *prefix, const char *suffix) {
    char name[512];
    snprintf(name, sizeof name, "%s%s", prefix, suffix);
    return find_var(vars, name);
}

static float *falloc(size_t n) {
    float *p = (float *) malloc(sizeof(float) * (n ? n : 1));
    if (!p) {
        fprintf(stderr, "oracle: out of memory (%zu floats)\n", n);
        abort();
    }
    return p;
}

/* reference: op_att/AttentionSelf.cpp:96-111; alpha/beta from :58-60 */
int oracle_attention_self(const oracle_vars *vars, const char *prefix, int batch, int seq_length,
                          int heads, int size_per_head, const float *in, const float *neg_mask,
                          float *context_out) {
    int S = seq_length, A = heads, d = size_per_head, H = A * d;
    size_t M = (size_t) batch * S;
    const float *qk_ = find_var2(vars, prefix, "/query/kernel"), *qb = find_var2(vars, prefix, "/query/bias");
    const float *kk = find_var2(vars, prefix, "/key/kernel"), *kb = find_var2(vars, prefix, "/key/bias");
    const float *vk = find_var2(vars, prefix, "/value/kernel"), *vb = find_var2(vars, prefix, "/value/bias");
    if (!qk_ || !qb || !kk || !kb || !vk || !vb) return -1;

    float *q = falloc(M * H), *k = falloc(M * H), *v = falloc(M * H);
    float *scores = falloc((size_t) batch * A * S * S);

    TIMED(ORACLE_PART_OTHER, memcpy(scores, neg_mask, sizeof(float) * (size_t) batch * A * S * S));
    TIMED(ORACLE_PART_DENSE, oracle_dense((int) M, H, H, qk_, qb, in, q));
    TIMED(ORACLE_PART_DENSE, oracle_dense((int) M, H, H, kk, kb, in, k));
    TIMED(ORACLE_PART_DENSE, oracle_dense((int) M, H, H, vk, vb, in, v));

    float alpha = (float) (1.0 / sqrt((double) d));
    TIMED(ORACLE_PART_ATTENTION_GEMM, oracle_att_q_k(batch, S, A, d, q, k, scores, alpha, -10000.0f));
    TIMED(ORACLE_PART_ROW_KERNELS, oracle_softmax_(scores, scores, batch * A * S, S));
    TIMED(ORACLE_PART_ATTENTION_GEMM, oracle_att_qk_v(batch, S, A, d, scores, v, context_out, 1.f, 0.f));

    free(scores);
    free(v);
    free(k);
    free(q);
    return 0;
}

/* reference: op_att/Transformer.cpp:145-175 */
int oracle_transformer(const oracle_vars *vars, const char *prefix, int batch, int seq_length,
                       int hidden, int layers, int heads, int intermediate, const float *in,
                       const int8_t *mask, float *out) {
    int S = seq_length, H = hidden, I = intermediate;
    size_t M = (size_t) batch * S;
    int rc = 0;

    float *neg_mask = falloc((size_t) batch * heads * S * S);
    TIMED(ORACLE_PART_OTHER, oracle_attention_mask(batch, S, heads, mask, neg_mask));

    float *prev = falloc(M * H);
    memcpy(prev, in, sizeof(float) * M * H);
    float *ctx = falloc(M * H), *att_out = falloc(M * H), *inter = falloc(M * I),
          *layer_out = falloc(M * H);

    for (int l = 0; l < layers && rc == 0; ++l) {
        char lp[256], ap[300];
        snprintf(lp, sizeof lp, "%s/layer_%d", prefix, l);
        snprintf(ap, sizeof ap, "%s/attention/self", lp);

        const float *aok = find_var2(vars, lp, "/attention/output/dense/kernel");
        const float *aob = find_var2(vars, lp, "/attention/output/dense/bias");
        const float *anb = find_var2(vars, lp, "/attention/output/LayerNorm/beta");
        const float *ang = find_var2(vars, lp, "/attention/output/LayerNorm/gamma");
        const float *ik = find_var2(vars, lp, "/intermediate/dense/kernel");
        const float *ib = find_var2(vars, lp, "/intermediate/dense/bias");
        const float *ok = find_var2(vars, lp, "/output/dense/kernel");
        const float *ob = find_var2(vars, lp, "/output/dense/bias");
        const float *onb = find_var2(vars, lp, "/output/LayerNorm/beta");
        const float *ong = find_var2(vars, lp, "/output/LayerNorm/gamma");
        if (!aok || !aob || !anb || !ang || !ik || !ib || !ok || !ob || !onb || !ong) {
            rc = -1;
            break;
        }

        /* attention/self */
        rc = oracle_attention_self(vars, ap, batch, S, heads, H / heads, prev, neg_mask, ctx);
        if (rc) break;
        /* attention/output: dense, then LayerNorm(residual = layer input) */
        TIMED(ORACLE_PART_DENSE, oracle_dense((int) M, H, H, aok, aob, ctx, att_out));
        TIMED(ORACLE_PART_ROW_KERNELS, oracle_layer_norm_(prev, att_out, (int) M, H, anb, ang));
        /* intermediate: dense + GELU */
        TIMED(ORACLE_PART_DENSE, oracle_dense((int) M, H, I, ik, ib, att_out, inter));
        TIMED(ORACLE_PART_ROW_KERNELS, oracle_gelu(M * I, inter));
        /* output: dense, then LayerNorm(residual = attention output) */
        TIMED(ORACLE_PART_DENSE, oracle_dense((int) M, I, H, ok, ob, inter, layer_out));
        TIMED(ORACLE_PART_ROW_KERNELS, oracle_layer_norm_(att_out, layer_out, (int) M, H, onb, ong));

        float *t = prev;
        prev = layer_out;
        layer_out = t;
    }
    if (rc == 0) memcpy(out, prev, sizeof(float) * M * H);

    free(layer_out);
    free(inter);
    free(att_out);
    free(ctx);
    free(prev);
    free(neg_mask);
    return rc;
}

/* reference: op_bert/BertEmbeddings.cpp:50-66 -- word rows into `out`,
 * token-type rows into a side buffer, positions added by a k=1 GEMM with
 * beta=1 (out[b] += pos[0:S]), then LayerNorm(in = type rows, inout = out). */
int oracle_bert_embeddings(const oracle_vars *vars, int batch, int seq_length, int hidden,
                           const int32_t *ids, const int8_t *segments, float *out) {
    const float *word = find_var(vars, "bert/embeddings/word_embeddings");
    const float *type = find_var(vars, "bert/embeddings/token_type_embeddings");
    const float *pos = find_var(vars, "bert/embeddings/position_embeddings");
    const float *beta = find_var(vars, "bert/embeddings/LayerNorm/beta");
    const float *gamma = find_var(vars, "bert/embeddings/LayerNorm/gamma");
    if (!word || !type || !pos || !beta || !gamma) return -1;

    int S = seq_length, H = hidden;
    size_t M = (size_t) batch * S;
    float *type_out = falloc(M * H);
    float *ones = falloc(batch);
    for (int b = 0; b < batch; ++b) ones[b] = 1.f;

    oracle_embedding(ids, (int) M, word, H, out);
    oracle_embedding_i8(segments, (int) M, type, H, type_out);
    oracle_sgemm(0, 0, S * H, batch, 1, 1.f, pos, S * H, ones, 1, 1.f, out, S * H);
    oracle_layer_norm_(type_out, out, (int) M, H, beta, gamma);

    free(ones);
    free(type_out);
    return 0;
}

/* reference: op_bert/BertPooler.cpp:62-77 -- bias rows into out, gemm on the
 * first token of every sequence (ldb = H*S), tanh in place. */
void oracle_bert_pooler(int batch, int seq_length, int hidden, const float *kernel,
                        const float *bias, const float *in, float *out) {
    int H = hidden;
    for (int b = 0; b < batch; ++b) memcpy(out + (size_t) b * H, bias, sizeof(float) * H);
    oracle_sgemm(0, 0, H, batch, H, 1.f, kernel, H, in, H * seq_length, 1.f, out, H);
    oracle_tanh_(out, batch * H);
}

/* reference: op_bert/BertPooler.cpp:93-96 */
void oracle_mean_pooler(int batch, int seq_length, int hidden, const float *in, float *out) {
    oracle_reduce_mean_1(in, out, batch, seq_length, hidden);
}

/* reference: op_out/AdditionalOutputLayer.cpp:45-66 */
void oracle_classifier(int batch, int hidden, int labels, const float *weights, const float *bias,
                       const float *in, float *logits, float *probs) {
    if (bias) {
        for (int b = 0; b < batch; ++b) memcpy(logits + (size_t) b * labels, bias, sizeof(float) * labels);
    }
    float beta = bias ? 1.f : 0.f;
    oracle_sgemm(1, 0, labels, batch, hidden, 1.f, weights, hidden, in, hidden, beta, logits, labels);
    if (probs) oracle_softmax_(logits, probs, batch, labels);
}

/* reference: Bert.cpp:27-53 (which pooler / whether a classifier) and :98-136 */
int oracle_bert_forward(const oracle_vars *vars, int batch, int seq_length, int hidden, int layers,
                        int heads, int intermediate, int labels, const int32_t *ids,
                        const int8_t *mask, const int8_t *segments, float *embedding_output,
                        float *sequence_output, float *pooled_output, float *logits, float *probs) {
    int S = seq_length, H = hidden;
    size_t M = (size_t) batch * S;
    if (batch == 0) return 0;

    float *emb = embedding_output ? embedding_output : falloc(M * H);
    float *seq = sequence_output ? sequence_output : falloc(M * H);
    float *pooled = pooled_output ? pooled_output : falloc((size_t) batch * H);
    int rc;
    TIMED(ORACLE_PART_OTHER, rc = oracle_bert_embeddings(vars, batch, S, H, ids, segments, emb));
    if (rc == 0) {
        rc = oracle_transformer(vars, "bert/encoder", batch, S, H, layers, heads, intermediate, emb,
                                mask, seq);
    }
    if (rc == 0) {
        const float *pk = find_var(vars, "bert/pooler/dense/kernel");
        if (pk) {
            const float *pb = find_var(vars, "bert/pooler/dense/bias");
            if (!pb) rc = -1;
            else oracle_bert_pooler(batch, S, H, pk, pb, seq, pooled);
        } else {
            oracle_mean_pooler(batch, S, H, seq, pooled);
        }
    }
    if (rc == 0) {
        const float *ow = find_var(vars, "output_weights");
        if (ow && (logits || probs)) {
            float *lg = logits ? logits : falloc((size_t) batch * labels);
            oracle_classifier(batch, H, labels, ow, find_var(vars, "output_bias"), pooled, lg, probs);
            if (!logits) free(lg);
        }
    }
    if (!pooled_output) free(pooled);
    if (!sequence_output) free(seq);
    if (!embedding_output) free(emb);
    return rc;
}

/* ------------------------------------------------------ fp16 rounding */

/* IEEE binary32 -> binary16, round to nearest even, overflow to infinity,
 * subnormal results kept (half_float::half default: half.hpp:373-374). */
uint16_t oracle_float_to_half_bits(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t abs = x & 0x7fffffffu;
    if (abs >= 0x7f800000u) { /* inf / nan */
        return (uint16_t) (sign | 0x7c00u | ((abs > 0x7f800000u) ? (0x200u | ((abs >> 13) & 0x3ffu)) : 0));
    }
    if (abs >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t) (sign | 0x7c00u);
    }
    if (abs < 0x38800000u) { /* result is subnormal or zero: |f| < 2^-14 */
        if (abs < 0x33000000u) return (uint16_t) sign; /* < 2^-25 -> 0 */
        uint32_t e = abs >> 23;                         /* biased exponent, 102..112 */
        uint32_t m = (abs & 0x7fffffu) | 0x800000u;     /* 24-bit significand */
        uint32_t shift = 126 - e;                       /* 14..24: bits dropped to reach 2^-24 units */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t) (sign | q);
    }
    uint32_t e = (abs >> 23) - 112; /* half biased exponent 1..30 */
    uint32_t m = abs & 0x7fffffu;
    uint32_t q = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t) (sign | q);
}

float oracle_half_bits_to_float(uint16_t h) {
    uint32_t sign = ((uint32_t) h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    uint32_t x;
    if (e == 0) {
        if (m == 0) {
            x = sign;
        } else {
            int sh = 0;
            while (!(m & 0x400u)) {
                m <<= 1;
                ++sh;
            }
            m &= 0x3ffu;
            x = sign | ((uint32_t) (113 - sh) << 23) | (m << 13);
        }
    } else if (e == 31) {
        x = sign | 0x7f800000u | (m << 13);
    } else {
        x = sign | ((e + 112) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* reference: common.h:94-106 (float2half then half2float) */
void oracle_round_to_half(const float *in, float *out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = oracle_half_bits_to_float(oracle_float_to_half_bits(in[i]));
}
