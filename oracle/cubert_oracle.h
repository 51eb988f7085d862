/*
 * CPU oracle for the BERT forward pass of zhihu/cuBERT (its "mklBERT" path).
 *
 * TEST INFRASTRUCTURE ONLY.  This is the checker the HIP kernels are compared
 * against; nothing in the shipped library links, loads or calls it.  It is a
 * plain-C restatement (fp32 storage, fp32 arithmetic, serial accumulation in
 * the reference's loop order) of the reference's CPU code; every function
 * names the reference file:line it follows.
 *
 * Pinning status (what fixes each function besides this restatement):
 *   oracle_embedding            reference EmbeddingTest vector; reference op build (bit-exact)
 *   oracle_layer_norm_          reference LayerNormTest vector; reference op build; textbook LN in float64
 *   oracle_softmax_             reference SoftmaxTest vector; reference op build; scipy.special.softmax
 *   oracle_gelu                 reference GELUTest closed form; reference op build
 *   oracle_not                  reference AttentionMaskTest vector; reference op build
 *   oracle_tanh_, oracle_reduce_mean_1   reference BertPoolerTest vectors; reference op build
 *   oracle_sgemm                reference DenseTest / BatchMatMulTest integer vectors; numpy float64 matmul
 *   oracle_sgemm_batch          through oracle_att_q_k / qk_v: reference BatchMatMulTest vectors, both batch modes
 *   oracle_dense                reference DenseTest vector
 *   oracle_attention_mask       reference AttentionMaskTest vector (24 values)
 *   oracle_att_q_k / qk_v       reference BatchMatMulTest vectors
 *   oracle_attention_self       reference AttentionSelfTest vector (12 values, 1e-5)
 *   oracle_transformer          reference TransformerTest vectors (1 layer 1e-6, 2 layers 1e-5)
 *   oracle_bert_embeddings      reference BertEmbeddingsTest closed form (1e-6)
 *   oracle_bert_pooler / mean   reference BertPoolerTest vectors
 *   oracle_classifier           reference AdditionalOutputLayerTest vector; closed form softmax(x W^T + b)
 *   oracle_bert_forward         composition of the above; independent float64 numpy BERT at small shapes
 */
#ifndef CUBERT_ORACLE_H
#define CUBERT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- BLAS selection ------------------------------------------------------
 * The reference's contractions live in Intel MKL (cblas_sgemm).  The oracle
 * uses a CBLAS sgemm loaded at run time from `path` (symbol `sym`, e.g. the
 * OpenBLAS bundled with scipy: "scipy_cblas_sgemm"); when none is set it uses
 * its own plain triple loop.  Returns 0 on success. */
int oracle_use_cblas(const char *path, const char *sym);
void oracle_use_builtin_gemm(void);
const char *oracle_blas_name(void);

/* Column-major sgemm with cblas_sgemm's meaning: C = alpha*op(A)*op(B) + beta*C.
 * reference: src/cuBERT/common.cpp:224-258 (blas_gemm<float>, HAVE_MKL branch). */
void oracle_sgemm(int transA, int transB, int M, int N, int K, float alpha,
                  const float *A, int lda, const float *B, int ldb, float beta,
                  float *C, int ldc);

/* One group of `count` independent column-major sgemm problems of one shape, cblas_sgemm_batch's meaning.
 * reference: src/cuBERT/common.cpp:260-298 (blas_gemm_batch<float>, HAVE_MKL branch). */
void oracle_sgemm_batch(int transA, int transB, int M, int N, int K, float alpha, const float **A, int lda,
                        const float **B, int ldb, float beta, float **C, int ldc, int count);
/* on (default): the problems of a batch run as an OpenMP loop around single-threaded sgemm calls, which is how
 * MKL's cblas_sgemm_batch spreads a group; off: one multi-threaded sgemm after the other.  Same results. */
void oracle_set_batch_parallel(int on);
/* Thread count the loaded BLAS reports for itself (0 for the builtin loop, which follows OpenMP). */
int oracle_blas_threads(void);

/* Wall-clock seconds spent per part of oracle_bert_forward / oracle_transformer since the last reset. */
enum { ORACLE_PART_DENSE = 0, ORACLE_PART_ATTENTION_GEMM = 1, ORACLE_PART_ROW_KERNELS = 2, ORACLE_PART_OTHER = 3,
       ORACLE_PROFILE_PARTS = 4 };
void oracle_profile_reset(void);
void oracle_profile_read(double seconds[ORACLE_PROFILE_PARTS]);

/* ---- primitive ops (reference: src/cuBERT/op, op_att, op_bert) ---------- */

/* out[i,:] = table[ids[i],:]          reference: op/Embedding.cpp:10-33 */
void oracle_embedding(const int32_t *ids, int n, const float *table, int width, float *out);
void oracle_embedding_i8(const int8_t *ids, int n, const float *table, int width, float *out);

/* inout = beta + gamma * (inout+in - mean) / sqrt(var + 1e-12), var = E[x^2]-mean^2
 *                                      reference: op/LayerNorm.cpp:11-42 */
void oracle_layer_norm_(const float *in, float *inout, int rows, int channels,
                        const float *beta, const float *gamma);

/* row softmax: max, expf(x-max), sum, divide   reference: op/Softmax.cpp:12-37 */
void oracle_softmax_(const float *in, float *out, int rows, int channel);

/* x * 0.5 * (1 + erff(x * sqrtf(0.5)))         reference: op/GELU.cpp:10-15 */
void oracle_gelu(size_t n, float *inout);

/* out[i] = !in[i]                              reference: op_att/AttentionMask.cpp:9-17 */
void oracle_not(const int8_t *in, float *out, int n);

/* reference: op_bert/BertPooler.cpp:10-15 and :18-32 */
void oracle_tanh_(float *inout, int n);
void oracle_reduce_mean_1(const float *in, float *out, int batch, int seq_length, int hidden);

/* ---- composite ops ------------------------------------------------------ */

/* out = in * kernel + bias; kernel is [inputs, units] row-major.
 * Bias is written into `out` first and the GEMM accumulates with beta = 1.
 * reference: op/Dense.cpp:41-57 */
void oracle_dense(int rows, int inputs, int units, const float *kernel, const float *bias,
                  const float *in, float *out);

/* out[b, a*S+q, k] = !mask[b,k]                reference: op_att/AttentionMask.cpp:41-54 */
void oracle_attention_mask(int batch, int seq_length, int heads, const int8_t *mask, float *out);

/* scores[b,q,a,k] = alpha * sum_j query[b,q,a,j] key[b,k,a,j] + beta * scores[b,q,a,k]
 * reference: op_att/BatchMatMul.cpp:31-38,57-68 */
void oracle_att_q_k(int batch, int seq_length, int heads, int size_per_head,
                    const float *query, const float *key, float *scores, float alpha, float beta);

/* out[b,q,a,j] = alpha * sum_k qk[b,q,a,k] value[b,k,a,j] + beta * out
 * reference: op_att/BatchMatMul.cpp:103-110,129-140 */
void oracle_att_qk_v(int batch, int seq_length, int heads, int size_per_head,
                     const float *qk, const float *value, float *out, float alpha, float beta);

/* Named weights, the way the reference hands them to its host classes
 * (std::unordered_map<std::string, T*>, e.g. Transformer.cpp:54-101). */
typedef struct {
    int n;
    const char *const *names;
    const float *const *data;
} oracle_vars;

/* Self attention.  `neg_mask` is the already-broadcast [B, A*S, S] tensor of
 * 1.0 at masked keys (what oracle_attention_mask writes).
 * reference: op_att/AttentionSelf.cpp:58-60,96-111.  Returns 0, or -1 when a
 * weight name is missing (the reference throws std::out_of_range). */
int oracle_attention_self(const oracle_vars *vars, const char *prefix, int batch, int seq_length,
                          int heads, int size_per_head, const float *in, const float *neg_mask,
                          float *context_out);

/* Encoder stack.  reference: op_att/Transformer.cpp:145-175 */
int oracle_transformer(const oracle_vars *vars, const char *prefix, int batch, int seq_length,
                       int hidden, int layers, int heads, int intermediate, const float *in,
                       const int8_t *mask, float *out);

/* word + position + token-type, then LayerNorm.
 * reference: op_bert/BertEmbeddings.cpp:50-66 */
int oracle_bert_embeddings(const oracle_vars *vars, int batch, int seq_length, int hidden,
                           const int32_t *ids, const int8_t *segments, float *out);

/* tanh(first_token * kernel + bias)            reference: op_bert/BertPooler.cpp:62-77 */
void oracle_bert_pooler(int batch, int seq_length, int hidden, const float *kernel,
                        const float *bias, const float *in, float *out);
/* mean over the sequence axis, padding included   reference: op_bert/BertPooler.cpp:93-96 */
void oracle_mean_pooler(int batch, int seq_length, int hidden, const float *in, float *out);

/* logits = in * W^T (+ bias), W is [labels, hidden]; probs = softmax(logits) when non-NULL.
 * reference: op_out/AdditionalOutputLayer.cpp:52-66 */
void oracle_classifier(int batch, int hidden, int labels, const float *weights, const float *bias,
                       const float *in, float *logits, float *probs);

/* Whole model.  Any output pointer may be NULL.  Pooler = BertPooler when
 * "bert/pooler/dense/kernel" is present, MeanPooler otherwise; classifier only
 * when "output_weights" is present.      reference: Bert.cpp:27-53,98-136 */
int oracle_bert_forward(const oracle_vars *vars, int batch, int seq_length, int hidden, int layers,
                        int heads, int intermediate, int labels, const int32_t *ids,
                        const int8_t *mask, const int8_t *segments, float *embedding_output,
                        float *sequence_output, float *pooled_output, float *logits, float *probs);

/* fp32 -> fp16 -> fp32 with round-to-nearest-even, the rounding half_float::half
 * is configured with in the reference (common.h:94-106, half.hpp:373-374). */
void oracle_round_to_half(const float *in, float *out, size_t n);
uint16_t oracle_float_to_half_bits(float f);
float oracle_half_bits_to_float(uint16_t h);

#ifdef __cplusplus
}
#endif
#endif
