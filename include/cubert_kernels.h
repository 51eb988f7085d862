/*
 * Device layer of the library: the fused, bandwidth-bound layer kernels of the
 * BERT forward pass for gfx950 (MI355X) and the small runtime they sit on.
 * Plain C ABI: device pointers, sizes, a stream.  This is the boundary the
 * reference draws between its host classes (.cpp) and its device code (.cu):
 * free launchers that take raw device pointers plus `void* stream`, run
 * asynchronously on that stream and report nothing back.
 *
 * Every kernel exists for fp32 storage (`_f32`) and for IEEE binary16 storage
 * (`_f16`, arithmetic in fp32, one rounding at the store).  `cubert_half` is
 * the 16-bit pattern of a binary16 value.
 *
 * Return value of every function that returns int: 0 on success; a positive
 * hipError_t when the launch failed; CUBERT_BAD_ARGUMENT (-1) when an argument
 * is outside what the kernel supports (nothing is launched then).  The host
 * classes above treat any non-zero value as fatal, as the reference does with
 * CUDA_CHECK (src/cuBERT/common.cpp:79-93).
 *
 * Pointers must be aligned to their element type; the fast paths additionally
 * need 16-byte aligned rows and are selected at launch time, other shapes take
 * a generic path with identical results.
 */
#ifndef CUBERT_KERNELS_H
#define CUBERT_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t cubert_half;
#define CUBERT_BAD_ARGUMENT (-1)
#define CUBERT_UNSUPPORTED (-2) /* valid arguments, but no kernel for this shape: the caller takes another route */
#define CUBERT_TOO_LARGE (-3)   /* beyond the fixed capacity of an entry point that allocates nothing */

/* ------------------------------------------------------------------ kernels */

/* out[i, :] = table[ids[i], :]  (no bounds check on ids, as in the reference).
 * replaces: embedding<int,T> / embedding<int8_t,T>, reference src/cuBERT/op/Embedding.h:9-15
 * (kernel op/Embedding.cu:8-41). */
int cubert_gather_f32(const int32_t *ids, int n, const float *table, int width, float *out, void *stream);
int cubert_gather_f16(const int32_t *ids, int n, const cubert_half *table, int width, cubert_half *out, void *stream);
int cubert_gather_i8_f32(const int8_t *ids, int n, const float *table, int width, float *out, void *stream);
int cubert_gather_i8_f16(const int8_t *ids, int n, const cubert_half *table, int width, cubert_half *out, void *stream);

/* BertEmbeddings in one pass:
 *   x = word[ids[m]] + pos[m mod seq_length] + type[segments[m]]        (m < batch*seq_length)
 *   out[m] = beta + gamma * (x - mean) / sqrt(E[x^2] - mean^2 + 1e-12)
 * replaces: the two embedding<> launches, the k=1 position GEMM and layer_norm_ of
 * reference src/cuBERT/op_bert/BertEmbeddings.cpp:50-66. */
int cubert_embed_ln_f32(const int32_t *ids, const int8_t *segments, const float *word, const float *pos,
                        const float *type, const float *beta, const float *gamma, float *out, int batch,
                        int seq_length, int hidden, void *stream);
int cubert_embed_ln_f16(const int32_t *ids, const int8_t *segments, const cubert_half *word,
                        const cubert_half *pos, const cubert_half *type, const cubert_half *beta,
                        const cubert_half *gamma, cubert_half *out, int batch, int seq_length, int hidden,
                        void *stream);

/* bias + residual + LayerNorm, in place on `inout`:
 *   x = inout[r] + bias + residual[r];  inout[r] = beta + gamma * (x - mean) / sqrt(var + 1e-12)
 * `bias` may be NULL (then this is exactly the reference launcher).
 * replaces: layer_norm_<T>(in=residual, inout, rows, hidden, mean, var, beta, gamma, stream),
 * reference src/cuBERT/op/LayerNorm.h:5-14 (kernels op/LayerNorm.cu:11-100), plus the bias
 * prefill of Dense::_pre_compute (op/Dense.cpp:41-44). */
int cubert_bias_res_ln_f32(float *inout, const float *residual, const float *bias, const float *beta,
                           const float *gamma, int rows, int hidden, void *stream);
int cubert_bias_res_ln_f16(cubert_half *inout, const cubert_half *residual, const cubert_half *bias,
                           const cubert_half *beta, const cubert_half *gamma, int rows, int hidden,
                           void *stream);

/* cubert_bias_res_ln_* on a Dense output that cubert_gemm_skinny_partials_* left as K slices (at most 64 rows; R is
 * `rows` rounded up to a multiple of 32, the token rows each slice holds):
 *   a = storage type of (0.f + partials[(0 * R + r) * pitch + c] + partials[(1 * R + r) * pitch + c] + ...)
 *   x = a + bias + residual[r];  out[r] = beta + gamma * (x - mean) / sqrt(var + 1e-12)
 * i.e. cubert_gemm_skinny_* (alpha 1, no bias) followed by cubert_bias_res_ln_*, without the GEMM's hand-over between
 * workgroups.  Given the slices, the fp32 result has the bits of cubert_bias_res_ln_f32 on their sum; in half
 * precision the inputs to the LayerNorm are the same and a few results differ in the last bit (separately compiled
 * kernels; at 768 halves cubert_bias_res_ln_f16 also adds a row's sums in another order).  `out` is written only (it may be any buffer but `residual`).  Shapes the
 * register-resident LayerNorm kernels do not take (hidden not 64 * {2,4,8} * {1..5}) return CUBERT_UNSUPPORTED
 * and launch nothing.
 * replaces: Dense + layer_norm_<T> of BertOutput / the attention output for a request of at most 64 tokens,
 * reference src/cuBERT/op_att/Transformer.cpp:160-169 (op/Dense.cpp:47-57, op/LayerNorm.h:5-14). */
int cubert_bias_res_ln_partials_f32(float *out, const float *partials, int slices, int pitch, const float *residual,
                                    const float *bias, const float *beta, const float *gamma, int rows, int hidden,
                                    void *stream);
int cubert_bias_res_ln_partials_f16(cubert_half *out, const float *partials, int slices, int pitch,
                                    const cubert_half *residual, const cubert_half *bias, const cubert_half *beta,
                                    const cubert_half *gamma, int rows, int hidden, void *stream);

/* bias + GELU (erf form), in place:  x = inout[r,c] + bias[c];  inout = x * 0.5 * (1 + erf(x / sqrt 2)).
 * `bias` may be NULL.
 * replaces: gelu<T>(N, inout, stream), reference src/cuBERT/op/GELU.h:6-7 (op/GELU.cu:14-26),
 * plus the bias prefill of the intermediate Dense. */
int cubert_bias_gelu_f32(float *inout, const float *bias, int rows, int width, void *stream);
int cubert_bias_gelu_f16(cubert_half *inout, const cubert_half *bias, int rows, int width, void *stream);

/* Attention mask + scale + softmax over the last axis of scores[batch, heads, seq_length, seq_length],
 * in place:   s = scores * scale + (mask[b, k] == 0 ? -10000 : 0);   p = exp(s - max_k s) / sum_k
 * `mask` is the caller's int8 [batch, seq_length] input mask (any non-zero byte keeps the key) and
 * may be NULL (no masking).
 * replaces: _not<T> + the k=1 broadcast GEMM of AttentionMask (reference src/cuBERT/op_att/
 * AttentionMask.h:8-12, AttentionMask.cpp:41-54), the per-layer mask copy and the alpha/beta of the
 * QK GEMM (op_att/AttentionSelf.cpp:58-60,99-101) and softmax_<T> (op/Softmax.h:8-14, five kernels
 * in op/Softmax.cu:104-115). */
int cubert_mask_scale_softmax_f32(float *scores, const int8_t *mask, float scale, int batch, int heads,
                                  int seq_length, void *stream);
int cubert_mask_scale_softmax_f16(cubert_half *scores, const int8_t *mask, float scale, int batch, int heads,
                                  int seq_length, void *stream);

/* The two attention contractions over all (batch, head) problems in one launch each.
 *   scores[b, a, q, k] = alpha * sum_j Q[b, q, a, j] * K[b, k, a, j]      (scores is [batch, heads, seq, seq])
 *   ctx[b, q, a, j]    = sum_k P[b, a, q, k] * V[b, k, a, j]              (ctx row stride ld_ctx >= heads*head_size)
 * q, k, v point at element (0, 0) of their [batch*seq, heads*head_size] views, row stride `ld` elements
 * (3*hidden for a packed QKV buffer).  Matrix-core kernels, fp32 accumulation.  Supported: seq a multiple of
 * 32, head_size 32 / 64 / 128, 16-byte aligned pointers, batch*heads <= 65535; anything else returns
 * CUBERT_UNSUPPORTED and launches nothing (the host classes then loop a strided-batched GEMM).
 * replaces: Att_Q_K<T>::compute and Att_QK_V<T>::compute (pointer-array batched GEMMs), reference
 * src/cuBERT/op_att/BatchMatMul.h:17-74 (BatchMatMul.cpp:57-68,129-140); alpha as AttentionSelf.cpp:58-60. */
int cubert_attention_scores_f32(const float *q, const float *k, int ld, float *scores, float alpha, int batch,
                                int heads, int seq_length, int head_size, void *stream);
int cubert_attention_scores_f16(const cubert_half *q, const cubert_half *k, int ld, cubert_half *scores, float alpha,
                                int batch, int heads, int seq_length, int head_size, void *stream);
int cubert_attention_context_f32(const float *probs, const float *v, int ld, float *ctx, int ld_ctx, int batch,
                                 int heads, int seq_length, int head_size, void *stream);
int cubert_attention_context_f16(const cubert_half *probs, const cubert_half *v, int ld, cubert_half *ctx, int ld_ctx,
                                 int batch, int heads, int seq_length, int head_size, void *stream);

/* The attention core of one layer in a single launch:
 *   ctx[b, q, a, :] = sum_k softmax_k(alpha * Q[b,q,a,:] . K[b,k,a,:] + (mask[b,k] == 0 ? -10000 : 0)) * V[b, k, a, :]
 * with the [batch, heads, seq, seq] scores held in registers in fp32 (never written to memory, never rounded to
 * the storage type as the three-kernel sequence cubert_attention_scores, cubert_mask_scale_softmax,
 * cubert_attention_context does; fp32 storage gives the same result up to summation order, fp16 storage agrees
 * within its tolerance).  Up to seq_length 128 the softmax is the exact two-pass one; from 129 to 512 it runs
 * online over chunks of 64 keys and is normalised once at the end.  mask may be NULL.  Shape support as the two contractions, and seq_length <= 512
 * (<= 128 for head_size 128, and K, V of one head must fit 160 KB of LDS: fp32 up to seq_length 256 at head size
 * 64); anything else returns CUBERT_UNSUPPORTED and launches nothing.
 * replaces: AttentionSelf<T>::_in_compute's Att_Q_K -> Softmax -> Att_QK_V sequence and the mask tensor of
 * AttentionMask<T>::compute, reference src/cuBERT/op_att/AttentionSelf.cpp:96-111, AttentionMask.cpp:41-54. */
int cubert_attention_fused_f32(const float *q, const float *k, const float *v, int ld, const int8_t *mask, float *ctx,
                               int ld_ctx, float alpha, int batch, int heads, int seq_length, int head_size,
                               void *stream);
int cubert_attention_fused_f16(const cubert_half *q, const cubert_half *k, const cubert_half *v, int ld,
                               const int8_t *mask, cubert_half *ctx, int ld_ctx, float alpha, int batch, int heads,
                               int seq_length, int head_size, void *stream);

/* Longest sequences first.  The long-sequence kernels (seq_length > 128) leave out key tiles (32 keys) whose mask
 * bytes are all zero, so a workgroup's time goes with its sequence's number of live tiles, and workgroups are handed
 * to the compute units in index order: a long sequence late in the batch starts late and the launch waits for it.
 * cubert_attention_order writes the sequence indices 0..batch-1 by falling live-tile count into order[0 .. batch) and,
 * from order[4 * batch] on, a record of 4 ints for the sequence at each position {number of live tiles, their tile
 * numbers in ascending order 4 bits each (low word, high word), the live tiles as a bit mask}: `order` holds
 * 8 * batch ints and is 16-byte aligned (one small launch; the mask is the same for every layer of a forward pass,
 * so once per pass).  cubert_attention_fused_ordered_* is cubert_attention_fused_* taking sequence order[i] where it
 * would take i, and the tiles to compute from that position's record (order may be NULL: batch order, tiles from
 * the mask; shapes of at most 128 keys ignore it).  Results are identical with any order, i.e. with any permutation
 * of the positions that moves the records along with the indices.
 * CUBERT_UNSUPPORTED from cubert_attention_order (seq_length not a multiple of 32 or above 512, more than 4096
 * sequences, a mask that is not 4-byte aligned, an order array that is not 16-byte aligned): pass NULL.
 * No counterpart in the reference, which computes every key of every sequence (src/cuBERT/op_att/AttentionSelf.cpp:96-111). */
int cubert_attention_order(const int8_t *mask, int batch, int seq_length, int *order, void *stream);
int cubert_attention_fused_ordered_f32(const float *q, const float *k, const float *v, int ld, const int8_t *mask,
                                       const int *order, float *ctx, int ld_ctx, float alpha, int batch, int heads,
                                       int seq_length, int head_size, void *stream);
int cubert_attention_fused_ordered_f16(const cubert_half *q, const cubert_half *k, const cubert_half *v, int ld,
                                       const int8_t *mask, const int *order, cubert_half *ctx, int ld_ctx, float alpha,
                                       int batch, int heads, int seq_length, int head_size, void *stream);


/* Row softmax of a [rows, channel] matrix, in place or not (classifier probabilities).
 * replaces: softmax_<T>(in, out, rows, channel, sum_buf, stream), reference src/cuBERT/op/Softmax.h:8-14. */
int cubert_row_softmax_f32(const float *in, float *out, int rows, int channel, void *stream);
int cubert_row_softmax_f16(const cubert_half *in, cubert_half *out, int rows, int channel, void *stream);

/* bias + tanh, in place on [rows, width]; `bias` may be NULL.
 * replaces: tanh_<T>(inout, N, stream), reference src/cuBERT/op_bert/BertPooler.h:8-11
 * (op_bert/BertPooler.cu:14-26), plus the pooler's bias prefill (BertPooler.cpp:65). */
int cubert_bias_tanh_f32(float *inout, const float *bias, int rows, int width, void *stream);
int cubert_bias_tanh_f16(cubert_half *inout, const cubert_half *bias, int rows, int width, void *stream);

/* out[b, c] = (sum_s in[b, s, c]) / seq_length  -- every position counts, padding included.
 * replaces: reduce_mean_1<T>(in, out, batch, seq_length, hidden, stream),
 * reference src/cuBERT/op_bert/BertPooler.h:13-16 (op_bert/BertPooler.cu:35-66). */
int cubert_mean_pool_f32(const float *in, float *out, int batch, int seq_length, int hidden, void *stream);
int cubert_mean_pool_f16(const cubert_half *in, cubert_half *out, int batch, int seq_length, int hidden,
                         void *stream);

/* The tail of a classification model in one launch (one workgroup per sequence):
 *     pooled = tanh(pooled + pooler_bias)   in place; skipped when pooler_bias is NULL
 *     logits = pooled W^T + out_bias        W [labels, hidden] row-major, out_bias may be NULL
 *     probs  = softmax(logits)
 * for up to 64 labels (more: CUBERT_UNSUPPORTED, nothing launched; use cubert_bias_tanh_*, cubert_gemm_* and
 * cubert_row_softmax_*).
 * replaces: tanh_<T> (op_bert/BertPooler.cpp:65-76), ClassifierOutputLayer<T>::_in_compute and its Softmax<T>
 * (op_out/AdditionalOutputLayer.cpp:30,52-66). */
int cubert_classifier_head_f32(float *pooled, const float *pooler_bias, const float *weights, const float *out_bias,
                               float *logits, float *probs, int batch, int hidden, int labels, void *stream);
int cubert_classifier_head_f16(cubert_half *pooled, const cubert_half *pooler_bias, const cubert_half *weights,
                               const cubert_half *out_bias, cubert_half *logits, cubert_half *probs, int batch,
                               int hidden, int labels, void *stream);

/* out[c, r] = in[r, c] for a row-major [rows, cols] matrix (out must not alias in).  No counterpart in the
 * reference, which keeps every Dense kernel [in, out] (op/Dense.cpp:47-57): half-precision models here store
 * them [out, in], the operand order the library's fp16 GEMMs run fastest on. */
int cubert_transpose_f32(const float *in, int rows, int cols, float *out, void *stream);
int cubert_transpose_f16(const cubert_half *in, int rows, int cols, cubert_half *out, void *stream);

/* ------------------------------------------------------------------ runtime
 * replaces: reference src/cuBERT/common.h:17-92 (cudart + cuBLAS side). */

int cubert_get_gpu_count(void);
int cubert_set_gpu(int device);
int cubert_gpu_info(int device); /* prints name, memory and clock to stderr */

void *cubert_malloc(size_t size); /* device memory; NULL on failure */
int cubert_free(void *ptr);
/* Free and total device memory of the current GPU in bytes (either pointer may be NULL): what the reference prints
 * when an allocation fails (src/cuBERT/common.cpp:158-161), here also readable by a caller that wants to see what a
 * model or a call took. */
int cubert_mem_info(size_t *free_bytes, size_t *total_bytes);
/* kind: 1 host->device, 2 device->host, 3 device->device (cudaMemcpyKind numbering, common.h:31-40) */
int cubert_memcpy(void *dst, const void *src, size_t n, int kind);
int cubert_memcpy_async(void *dst, const void *src, size_t n, int kind, void *stream);

void *cubert_stream_create(void);
int cubert_stream_destroy(void *stream);
int cubert_stream_synchronize(void *stream);

/* Page-locked host memory, for staging buffers that asynchronous copies read or write directly
 * (the reference copies from the caller's pageable memory, src/cuBERT/common.cpp:176-195). */
void *cubert_malloc_host(size_t size); /* NULL on failure */
int cubert_free_host(void *ptr);

/* Events on a stream (no counterpart in the reference, which has no built-in profiling): they time single
 * kernels of a forward pass where they run and tell the host when a staging buffer may be written again. */
void *cubert_event_create(void);
int cubert_event_synchronize(void *event); /* blocks the calling thread until the event has completed */
int cubert_event_destroy(void *event);
int cubert_event_record(void *event, void *stream);
int cubert_event_elapsed_ms(void *start, void *stop, float *ms); /* both events must have completed */
/* The next layer kernel launched from the calling thread writes its own start and stop timestamps into the
 * two events (the kernel's dispatch packet carries them), so cubert_event_elapsed_ms(start, stop) is that
 * kernel's execution time alone.  One shot: cleared by the launch.  NULL, NULL cancels. */
int cubert_time_next_launch(void *start_event, void *stop_event);

/* A BLAS context: a hipBLASLt handle, a workspace, a plan cache and the few-token kernel's scratch (partial tiles
 * and arrival counters), bound to one stream.  One set of each per context, so a context's GEMMs belong on ONE
 * stream and come from one thread at a time: the library serialises the calls of several threads on one handle
 * (a mutex), and cubert_blas_set_stream to a different stream first waits for what the context launched on the
 * old one, but launches of one context never overlap on the device.  Callers that want GEMMs to overlap use one
 * context per stream (as Bert<T> does: one context and one stream per model instance, the reference's
 * arrangement, src/cuBERT/Bert.cpp:23-25). */
void *cubert_blas_create(void);
int cubert_blas_destroy(void *handle);
int cubert_blas_set_stream(void *handle, void *stream);
void *cubert_blas_get_stream(void *handle);

/* Column-major GEMM with the meaning of cublasGemmEx / cblas_sgemm:
 *   C = alpha * op(A) * op(B) + beta * C        (fp32 accumulation for both storage types)
 * When `bias` is not NULL it is a length-M vector added to every column of the product before
 * beta*C (GEMM epilogue), which is how a Dense bias is applied for row-major activations.
 * replaces: blas_gemm<T>, reference src/cuBERT/common.h:59-68 (common.cpp:224-258,351-372). */
int cubert_gemm_f32(void *handle, int transA, int transB, int M, int N, int K, float alpha, const float *A,
                    int lda, const float *B, int ldb, float beta, float *C, int ldc, const float *bias);
int cubert_gemm_f16(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                    const cubert_half *A, int lda, const cubert_half *B, int ldb, float beta, cubert_half *C,
                    int ldc, const cubert_half *bias);
/* The same with fp16 operands and an fp32 result (C and bias are float; the products are exact and accumulate in
 * fp32).  With operands written by cubert_split3_f32 this is the Dense GEMM of an fp32 model on the fp16 matrix
 * cores.  replaces: blas_gemm<float>, reference src/cuBERT/common.h:59-68 (common.cpp:224-258), as an opt-in
 * alternative to cubert_gemm_f32. */
int cubert_gemm_f16_f32(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                        const cubert_half *A, int lda, const cubert_half *B, int ldb, float beta, float *C, int ldc,
                        const float *bias);

/* fp32 rows as sums of two fp16 numbers: with hi = fp16(scale * x) and lo = fp16(scale * x - hi),
 *   out[r] = [hi(in[r]) | hi(in[r]) | lo(in[r])]      (lo_in_middle = 0: the token side of a Dense GEMM)
 *   out[r] = [hi(in[r]) | lo(in[r]) | hi(in[r])]      (lo_in_middle = 1: the weight side, rows = output features)
 * each part `width` halves, so that a dot product of a token row with a weight row over 3 * width is
 * hi*hi + hi*lo + lo*hi = the fp32 product up to 2^-22 relative.  Values are clamped to the fp16 range; `scale`
 * (a power of two, undone by the GEMM's alpha) keeps small values out of the fp16 subnormals.  A value that had
 * to be clamped (|scale * x| > 65504) or is not a number no longer equals its two terms: this and the three entry
 * points below then store 1 to *overflow (device memory, or page-locked host memory from cubert_malloc_host;
 * NULL = not wanted; never written otherwise, so the caller clears it), and the caller must not use the product
 * (the host classes recompute the request with cubert_gemm_f32).
 * replaces: nothing in the reference by itself; it is the operand preparation of the opt-in form of
 * Dense<float>::compute (reference src/cuBERT/op/Dense.cpp:47-57) that runs on the fp16 matrix cores. */
int cubert_split3_f32(const float *in, int rows, int width, float scale, int lo_in_middle, cubert_half *out,
                      int *overflow, void *stream);
/* bias + GELU as cubert_bias_gelu_f32 computes it, times `scale` (a power of two), written as [hi | hi | lo] rows
 * for the GEMM that follows instead of in place.  replaces: gelu<float>, reference src/cuBERT/op/GELU.h:6-7 (op/GELU.cu:14-26), followed
 * by the operand preparation above. */
int cubert_bias_gelu_split3_f32(const float *in, const float *bias, int rows, int width, float scale,
                                cubert_half *out, int *overflow, void *stream);
/* cubert_attention_fused_f32 with the context, times `scale` (a power of two), written as [hi | hi | lo] rows,
 * split_ctx[batch * seq_length, 3 * heads * head_size], for the GEMM that follows, instead of as fp32.  Same shape limits and return codes.
 * replaces: AttentionSelf<float>::_in_compute between the projections, reference
 * src/cuBERT/op_att/AttentionSelf.cpp:96-111, followed by the operand preparation above. */
int cubert_attention_fused_split3_f32(const float *q, const float *k, const float *v, int ld, const int8_t *mask,
                                      float scale, cubert_half *split_ctx, float alpha, int batch, int heads, int seq_length,
                                      int head_size, int *overflow, void *stream);
/* cubert_bias_res_ln_f32, and its result times `scale` (a power of two) again as [hi | hi | lo] rows in
 * split_out[rows, 3 * hidden] for the GEMM that follows.  hidden must be 256 k (k = 1..6, 8) with 16-byte aligned operands, otherwise CUBERT_UNSUPPORTED is
 * returned and nothing is done.  replaces: layer_norm_<float>, reference src/cuBERT/op/LayerNorm.h:5-14
 * (op/LayerNorm.cu:11-100), followed by the operand preparation above. */
int cubert_bias_res_ln_split3_f32(float *inout, const float *residual, const float *bias, const float *beta,
                                  const float *gamma, int rows, int hidden, float scale, cubert_half *split_out,
                                  int *overflow, void *stream);

/* C = alpha * A * B + bias for N <= 64 columns (no transposes, beta = 0): the Dense layer of a request with at
 * most 64 tokens, where A is the [in, out] weight matrix (M = out, K = in) and each column of B one token.
 * One pass over the weights on the matrix cores with every load in flight at once (from 33 tokens on a wavefront
 * multiplies its weights with two blocks of 32 tokens); K is cut into slices that are added in a fixed order, so
 * results do not depend on scheduling.  cubert_gemm_* takes this path by itself when the problem fits and
 * N <= 32 (CUBERT_GEMM=library in the environment turns that off); beyond 32 tokens the library is the faster one
 * for some shapes and the caller chooses (the host classes: see csrc/host/Transformer.cpp).  Needs K a multiple
 * of 16 and B 16-byte aligned with ldb a multiple of 16 bytes; anything else returns CUBERT_UNSUPPORTED and
 * launches nothing (also with CUBERT_GEMM=library or naive in the environment).  activation: 0 = none, 1 = the
 * erf-form GELU of cubert_bias_gelu applied to the result (Dense + bias + GELU of BertIntermediate in one
 * launch; reference src/cuBERT/op_att/Transformer.cpp:164-165).  Launches of one handle share its partial-tile
 * workspace and counters and are ordered by the handle's one stream (see cubert_blas_create); they never run
 * concurrently.
 * replaces: Dense<T>::compute -> blas_gemm<T> for small batch * seq_length, reference
 * src/cuBERT/op/Dense.cpp:47-57 (bias: Dense.cpp:41-44). */
int cubert_gemm_skinny_f32(void *handle, int M, int N, int K, float alpha, const float *A, int lda, const float *B,
                           int ldb, float *C, int ldc, const float *bias, int activation);
int cubert_gemm_skinny_f16(void *handle, int M, int N, int K, float alpha, const cubert_half *A, int lda,
                           const cubert_half *B, int ldb, cubert_half *C, int ldc, const cubert_half *bias,
                           int activation);

/* cubert_gemm_skinny_f32 for callers that cannot allocate device memory or hold a BLAS context: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference
 * (whose GEMMs all go through a cuBLAS handle) and none is needed by the host classes here.  Same kernel, same
 * arguments and return codes, same results bit for bit; instead of a handle it takes the stream, and the split-K
 * partial tiles and arrival counters live in a fixed array inside the library's device image (4 MiB + 16 KiB on
 * every GPU the library runs on, until the process ends).  The call allocates and frees nothing.  The array's
 * size fixes the largest problem: M <= CUBERT_GEMM_SKINNY_NOALLOC_MAX_M output features and
 * K <= CUBERT_GEMM_SKINNY_NOALLOC_MAX_K; beyond that CUBERT_TOO_LARGE is returned, a message goes to stderr and
 * nothing is launched.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams,
 * two threads) race on it; keep them on one stream or order them yourself.  The first call on a device looks up
 * the array's address there (hipGetSymbolAddress), which is the only set-up. */
#define CUBERT_GEMM_SKINNY_NOALLOC_MAX_M 32768
#define CUBERT_GEMM_SKINNY_NOALLOC_MAX_K 65536
int cubert_gemm_skinny_noalloc_f32(void *stream, int M, int N, int K, float alpha, const float *A, int lda,
                                   const float *B, int ldb, float *C, int ldc, const float *bias, int activation);

/* The few-token kernel on weights re-ordered once into the order it consumes them (a workgroup then streams
 * one contiguous run with 16-byte loads instead of 128-byte pieces at a stride of a weight row).
 * cubert_gemm_skinny_packed_elements(M, K) elements are needed for the packed copy of an A of M x K;
 * cubert_gemm_skinny_pack_* fills it (asynchronous, on the handle's stream; K a multiple of 16, packed 16-byte
 * aligned, else CUBERT_UNSUPPORTED); cubert_gemm_skinny_packed_* is cubert_gemm_skinny_* on the packed copy.
 * No counterpart in the reference (its weights stay in the TensorFlow layout, src/cuBERT/op/Dense.cpp:14-38). */
size_t cubert_gemm_skinny_packed_elements(int M, int K);
int cubert_gemm_skinny_pack_f32(void *handle, const float *A, int lda, int M, int K, float *packed);
int cubert_gemm_skinny_pack_f16(void *handle, const cubert_half *A, int lda, int M, int K, cubert_half *packed);
int cubert_gemm_skinny_packed_f32(void *handle, int M, int N, int K, float alpha, const float *packedA, const float *B,
                                  int ldb, float *C, int ldc, const float *bias, int activation);
int cubert_gemm_skinny_packed_f16(void *handle, int M, int N, int K, float alpha, const cubert_half *packedA,
                                  const cubert_half *B, int ldb, cubert_half *C, int ldc, const cubert_half *bias,
                                  int activation);

/* The few-token product left as partial sums, for a consumer kernel that adds them while it loads its operand
 * (cubert_bias_res_ln_partials_*).  A few-token Dense kernel spends 2 of its 7-10 us
 * handing the K slices over to the workgroup that adds them; here every workgroup stores its slice and is done:
 *   partials[(slice * R + token) * pitch + feature] = sum over the slice's k of A[k, feature] * B[k, token]
 * for *slices slices, all R token rows (R = N rounded up to a multiple of 32; rows from N on are zero) and
 * *pitch >= M features per row (fp32 whatever the
 * storage type; no alpha, bias or activation).  Adding the slices in slice order, starting from 0.f, and rounding
 * to the storage type is what a consumer does; the result is cubert_gemm_skinny_*'s for alpha = 1 and no bias up to
 * the order of the additions (the reduction may be cut into more slices here: nobody in this kernel has to add them,
 * and a weight matrix with few feature blocks streams faster when more workgroups pull on it).  packed != 0: A is the
 * output of cubert_gemm_skinny_pack_* (lda ignored).  partials must
 * hold partial_floats >= *slices * R * *pitch floats (1 << 20 is enough for every BERT-base/large Dense layer),
 * else CUBERT_UNSUPPORTED and nothing is launched; same conditions on K, B and ldb as cubert_gemm_skinny_*.
 * Asynchronous on the handle's stream.  No counterpart in the reference; same place as cubert_gemm_skinny_*
 * (src/cuBERT/op/Dense.cpp:47-57). */
int cubert_gemm_skinny_partials_f32(void *handle, int M, int N, int K, const float *A, int lda, int packed,
                                    const float *B, int ldb, float *partials, size_t partial_floats, int *slices,
                                    int *pitch);
int cubert_gemm_skinny_partials_f16(void *handle, int M, int N, int K, const cubert_half *A, int lda, int packed,
                                    const cubert_half *B, int ldb, float *partials, size_t partial_floats, int *slices,
                                    int *pitch);

/* The same over `batch_count` problems at fixed strides (in elements).
 * replaces: blas_gemm_strided_batch<T>, reference src/cuBERT/common.h:82-92. */
int cubert_gemm_strided_batch_f32(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                                  const float *A, int lda, long long strideA, const float *B, int ldb,
                                  long long strideB, float beta, float *C, int ldc, long long strideC,
                                  int batch_count);
int cubert_gemm_strided_batch_f16(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                                  const cubert_half *A, int lda, long long strideA, const cubert_half *B,
                                  int ldb, long long strideB, float beta, cubert_half *C, int ldc,
                                  long long strideC, int batch_count);

/* The same over `batch_count` problems given as arrays of pointers: A_array, B_array and C_array are DEVICE arrays
 * of batch_count device pointers (one problem each, as cublasGemmBatchedEx takes them); lda, ldb, ldc and the
 * transposes are shared.  fp32 accumulation; with beta = 0 the C matrices are not read.  Runs on the handle's
 * stream, asynchronously.  This is the interface of the reference's attention contractions (Att_Q_K / Att_QK_V
 * build one pointer per (batch, head), src/cuBERT/op_att/BatchMatMul.cpp:31-38,57-68,103-110,129-140); the host
 * classes here use cubert_attention_* instead, which is the fast path.  This entry point is the compatibility
 * path for a host program that keeps the reference's BatchMatMul classes: shapes whose M, N and K are multiples of
 * 32 run on the matrix cores (a wavefront per 32 x 32 tile of C), any other shape on plain fused multiply-adds.
 * What it costs, measured on one MI355X on the QK^T contraction of 1536 (batch, head) problems of head size 64,
 * microseconds per launch, this entry point / cubert_attention_scores_* on the same operands:
 *   fp32  seq 32:  8.3 / 10.0    seq 128:  73.6 / 128.3
 *   fp16  seq 32:  4.9 /  4.5    seq 128:  40.5 /  17.3
 * (before the matrix-core kernel: 21.3, 114.3, 19.4 and 96.8).  Either way a host that goes through this interface
 * writes the [batch, heads, seq, seq] tensor to memory and reads it back twice, which cubert_attention_fused_* does
 * not: one launch of 12.7 us (fp32, seq 32) instead of three.
 * replaces: blas_gemm_batch<T>, reference src/cuBERT/common.h:70-80 (src/cuBERT/common.cpp:261-298,375-396). */
int cubert_gemm_batch_f32(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                          const float *const *A_array, int lda, const float *const *B_array, int ldb, float beta,
                          float *const *C_array, int ldc, int batch_count);
int cubert_gemm_batch_f16(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                          const cubert_half *const *A_array, int lda, const cubert_half *const *B_array, int ldb,
                          float beta, cubert_half *const *C_array, int ldc, int batch_count);

#ifdef __cplusplus
}
#endif
#endif /* CUBERT_KERNELS_H */
