// Host-side view of the device layer, in the vocabulary of the reference's
// cuBERT::common.h (src/cuBERT/common.h:17-112): typed malloc/memcpy/stream/
// blas helpers and the layer launchers, overloaded on the storage type
// (float, half) and forwarding to the C ABI of include/cubert_kernels.h.
// Any device error is fatal: message to stderr, exit(EXIT_FAILURE), as the
// reference's CUDA_CHECK does (common.cpp:79-93).
#ifndef CUBERT_HOST_COMMON_H
#define CUBERT_HOST_COMMON_H

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "cubert_kernels.h"

namespace cuBERT {

typedef _Float16 half;  // IEEE binary16; float <-> half conversions round to nearest even

#define CUBERT_CHECK(call)                                                                            \
    do {                                                                                              \
        int rc_ = (call);                                                                             \
        if (rc_ != 0) {                                                                               \
            fprintf(stderr, "cuBERT device error %d in file '%s' in line %i : %s\n", rc_, __FILE__,   \
                    __LINE__, #call);                                                                 \
            exit(EXIT_FAILURE);                                                                       \
        }                                                                                             \
    } while (0)

inline void initialize() {}
inline void finalize() {}

inline int get_gpu_count() { return cubert_get_gpu_count(); }
inline void set_gpu(int device) { CUBERT_CHECK(cubert_set_gpu(device)); }
inline void gpu_info(int device) { CUBERT_CHECK(cubert_gpu_info(device)); }

inline void *cuda_stream_create() {
    void *s = cubert_stream_create();
    if (s == nullptr) {
        fprintf(stderr, "cuBERT: could not create a stream\n");
        exit(EXIT_FAILURE);
    }
    return s;
}
inline void cuda_stream_destroy(void *stream) { CUBERT_CHECK(cubert_stream_destroy(stream)); }
inline void cuda_stream_synchronize(void *stream) { CUBERT_CHECK(cubert_stream_synchronize(stream)); }

inline void *malloc(size_t size) {
    void *p = cubert_malloc(size);
    if (p == nullptr) exit(EXIT_FAILURE);  // cubert_malloc has printed sizes and free memory
    return p;
}
inline void free(void *ptr) { CUBERT_CHECK(cubert_free(ptr)); }
inline void memcpy(void *dst, const void *src, size_t n, int kind) { CUBERT_CHECK(cubert_memcpy(dst, src, n, kind)); }
inline void memcpyAsync(void *dst, const void *src, size_t n, int kind, void *stream) {
    CUBERT_CHECK(cubert_memcpy_async(dst, src, n, kind, stream));
}

inline void *blas_create() {
    void *h = cubert_blas_create();
    if (h == nullptr) {
        fprintf(stderr, "cuBERT: could not create a hipBLASLt context\n");
        exit(EXIT_FAILURE);
    }
    return h;
}
inline void blas_destroy(void *handle) { CUBERT_CHECK(cubert_blas_destroy(handle)); }
inline void *blas_get_stream(void *handle) { return cubert_blas_get_stream(handle); }
inline void blas_set_stream(void *handle, void *stream) { CUBERT_CHECK(cubert_blas_set_stream(handle, stream)); }

inline const cubert_half *h(const half *p) { return reinterpret_cast<const cubert_half *>(p); }
inline cubert_half *h(half *p) { return reinterpret_cast<cubert_half *>(p); }

// Column-major GEMM, C = alpha*op(A)*op(B) + beta*C (+ bias per row of C), fp32 accumulation.
inline void blas_gemm(void *handle, bool TransA, bool TransB, int M, int N, int K, float alpha, const float *A,
                      int lda, const float *B, int ldb, float beta, float *C, int ldc, const float *bias = nullptr) {
    CUBERT_CHECK(cubert_gemm_f32(handle, TransA, TransB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc, bias));
}
inline void blas_gemm(void *handle, bool TransA, bool TransB, int M, int N, int K, float alpha, const half *A, int lda,
                      const half *B, int ldb, float beta, half *C, int ldc, const half *bias = nullptr) {
    CUBERT_CHECK(cubert_gemm_f16(handle, TransA, TransB, M, N, K, alpha, h(A), lda, h(B), ldb, beta, h(C), ldc, h(bias)));
}
// A Dense layer for at most 64 tokens on the few-token kernel (column-major C[M, N] = [gelu](A B + bias), N <= 64),
// on the weights in its own order when `packed` is given; false when the kernel does not take the problem
// (the caller then runs blas_gemm).  No counterpart in the reference.
inline bool dense_few_tokens(void *handle, int M, int N, int K, const float *A, int lda, const float *packed,
                             const float *B, int ldb, float *C, int ldc, const float *bias, bool gelu) {
    const int rc = packed ? cubert_gemm_skinny_packed_f32(handle, M, N, K, 1.f, packed, B, ldb, C, ldc, bias, gelu)
                          : cubert_gemm_skinny_f32(handle, M, N, K, 1.f, A, lda, B, ldb, C, ldc, bias, gelu);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline bool dense_few_tokens(void *handle, int M, int N, int K, const half *A, int lda, const half *packed,
                             const half *B, int ldb, half *C, int ldc, const half *bias, bool gelu) {
    const int rc = packed ? cubert_gemm_skinny_packed_f16(handle, M, N, K, 1.f, h(packed), h(B), ldb, h(C), ldc, h(bias),
                                                          gelu)
                          : cubert_gemm_skinny_f16(handle, M, N, K, 1.f, h(A), lda, h(B), ldb, h(C), ldc, h(bias), gelu);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
// The same product left as K slices for the kernel that consumes it (layer_norm_partials):
// partials[(slice * R + token) * pitch + feature], fp32, R = N rounded up to 32; false when the kernel does not take
// the problem.
inline bool dense_few_tokens_partials(void *handle, int M, int N, int K, const float *A, int lda, const float *packed,
                                      const float *B, int ldb, float *partials, size_t partial_floats, int *slices,
                                      int *pitch) {
    const int rc = cubert_gemm_skinny_partials_f32(handle, M, N, K, packed ? packed : A, lda, packed != nullptr, B, ldb,
                                                   partials, partial_floats, slices, pitch);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline bool dense_few_tokens_partials(void *handle, int M, int N, int K, const half *A, int lda, const half *packed,
                                      const half *B, int ldb, float *partials, size_t partial_floats, int *slices,
                                      int *pitch) {
    const int rc = cubert_gemm_skinny_partials_f16(handle, M, N, K, h(packed ? packed : A), lda, packed != nullptr, h(B),
                                                   ldb, partials, partial_floats, slices, pitch);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
// out = LayerNorm(storage type of (sum of the slices) + bias + residual) for at most 64 rows; false when declined
inline bool layer_norm_partials(float *out, const float *partials, int slices, int pitch, const float *residual,
                                const float *bias, const float *beta, const float *gamma, int rows, int hidden,
                                void *stream) {
    const int rc = cubert_bias_res_ln_partials_f32(out, partials, slices, pitch, residual, bias, beta, gamma, rows,
                                                   hidden, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline bool layer_norm_partials(half *out, const float *partials, int slices, int pitch, const half *residual,
                                const half *bias, const half *beta, const half *gamma, int rows, int hidden,
                                void *stream) {
    const int rc = cubert_bias_res_ln_partials_f16(h(out), partials, slices, pitch, h(residual), h(bias), h(beta),
                                                   h(gamma), rows, hidden, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline void pack_few_token_weights(void *handle, const float *A, int lda, int M, int K, float *packed) {
    CUBERT_CHECK(cubert_gemm_skinny_pack_f32(handle, A, lda, M, K, packed));
}
inline void pack_few_token_weights(void *handle, const half *A, int lda, int M, int K, half *packed) {
    CUBERT_CHECK(cubert_gemm_skinny_pack_f16(handle, h(A), lda, M, K, h(packed)));
}

// fp16 operands, fp32 result: the Dense GEMM of an fp32 model in its two-term fp16 form (kernels/split.hip)
inline void blas_gemm_f16_f32(void *handle, bool TransA, bool TransB, int M, int N, int K, float alpha, const half *A,
                              int lda, const half *B, int ldb, float beta, float *C, int ldc,
                              const float *bias = nullptr) {
    CUBERT_CHECK(cubert_gemm_f16_f32(handle, TransA, TransB, M, N, K, alpha, h(A), lda, h(B), ldb, beta, C, ldc, bias));
}
// (`overflow` in this and the next three: where 1 is stored when a value did not fit its two terms; may be null)
inline void split3(const float *in, int rows, int width, float scale, bool lo_in_middle, half *out, int *overflow,
                   void *stream) {
    CUBERT_CHECK(cubert_split3_f32(in, rows, width, scale, lo_in_middle, h(out), overflow, stream));
}
// false: the shape is not one the fused kernel takes (the caller runs layer_norm_ and split3)
inline bool layer_norm_split3(const float *in, float *inout, int rows, int channels, const float *bias,
                              const float *beta, const float *gamma, float scale, half *split_out, int *overflow,
                              void *stream) {
    const int rc = cubert_bias_res_ln_split3_f32(inout, in, bias, beta, gamma, rows, channels, scale, h(split_out),
                                                 overflow, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
// the one-launch attention core with its context in two-term rows; false when the shape is not taken
inline bool attention_fused_split3(const float *q, const float *k, const float *v, int ld, const int8_t *mask,
                                   float scale, half *split_ctx, float alpha, int batch, int heads, int seq,
                                   int head_size, int *overflow, void *stream) {
    const int rc = cubert_attention_fused_split3_f32(q, k, v, ld, mask, scale, h(split_ctx), alpha, batch, heads, seq,
                                                     head_size, overflow, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline void bias_gelu_split3(const float *in, const float *bias, int rows, int width, float scale, half *out,
                             int *overflow, void *stream) {
    CUBERT_CHECK(cubert_bias_gelu_split3_f32(in, bias, rows, width, scale, h(out), overflow, stream));
}

inline void transpose(const float *in, int rows, int cols, float *out, void *stream) {
    CUBERT_CHECK(cubert_transpose_f32(in, rows, cols, out, stream));
}
inline void transpose(const half *in, int rows, int cols, half *out, void *stream) {
    CUBERT_CHECK(cubert_transpose_f16(h(in), rows, cols, h(out), stream));
}

inline void blas_gemm_strided_batch(void *handle, bool TransA, bool TransB, int m, int n, int k, float alpha,
                                    const float *A, int lda, long long strideA, const float *B, int ldb,
                                    long long strideB, float beta, float *C, int ldc, long long strideC,
                                    int batchCount) {
    CUBERT_CHECK(cubert_gemm_strided_batch_f32(handle, TransA, TransB, m, n, k, alpha, A, lda, strideA, B, ldb, strideB,
                                               beta, C, ldc, strideC, batchCount));
}
inline void blas_gemm_strided_batch(void *handle, bool TransA, bool TransB, int m, int n, int k, float alpha,
                                    const half *A, int lda, long long strideA, const half *B, int ldb,
                                    long long strideB, float beta, half *C, int ldc, long long strideC,
                                    int batchCount) {
    CUBERT_CHECK(cubert_gemm_strided_batch_f16(handle, TransA, TransB, m, n, k, alpha, h(A), lda, strideA, h(B), ldb,
                                               strideB, beta, h(C), ldc, strideC, batchCount));
}

// reference: common.h:70-80 (arrays of device pointers, themselves in device memory)
inline void blas_gemm_batch(void *handle, bool TransA, bool TransB, int m, int n, int k, float alpha,
                            const float **Aarray, int lda, const float **Barray, int ldb, float beta, float **Carray,
                            int ldc, int batchCount) {
    CUBERT_CHECK(cubert_gemm_batch_f32(handle, TransA, TransB, m, n, k, alpha, Aarray, lda, Barray, ldb, beta, Carray,
                                       ldc, batchCount));
}
inline void blas_gemm_batch(void *handle, bool TransA, bool TransB, int m, int n, int k, float alpha,
                            const half **Aarray, int lda, const half **Barray, int ldb, float beta, half **Carray,
                            int ldc, int batchCount) {
    CUBERT_CHECK(cubert_gemm_batch_f16(handle, TransA, TransB, m, n, k, alpha,
                                       reinterpret_cast<const cubert_half *const *>(Aarray), lda,
                                       reinterpret_cast<const cubert_half *const *>(Barray), ldb, beta,
                                       reinterpret_cast<cubert_half *const *>(Carray), ldc, batchCount));
}

// ---- layer launchers (names of the reference's launchers where one exists) ----

// reference: op/Embedding.h:9-15
inline void embedding(const int *ids, int n, const float *table, int width, float *out, void *stream) {
    CUBERT_CHECK(cubert_gather_f32(ids, n, table, width, out, stream));
}
inline void embedding(const int *ids, int n, const half *table, int width, half *out, void *stream) {
    CUBERT_CHECK(cubert_gather_f16(ids, n, h(table), width, h(out), stream));
}
inline void embedding(const int8_t *ids, int n, const float *table, int width, float *out, void *stream) {
    CUBERT_CHECK(cubert_gather_i8_f32(ids, n, table, width, out, stream));
}
inline void embedding(const int8_t *ids, int n, const half *table, int width, half *out, void *stream) {
    CUBERT_CHECK(cubert_gather_i8_f16(ids, n, h(table), width, h(out), stream));
}

// BertEmbeddings::compute in one launch (reference: op_bert/BertEmbeddings.cpp:50-66)
inline void embed_layer_norm(const int *ids, const int8_t *segments, const float *word, const float *pos,
                             const float *type, const float *beta, const float *gamma, float *out, int batch, int seq,
                             int hidden, void *stream) {
    CUBERT_CHECK(cubert_embed_ln_f32(ids, segments, word, pos, type, beta, gamma, out, batch, seq, hidden, stream));
}
inline void embed_layer_norm(const int *ids, const int8_t *segments, const half *word, const half *pos,
                             const half *type, const half *beta, const half *gamma, half *out, int batch, int seq,
                             int hidden, void *stream) {
    CUBERT_CHECK(cubert_embed_ln_f16(ids, segments, h(word), h(pos), h(type), h(beta), h(gamma), h(out), batch, seq,
                                     hidden, stream));
}

// reference: op/LayerNorm.h:5-14, with the Dense bias folded in (bias may be null)
inline void layer_norm_(const float *in, float *inout, int rows, int channels, const float *bias, const float *beta,
                        const float *gamma, void *stream) {
    CUBERT_CHECK(cubert_bias_res_ln_f32(inout, in, bias, beta, gamma, rows, channels, stream));
}
inline void layer_norm_(const half *in, half *inout, int rows, int channels, const half *bias, const half *beta,
                        const half *gamma, void *stream) {
    CUBERT_CHECK(cubert_bias_res_ln_f16(h(inout), h(in), h(bias), h(beta), h(gamma), rows, channels, stream));
}

// Pooler bias + tanh (pooler_bias null: none), classifier and its softmax in one launch; false when the kernel
// does not take the problem (many labels).  reference: op_bert/BertPooler.cpp:65-76, op_out/AdditionalOutputLayer.cpp:52-66
inline bool classifier_head(float *pooled, const float *pooler_bias, const float *weights, const float *out_bias,
                            float *logits, float *probs, int batch, int hidden, int labels, void *stream) {
    const int rc = cubert_classifier_head_f32(pooled, pooler_bias, weights, out_bias, logits, probs, batch, hidden, labels,
                                              stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline bool classifier_head(half *pooled, const half *pooler_bias, const half *weights, const half *out_bias,
                            half *logits, half *probs, int batch, int hidden, int labels, void *stream) {
    const int rc = cubert_classifier_head_f16(h(pooled), h(pooler_bias), h(weights), h(out_bias), h(logits), h(probs),
                                              batch, hidden, labels, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}

// reference: op/GELU.h:6-7, with the Dense bias folded in (bias may be null)
inline void gelu(float *inout, const float *bias, int rows, int width, void *stream) {
    CUBERT_CHECK(cubert_bias_gelu_f32(inout, bias, rows, width, stream));
}
inline void gelu(half *inout, const half *bias, int rows, int width, void *stream) {
    CUBERT_CHECK(cubert_bias_gelu_f16(h(inout), h(bias), rows, width, stream));
}

// AttentionMask + QK scale + softmax_ (reference: op_att/AttentionMask.h:8-12, op/Softmax.h:8-14)
inline void mask_scale_softmax_(float *scores, const int8_t *mask, float scale, int batch, int heads, int seq,
                                void *stream) {
    CUBERT_CHECK(cubert_mask_scale_softmax_f32(scores, mask, scale, batch, heads, seq, stream));
}
inline void mask_scale_softmax_(half *scores, const int8_t *mask, float scale, int batch, int heads, int seq,
                                void *stream) {
    CUBERT_CHECK(cubert_mask_scale_softmax_f16(h(scores), mask, scale, batch, heads, seq, stream));
}

// Att_Q_K / Att_QK_V over every (batch, head) problem in one launch (reference: op_att/BatchMatMul.h:17-74).
// Return false when the shape has no matrix-core kernel; the caller then loops a strided-batched GEMM.
inline bool attention_scores(const float *q, const float *k, int ld, float *scores, float alpha, int batch, int heads,
                             int seq, int head_size, void *stream) {
    const int rc = cubert_attention_scores_f32(q, k, ld, scores, alpha, batch, heads, seq, head_size, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline bool attention_scores(const half *q, const half *k, int ld, half *scores, float alpha, int batch, int heads,
                             int seq, int head_size, void *stream) {
    const int rc = cubert_attention_scores_f16(h(q), h(k), ld, h(scores), alpha, batch, heads, seq, head_size, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline bool attention_context(const float *probs, const float *v, int ld, float *ctx, int ld_ctx, int batch, int heads,
                              int seq, int head_size, void *stream) {
    const int rc = cubert_attention_context_f32(probs, v, ld, ctx, ld_ctx, batch, heads, seq, head_size, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline bool attention_context(const half *probs, const half *v, int ld, half *ctx, int ld_ctx, int batch, int heads,
                              int seq, int head_size, void *stream) {
    const int rc = cubert_attention_context_f16(h(probs), h(v), ld, h(ctx), ld_ctx, batch, heads, seq, head_size, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}

// Sequence indices by falling number of live key tiles, for the long-sequence attention kernels; false when the
// shape or the mask's alignment is not taken (then pass no order).
inline bool attention_order(const int8_t *mask, int batch, int seq, int *order, void *stream) {
    const int rc = cubert_attention_order(mask, batch, seq, order, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}

// The whole attention core (scores, mask, softmax, context) in one launch (seq_length <= 512); false when
// the shape has no such kernel (reference: AttentionSelf.cpp:96-111 runs it as three operators).
inline bool attention_fused(const float *q, const float *k, const float *v, int ld, const int8_t *mask, float *ctx,
                            int ld_ctx, float alpha, int batch, int heads, int seq, int head_size, void *stream,
                            const int *order = nullptr) {
    const int rc = cubert_attention_fused_ordered_f32(q, k, v, ld, mask, order, ctx, ld_ctx, alpha, batch, heads, seq,
                                                      head_size, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}
inline bool attention_fused(const half *q, const half *k, const half *v, int ld, const int8_t *mask, half *ctx,
                            int ld_ctx, float alpha, int batch, int heads, int seq, int head_size, void *stream,
                            const int *order = nullptr) {
    const int rc = cubert_attention_fused_ordered_f16(h(q), h(k), h(v), ld, mask, order, h(ctx), ld_ctx, alpha, batch,
                                                      heads, seq, head_size, stream);
    if (rc == CUBERT_UNSUPPORTED) return false;
    CUBERT_CHECK(rc);
    return true;
}

// reference: op/Softmax.h:8-14
inline void softmax_(const float *in, float *out, int rows, int channel, void *stream) {
    CUBERT_CHECK(cubert_row_softmax_f32(in, out, rows, channel, stream));
}
inline void softmax_(const half *in, half *out, int rows, int channel, void *stream) {
    CUBERT_CHECK(cubert_row_softmax_f16(h(in), h(out), rows, channel, stream));
}

// reference: op_bert/BertPooler.h:8-11, with the pooler bias folded in
inline void tanh_(float *inout, const float *bias, int rows, int width, void *stream) {
    CUBERT_CHECK(cubert_bias_tanh_f32(inout, bias, rows, width, stream));
}
inline void tanh_(half *inout, const half *bias, int rows, int width, void *stream) {
    CUBERT_CHECK(cubert_bias_tanh_f16(h(inout), h(bias), rows, width, stream));
}

// reference: op_bert/BertPooler.h:13-16
inline void reduce_mean_1(const float *in, float *out, int batch, int seq, int hidden, void *stream) {
    CUBERT_CHECK(cubert_mean_pool_f32(in, out, batch, seq, hidden, stream));
}
inline void reduce_mean_1(const half *in, half *out, int batch, int seq, int hidden, void *stream) {
    CUBERT_CHECK(cubert_mean_pool_f16(h(in), h(out), batch, seq, hidden, stream));
}

// Host-side conversions (reference: common.h:94-106); round to nearest even.
inline void float2half(const float *fs, void *hs, size_t n) {
    half *o = static_cast<half *>(hs);
    for (size_t i = 0; i < n; ++i) o[i] = (half) fs[i];
}
inline void half2float(const void *hs, float *fs, size_t n) {
    const half *i_ = static_cast<const half *>(hs);
    for (size_t i = 0; i < n; ++i) fs[i] = (float) i_[i];
}
inline void T2T(const float *in, float *out, size_t n) { std::memcpy(out, in, n * sizeof(float)); }
inline void T2T(const half *in, half *out, size_t n) { std::memcpy(out, in, n * sizeof(half)); }
inline void T2T(const float *in, half *out, size_t n) { float2half(in, out, n); }
inline void T2T(const half *in, float *out, size_t n) { half2float(in, out, n); }

}  // namespace cuBERT

#endif  // CUBERT_HOST_COMMON_H
