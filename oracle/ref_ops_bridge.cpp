/*
 * C entry points onto the reference's own CPU launchers (TEST INFRASTRUCTURE ONLY).
 *
 * Compiled together with the reference's op translation units, taken where
 * they lie under /root/reference/src (never copied): op/{Embedding,LayerNorm,
 * Softmax,GELU}.cpp, op_att/AttentionMask.cpp, op_bert/BertPooler.cpp, with
 * -DHAVE_MKL so their OpenMP/CPU specialisations are the ones built.  Only the
 * free launcher templates are reachable from here; the reference's classes in
 * the same files (which need its MKL-backed runtime) are dropped at link time
 * by --gc-sections, so the library has no unresolved runtime symbols.
 */
#include <cstddef>
#include <cstdint>

#include "cuBERT/op/Embedding.h"
#include "cuBERT/op/GELU.h"
#include "cuBERT/op/LayerNorm.h"
#include "cuBERT/op/Softmax.h"
#include "cuBERT/op_att/AttentionMask.h"
#include "cuBERT/op_bert/BertPooler.h"

#define REF_API extern "C" __attribute__((visibility("default")))

REF_API void ref_embedding(const int32_t *ids, int n, const float *table, int width, float *out) {
    cuBERT::embedding<int, float>(ids, n, table, width, out, nullptr);
}

REF_API void ref_embedding_i8(const int8_t *ids, int n, const float *table, int width, float *out) {
    cuBERT::embedding<int8_t, float>(ids, n, table, width, out, nullptr);
}

REF_API void ref_layer_norm_(const float *in, float *inout, int rows, int channels,
                             const float *beta, const float *gamma) {
    cuBERT::layer_norm_<float>(in, inout, rows, channels, nullptr, nullptr, beta, gamma, nullptr);
}

REF_API void ref_softmax_(float *in, float *out, int rows, int channel) {
    cuBERT::softmax_<float>(in, out, rows, channel, nullptr, nullptr);
}

REF_API void ref_gelu(size_t n, float *inout) { cuBERT::gelu<float>(n, inout, nullptr); }

REF_API void ref_not(const int8_t *in, float *out, int n) { cuBERT::_not<float>(in, out, n, nullptr); }

REF_API void ref_tanh_(float *inout, int n) { cuBERT::tanh_<float>(inout, n, nullptr); }

REF_API void ref_reduce_mean_1(const float *in, float *out, int batch, int seq_length, int hidden) {
    cuBERT::reduce_mean_1<float>(in, out, batch, seq_length, hidden, nullptr);
}
