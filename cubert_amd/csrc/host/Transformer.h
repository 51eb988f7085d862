// The encoder stack on one device.  Public surface of the reference's
// Transformer<T> (src/cuBERT/op_att/Transformer.h:17-39): construct from the
// named-weight map under a variable prefix, then compute(batch, input, mask)
// with device pointers, returning a device pointer to [batch, seq, hidden].
//
// Inside, a layer is 8 launches (7 for at most 32 tokens, where the two Dense kernels in front of a LayerNorm also
// leave their K slices to it instead of adding them up themselves; up to 64 tokens those two, and in half precision
// the intermediate one, still run on the few-token kernel):
//   qkv   = x * [Wq|Wk|Wv] + [bq|bk|bv]          one GEMM, bias in its epilogue
//   ctx   = softmax((1/sqrt d) Q K^T + mask) V    one attention kernel (scores stay in registers); where its
//                                                 shape limits do not hold: scores kernel or batched GEMM into
//                                                 scores[B, A, S, S], mask_scale_softmax_, context kernel or GEMM
//   a     = LN(ctx * Wo + bo + x)                 GEMM, then layer_norm_   (fused kernel)
//   i     = GELU(a * Wi + bi)                     GEMM, then gelu          (fused kernel; one launch for both at
//                                                 <= 32 tokens)
//   out   = LN(i * Wout + bout + a)               GEMM, then layer_norm_   (fused kernel)
// Activation buffers are shared by all layers (the reference keeps four private
// buffers per layer); weights live in one device allocation.  A half-precision model whose seq_length allows
// requests of at most 32 tokens also keeps its four Dense kernels in the few-token GEMM kernel's own order.
//
// CUBERT_FP32_DENSE=f16x3 in the environment when an fp32 model is opened makes its Dense layers run on the fp16
// matrix cores for requests of at least 384 tokens (measured break-even at BERT-base: below it the GEMMs are bound
// by reading the weights, and two-term weights are the larger ones): every fp32 operand is written as the sum of two fp16 numbers and the
// product as hi*hi + hi*lo + lo*hi with fp32 accumulation (one GEMM over three times the reduction length), which
// keeps the error of an fp32 GEMM for activations up to 2^12 in size (see kernels/split.hip).
// Everything between the GEMMs stays fp32.  The default is the fp32 GEMM.
#ifndef CUBERT_HOST_TRANSFORMER_H
#define CUBERT_HOST_TRANSFORMER_H

#include <cstddef>
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "Arena.h"
#include "common.h"
#include "Profiler.h"

namespace cuBERT {

template <typename T>
class Transformer {
public:
    explicit Transformer(void *cublas, const std::string &var_prefix, const std::unordered_map<std::string, T *> &var,
                         size_t max_batch_size, size_t seq_length, size_t hidden_size, size_t num_hidden_layers,
                         size_t num_attention_heads, size_t intermediate_size);

    virtual ~Transformer();

    Transformer(const Transformer &) = delete;
    Transformer &operator=(const Transformer &) = delete;

    T *compute(size_t batch_size, T *input_gpu, int8_t *attention_mask);

    // Kept for source compatibility with callers of the reference: there the
    // Dense outputs had to be pre-filled with their biases before a request;
    // here biases are applied inside the GEMM epilogue or the fused kernels.
    void _pre_compute(size_t batch_size);

    T *_in_compute(size_t batch_size, T *input_gpu, int8_t *attention_mask);

    // Optional per-kernel timing (owned by the caller; null = off).
    void set_profiler(Profiler *p) { profiler = p; }

    // Two-term fp16 Dense form only (CUBERT_FP32_DENSE=f16x3).  An activation beyond the fp16 range (|16 x| > 65504)
    // cannot be written as two fp16 terms; the kernels that write two-term rows then raise a flag instead of
    // handing a clamped operand to the GEMM in silence.  Once the stream has drained, two_term_overflowed() says
    // whether any request since the last call raised it (and clears it); the caller then runs the request again
    // after use_fp32_dense_once(), which makes the next _in_compute take the fp32 GEMMs whatever its size.
    bool two_term_overflowed();
    void use_fp32_dense_once() { fp32_dense_once = true; }

private:
    // A Dense kernel for the two-term fp16 form: rows [hi | lo | hi] of scale * W^T, [out, 3 * in]; unscale = 1 / scale
    static constexpr size_t kTwoTermMinTokens = 384;
    // activations are multiplied by this before they are taken apart (undone by the GEMM's alpha): rows whose
    // entries are of order 2^-7 .. 2^12 keep full accuracy (fp16 subnormals below, clamping above)
    static constexpr float kTwoTermActivationScale = 16.f;
    struct SplitKernel {
        half *weights = nullptr;
        float unscale = 1.f;
    };

    struct Layer {
        // Dense kernels are [in, out] as in the model file, or [out, in] when transposed_kernels is set
        T *qkv_kernel, *qkv_bias;            // [hidden, 3*hidden] (query | key | value side by side), [3*hidden]
        T *attention_output_kernel, *attention_output_bias;
        T *attention_norm_beta, *attention_norm_gamma;
        T *intermediate_kernel, *intermediate_bias;
        T *output_kernel, *output_bias;
        T *output_norm_beta, *output_norm_gamma;
        // the Dense kernels again, in the few-token GEMM kernel's order (null when not kept)
        T *qkv_packed = nullptr, *attention_output_packed = nullptr, *intermediate_packed = nullptr,
          *output_packed = nullptr;
        SplitKernel qkv_split, attention_output_split, intermediate_split, output_split;  // (null when not kept)
    };

    void layout_weights();
    void layout_buffers();
    // The [max_batch, heads, seq, seq] score tensor.  Only the three-kernel attention path touches it, and the
    // one-launch kernel takes every BERT shape up to seq_length 512, so it is not part of `buffers` (it would be the
    // largest of them: 403 MB at batch 64 x 12 heads x seq 512 in fp16) but allocated on first use.
    T *scores();
    // context_out = attention(qkv); with `split_context` (fp32 models in the two-term Dense form) the one-launch
    // kernel writes the context there as two-term rows instead and true is returned
    bool attention(size_t batch_size, const T *qkv, const int8_t *mask, half *split_context = nullptr);
    // out[tokens, out_features] = in[tokens, in_features] * kernel (+ bias) (, GELU); returns whether bias and
    // activation were applied (false: the caller's fused kernel still has to).
    bool dense(int out_features, int tokens, int in_features, const T *kernel, const T *packed, const T *in, T *out,
               const T *bias, bool bias_in_gemm, bool gelu, Profiler::Kind kind, int ld_out = 0);
    // The same on the fp16 matrix cores from two-term operands (fp32 models only): `in` is split into
    // split_operand first, or, when null, split_operand already holds the [hi | hi | lo] rows.  `bias` may be null.
    void dense_split(int out_features, int tokens, int in_features, const SplitKernel &kernel, const T *in, T *out,
                     const T *bias, Profiler::Kind kind, int ld_out = 0);
    // out = LayerNorm(in * kernel + bias + residual): dense(), then layer_norm_; for at most 32 tokens the few-token
    // GEMM leaves its K slices in few_token_partials and the LayerNorm kernel adds them while it loads (same values,
    // without the GEMM's 2 us hand-over between workgroups).
    void dense_norm(int tokens, int in_features, const T *kernel, const T *packed, const T *in, const T *bias,
                    const T *residual, const T *beta, const T *gamma, T *out, Profiler::Kind kind);

    // up to how many tokens the Dense layer of this kind runs on the few-token kernel (32 or 64)
    int few_token_limit(Profiler::Kind kind) const;

    void *cublas;
    Profiler *profiler = nullptr;
    bool slices_to_norm = true;        // few-token Dense layers hand their K slices to the LayerNorm (cleared when declined)
    bool dense_gelu_fits = true;       // cleared when the few-token Dense + GELU kernel declines this model's shape
    bool keep_packed = false;          // Dense kernels are also kept in the few-token kernel's order
    bool transposed_kernels = false;   // Dense kernels are stored [out, in] instead of [in, out] (half precision)
    bool split_dense = false;          // fp32 model with Dense layers in the two-term fp16 form (opt-in)
    bool fp32_dense_once = false;      // the next request takes the fp32 GEMMs (set after a two-term overflow)
    int *split_overflow = nullptr;     // page-locked host word the two-term kernels set to 1 on overflow (split_dense)
    bool norm_writes_operand = true;   // cleared when the LayerNorm that also writes two-term rows declines the hidden size
    bool fused_attention_fits = true;  // cleared when the one-launch attention kernel declines this model's shape
    size_t max_batch_size, seq_length, hidden_size, num_hidden_layers, num_attention_heads, intermediate_size;

    Arena weights;
    Arena buffers;
    Arena score_memory;  // the score tensor of the three-kernel attention path: claimed when a request first takes it
    std::vector<Layer> layers;

    size_t qkv_ld = 0;       // elements from one token's Q | K | V row to the next (>= 3*hidden)
    T *qkv_out;              // [M, qkv_ld]
    T *attention_scores = nullptr;  // [B, heads, seq, seq], in score_memory (null until scores() is first called)
    T *context_out;          // [M, hidden]
    int *attention_order = nullptr;  // [8 * max_batch]: sequence indices, most live key tiles first, and their tile lists (seq_length > 128)
    bool order_ready = false;        // attention_order holds the current request's order
    T *attention_output;     // [M, hidden]
    T *intermediate_output;  // [M, intermediate]
    T *layer_output[2];      // [M, hidden], alternating between layers
    half *split_operand = nullptr;  // [M, 3 * max(hidden, intermediate)] two-term rows of the current Dense input
    static constexpr size_t kFewTokenPartialFloats = (size_t) 1 << 20;
    float *few_token_partials = nullptr;  // K slices of the current few-token Dense layer (seq_length <= 64 only)
};

}  // namespace cuBERT

#endif  // CUBERT_HOST_TRANSFORMER_H
