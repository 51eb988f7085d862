#include "Transformer.h"

#include <cmath>
#include <cstdlib>
#include <string>
#include <stdexcept>

namespace cuBERT {

namespace {
template <typename T>
void upload(T *dst, const T *src, size_t count) {
    if (dst != nullptr) cuBERT::memcpy(dst, src, count * sizeof(T), 1);
}

// device memory for the duration of a scope (a missing weight name throws out of the constructor)
struct ScopedDeviceBuffer {
    void *ptr = nullptr;
    explicit ScopedDeviceBuffer(size_t bytes) : ptr(bytes ? cuBERT::malloc(bytes) : nullptr) {}
    ScopedDeviceBuffer(const ScopedDeviceBuffer &) = delete;
    ScopedDeviceBuffer &operator=(const ScopedDeviceBuffer &) = delete;
    ~ScopedDeviceBuffer() {
        if (ptr != nullptr) cubert_free(ptr);
    }
};
}  // namespace

template <typename T>
Transformer<T>::Transformer(void *cublas, const std::string &var_prefix,
                            const std::unordered_map<std::string, T *> &var, size_t max_batch_size,
                            size_t seq_length, size_t hidden_size, size_t num_hidden_layers,
                            size_t num_attention_heads, size_t intermediate_size)
        : cublas(cublas), max_batch_size(max_batch_size), seq_length(seq_length), hidden_size(hidden_size),
          num_hidden_layers(num_hidden_layers), num_attention_heads(num_attention_heads),
          intermediate_size(intermediate_size), layers(num_hidden_layers) {
    if (num_attention_heads == 0 || hidden_size % num_attention_heads != 0) {
        throw std::invalid_argument("hidden_size must be a multiple of num_attention_heads");
    }
    const size_t H = hidden_size, I = intermediate_size;
    // The re-ordered copies pay off for 2-byte weights (the plain layout makes the few-token kernel read 64-byte
    // pieces): measured 2 us per GEMM at hidden 768; for 4-byte weights the gain is within 5 %, not worth the memory.
    keep_packed = sizeof(T) == 2 && seq_length <= 64 && H % 16 == 0 && I % 16 == 0;
    // The library's fp16 GEMMs are 10-19 % faster with both operands contiguous along the reduction (measured at
    // 32768 tokens on every Dense shape of BERT-base and BERT-large, same bits out); its fp32 GEMMs do not care.
    // Half-precision models therefore keep their Dense kernels [out, in], transposed once here.
    transposed_kernels = sizeof(T) == 2;
    const char *dense_mode = std::getenv("CUBERT_FP32_DENSE");
    if (dense_mode != nullptr && std::string(dense_mode) != "f16x3" && std::string(dense_mode) != "f32" &&
        std::string(dense_mode) != "") {
        fprintf(stderr, "cuBERT: CUBERT_FP32_DENSE=%s is not understood (f32 or f16x3); using f32\n", dense_mode);
    }
    split_dense = sizeof(T) == 4 && dense_mode != nullptr && std::string(dense_mode) == "f16x3" &&
                  max_batch_size * seq_length >= kTwoTermMinTokens;

    if (split_dense) {
        split_overflow = static_cast<int *>(cubert_malloc_host(64));
        if (split_overflow == nullptr) throw std::runtime_error("no page-locked host memory for the two-term overflow flag");
        *split_overflow = 0;
    }

    // Weight names as the reference resolves them (Transformer.cpp:54-101, AttentionSelf.cpp:27-44);
    // a missing name throws std::out_of_range from unordered_map::at, as it does there.
    layout_weights();
    weights.allocate();
    layout_weights();

    void *stream = cuBERT::blas_get_stream(cublas);
    const size_t largest = H * (3 * H > I ? 3 * H : I);
    ScopedDeviceBuffer staging_memory(transposed_kernels || split_dense ? largest * sizeof(T) : 0);
    T *staging = static_cast<T *>(staging_memory.ptr);
    // one Dense kernel, [in, out] on the host, into its place on the device (and its few-token copy)
    auto load_kernel = [&](T *dst, T *few_token_copy, SplitKernel &split, const T *host, size_t in, size_t out) {
        T *plain = transposed_kernels ? staging : dst;
        upload(plain, host, in * out);
        if (keep_packed) cuBERT::pack_few_token_weights(cublas, plain, (int) out, (int) out, (int) in, few_token_copy);
        if (transposed_kernels) {
            cuBERT::transpose(plain, (int) in, (int) out, dst, stream);
            cuBERT::cuda_stream_synchronize(stream);  // the staging buffer is written again by the next upload
        }
        if constexpr (sizeof(T) == 4) {
            if (split_dense) {
                // a power of two that brings the largest weight to [512, 1024): far from fp16's subnormals and its limit
                float largest_weight = 0.f;
                for (size_t i = 0; i < in * out; ++i) largest_weight = std::fmax(largest_weight, std::fabs(host[i]));
                int exponent = 0;
                if (largest_weight > 0.f && std::isfinite(largest_weight)) {
                    (void) std::frexp(largest_weight, &exponent);  // largest = f * 2^exponent, f in [0.5, 1)
                    exponent = 10 - exponent;
                }
                split.unscale = std::ldexp(1.f, -exponent);
                cuBERT::transpose(dst, (int) in, (int) out, staging, stream);
                // (weights are scaled into [512, 1024): no overflow flag needed on this side)
                cuBERT::split3(staging, (int) out, (int) in, std::ldexp(1.f, exponent), true, split.weights, nullptr,
                               stream);
                cuBERT::cuda_stream_synchronize(stream);
            }
        }
    };

    std::vector<T> packed(H * 3 * H), packed_bias(3 * H);
    for (size_t l = 0; l < num_hidden_layers; ++l) {
        const std::string p = var_prefix + "/layer_" + std::to_string(l);
        const T *q = var.at(p + "/attention/self/query/kernel"), *qb = var.at(p + "/attention/self/query/bias");
        const T *k = var.at(p + "/attention/self/key/kernel"), *kb = var.at(p + "/attention/self/key/bias");
        const T *v = var.at(p + "/attention/self/value/kernel"), *vb = var.at(p + "/attention/self/value/bias");
        // [in, out] row-major kernels side by side: row i = [Wq[i,:] | Wk[i,:] | Wv[i,:]]
        for (size_t i = 0; i < H; ++i) {
            std::memcpy(&packed[i * 3 * H], q + i * H, H * sizeof(T));
            std::memcpy(&packed[i * 3 * H + H], k + i * H, H * sizeof(T));
            std::memcpy(&packed[i * 3 * H + 2 * H], v + i * H, H * sizeof(T));
        }
        std::memcpy(&packed_bias[0], qb, H * sizeof(T));
        std::memcpy(&packed_bias[H], kb, H * sizeof(T));
        std::memcpy(&packed_bias[2 * H], vb, H * sizeof(T));
        Layer &w = layers[l];
        load_kernel(w.qkv_kernel, w.qkv_packed, w.qkv_split, packed.data(), H, 3 * H);
        upload(w.qkv_bias, packed_bias.data(), 3 * H);
        load_kernel(w.attention_output_kernel, w.attention_output_packed, w.attention_output_split,
                    var.at(p + "/attention/output/dense/kernel"), H, H);
        upload(w.attention_output_bias, var.at(p + "/attention/output/dense/bias"), H);
        upload(w.attention_norm_beta, var.at(p + "/attention/output/LayerNorm/beta"), H);
        upload(w.attention_norm_gamma, var.at(p + "/attention/output/LayerNorm/gamma"), H);
        load_kernel(w.intermediate_kernel, w.intermediate_packed, w.intermediate_split,
                    var.at(p + "/intermediate/dense/kernel"), H, I);
        upload(w.intermediate_bias, var.at(p + "/intermediate/dense/bias"), I);
        load_kernel(w.output_kernel, w.output_packed, w.output_split, var.at(p + "/output/dense/kernel"), I, H);
        upload(w.output_bias, var.at(p + "/output/dense/bias"), H);
        upload(w.output_norm_beta, var.at(p + "/output/LayerNorm/beta"), H);
        upload(w.output_norm_gamma, var.at(p + "/output/LayerNorm/gamma"), H);
    }
    cuBERT::cuda_stream_synchronize(stream);  // nothing reads the staging buffer after this

    layout_buffers();
    buffers.allocate();
    layout_buffers();
}

template <typename T>
Transformer<T>::~Transformer() {
    cubert_free_host(split_overflow);  // null is accepted
}

template <typename T>
bool Transformer<T>::two_term_overflowed() {
    if (split_overflow == nullptr || *static_cast<volatile int *>(split_overflow) == 0) return false;
    *split_overflow = 0;
    return true;
}

template <typename T>
void Transformer<T>::layout_weights() {
    const size_t H = hidden_size, I = intermediate_size;
    for (Layer &w : layers) {
        w.qkv_kernel = weights.take<T>(H * 3 * H);
        w.qkv_bias = weights.take<T>(3 * H);
        w.attention_output_kernel = weights.take<T>(H * H);
        w.attention_output_bias = weights.take<T>(H);
        w.attention_norm_beta = weights.take<T>(H);
        w.attention_norm_gamma = weights.take<T>(H);
        w.intermediate_kernel = weights.take<T>(H * I);
        w.intermediate_bias = weights.take<T>(I);
        w.output_kernel = weights.take<T>(I * H);
        w.output_bias = weights.take<T>(H);
        w.output_norm_beta = weights.take<T>(H);
        w.output_norm_gamma = weights.take<T>(H);
        if (keep_packed) {
            w.qkv_packed = weights.take<T>(cubert_gemm_skinny_packed_elements(3 * (int) H, (int) H));
            w.attention_output_packed = weights.take<T>(cubert_gemm_skinny_packed_elements((int) H, (int) H));
            w.intermediate_packed = weights.take<T>(cubert_gemm_skinny_packed_elements((int) I, (int) H));
            w.output_packed = weights.take<T>(cubert_gemm_skinny_packed_elements((int) H, (int) I));
        }
        if (split_dense) {
            w.qkv_split.weights = weights.take<half>(3 * H * 3 * H);
            w.attention_output_split.weights = weights.take<half>(3 * H * H);
            w.intermediate_split.weights = weights.take<half>(3 * H * I);
            w.output_split.weights = weights.take<half>(3 * I * H);
        }
    }
}

template <typename T>
void Transformer<T>::layout_buffers() {
    const size_t M = max_batch_size * seq_length, H = hidden_size;
    // 64 elements between one token's Q | K | V row and the next: the attention kernels read 128-byte pieces of these
    // rows at the row pitch, and a pitch of 3 * hidden elements (6 KB for BERT-large in fp16) spreads those pieces
    // badly over the memory channels.  Measured at 256 sequences x 16 heads x 128 keys, fp16, with and without the
    // padding in alternation on one box: attention kernel 57.4 -> 51.3 us, forward pass 20.34 -> 20.24 ms; BERT-base
    // shapes (pitch 4.5 KB fp16, 9 KB fp32) move by less than the run-to-run noise.
    qkv_ld = 3 * H + 64;
    qkv_out = buffers.take<T>(M * qkv_ld);
    context_out = buffers.take<T>(M * H);
    attention_order = buffers.take<int>(8 * max_batch_size);  // indices, then a record of live tiles per position
    attention_output = buffers.take<T>(M * H);
    intermediate_output = buffers.take<T>(M * intermediate_size);
    layer_output[0] = buffers.take<T>(M * H);
    layer_output[1] = buffers.take<T>(M * H);
    if (split_dense) split_operand = buffers.take<half>(M * 3 * (H > intermediate_size ? H : intermediate_size));
    if (seq_length <= 64) few_token_partials = buffers.take<float>(kFewTokenPartialFloats);
}

template <typename T>
T *Transformer<T>::scores() {
    if (attention_scores == nullptr) {
        const size_t count = max_batch_size * num_attention_heads * seq_length * seq_length;
        score_memory.take<T>(count);
        score_memory.allocate();
        attention_scores = score_memory.take<T>(count);
    }
    return attention_scores;
}

template <typename T>
T *Transformer<T>::compute(size_t batch_size, T *input_gpu, int8_t *attention_mask) {
    _pre_compute(batch_size);
    return _in_compute(batch_size, input_gpu, attention_mask);
}

template <typename T>
void Transformer<T>::_pre_compute(size_t) {}

// scores[b, a, q, k] = (1/sqrt d) * sum_j Q[b, q, a, j] K[b, k, a, j];  softmax with mask;
// ctx[b, q, a, :] = sum_k p[b, a, q, k] V[b, k, a, :].   Q, K, V are column blocks of qkv[M, 3H].
// The contractions run as one matrix-core launch each where the shape allows.  Otherwise: the (b, a)
// problems have two strides (b: seq*3H, a: d), a strided-batched GEMM has one, so the shorter of the two
// axes is looped on the host and the longer one is the GEMM batch.
template <typename T>
bool Transformer<T>::attention(size_t batch_size, const T *qkv, const int8_t *mask, half *split_context) {
    void *stream = cuBERT::blas_get_stream(cublas);
    const int S = (int) seq_length, A = (int) num_attention_heads, H = (int) hidden_size, d = H / A;
    const int B = (int) batch_size, ld = (int) qkv_ld;
    const float alpha = (float) (1.0 / std::sqrt((double) d));
    const T *Q = qkv, *K = qkv + H, *V = qkv + 2 * H;
    const long long seq_stride = (long long) S * ld, head_stride = d;
    const long long score_b = (long long) A * S * S, score_a = (long long) S * S;

    // One launch with the score tensor held in registers where the shape allows (seq_length <= 512, K and V
    // of a head within LDS).  CUBERT_ATTENTION=split in the
    // environment keeps the three-operator path below (scores, mask + softmax, context) for every shape.
    static const bool split_only = [] {
        const char *e = std::getenv("CUBERT_ATTENTION");
        return e != nullptr && std::string(e) == "split";
    }();
    if (!split_only && fused_attention_fits) {
        Timed t(profiler, Profiler::kAttentionFused, stream);
        if constexpr (sizeof(T) == 4) {
            if (split_context != nullptr &&
                cuBERT::attention_fused_split3(Q, K, V, ld, mask, kTwoTermActivationScale, split_context, alpha, B, A, S,
                                               d, split_overflow, stream)) {
                return true;
            }
        }
        if (cuBERT::attention_fused(Q, K, V, ld, mask, context_out, H, alpha, B, A, S, d, stream,
                                    order_ready ? attention_order : nullptr)) {
            return false;
        }
        fused_attention_fits = false;  // seq_length and head size are fixed per model: do not ask again
        t.cancel();
    }

    T *score_tensor = scores();
    const bool loop_heads = A <= B;
    const int outer = loop_heads ? A : B, inner = loop_heads ? B : A;
    const long long in_outer = loop_heads ? head_stride : seq_stride, in_inner = loop_heads ? seq_stride : head_stride;
    const long long sc_outer = loop_heads ? score_a : score_b, sc_inner = loop_heads ? score_b : score_a;
    const long long ctx_outer = loop_heads ? (long long) d : (long long) S * H;
    const long long ctx_inner = loop_heads ? (long long) S * H : (long long) d;

    {
        Timed t(profiler, Profiler::kAttentionGemm, stream);
        if (!cuBERT::attention_scores(Q, K, ld, score_tensor, alpha, B, A, S, d, stream)) {
            for (int o = 0; o < outer; ++o) {
                // column-major: scores_ba (S_k x S_q, ld S) = K_ba^T (d x S_k, ld 3H)^T * Q_ba (d x S_q, ld 3H)
                cuBERT::blas_gemm_strided_batch(cublas, true, false, S, S, d, alpha, K + o * in_outer, ld, in_inner,
                                                Q + o * in_outer, ld, in_inner, 0.f, score_tensor + o * sc_outer,
                                                S, sc_inner, inner);
            }
        }
    }
    {
        Timed t(profiler, Profiler::kMaskScaleSoftmax, stream);
        cuBERT::mask_scale_softmax_(score_tensor, mask, 1.0f, B, A, S, stream);
    }
    Timed t(profiler, Profiler::kAttentionGemm, stream);
    if (!cuBERT::attention_context(score_tensor, V, ld, context_out, H, B, A, S, d, stream)) {
        for (int o = 0; o < outer; ++o) {
            // column-major: ctx_ba (d x S_q, ld H) = V_ba (d x S_k, ld 3H) * p_ba (S_k x S_q, ld S)
            cuBERT::blas_gemm_strided_batch(cublas, false, false, d, S, S, 1.f, V + o * in_outer, ld, in_inner,
                                            score_tensor + o * sc_outer, S, sc_inner, 0.f,
                                            context_out + o * ctx_outer, H, ctx_inner, inner);
        }
    }
    return false;
}

// One Dense layer.  The bias goes into the GEMM only where the caller asks for it (bias_in_gemm: the Q/K/V
// projection, whose consumer has no fused bias) or where the few-token kernel applies it together with the GELU;
// otherwise it is left to the fused kernel that follows (which then reads the GEMM output once anyway).
template <typename T>
bool Transformer<T>::dense(int out_features, int tokens, int in_features, const T *kernel, const T *packed, const T *in,
                           T *out, const T *bias, bool bias_in_gemm, bool gelu, Profiler::Kind kind, int ld_out) {
    void *stream = cuBERT::blas_get_stream(cublas);
    Timed t(profiler, profiler != nullptr ? profiler->dense_kind(kind) : Profiler::kDenseGemm, stream);
    if (ld_out == 0) ld_out = out_features;
    // (the few-token kernel reads [in, out] kernels or its own copy of them, not transposed ones)
    if (tokens <= few_token_limit(kind) && (packed != nullptr || (!transposed_kernels && (gelu || tokens > 32) && dense_gelu_fits))) {
        const bool with_bias = bias_in_gemm || gelu;
        if (cuBERT::dense_few_tokens(cublas, out_features, tokens, in_features, kernel, out_features, packed, in,
                                     in_features, out, ld_out, with_bias ? bias : nullptr, gelu)) {
            return with_bias;
        }
        if (gelu) dense_gelu_fits = false;  // the layer sizes are fixed per model: do not ask again
    }
    cuBERT::blas_gemm(cublas, transposed_kernels, false, out_features, tokens, in_features, 1.f, kernel,
                      transposed_kernels ? in_features : out_features, in, in_features, 0.f, out, ld_out,
                      bias_in_gemm ? bias : nullptr);
    return bias_in_gemm;
}

template <typename T>
void Transformer<T>::dense_split(int out_features, int tokens, int in_features, const SplitKernel &kernel, const T *in,
                                 T *out, const T *bias, Profiler::Kind kind, int ld_out) {
    if (ld_out == 0) ld_out = out_features;
    if constexpr (sizeof(T) == 4) {
        void *stream = cuBERT::blas_get_stream(cublas);
        if (in != nullptr) {
            Timed t(profiler, Profiler::kDenseSplit, stream);
            cuBERT::split3(in, tokens, in_features, kTwoTermActivationScale, false, split_operand, split_overflow,
                           stream);
        }
        Timed t(profiler, profiler != nullptr ? profiler->dense_kind(kind) : Profiler::kDenseGemm, stream);
        cuBERT::blas_gemm_f16_f32(cublas, true, false, out_features, tokens, 3 * in_features,
                                  kernel.unscale / kTwoTermActivationScale,
                                  kernel.weights, 3 * in_features, split_operand, 3 * in_features, 0.f, out,
                                  ld_out, bias);
    } else {
        throw std::logic_error("the two-term fp16 Dense form is for fp32 models");
    }
}

// Up to how many tokens a Dense layer runs on the few-token kernel.  32 for all of them; 64 where the kernel with two
// blocks of 32 tokens per wavefront is ahead of the library.  Measured at BERT-base, batch 2 x seq 32, a launch
// event-timed inside the forward pass, library against kernel -- fp32: attention output 9.1 / 7.6 us, output
// 20.4 / 15.1 us, but Q|K|V 11.7 / 12.5 and intermediate + GELU 16.4 / 18.7 (the fp32 MFMAs of a second token block
// cost what the library's tiles do not); fp16: attention output 8.6 / 6.5, intermediate + GELU 14.6 / 10.7, output
// 10.4 / 7.7, Q|K|V 8.5 / 10.1.  Forward pass 0.665 -> 0.61 ms (fp32), 0.541 -> 0.423 ms (fp16).
template <typename T>
int Transformer<T>::few_token_limit(Profiler::Kind kind) const {
    switch (kind) {
        case Profiler::kDenseAttentionOutput:
        case Profiler::kDenseOutput: return 64;
        case Profiler::kDenseIntermediate: return sizeof(T) == 2 ? 64 : 32;
        default: return 32;
    }
}

// CUBERT_FEW_TOKEN_SLICES=0 in the environment keeps the few-token Dense kernels adding their own K slices.
static bool few_token_slices_enabled() {
    static const bool on = [] {
        const char *e = std::getenv("CUBERT_FEW_TOKEN_SLICES");
        return e == nullptr || std::string(e) != "0";
    }();
    return on;
}

template <typename T>
void Transformer<T>::dense_norm(int tokens, int in_features, const T *kernel, const T *packed, const T *in, const T *bias,
                                const T *residual, const T *beta, const T *gamma, T *out, Profiler::Kind kind) {
    void *stream = cuBERT::blas_get_stream(cublas);
    const int H = (int) hidden_size;
    if (tokens <= few_token_limit(kind) && slices_to_norm && few_token_partials != nullptr && few_token_slices_enabled() &&
        (packed != nullptr || !transposed_kernels)) {
        int slices = 0, pitch = 0;
        bool done = false;
        {
            Timed t(profiler, profiler != nullptr ? profiler->dense_kind(kind) : Profiler::kDenseGemm, stream);
            done = cuBERT::dense_few_tokens_partials(cublas, H, tokens, in_features, kernel, H, packed, in, in_features,
                                                     few_token_partials, kFewTokenPartialFloats, &slices, &pitch);
            if (!done) t.cancel();
        }
        if (done) {
            Timed t(profiler, Profiler::kBiasResLayerNorm, stream);
            if (cuBERT::layer_norm_partials(out, few_token_partials, slices, pitch, residual, bias, beta, gamma, tokens, H,
                                            stream)) {
                return;
            }
            t.cancel();
        }
        slices_to_norm = false;  // the layer sizes are fixed per model: do not ask again
    }
    const bool bias_done = dense(H, tokens, in_features, kernel, packed, in, out, bias, false, false, kind);
    Timed t(profiler, Profiler::kBiasResLayerNorm, stream);
    cuBERT::layer_norm_(residual, out, tokens, H, bias_done ? nullptr : bias, beta, gamma, stream);
}

template <typename T>
T *Transformer<T>::_in_compute(size_t batch_size, T *input_gpu, int8_t *attention_mask) {
    if (batch_size > max_batch_size) throw std::invalid_argument("batch_size > max_batch_size");
    void *stream = cuBERT::blas_get_stream(cublas);
    const int M = (int) (batch_size * seq_length), H = (int) hidden_size, I = (int) intermediate_size;

    // (small requests are bound by the pass over the weights, which are 6 bytes per parameter in two-term form and 4
    // in fp32: they keep the fp32 kernels)
    const bool split = split_dense && (size_t) M >= kTwoTermMinTokens && !fp32_dense_once;
    fp32_dense_once = false;
    bool operand_ready = false;

    // long sequences: the attention kernels take the sequences longest first (the mask is the same for every layer)
    order_ready = seq_length > 128 && attention_mask != nullptr && fused_attention_fits &&
                  cuBERT::attention_order(attention_mask, (int) batch_size, (int) seq_length, attention_order, stream);

    T *prev_output = input_gpu;
    for (size_t l = 0; l < num_hidden_layers; ++l) {
        const Layer &w = layers[l];
        T *layer_input = prev_output;
        T *out = layer_output[l & 1];

        if (split) {
            if constexpr (sizeof(T) == 4) {
                // split_operand holds the two-term rows of the next Dense input whenever the kernel before it could
                // write them itself (LayerNorm, GELU); otherwise dense_split makes them from the fp32 rows
                dense_split(3 * H, M, H, w.qkv_split, operand_ready ? nullptr : layer_input, qkv_out, w.qkv_bias,
                            Profiler::kDenseQkv, (int) qkv_ld);
                const bool context_ready = attention(batch_size, qkv_out, attention_mask, split_operand);
                dense_split(H, M, H, w.attention_output_split, context_ready ? nullptr : context_out, attention_output,
                            nullptr, Profiler::kDenseAttentionOutput);
                {
                    Timed t(profiler, Profiler::kBiasResLayerNorm, stream);
                    operand_ready = norm_writes_operand &&
                                    cuBERT::layer_norm_split3(layer_input, attention_output, M, H, w.attention_output_bias,
                                                              w.attention_norm_beta, w.attention_norm_gamma,
                                                              kTwoTermActivationScale, split_operand, split_overflow,
                                                              stream);
                    if (!operand_ready) {
                        norm_writes_operand = false;  // the hidden size is fixed per model: do not ask again
                        cuBERT::layer_norm_(layer_input, attention_output, M, H, w.attention_output_bias,
                                            w.attention_norm_beta, w.attention_norm_gamma, stream);
                    }
                }
                dense_split(I, M, H, w.intermediate_split, operand_ready ? nullptr : attention_output,
                            intermediate_output, nullptr, Profiler::kDenseIntermediate);
                {
                    // bias + GELU straight into the two-term rows the output Dense reads
                    Timed t(profiler, Profiler::kBiasGelu, stream);
                    cuBERT::bias_gelu_split3(intermediate_output, w.intermediate_bias, M, I, kTwoTermActivationScale,
                                             split_operand, split_overflow, stream);
                }
                dense_split(H, M, I, w.output_split, nullptr, out, nullptr, Profiler::kDenseOutput);
                {
                    Timed t(profiler, Profiler::kBiasResLayerNorm, stream);
                    operand_ready = norm_writes_operand &&
                                    cuBERT::layer_norm_split3(attention_output, out, M, H, w.output_bias,
                                                              w.output_norm_beta, w.output_norm_gamma,
                                                              kTwoTermActivationScale, split_operand, split_overflow,
                                                              stream);
                    if (!operand_ready) {
                        norm_writes_operand = false;
                        cuBERT::layer_norm_(attention_output, out, M, H, w.output_bias, w.output_norm_beta,
                                            w.output_norm_gamma, stream);
                    }
                }
            }
            prev_output = out;
            continue;
        }

        // attention/self: row-major Y[M, N] = X[M, K] W[K, N] is the column-major gemm(N, M, K) on (W, X)
        dense(3 * H, M, H, w.qkv_kernel, w.qkv_packed, layer_input, qkv_out, w.qkv_bias, true, false, Profiler::kDenseQkv,
              (int) qkv_ld);
        attention(batch_size, qkv_out, attention_mask);

        // attention/output: dense, then bias + residual(layer input) + LayerNorm
        dense_norm(M, H, w.attention_output_kernel, w.attention_output_packed, context_out, w.attention_output_bias,
                   layer_input, w.attention_norm_beta, w.attention_norm_gamma, attention_output,
                   Profiler::kDenseAttentionOutput);

        // intermediate: dense, then bias + GELU (one launch for all three at <= 32 tokens)
        if (!dense(I, M, H, w.intermediate_kernel, w.intermediate_packed, attention_output, intermediate_output,
                   w.intermediate_bias, false, true, Profiler::kDenseIntermediate)) {
            Timed t(profiler, Profiler::kBiasGelu, stream);
            cuBERT::gelu(intermediate_output, w.intermediate_bias, M, I, stream);
        }

        // output: dense, then bias + residual(attention output) + LayerNorm
        dense_norm(M, I, w.output_kernel, w.output_packed, intermediate_output, w.output_bias, attention_output,
                   w.output_norm_beta, w.output_norm_gamma, out, Profiler::kDenseOutput);

        prev_output = out;
    }
    return prev_output;
}

template class Transformer<float>;
template class Transformer<half>;

}  // namespace cuBERT
