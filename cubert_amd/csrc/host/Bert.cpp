#include "Bert.h"

#include <cstdlib>
#include <cstring>
#include <iostream>
#include <stdexcept>
#include <string>
#include <vector>

namespace cuBERT {

namespace {
inline size_t round_up_16(size_t n) { return (n + 15) & ~size_t(15); }
// bytes of the input block for M tokens: int ids, then int8 mask, then int8 segment ids, each 16-byte aligned
inline size_t input_block_bytes(size_t M) { return round_up_16(round_up_16(sizeof(int) * M) + M) + M; }
}  // namespace

// Every id indexes a row of an embedding table on the device, where nothing checks it (nor does the reference,
// src/cuBERT/op/Embedding.cpp:16-19): ids are checked here, on the host, before anything is enqueued.
void check_input_range(const int *input_ids, const int8_t *segment_ids, size_t count, size_t vocab_size,
                       size_t type_vocab_size) {
    unsigned bad_id = 0, bad_segment = 0;
    const unsigned vocab = vocab_size > 0x7fffffffu ? 0x80000000u : (unsigned) vocab_size;
    const unsigned types = type_vocab_size > 127 ? 128u : (unsigned) type_vocab_size;
    for (size_t i = 0; i < count; ++i) bad_id |= (unsigned) input_ids[i] >= vocab;  // a negative id wraps to a large one
    for (size_t i = 0; i < count; ++i) bad_segment |= (unsigned) (uint8_t) segment_ids[i] >= types;
    if (!bad_id && !bad_segment) return;
    for (size_t i = 0; i < count; ++i) {
        if ((unsigned) input_ids[i] >= vocab) {
            throw std::invalid_argument("input id out of range: input_ids[" + std::to_string(i) + "] = " +
                                        std::to_string(input_ids[i]) + ", vocab_size = " + std::to_string(vocab_size));
        }
    }
    for (size_t i = 0; i < count; ++i) {
        if ((unsigned) (uint8_t) segment_ids[i] >= types) {
            throw std::invalid_argument("segment id out of range: segment_ids[" + std::to_string(i) + "] = " +
                                        std::to_string((int) segment_ids[i]) + ", type_vocab_size = " +
                                        std::to_string(type_vocab_size));
        }
    }
}

// Batch sizes to prepare when a model is opened, from CUBERT_OPEN_WARMUP: unset = the maximum batch only (what the
// reference prepares, src/cuBERT/Bert.cpp:62-64); "0" = none; otherwise a comma-separated list of batch sizes, in
// which "max" stands for max_batch_size ("1,8,max").  Entries that are not a size in [1, max_batch_size] are named
// on stderr and skipped.
std::vector<size_t> open_warmup_batches(const char *setting, size_t max_batch_size) {
    std::vector<size_t> batches;
    if (setting == nullptr) {
        batches.push_back(max_batch_size);
        return batches;
    }
    const std::string text(setting);
    if (text == "0") return batches;
    size_t at = 0;
    while (at <= text.size()) {
        size_t end = text.find(',', at);
        if (end == std::string::npos) end = text.size();
        std::string item = text.substr(at, end - at);
        at = end + 1;
        while (!item.empty() && (item.back() == ' ' || item.back() == '\t')) item.pop_back();
        while (!item.empty() && (item.front() == ' ' || item.front() == '\t')) item.erase(item.begin());
        if (item.empty()) continue;
        size_t batch = 0;
        bool ok = true;
        if (item == "max") {
            batch = max_batch_size;
        } else {
            for (char c : item) {
                if (c < '0' || c > '9' || batch > (size_t) 1 << 40) {
                    ok = false;
                    break;
                }
                batch = batch * 10 + (size_t) (c - '0');
            }
        }
        if (!ok || batch == 0 || batch > max_batch_size) {
            std::cerr << "cuBERT: CUBERT_OPEN_WARMUP entry \"" << item << "\" is not a batch size in [1, " << max_batch_size
                      << "]; skipped" << std::endl;
            continue;
        }
        bool seen = false;
        for (size_t b : batches) seen = seen || b == batch;
        if (!seen) batches.push_back(batch);
    }
    return batches;
}

template <typename T>
Bert<T>::Bert(const std::unordered_map<std::string, T *> &var, size_t max_batch_size, size_t seq_length,
              size_t vocab_size, size_t type_vocab_size, size_t hidden_size, size_t num_hidden_layers,
              size_t num_attention_heads, size_t intermediate_size, size_t num_labels)
        : max_batch_size(max_batch_size), seq_length(seq_length), hidden_size(hidden_size), num_labels(num_labels),
          vocab_size(vocab_size), type_vocab_size(type_vocab_size), transformer(nullptr), _sequence_output(nullptr) {
    try {
        this->stream = cuBERT::cuda_stream_create();
        this->cublas = cuBERT::blas_create();
        cuBERT::blas_set_stream(cublas, stream);

        has_pooler_dense = var.count("bert/pooler/dense/kernel") != 0;
        has_classifier = var.count("output_weights") != 0;
        has_classifier_bias = has_classifier && var.count("output_bias") != 0;

        const size_t H = hidden_size;
        layout_weights(vocab_size, type_vocab_size);
        weights.allocate();
        layout_weights(vocab_size, type_vocab_size);

        cuBERT::memcpy(word_embeddings, var.at("bert/embeddings/word_embeddings"), vocab_size * H * sizeof(T), 1);
        cuBERT::memcpy(token_type_embeddings, var.at("bert/embeddings/token_type_embeddings"),
                       type_vocab_size * H * sizeof(T), 1);
        // only the positions a sequence of seq_length tokens can use are kept on the device
        cuBERT::memcpy(position_embeddings, var.at("bert/embeddings/position_embeddings"), seq_length * H * sizeof(T), 1);
        cuBERT::memcpy(embedding_norm_beta, var.at("bert/embeddings/LayerNorm/beta"), H * sizeof(T), 1);
        cuBERT::memcpy(embedding_norm_gamma, var.at("bert/embeddings/LayerNorm/gamma"), H * sizeof(T), 1);
        if (has_pooler_dense) {
            cuBERT::memcpy(pooler_kernel, var.at("bert/pooler/dense/kernel"), H * H * sizeof(T), 1);
            cuBERT::memcpy(pooler_bias, var.at("bert/pooler/dense/bias"), H * sizeof(T), 1);
        }
        if (has_classifier) {
            cuBERT::memcpy(output_weights, var.at("output_weights"), num_labels * H * sizeof(T), 1);
            if (has_classifier_bias) cuBERT::memcpy(output_bias, var.at("output_bias"), num_labels * sizeof(T), 1);
        }

        this->transformer = new Transformer<T>(cublas, "bert/encoder", var, max_batch_size, seq_length, hidden_size,
                                               num_hidden_layers, num_attention_heads, intermediate_size);
        this->transformer->set_profiler(&profiler);

        layout_buffers();
        buffers.allocate();
        layout_buffers();

        input_staging = static_cast<unsigned char *>(cubert_malloc_host(input_block_bytes(max_batch_size * seq_length)));
        if (input_staging == nullptr) throw std::runtime_error("no page-locked host memory for the request inputs");
        output_staging = static_cast<unsigned char *>(cubert_malloc_host(kOutputStagingBytes));
        if (output_staging == nullptr) throw std::runtime_error("no page-locked host memory for the outputs");

        for (size_t batch : open_warmup_batches(std::getenv("CUBERT_OPEN_WARMUP"), max_batch_size)) _pre_compute(batch);
    } catch (...) {
        release();
        throw;
    }
}

template <typename T>
Bert<T>::~Bert() {
    release();
}

template <typename T>
void Bert<T>::release() noexcept {
    if (stream != nullptr) cubert_stream_synchronize(stream);
    cubert_free_host(input_staging);  // null is accepted
    cubert_free_host(output_staging);
    delete transformer;
    if (cublas != nullptr) cubert_blas_destroy(cublas);
    if (stream != nullptr) cubert_stream_destroy(stream);
    input_staging = nullptr, output_staging = nullptr, transformer = nullptr, cublas = nullptr, stream = nullptr;
}

template <typename T>
void Bert<T>::layout_weights(size_t vocab_size, size_t type_vocab_size) {
    const size_t H = hidden_size;
    word_embeddings = weights.take<T>(vocab_size * H);
    token_type_embeddings = weights.take<T>(type_vocab_size * H);
    position_embeddings = weights.take<T>(seq_length * H);
    embedding_norm_beta = weights.take<T>(H);
    embedding_norm_gamma = weights.take<T>(H);
    pooler_kernel = has_pooler_dense ? weights.take<T>(H * H) : nullptr;
    pooler_bias = has_pooler_dense ? weights.take<T>(H) : nullptr;
    output_weights = has_classifier ? weights.take<T>(num_labels * H) : nullptr;
    output_bias = has_classifier_bias ? weights.take<T>(num_labels) : nullptr;
}

template <typename T>
void Bert<T>::layout_buffers() {
    const size_t M = max_batch_size * seq_length;
    input_block = buffers.take<unsigned char>(input_block_bytes(M));
    input_ids_buf = nullptr, input_mask_buf = nullptr, segment_ids_buf = nullptr;  // set per request
    _embedding_output = buffers.take<T>(M * hidden_size);
    _pooled_output = buffers.take<T>(max_batch_size * hidden_size);
    _logits = has_classifier ? buffers.take<T>(max_batch_size * num_labels) : nullptr;
    _probs = has_classifier ? buffers.take<T>(max_batch_size * num_labels) : nullptr;
}

// What a first request of `batch_size` sequences would otherwise pay for: one forward pass on made-up inputs, so
// that every GEMM shape of that batch size is planned and, where that applies, its algorithm chosen by timing
// (tens of milliseconds) before a caller waits on it.  The reference also prepares the maximum batch when a model
// is built (src/cuBERT/Bert.cpp:62-64, there: bias rows copied into the Dense outputs).  Other batch sizes are
// still planned on their first request.
template <typename T>
void Bert<T>::_pre_compute(size_t batch_size) {
    if (batch_size == 0 || batch_size > max_batch_size || vocab_size == 0) return;
    const size_t M = batch_size * seq_length;
    const size_t mask_at = round_up_16(sizeof(int) * M), segments_at = round_up_16(mask_at + M);
    if (input_copy_pending) synchronize();
    // ids spread over the vocabulary (a multiplicative hash of the position), every position valid, segment 0:
    // activations like those of a real request, which is what the timing of GEMM algorithms should see
    int *ids = reinterpret_cast<int *>(input_staging);
    for (size_t i = 0; i < M; ++i) ids[i] = (int) ((uint32_t) (i * 2654435761u) % (uint32_t) vocab_size);
    std::memset(input_staging + mask_at, 1, M);
    std::memset(input_staging + segments_at, 0, M);
    cuBERT::memcpyAsync(input_block, input_staging, segments_at + M, 1, stream);
    input_ids_buf = reinterpret_cast<int *>(input_block);
    input_mask_buf = reinterpret_cast<int8_t *>(input_block + mask_at);
    segment_ids_buf = reinterpret_cast<int8_t *>(input_block + segments_at);
    forward(batch_size);
    synchronize();
    (void) transformer->two_term_overflowed();  // what the made-up inputs did says nothing about a request
    input_ids_buf = nullptr, input_mask_buf = nullptr, segment_ids_buf = nullptr;  // no request is resident
}

template <typename T>
void Bert<T>::synchronize() {
    cuBERT::cuda_stream_synchronize(stream);
    input_copy_pending = false;
}

// One output on its way to the caller.  A copy into pageable memory costs about 11 us more than one into
// page-locked memory (measured: 3 KB, 23.0 against 11.8 us including the wait), so small outputs land in a
// page-locked block first and reach the caller's array after the stream has drained.
template <typename T>
void Bert<T>::fetch(void *dst, const void *src, size_t bytes) {
    requested.push_back(RequestedOutput{dst, src, bytes});
    enqueue_fetch(dst, src, bytes);
}

template <typename T>
void Bert<T>::enqueue_fetch(void *dst, const void *src, size_t bytes) {
    const size_t at = round_up_16(staged_bytes);
    if (output_staging != nullptr && at + bytes <= kOutputStagingBytes) {
        cuBERT::memcpyAsync(output_staging + at, src, bytes, 2, stream);
        staged.push_back(StagedOutput{dst, at, bytes});
        staged_bytes = at + bytes;
    } else {
        cuBERT::memcpyAsync(dst, src, bytes, 2, stream);
    }
}

template <typename T>
void Bert<T>::finish_outputs() {
    synchronize();
    // An fp32 model in the two-term fp16 Dense form (opt-in): an activation beyond what two fp16 terms can hold
    // raised a flag while the request ran.  Its results are not to be trusted: the same request, whose inputs are
    // still on the device, runs again on the fp32 GEMMs, and the copies this call asked for are made again.
    if (transformer != nullptr && transformer->two_term_overflowed() && last_batch > 0 && input_ids_buf != nullptr) {
        transformer->use_fp32_dense_once();
        forward(last_batch);
        staged.clear();
        staged_bytes = 0;
        for (const RequestedOutput &o : requested) enqueue_fetch(o.dst, o.src, o.bytes);
        synchronize();
        (void) transformer->two_term_overflowed();  // (the fp32 pass writes no two-term rows; nothing to clear)
    }
    for (const StagedOutput &o : staged) std::memcpy(o.dst, output_staging + o.offset, o.bytes);
    staged.clear();
    staged_bytes = 0;
    requested.clear();
}

template <typename T>
void Bert<T>::compute(size_t batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids) {
    if (batch_size > max_batch_size) {
        throw std::invalid_argument("batch_size > max_batch_size");
    } else if (batch_size == 0) {
        return;
    }
    const size_t M = batch_size * seq_length;
    check_input_range(input_ids, segment_ids, M, vocab_size, type_vocab_size);
    const size_t mask_at = round_up_16(sizeof(int) * M), segments_at = round_up_16(mask_at + M);
    // The staging memory may still be being read by the previous request's copy when that request's outputs
    // were never fetched (every output method drains the stream); no event sits on a request's own path.
    if (input_copy_pending) synchronize();
    std::memcpy(input_staging, input_ids, sizeof(int) * M);
    std::memcpy(input_staging + mask_at, input_mask, M);
    std::memcpy(input_staging + segments_at, segment_ids, M);
    cuBERT::memcpyAsync(input_block, input_staging, segments_at + M, 1, stream);
    input_copy_pending = true;
    input_ids_buf = reinterpret_cast<int *>(input_block);
    input_mask_buf = reinterpret_cast<int8_t *>(input_block + mask_at);
    segment_ids_buf = reinterpret_cast<int8_t *>(input_block + segments_at);
    forward(batch_size);
}

template <typename T>
void Bert<T>::compute_resident(size_t batch_size) {
    if (batch_size > max_batch_size) {
        throw std::invalid_argument("batch_size > max_batch_size");
    } else if (batch_size == 0) {
        return;
    }
    if (input_ids_buf == nullptr) throw std::invalid_argument("compute_resident needs a compute call before it");
    forward(batch_size);
}

template <typename T>
void Bert<T>::forward(size_t batch_size) {
    last_batch = batch_size;
    const int B = (int) batch_size, S = (int) seq_length, H = (int) hidden_size, L = (int) num_labels;

    // bert/embeddings
    {
        Timed t(&profiler, Profiler::kEmbedLayerNorm, stream);
        cuBERT::embed_layer_norm(input_ids_buf, segment_ids_buf, word_embeddings, position_embeddings,
                                 token_type_embeddings, embedding_norm_beta, embedding_norm_gamma, _embedding_output,
                                 B, S, H, stream);
    }

    // bert/encoder
    _sequence_output = transformer->_in_compute(batch_size, _embedding_output, input_mask_buf);

    // bert/pooler
    bool tanh_pending = false;
    if (has_pooler_dense) {
        // first token of every sequence: the B rows are seq_length*hidden apart
        Timed t(&profiler, profiler.dense_kind(Profiler::kDensePooler), stream);
        cuBERT::blas_gemm(cublas, false, false, H, B, H, 1.f, pooler_kernel, H, _sequence_output, H * S, 0.f,
                          _pooled_output, H);
        tanh_pending = true;
    } else {
        Timed t(&profiler, Profiler::kMeanPool, stream);
        cuBERT::reduce_mean_1(_sequence_output, _pooled_output, B, S, H, stream);
    }

    // classifier head: pooler bias + tanh, logits = pooled * W^T (+ bias) with W [num_labels, hidden] row-major, and
    // their softmax -- one launch for few labels, else the three kernels of the reference
    if (has_classifier && classifier_head_fits) {
        Timed t(&profiler, Profiler::kClassifierHead, stream);
        if (cuBERT::classifier_head(_pooled_output, tanh_pending ? pooler_bias : nullptr, output_weights, output_bias,
                                    _logits, _probs, B, H, L, stream)) {
            return;
        }
        classifier_head_fits = false;  // the sizes are fixed per model: do not ask again
        t.cancel();
    }
    if (tanh_pending) {
        Timed t(&profiler, Profiler::kBiasTanh, stream);
        cuBERT::tanh_(_pooled_output, pooler_bias, B, H, stream);
    }
    if (has_classifier) {
        {
            Timed t(&profiler, Profiler::kDenseGemm, stream);
            cuBERT::blas_gemm(cublas, true, false, L, B, H, 1.f, output_weights, H, _pooled_output, H, 0.f, _logits, L,
                              output_bias);
        }
        Timed t(&profiler, Profiler::kRowSoftmax, stream);
        cuBERT::softmax_(_logits, _probs, B, L, stream);
    }
}

template <typename T>
void Bert<T>::logits(size_t batch_size, T *logits, T *probs) {
    if (!has_classifier) {
        std::cerr << "model does not have additional_output_layer, the output logits is wrong." << std::endl;
    }
    if (has_classifier && logits != nullptr) {
        fetch(logits, _logits, sizeof(T) * batch_size * num_labels);
    }
    if (has_classifier && probs != nullptr) {
        fetch(probs, _probs, sizeof(T) * batch_size * num_labels);
    }
    finish_outputs();
}

template <typename T>
void Bert<T>::pooled_output(size_t batch_size, T *pooled_output) {
    fetch(pooled_output, _pooled_output, sizeof(T) * batch_size * hidden_size);
    finish_outputs();
}

template <typename T>
void Bert<T>::sequence_output(size_t batch_size, T *sequence_output) {
    fetch(sequence_output, _sequence_output, sizeof(T) * batch_size * seq_length * hidden_size);
    finish_outputs();
}

template <typename T>
void Bert<T>::embedding_output(size_t batch_size, T *embedding_output) {
    fetch(embedding_output, _embedding_output, sizeof(T) * batch_size * seq_length * hidden_size);
    finish_outputs();
}

template <typename T>
void Bert<T>::output(size_t batch_size, cuBERT_Output *output) {
    const size_t tokens = batch_size * seq_length * hidden_size;
    if (output->logits != nullptr && has_classifier) {
        fetch(output->logits, _logits, sizeof(T) * batch_size * num_labels);
    }
    if (output->probs != nullptr && has_classifier) {
        fetch(output->probs, _probs, sizeof(T) * batch_size * num_labels);
    }
    if (output->pooled_output != nullptr) {
        fetch(output->pooled_output, _pooled_output, sizeof(T) * batch_size * hidden_size);
    }
    if (output->sequence_output != nullptr) {
        fetch(output->sequence_output, _sequence_output, sizeof(T) * tokens);
    }
    if (output->embedding_output != nullptr) {
        fetch(output->embedding_output, _embedding_output, sizeof(T) * tokens);
    }
    finish_outputs();
}

template <>
void Bert<float>::output_to_float(size_t batch_size, cuBERT_Output *output) {
    this->output(batch_size, output);
}

template <>
void Bert<half>::output_to_float(size_t batch_size, cuBERT_Output *output) {
    const size_t tokens = batch_size * seq_length * hidden_size;
    std::vector<half> lg(output->logits ? batch_size * num_labels : 0), pr(output->probs ? batch_size * num_labels : 0),
            po(output->pooled_output ? batch_size * hidden_size : 0), sq(output->sequence_output ? tokens : 0),
            em(output->embedding_output ? tokens : 0);
    cuBERT_Output tmp;
    tmp.logits = output->logits ? lg.data() : nullptr;
    tmp.probs = output->probs ? pr.data() : nullptr;
    tmp.pooled_output = output->pooled_output ? po.data() : nullptr;
    tmp.sequence_output = output->sequence_output ? sq.data() : nullptr;
    tmp.embedding_output = output->embedding_output ? em.data() : nullptr;
    this->output(batch_size, &tmp);
    if (output->logits) half2float(lg.data(), (float *) output->logits, lg.size());
    if (output->probs) half2float(pr.data(), (float *) output->probs, pr.size());
    if (output->pooled_output) half2float(po.data(), (float *) output->pooled_output, po.size());
    if (output->sequence_output) half2float(sq.data(), (float *) output->sequence_output, sq.size());
    if (output->embedding_output) half2float(em.data(), (float *) output->embedding_output, em.size());
}

template class Bert<float>;
template class Bert<half>;

}  // namespace cuBERT
