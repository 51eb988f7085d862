// One BERT model on one device: owns a stream, a BLAS context, the device
// copies of the weights and all activation buffers.  Public surface of the
// reference's Bert<T> (src/cuBERT/Bert.h:17-44).  Not thread-safe; BertM
// serialises access.
#ifndef CUBERT_HOST_BERT_H
#define CUBERT_HOST_BERT_H

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>
#include <unordered_map>

#include "Arena.h"
#include "Transformer.h"
#include "cuBERT.h"

namespace cuBERT {

// Throws std::invalid_argument naming the first input id outside [0, vocab_size) or segment id outside
// [0, type_vocab_size).  Bert<T>::compute runs it on every request before anything is enqueued.
void check_input_range(const int *input_ids, const int8_t *segment_ids, size_t count, size_t vocab_size,
                       size_t type_vocab_size);

// The batch sizes a model prepares when it is opened, read from the text of CUBERT_OPEN_WARMUP (nullptr = unset):
// unset = max_batch_size only, "0" = none, else a comma-separated list in which "max" stands for max_batch_size.
std::vector<size_t> open_warmup_batches(const char *setting, size_t max_batch_size);

template <typename T>
class Bert {
public:
    // `var` maps TensorFlow variable names to host arrays (see Transformer.cpp and Bert.cpp for the
    // names).  "bert/pooler/dense/kernel" present -> first-token dense+tanh pooler, absent -> mean
    // pooler; "output_weights" present -> classifier head with `num_labels` rows ("output_bias" optional).
    explicit Bert(const std::unordered_map<std::string, T *> &var, size_t max_batch_size, size_t seq_length,
                  size_t vocab_size, size_t type_vocab_size, size_t hidden_size = 768, size_t num_hidden_layers = 12,
                  size_t num_attention_heads = 12, size_t intermediate_size = 3072, size_t num_labels = 1);

    virtual ~Bert();

    Bert(const Bert &) = delete;
    Bert &operator=(const Bert &) = delete;

    // One forward pass of `batch_size` sequences on made-up inputs: plans (and where it applies times) every GEMM
    // shape of that batch size, so that the first request of that size does not pay for it.  The constructor runs
    // it for max_batch_size (CUBERT_OPEN_WARMUP=0 in the environment skips that, a list such as 1,8,max names the
    // batch sizes to prepare instead).  Nothing needs preparing
    // between requests, unlike in the reference, whose _pre_compute refills the Dense outputs with their biases.
    void _pre_compute(size_t batch_size);

    // Copies the three host input arrays to the device and enqueues the forward pass.  Asynchronous:
    // one of the output methods below must follow to wait for and fetch results.
    void compute(size_t batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids);

    // Output methods: copy to host arrays (nullptr = skip) and synchronise the stream.
    void logits(size_t batch_size, T *logits, T *probs);
    void pooled_output(size_t batch_size, T *pooled_output);
    void sequence_output(size_t batch_size, T *sequence_output);
    void embedding_output(size_t batch_size, T *embedding_output);
    void output(size_t batch_size, cuBERT_Output *output);
    // Same, but a half model converts to float on the host first.
    void output_to_float(size_t batch_size, cuBERT_Output *output);

    // The stream all of this model's work runs on (for timing with events).
    void *get_stream() const { return stream; }

    // The forward pass again on the inputs the last compute() left on the device (no host copies):
    // the steady-state device work of a request, used for throughput measurements.
    void compute_resident(size_t batch_size);

    // Per-kernel timing: switch kinds on (bit k = Profiler::Kind k), run, synchronise, then read.
    void profile(unsigned kinds) { profiler.enable(kinds); }
    void profile_read(double *total_ms, int *count) {
        synchronize();
        profiler.collect(total_ms, count);
    }

private:
    void forward(size_t batch_size);
    void synchronize();       // drains the stream
    void fetch(void *dst, const void *src, size_t bytes);  // queue one device-to-host output copy and remember it
    void enqueue_fetch(void *dst, const void *src, size_t bytes);
    void finish_outputs();    // drain the stream and hand staged outputs to the caller's arrays
    void release() noexcept;  // everything the constructor acquired so far (also run when it throws)
    void layout_weights(size_t vocab_size, size_t type_vocab_size);
    void layout_buffers();

    void *cublas = nullptr;
    void *stream = nullptr;

    size_t max_batch_size, seq_length, hidden_size, num_labels;
    size_t vocab_size, type_vocab_size;  // rows of the word and token-type tables: bounds of a request's ids
    bool has_pooler_dense, has_classifier, has_classifier_bias;
    bool classifier_head_fits = true;  // cleared when the one-launch classifier head declines this model's shape

    Transformer<T> *transformer = nullptr;
    Profiler profiler;

    Arena weights;
    T *word_embeddings, *token_type_embeddings, *position_embeddings;  // position: first seq_length rows only
    T *embedding_norm_beta, *embedding_norm_gamma;
    T *pooler_kernel, *pooler_bias;
    T *output_weights, *output_bias;

    Arena buffers;
    // The three inputs of a request travel as one block: ids, then the mask, then the segment ids, each
    // starting at a multiple of 16 bytes.  A request is packed into page-locked host memory in that layout and
    // reaches the device in a single asynchronous copy; the pointers below are set per request.
    unsigned char *input_block;          // device
    unsigned char *input_staging = nullptr;  // page-locked host memory, same size
    // small outputs pass through page-locked memory on their way to the caller's (pageable) arrays
    static constexpr size_t kOutputStagingBytes = 32 * 1024;
    struct StagedOutput {
        void *dst;
        size_t offset, bytes;
    };
    unsigned char *output_staging = nullptr;
    std::vector<StagedOutput> staged;
    size_t staged_bytes = 0;
    // every copy an output call has asked for, so that the call can be repeated after the request was recomputed
    struct RequestedOutput {
        void *dst;
        const void *src;
        size_t bytes;
    };
    std::vector<RequestedOutput> requested;
    size_t last_batch = 0;               // batch size of the forward pass whose results the buffers hold
    bool input_copy_pending = false;     // a copy out of input_staging was queued and the stream not drained since
    int *input_ids_buf;
    int8_t *input_mask_buf;
    int8_t *segment_ids_buf;
    T *_embedding_output;
    T *_sequence_output;  // points into the transformer's buffers
    T *_pooled_output;
    T *_logits;
    T *_probs;
};

}  // namespace cuBERT

#endif  // CUBERT_HOST_BERT_H
