// A loaded model replicated on every visible GPU, safe to call from many host
// threads: requests go round-robin over the replicas and hold that replica's
// mutex for the whole compute + copy-out.  Public surface of the reference's
// BertM<T> (src/cuBERT/BertM.h:17-37).  CUBERT_MODELS_PER_GPU=n in the environment
// keeps n replicas per device (own weights, buffers and stream each), which
// lets small concurrent requests overlap on one device.
#ifndef CUBERT_HOST_BERTM_H
#define CUBERT_HOST_BERTM_H

#include <atomic>
#include <cstdint>
#include <memory>
#include <mutex>
#include <vector>

#include "Bert.h"
#include "Graph.h"
#include "cuBERT.h"

namespace cuBERT {

template <typename T>
class BertM {
public:
    explicit BertM(const char *model_file, size_t max_batch_size, size_t seq_length, size_t num_hidden_layers = 12,
                   size_t num_attention_heads = 12);

    virtual ~BertM();

    // Returns the index of the replica that served the request.
    unsigned int compute(size_t batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids, T *output,
                         cuBERT_OutputType output_type = cuBERT_LOGITS);

    unsigned int compute(size_t batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids,
                         cuBERT_Output *output, bool output_to_float = false);

    size_t seq_length;

    // Shape facts read from the model file, for callers that size output buffers.
    size_t hidden_size() const { return graph.hidden_size; }
    size_t num_labels() const { return graph.num_labels; }
    Bert<T> *replica(size_t i) { return bert_instances[i].get(); }

private:
    Graph<T> graph;
    // owned: a constructor that throws half way (a later device fails) releases the replicas built so far
    std::vector<std::unique_ptr<Bert<T>>> bert_instances;
    std::vector<std::unique_ptr<std::mutex>> mutex_instances;
    std::vector<int> device_of_instance;  // instance i runs on device i % gpu_count (CUBERT_MODELS_PER_GPU instances each)
    std::atomic<uint8_t> rr;
};

}  // namespace cuBERT

#endif  // CUBERT_HOST_BERTM_H
