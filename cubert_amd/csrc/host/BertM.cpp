#include "BertM.h"

#include <chrono>
#include <cstdlib>
#include <iostream>
#include <stdexcept>
#include <string>

namespace cuBERT {

namespace {

// Every tensor the model will read must hold as many elements as the sizes found in the file and the
// arguments of cuBERT_open imply; the constructors below copy that many elements without looking again.
// (The reference trusts the file.)  A tensor that is absent is left to the lookup that needs it.
template <typename T>
void check_tensor_sizes(const Graph<T> &g, size_t seq_length, size_t num_hidden_layers) {
    const size_t H = g.hidden_size, I = g.intermediate_size;
    auto expect = [&](const std::string &name, size_t want, bool at_least = false) {
        auto it = g.size.find(name);
        if (it == g.size.end()) return;
        if (at_least ? it->second < want : it->second != want) {
            throw std::invalid_argument("model file invalid: " + name + " holds " + std::to_string(it->second) +
                                        " elements, the model needs " + std::to_string(want));
        }
    };
    if (H == 0) throw std::invalid_argument("model file invalid: no embedding tables");
    expect("bert/embeddings/word_embeddings", g.vocab_size * H);
    expect("bert/embeddings/token_type_embeddings", g.type_vocab_size * H);
    expect("bert/embeddings/position_embeddings", seq_length * H, true);
    expect("bert/embeddings/LayerNorm/beta", H);
    expect("bert/embeddings/LayerNorm/gamma", H);
    for (size_t l = 0; l < num_hidden_layers; ++l) {
        const std::string p = "bert/encoder/layer_" + std::to_string(l);
        for (const char *n : {"query", "key", "value"}) {
            expect(p + "/attention/self/" + n + "/kernel", H * H);
            expect(p + "/attention/self/" + n + "/bias", H);
        }
        expect(p + "/attention/output/dense/kernel", H * H);
        expect(p + "/attention/output/dense/bias", H);
        expect(p + "/attention/output/LayerNorm/beta", H);
        expect(p + "/attention/output/LayerNorm/gamma", H);
        expect(p + "/intermediate/dense/kernel", H * I);
        expect(p + "/intermediate/dense/bias", I);
        expect(p + "/output/dense/kernel", I * H);
        expect(p + "/output/dense/bias", H);
        expect(p + "/output/LayerNorm/beta", H);
        expect(p + "/output/LayerNorm/gamma", H);
    }
    expect("bert/pooler/dense/kernel", H * H);
    expect("bert/pooler/dense/bias", H);
    expect("output_weights", g.num_labels * H);
    expect("output_bias", g.num_labels);
}

}  // namespace

template <typename T>
BertM<T>::BertM(const char *model_file, size_t max_batch_size, size_t seq_length, size_t num_hidden_layers,
                size_t num_attention_heads)
        : seq_length(seq_length), graph(model_file), rr(0) {
    check_tensor_sizes(graph, seq_length, num_hidden_layers);
    const int count = cuBERT::get_gpu_count();
    if (count == 0) {
        throw std::invalid_argument("No GPU device detected");
    }
    std::cerr << "Found GPU count: " << count << std::endl;

    // CUBERT_MODELS_PER_GPU=n in the environment (default 1) keeps n instances per device, each with its own stream:
    // requests of a few tokens leave most of the chip idle (their kernels wait on memory latency), so concurrent
    // callers get more requests per second when they do not queue behind one instance per device.  (The reference
    // has the same knob for its CPU build, CUBERT_NUM_CPU_MODELS, src/cuBERT/BertM.cpp:25-28.)
    int per_device = 1;
    if (const char *text = std::getenv("CUBERT_MODELS_PER_GPU")) {
        per_device = std::atoi(text);
        if (per_device < 1 || count * per_device > 255) {
            throw std::invalid_argument("CUBERT_MODELS_PER_GPU must be at least 1 and give at most 255 instances");
        }
        std::cerr << "Found CUBERT_MODELS_PER_GPU: " << per_device << std::endl;
    }

    for (int instance = 0; instance < count * per_device; ++instance) {
        const int device = instance % count;  // round-robin over instances visits the devices in turn
        const auto start = std::chrono::high_resolution_clock::now();
        cuBERT::set_gpu(device);
        cuBERT::gpu_info(device);
        bert_instances.emplace_back(new Bert<T>(graph.var, max_batch_size, seq_length, graph.vocab_size,
                                                graph.type_vocab_size, graph.hidden_size, num_hidden_layers,
                                                num_attention_heads, graph.intermediate_size, graph.num_labels));
        mutex_instances.emplace_back(new std::mutex());
        device_of_instance.push_back(device);
        const auto finish = std::chrono::high_resolution_clock::now();
        std::cerr << "device setup: " << device << ". Took "
                  << std::chrono::duration_cast<std::chrono::milliseconds>(finish - start).count() << " milliseconds."
                  << std::endl;
    }
}

template <typename T>
BertM<T>::~BertM() {
    for (size_t i = 0; i < bert_instances.size(); ++i) {
        cuBERT::set_gpu(device_of_instance[i]);
        bert_instances[i].reset();
    }
}

template <typename T>
unsigned int BertM<T>::compute(size_t batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids, T *output,
                               cuBERT_OutputType output_type) {
    const uint8_t count = rr++;
    const unsigned int choice = count % bert_instances.size();

    cuBERT::set_gpu(device_of_instance[choice]);
    Bert<T> *bert = bert_instances[choice].get();
    std::lock_guard<std::mutex> lg(*mutex_instances[choice]);

    bert->compute(batch_size, input_ids, input_mask, segment_ids);
    switch (output_type) {
        case cuBERT_LOGITS: bert->logits(batch_size, output, nullptr); break;
        case cuBERT_PROBS: bert->logits(batch_size, nullptr, output); break;
        case cuBERT_POOLED_OUTPUT: bert->pooled_output(batch_size, output); break;
        case cuBERT_EMBEDDING_OUTPUT: bert->embedding_output(batch_size, output); break;
        case cuBERT_SEQUENCE_OUTPUT: bert->sequence_output(batch_size, output); break;
        default: throw std::invalid_argument("invalid output type");
    }
    return choice;
}

template <typename T>
unsigned int BertM<T>::compute(size_t batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids,
                               cuBERT_Output *output, bool output_to_float) {
    const uint8_t count = rr++;
    const unsigned int choice = count % bert_instances.size();

    cuBERT::set_gpu(device_of_instance[choice]);
    Bert<T> *bert = bert_instances[choice].get();
    std::lock_guard<std::mutex> lg(*mutex_instances[choice]);

    bert->compute(batch_size, input_ids, input_mask, segment_ids);
    if (output_to_float) {
        bert->output_to_float(batch_size, output);
    } else {
        bert->output(batch_size, output);
    }
    return choice;
}

template class BertM<float>;
template class BertM<half>;

}  // namespace cuBERT
