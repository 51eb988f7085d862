// The public C API (include/cuBERT.h) and the exception-free host entry points
// (include/cubert_host.h).
#include <cstring>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "Bert.h"
#include "BertM.h"
#include "Transformer.h"
#include "cuBERT.h"
#include "tokenization.h"
#include "cubert_host.h"

using cuBERT::half;

// ------------------------------------------------------------------ cuBERT.h

void cuBERT_initialize() { cuBERT::initialize(); }

void cuBERT_finalize() { cuBERT::finalize(); }

int cuBERT_get_gpu_count() { return cuBERT::get_gpu_count(); }

void *cuBERT_open(const char *model_file, int max_batch_size, int seq_length, int num_hidden_layers,
                  int num_attention_heads, cuBERT_ComputeType compute_type) {
    if (compute_type == cuBERT_COMPUTE_FLOAT) {
        return new cuBERT::BertM<float>(model_file, max_batch_size, seq_length, num_hidden_layers, num_attention_heads);
    }
    return new cuBERT::BertM<half>(model_file, max_batch_size, seq_length, num_hidden_layers, num_attention_heads);
}

void cuBERT_compute(void *model, int batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids, void *output,
                    cuBERT_OutputType output_type, cuBERT_ComputeType compute_type) {
    if (compute_type == cuBERT_COMPUTE_FLOAT) {
        ((cuBERT::BertM<float> *) model)->compute(batch_size, input_ids, input_mask, segment_ids, (float *) output,
                                                  output_type);
    } else {
        ((cuBERT::BertM<half> *) model)->compute(batch_size, input_ids, input_mask, segment_ids, (half *) output,
                                                 output_type);
    }
}

void cuBERT_compute_m(void *model, int batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids,
                      cuBERT_Output *output, cuBERT_ComputeType compute_type, int output_to_float) {
    if (compute_type == cuBERT_COMPUTE_FLOAT) {
        ((cuBERT::BertM<float> *) model)->compute(batch_size, input_ids, input_mask, segment_ids, output,
                                                  output_to_float != 0);
    } else {
        ((cuBERT::BertM<half> *) model)->compute(batch_size, input_ids, input_mask, segment_ids, output,
                                                 output_to_float != 0);
    }
}

void cuBERT_close(void *model, cuBERT_ComputeType compute_type) {
    if (compute_type == cuBERT_COMPUTE_FLOAT) {
        delete (cuBERT::BertM<float> *) model;
    } else {
        delete (cuBERT::BertM<half> *) model;
    }
}

void *cuBERT_open_tokenizer(const char *vocab_file, int do_lower_case) {
    return new cuBERT::FullTokenizer(vocab_file, do_lower_case != 0);
}

void cuBERT_close_tokenizer(void *tokenizer) { delete (cuBERT::FullTokenizer *) tokenizer; }

namespace {

size_t model_seq_length(void *model, cuBERT_ComputeType compute_type) {
    if (model == nullptr) throw std::invalid_argument("null model");
    return compute_type == cuBERT_COMPUTE_FLOAT ? ((cuBERT::BertM<float> *) model)->seq_length
                                                : ((cuBERT::BertM<half> *) model)->seq_length;
}

// text -> ids, mask, segment ids for a batch (reference: cuBERT.cpp:216-247; heap instead of stack arrays)
struct TokenizedBatch {
    std::vector<int> input_ids;
    std::vector<int8_t> input_mask, segment_ids;

    TokenizedBatch(void *tokenizer, size_t seq_length, int batch_size, const char **text_a, const char **text_b) {
        if (tokenizer == nullptr || batch_size < 0 || (batch_size > 0 && text_a == nullptr)) {
            throw std::invalid_argument("tokenizer, text_a and a non-negative batch_size are required");
        }
        const size_t n = (size_t) batch_size * seq_length;
        input_ids.resize(n);
        input_mask.resize(n);
        segment_ids.resize(n);
        const auto *tok = (const cuBERT::FullTokenizer *) tokenizer;
        for (int i = 0; i < batch_size; ++i) {
            tok->convert_single_example(seq_length, text_a[i], text_b == nullptr ? nullptr : text_b[i],
                                        input_ids.data() + seq_length * i, input_mask.data() + seq_length * i,
                                        segment_ids.data() + seq_length * i);
        }
    }
};

}  // namespace

void cuBERT_tokenize_compute(void *model, void *tokenizer, int batch_size, const char **text_a, const char **text_b,
                             void *output, cuBERT_OutputType output_type, cuBERT_ComputeType compute_type) {
    TokenizedBatch t(tokenizer, model_seq_length(model, compute_type), batch_size, text_a, text_b);
    cuBERT_compute(model, batch_size, t.input_ids.data(), t.input_mask.data(), t.segment_ids.data(), output,
                   output_type, compute_type);
}

void cuBERT_tokenize_compute_m(void *model, void *tokenizer, int batch_size, const char **text_a, const char **text_b,
                               cuBERT_Output *output, cuBERT_ComputeType compute_type, int output_to_float) {
    TokenizedBatch t(tokenizer, model_seq_length(model, compute_type), batch_size, text_a, text_b);
    cuBERT_compute_m(model, batch_size, t.input_ids.data(), t.input_mask.data(), t.segment_ids.data(), output,
                     compute_type, output_to_float);
}

// ------------------------------------------------------------- cubert_host.h

namespace {

thread_local std::string g_last_error;

template <typename F>
int guarded(F &&f) {
    try {
        g_last_error.clear();
        f();
        return 0;
    } catch (const std::invalid_argument &e) {
        g_last_error = e.what();
        return CUBERT_E_INVALID_ARGUMENT;
    } catch (const std::out_of_range &e) {
        g_last_error = e.what();
        return CUBERT_E_OUT_OF_RANGE;
    } catch (const std::exception &e) {
        g_last_error = e.what();
        return CUBERT_E_OTHER;
    }
}

template <typename T>
std::unordered_map<std::string, T *> var_map(int n, const char *const *names, const void *const *data) {
    std::unordered_map<std::string, T *> var;
    for (int i = 0; i < n; ++i) var[names[i]] = (T *) data[i];
    return var;
}

template <typename T>
void transformer_run(const char *prefix, int n, const char *const *names, const void *const *data, int batch, int seq,
                     int hidden, int layers, int heads, int intermediate, const void *input, const int8_t *mask,
                     void *output) {
    void *stream = cuBERT::cuda_stream_create();
    void *blas = cuBERT::blas_create();
    cuBERT::blas_set_stream(blas, stream);
    {
        cuBERT::Transformer<T> transformer(blas, prefix, var_map<T>(n, names, data), batch, seq, hidden, layers, heads,
                                           intermediate);
        const size_t count = (size_t) batch * seq * hidden;
        T *in_gpu = (T *) cuBERT::malloc(count * sizeof(T));
        int8_t *mask_gpu = (int8_t *) cuBERT::malloc((size_t) batch * seq);
        cuBERT::memcpy(in_gpu, input, count * sizeof(T), 1);
        cuBERT::memcpy(mask_gpu, mask, (size_t) batch * seq, 1);
        T *out_gpu = transformer.compute(batch, in_gpu, mask_gpu);
        cuBERT::memcpyAsync(output, out_gpu, count * sizeof(T), 2, stream);
        cuBERT::cuda_stream_synchronize(stream);
        if (transformer.two_term_overflowed()) {  // opt-in two-term fp16 Dense form: an activation did not fit, again in fp32
            transformer.use_fp32_dense_once();
            out_gpu = transformer.compute(batch, in_gpu, mask_gpu);
            cuBERT::memcpyAsync(output, out_gpu, count * sizeof(T), 2, stream);
            cuBERT::cuda_stream_synchronize(stream);
        }
        cuBERT::free(mask_gpu);
        cuBERT::free(in_gpu);
    }
    cuBERT::blas_destroy(blas);
    cuBERT::cuda_stream_destroy(stream);
}

template <typename T>
const void *graph_var(const cuBERT::Graph<T> *g, const char *name, size_t *elements, long long *dims, int max_dims,
                      int *n_dims) {
    auto it = g->var.find(name);
    if (it == g->var.end()) return nullptr;
    if (elements != nullptr) *elements = g->size.at(name);
    const std::vector<long long> &shape = g->shape.at(name);
    if (n_dims != nullptr) *n_dims = (int) shape.size();
    for (int i = 0; dims != nullptr && i < max_dims && i < (int) shape.size(); ++i) dims[i] = shape[i];
    return it->second;
}

}  // namespace

extern "C" {

const char *cubert_last_error(void) { return g_last_error.c_str(); }

int cubert_try_open(const char *model_file, int max_batch_size, int seq_length, int num_hidden_layers,
                    int num_attention_heads, int compute_type, void **model) {
    return guarded([&] {
        *model = cuBERT_open(model_file, max_batch_size, seq_length, num_hidden_layers, num_attention_heads,
                             (cuBERT_ComputeType) compute_type);
    });
}

int cubert_try_compute(void *model, int batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids,
                       void *output, int output_type, int compute_type) {
    return guarded([&] {
        cuBERT_compute(model, batch_size, input_ids, input_mask, segment_ids, output, (cuBERT_OutputType) output_type,
                       (cuBERT_ComputeType) compute_type);
    });
}

int cubert_try_compute_m(void *model, int batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids,
                         cuBERT_Output *output, int compute_type, int output_to_float) {
    return guarded([&] {
        cuBERT_compute_m(model, batch_size, input_ids, input_mask, segment_ids, output,
                         (cuBERT_ComputeType) compute_type, output_to_float);
    });
}

int cubert_try_close(void *model, int compute_type) {
    return guarded([&] { cuBERT_close(model, (cuBERT_ComputeType) compute_type); });
}

namespace {

// tokens joined by '\n' into a caller buffer
void emit_tokens(const std::vector<std::string> &tokens, const char *sep, char *out, size_t capacity, int *n_tokens,
                 size_t *needed) {
    size_t bytes = 1;
    for (const auto &t : tokens) bytes += t.size();
    if (!tokens.empty()) bytes += (tokens.size() - 1) * std::strlen(sep);
    if (n_tokens) *n_tokens = (int) tokens.size();
    if (needed) *needed = bytes;
    if (out == nullptr || capacity < bytes) return;
    char *p = out;
    for (size_t i = 0; i < tokens.size(); ++i) {
        if (i) {
            std::memcpy(p, sep, std::strlen(sep));
            p += std::strlen(sep);
        }
        std::memcpy(p, tokens[i].data(), tokens[i].size());
        p += tokens[i].size();
    }
    *p = 0;
}

}  // namespace

int cubert_try_open_tokenizer(const char *vocab_file, int do_lower_case, void **tokenizer) {
    return guarded([&] {
        if (vocab_file == nullptr || tokenizer == nullptr) throw std::invalid_argument("null argument");
        *tokenizer = cuBERT_open_tokenizer(vocab_file, do_lower_case);
    });
}

int cubert_try_tokenize_compute(void *model, void *tokenizer, int batch_size, const char **text_a, const char **text_b,
                                void *output, int output_type, int compute_type) {
    return guarded([&] {
        cuBERT_tokenize_compute(model, tokenizer, batch_size, text_a, text_b, output, (cuBERT_OutputType) output_type,
                                (cuBERT_ComputeType) compute_type);
    });
}

int cubert_try_tokenize_compute_m(void *model, void *tokenizer, int batch_size, const char **text_a,
                                  const char **text_b, cuBERT_Output *output, int compute_type, int output_to_float) {
    return guarded([&] {
        cuBERT_tokenize_compute_m(model, tokenizer, batch_size, text_a, text_b, output,
                                  (cuBERT_ComputeType) compute_type, output_to_float);
    });
}

int cubert_tokenizer_tokenize(void *tokenizer, int do_lower_case, const char *text, int max_length, char *out,
                              size_t capacity, int *n_tokens, size_t *needed) {
    return guarded([&] {
        if (text == nullptr || max_length < 0) throw std::invalid_argument("text and a non-negative max_length are required");
        std::vector<std::string> tokens;
        if (tokenizer != nullptr) {
            ((const cuBERT::FullTokenizer *) tokenizer)->tokenize(text, &tokens, (size_t) max_length);
        } else {
            cuBERT::BasicTokenizer(do_lower_case != 0).tokenize(text, &tokens, (size_t) max_length);
        }
        emit_tokens(tokens, "\n", out, capacity, n_tokens, needed);
    });
}

int cubert_tokenizer_wordpiece(void *tokenizer, const char *token, char *out, size_t capacity, int *n_tokens,
                               size_t *needed) {
    return guarded([&] {
        if (tokenizer == nullptr || token == nullptr) throw std::invalid_argument("null argument");
        std::vector<std::string> tokens;
        ((const cuBERT::FullTokenizer *) tokenizer)->wordpiece(token, &tokens);
        emit_tokens(tokens, "\n", out, capacity, n_tokens, needed);
    });
}

long long cubert_tokenizer_token_id(void *tokenizer, const char *token) {
    if (tokenizer == nullptr || token == nullptr) return 0;
    return (long long) ((const cuBERT::FullTokenizer *) tokenizer)->convert_token_to_id(token);
}

int cubert_tokenizer_convert_example(void *tokenizer, int max_seq_length, const char *text_a, const char *text_b,
                                     int *input_ids, int8_t *input_mask, int8_t *segment_ids) {
    return guarded([&] {
        if (!tokenizer || !text_a || !input_ids || !input_mask || !segment_ids || max_seq_length < 0) {
            throw std::invalid_argument("null argument");
        }
        ((const cuBERT::FullTokenizer *) tokenizer)->convert_single_example((size_t) max_seq_length, text_a, text_b,
                                                                            input_ids, input_mask, segment_ids);
    });
}

int cubert_tokenizer_char_class(int which, int code_point) {
    switch (which) {
        case 0: return cuBERT::_is_whitespace(code_point);
        case 1: return cuBERT::_is_control(code_point);
        case 2: return cuBERT::_is_punctuation(code_point);
        default: return -1;
    }
}

int cubert_tokenizer_nfd(const char *text, char *out, size_t capacity, size_t *needed) {
    return guarded([&] {
        if (text == nullptr) throw std::invalid_argument("null text");
        std::vector<uint32_t> cps, decomposed;
        const unsigned char *s = (const unsigned char *) text;
        size_t left = std::strlen(text);
        while (left > 0) {
            uint32_t cp;
            const int len = cuBERT::unicode::decode_utf8(s, left, &cp);
            if (len < 0) throw std::invalid_argument("malformed UTF-8");
            cps.push_back(cp);
            s += len;
            left -= (size_t) len;
        }
        cuBERT::unicode::nfd(cps, &decomposed);
        std::vector<std::string> one(1);
        for (uint32_t cp : decomposed) cuBERT::unicode::append_utf8(cp, &one[0]);
        emit_tokens(one, "", out, capacity, nullptr, needed);
    });
}

const char *cubert_tokenizer_unicode_version(void) { return cuBERT::unicode::version(); }

int cubert_model_info(void *model, int compute_type, int *hidden_size, int *num_labels, int *seq_length) {
    return guarded([&] {
        if (model == nullptr) throw std::invalid_argument("null model");
        if (compute_type == cuBERT_COMPUTE_FLOAT) {
            auto *m = (cuBERT::BertM<float> *) model;
            *hidden_size = (int) m->hidden_size(), *num_labels = (int) m->num_labels(), *seq_length = (int) m->seq_length;
        } else {
            auto *m = (cuBERT::BertM<half> *) model;
            *hidden_size = (int) m->hidden_size(), *num_labels = (int) m->num_labels(), *seq_length = (int) m->seq_length;
        }
    });
}

int cubert_bert_create(int dtype, int n_vars, const char *const *names, const void *const *data, int max_batch_size,
                       int seq_length, int vocab_size, int type_vocab_size, int hidden_size, int num_hidden_layers,
                       int num_attention_heads, int intermediate_size, int num_labels, void **bert) {
    return guarded([&] {
        if (dtype == 0) {
            *bert = new cuBERT::Bert<float>(var_map<float>(n_vars, names, data), max_batch_size, seq_length, vocab_size,
                                            type_vocab_size, hidden_size, num_hidden_layers, num_attention_heads,
                                            intermediate_size, num_labels);
        } else {
            *bert = new cuBERT::Bert<half>(var_map<half>(n_vars, names, data), max_batch_size, seq_length, vocab_size,
                                           type_vocab_size, hidden_size, num_hidden_layers, num_attention_heads,
                                           intermediate_size, num_labels);
        }
    });
}

int cubert_bert_compute(void *bert, int dtype, int batch_size, int *input_ids, int8_t *input_mask,
                        int8_t *segment_ids) {
    return guarded([&] {
        if (dtype == 0) ((cuBERT::Bert<float> *) bert)->compute(batch_size, input_ids, input_mask, segment_ids);
        else ((cuBERT::Bert<half> *) bert)->compute(batch_size, input_ids, input_mask, segment_ids);
    });
}

int cubert_bert_output(void *bert, int dtype, int batch_size, cuBERT_Output *output, int output_to_float) {
    return guarded([&] {
        if (dtype == 0) {
            ((cuBERT::Bert<float> *) bert)->output(batch_size, output);
        } else if (output_to_float) {
            ((cuBERT::Bert<half> *) bert)->output_to_float(batch_size, output);
        } else {
            ((cuBERT::Bert<half> *) bert)->output(batch_size, output);
        }
    });
}

int cubert_bert_compute_resident(void *bert, int dtype, int batch_size) {
    return guarded([&] {
        if (dtype == 0) ((cuBERT::Bert<float> *) bert)->compute_resident(batch_size);
        else ((cuBERT::Bert<half> *) bert)->compute_resident(batch_size);
    });
}

int cubert_bert_profile(void *bert, int dtype, unsigned kinds) {
    return guarded([&] {
        if (dtype == 0) ((cuBERT::Bert<float> *) bert)->profile(kinds);
        else ((cuBERT::Bert<half> *) bert)->profile(kinds);
    });
}

int cubert_bert_profile_read(void *bert, int dtype, double *total_ms, int *count, int n_kinds) {
    return guarded([&] {
        if (n_kinds < (int) cuBERT::Profiler::kKinds) throw std::invalid_argument("n_kinds too small");
        if (dtype == 0) ((cuBERT::Bert<float> *) bert)->profile_read(total_ms, count);
        else ((cuBERT::Bert<half> *) bert)->profile_read(total_ms, count);
    });
}

void *cubert_bert_stream(void *bert, int dtype) {
    return dtype == 0 ? ((cuBERT::Bert<float> *) bert)->get_stream() : ((cuBERT::Bert<half> *) bert)->get_stream();
}

int cubert_bert_destroy(void *bert, int dtype) {
    return guarded([&] {
        if (dtype == 0) delete (cuBERT::Bert<float> *) bert;
        else delete (cuBERT::Bert<half> *) bert;
    });
}

int cubert_check_input_range(const int *input_ids, const int8_t *segment_ids, size_t count, size_t vocab_size,
                             size_t type_vocab_size) {
    return guarded([&] {
        if (count > 0 && (input_ids == nullptr || segment_ids == nullptr)) throw std::invalid_argument("null argument");
        cuBERT::check_input_range(input_ids, segment_ids, count, vocab_size, type_vocab_size);
    });
}

long long cubert_open_warmup_batches(const char *setting, size_t max_batch_size, size_t *batches, size_t capacity) {
    const std::vector<size_t> found = cuBERT::open_warmup_batches(setting, max_batch_size);
    for (size_t i = 0; i < found.size() && i < capacity && batches != nullptr; ++i) batches[i] = found[i];
    return (long long) found.size();
}

int cubert_graph_open(const char *model_file, int dtype, void **graph) {
    return guarded([&] {
        if (graph == nullptr || model_file == nullptr) throw std::invalid_argument("null argument");
        *graph = dtype == 0 ? (void *) new cuBERT::Graph<float>(model_file) : (void *) new cuBERT::Graph<half>(model_file);
    });
}

long long cubert_graph_count(void *graph, int dtype) {
    if (graph == nullptr) return -1;
    return dtype == 0 ? (long long) ((cuBERT::Graph<float> *) graph)->var.size()
                      : (long long) ((cuBERT::Graph<half> *) graph)->var.size();
}

const void *cubert_graph_var(void *graph, int dtype, const char *name, size_t *elements, long long *dims,
                             int max_dims, int *n_dims) {
    if (graph == nullptr || name == nullptr) return nullptr;
    return dtype == 0 ? graph_var((const cuBERT::Graph<float> *) graph, name, elements, dims, max_dims, n_dims)
                      : graph_var((const cuBERT::Graph<half> *) graph, name, elements, dims, max_dims, n_dims);
}

int cubert_graph_sizes(void *graph, int dtype, size_t sizes[5]) {
    return guarded([&] {
        if (graph == nullptr || sizes == nullptr) throw std::invalid_argument("null argument");
        auto fill = [&](auto *g) {
            sizes[0] = g->vocab_size;
            sizes[1] = g->type_vocab_size;
            sizes[2] = g->hidden_size;
            sizes[3] = g->intermediate_size;
            sizes[4] = g->num_labels;
        };
        if (dtype == 0) fill((cuBERT::Graph<float> *) graph);
        else fill((cuBERT::Graph<half> *) graph);
    });
}

int cubert_graph_close(void *graph, int dtype) {
    return guarded([&] {
        if (dtype == 0) delete (cuBERT::Graph<float> *) graph;
        else delete (cuBERT::Graph<half> *) graph;
    });
}

int cubert_transformer_run(int dtype, const char *var_prefix, int n_vars, const char *const *names,
                           const void *const *data, int batch_size, int seq_length, int hidden_size,
                           int num_hidden_layers, int num_attention_heads, int intermediate_size, const void *input,
                           const int8_t *mask, void *output) {
    return guarded([&] {
        if (dtype == 0) {
            transformer_run<float>(var_prefix, n_vars, names, data, batch_size, seq_length, hidden_size,
                                   num_hidden_layers, num_attention_heads, intermediate_size, input, mask, output);
        } else {
            transformer_run<half>(var_prefix, n_vars, names, data, batch_size, seq_length, hidden_size,
                                  num_hidden_layers, num_attention_heads, intermediate_size, input, mask, output);
        }
    });
}

}  // extern "C"
