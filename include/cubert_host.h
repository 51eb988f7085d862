/*
 * C entry points onto the host classes, for callers that cannot take a C++
 * exception or a C++ object across their FFI (ctypes, JNA, cgo).
 *
 * Two groups:
 *  1. cubert_try_*: the public API of cuBERT.h with the same arguments, but an
 *     argument error (std::invalid_argument, std::out_of_range ...) is caught
 *     and returned as a code; cubert_last_error() gives its message.  The
 *     reference lets such exceptions cross the C boundary and its Cython
 *     binding turns them into Python exceptions (python/_cuBERT.pxd:8-66,
 *     "except +"); a ctypes/JNA caller would abort instead.
 *  2. cubert_bert_* / cubert_transformer_*: the constructors and methods of
 *     cuBERT::Bert<T> (reference src/cuBERT/Bert.h:17-44) and
 *     cuBERT::Transformer<T> (reference src/cuBERT/op_att/Transformer.h:17-39)
 *     taking the weights as parallel arrays of names and host pointers, which
 *     is the reference's std::unordered_map<std::string, T*> spelled in C.
 *     dtype: 0 = float weights/outputs, 1 = binary16 weights/outputs.
 *
 * Return codes: 0 ok, CUBERT_E_INVALID_ARGUMENT (std::invalid_argument),
 * CUBERT_E_OUT_OF_RANGE (std::out_of_range, e.g. a missing weight name),
 * CUBERT_E_OTHER (any other exception).
 */
#ifndef CUBERT_HOST_API_H
#define CUBERT_HOST_API_H

#include <stddef.h>
#include <stdint.h>

#include "cuBERT.h"

#ifdef __cplusplus
extern "C" {
#endif

#define CUBERT_E_INVALID_ARGUMENT 1
#define CUBERT_E_OUT_OF_RANGE 2
#define CUBERT_E_OTHER 3

/* Message of the last error on the calling thread ("" if none). */
const char *cubert_last_error(void);

/* ---- 1. exception-free variants of cuBERT.h -------------------------------- */

/* replaces: cuBERT_open, reference src/cuBERT.cpp:23-44 */
int cubert_try_open(const char *model_file, int max_batch_size, int seq_length, int num_hidden_layers,
                    int num_attention_heads, int compute_type, void **model);
/* replaces: cuBERT_compute, reference src/cuBERT.cpp:46-67 */
int cubert_try_compute(void *model, int batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids,
                       void *output, int output_type, int compute_type);
/* replaces: cuBERT_compute_m, reference src/cuBERT.cpp:69-90 */
int cubert_try_compute_m(void *model, int batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids,
                         cuBERT_Output *output, int compute_type, int output_to_float);
/* The range check cuBERT_compute applies to a request before anything is enqueued: every input id in
 * [0, vocab_size), every segment id in [0, type_vocab_size); CUBERT_E_INVALID_ARGUMENT and a message naming the
 * first offender otherwise.  (The reference indexes its tables unchecked, src/cuBERT/op/Embedding.cpp:16-19.) */
int cubert_check_input_range(const int *input_ids, const int8_t *segment_ids, size_t count, size_t vocab_size,
                             size_t type_vocab_size);
/* The batch sizes a model prepares when it is opened (one forward pass each on made-up inputs, so that a first
 * request of that size does not pay for GEMM planning), as read from the text of the environment variable
 * CUBERT_OPEN_WARMUP (`setting`, NULL = unset): unset = max_batch_size only, which is what the reference prepares
 * (src/cuBERT/Bert.cpp:62-64); "0" = none; else a comma-separated list of batch sizes in which "max" stands for
 * max_batch_size, e.g. "1,8,max".  Entries outside [1, max_batch_size] are named on stderr and skipped.  Writes up
 * to `capacity` sizes to `batches` in the order they will run and returns how many there are.  CPU only. */
long long cubert_open_warmup_batches(const char *setting, size_t max_batch_size, size_t *batches, size_t capacity);
/* replaces: cuBERT_close, reference src/cuBERT.cpp:92-102 */
int cubert_try_close(void *model, int compute_type);
/* Shape facts of an opened model (hidden size, labels, seq_length) for sizing output arrays. */
int cubert_model_info(void *model, int compute_type, int *hidden_size, int *num_labels, int *seq_length);
/* replaces: Graph<T>::Graph(filename) and the public members of Graph<T>, reference
 * src/cuBERT/tensorflow/Graph.h:10-23, Graph.cpp:13-91: the float and binary16 constants of a frozen GraphDef
 * converted to dtype (0 float, 1 binary16), by node name.  CPU only.  cubert_graph_var gives the host pointer the
 * graph owns (NULL for an unknown name), the number of elements it holds and, when dims != NULL, up to max_dims
 * dimensions of the declared shape (*n_dims receives the rank).  The dimensions are the file's declaration, the
 * element count is what the file holds (bytes of tensor_content; a value list repeated up to the declared size; a
 * declared shape with no data at all read as zeros): the two may disagree for a malformed file, as in the reference
 * (Graph.cpp:50-56), and a model is checked against the shapes it needs when it is built.  cubert_graph_sizes gives vocab_size,
 * type_vocab_size, hidden_size, intermediate_size and num_labels in that order. */
int cubert_graph_open(const char *model_file, int dtype, void **graph);
long long cubert_graph_count(void *graph, int dtype);
const void *cubert_graph_var(void *graph, int dtype, const char *name, size_t *elements, long long *dims,
                             int max_dims, int *n_dims);
int cubert_graph_sizes(void *graph, int dtype, size_t sizes[5]);
int cubert_graph_close(void *graph, int dtype);
/* replaces: cuBERT_open_tokenizer, reference src/cuBERT.cpp:104-106 */
int cubert_try_open_tokenizer(const char *vocab_file, int do_lower_case, void **tokenizer);
/* replaces: cuBERT_tokenize_compute / cuBERT_tokenize_compute_m, reference src/cuBERT.cpp:216-280 */
int cubert_try_tokenize_compute(void *model, void *tokenizer, int batch_size, const char **text_a, const char **text_b,
                                void *output, int output_type, int compute_type);
int cubert_try_tokenize_compute_m(void *model, void *tokenizer, int batch_size, const char **text_a,
                                  const char **text_b, cuBERT_Output *output, int compute_type, int output_to_float);

/* ---- 1b. the tokenizer by itself (CPU only; no counterpart in the reference's C API, which reaches these
 *          only through cuBERT_tokenize_compute) ---------------------------------------------------------- */

/* FullTokenizer::tokenize (reference src/cuBERT/tokenization.cpp:218-228), or with tokenizer == NULL
 * BasicTokenizer(do_lower_case)::tokenize (tokenization.cpp:116-183).  The tokens are written to `out` separated
 * by '\n' (a token never contains white space) and NUL terminated; *n_tokens receives their number and *needed
 * the bytes required including the NUL.  When `capacity` is too small nothing is written and the call still
 * returns 0: call again with a buffer of *needed bytes. */
int cubert_tokenizer_tokenize(void *tokenizer, int do_lower_case, const char *text, int max_length, char *out,
                              size_t capacity, int *n_tokens, size_t *needed);
/* WordpieceTokenizer::tokenize on one basic token (tokenization.cpp:186-216); output as above. */
int cubert_tokenizer_wordpiece(void *tokenizer, const char *token, char *out, size_t capacity, int *n_tokens,
                               size_t *needed);
/* FullTokenizer::convert_token_to_id (tokenization.h:131-139): 0 and a message on stderr for an unknown token. */
long long cubert_tokenizer_token_id(void *tokenizer, const char *token);
/* convert_single_example (src/cuBERT.cpp:137-214): [CLS] a [SEP] (b [SEP]) -> ids, mask, segment ids, padded
 * to max_seq_length entries each.  text_b may be NULL. */
int cubert_tokenizer_convert_example(void *tokenizer, int max_seq_length, const char *text_a, const char *text_b,
                                     int *input_ids, int8_t *input_mask, int8_t *segment_ids);
/* _is_whitespace / _is_control / _is_punctuation (tokenization.cpp:84-94): which = 0 / 1 / 2. */
int cubert_tokenizer_char_class(int which, int code_point);
/* NFD of a UTF-8 string (what utf8proc_NFD gives the reference, tokenization.cpp:123-125); output as for
 * cubert_tokenizer_tokenize without separators.  Returns 1 (invalid argument) for malformed UTF-8. */
int cubert_tokenizer_nfd(const char *text, char *out, size_t capacity, size_t *needed);
/* Version of the Unicode database the tables were generated from, e.g. "13.0.0". */
const char *cubert_tokenizer_unicode_version(void);

/* ---- 2. host classes ------------------------------------------------------- */

/* replaces: Bert<T>::Bert(var, ...), reference src/cuBERT/Bert.cpp:8-65 */
int cubert_bert_create(int dtype, int n_vars, const char *const *names, const void *const *data, int max_batch_size,
                       int seq_length, int vocab_size, int type_vocab_size, int hidden_size, int num_hidden_layers,
                       int num_attention_heads, int intermediate_size, int num_labels, void **bert);
/* replaces: Bert<T>::compute, reference src/cuBERT/Bert.cpp:98-136 (asynchronous) */
int cubert_bert_compute(void *bert, int dtype, int batch_size, int *input_ids, int8_t *input_mask,
                        int8_t *segment_ids);
/* replaces: Bert<T>::output / output_to_float, reference src/cuBERT/Bert.cpp:185-259 (synchronises) */
int cubert_bert_output(void *bert, int dtype, int batch_size, cuBERT_Output *output, int output_to_float);
/* The forward pass again on the inputs the last cubert_bert_compute left on the device (no host copies;
 * asynchronous).  No counterpart in the reference: it is the device-resident step throughput is quoted on. */
int cubert_bert_compute_resident(void *bert, int dtype, int batch_size);
/* Per-kernel timing with stream events: bit k of `kinds` switches kind k on (0 embed+LN, 1 bias+residual+LN,
 * 2 bias+GELU, 3 mask+scale+softmax, 4 bias+tanh, 5 mean pool, 6 row softmax, 7 dense GEMM, 8 attention GEMM,
 * 9 fused attention, 10 classifier head, 11 two-term operand rows; 12-16 the Dense GEMMs one by one: Q|K|V,
 * attention output, intermediate, output, pooler -- a Dense launch is timed under its own kind when that is on and
 * under kind 7 otherwise).  cubert_bert_profile_read synchronises, adds the elapsed milliseconds and launch counts
 * seen since the last read to total_ms[kind] / count[kind] (arrays of n_kinds >= 17 entries) and forgets them. */
int cubert_bert_profile(void *bert, int dtype, unsigned kinds);
int cubert_bert_profile_read(void *bert, int dtype, double *total_ms, int *count, int n_kinds);
/* The HIP stream the model's work is enqueued on. */
void *cubert_bert_stream(void *bert, int dtype);
int cubert_bert_destroy(void *bert, int dtype);

/* replaces: Transformer<T>::Transformer + compute, reference src/cuBERT/op_att/Transformer.cpp:8-132,145-175.
 * `input` [batch, seq, hidden] and `mask` [batch, seq] are host arrays, `output` a host array of the
 * input's size; the call copies in, runs the encoder stack, copies out and synchronises. */
int cubert_transformer_run(int dtype, const char *var_prefix, int n_vars, const char *const *names,
                           const void *const *data, int batch_size, int seq_length, int hidden_size,
                           int num_hidden_layers, int num_attention_heads, int intermediate_size, const void *input,
                           const int8_t *mask, void *output);

#ifdef __cplusplus
}
#endif
#endif /* CUBERT_HOST_API_H */
