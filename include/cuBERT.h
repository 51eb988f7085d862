/*
 * Public C ABI of the library (libcuBERT.so), binary-compatible with
 * zhihu/cuBERT's src/cuBERT.h:10-97 so that its Python (Cython) and Java (JNA)
 * bindings and C callers keep working unchanged: same symbol names, same
 * argument order and types, same enum values, same cuBERT_Output field order.
 *
 * Conventions (as in the reference):
 *  - a model handle is opaque; the compute_type given to cuBERT_open must be
 *    passed again to cuBERT_compute / cuBERT_compute_m / cuBERT_close;
 *  - input_ids / input_mask / segment_ids are caller-owned host arrays of
 *    batch_size * seq_length elements; outputs are caller-owned host arrays
 *    whose element type is the model's compute type (float, or IEEE binary16
 *    for cuBERT_COMPUTE_HALF unless output_to_float is set);
 *  - a call returns after the results are in the caller's buffers;
 *  - batch_size == 0 is a no-op; batch_size > max_batch_size and other
 *    argument errors throw std::invalid_argument through the C boundary;
 *    device errors print a message and exit the process.
 */
#ifndef CUBERT_PUBLIC_API_H
#define CUBERT_PUBLIC_API_H

#ifdef __cplusplus
#include <cstdint>
#define CUBERT_DEFAULT(x) = x
extern "C" {
#else
#include <stdint.h>
#define CUBERT_DEFAULT(x)
#endif

/* Arithmetic/storage type of a model: fp32 everywhere, or fp16 storage with
 * fp32 arithmetic.            replaces: reference src/cuBERT.h:12-15 */
enum cuBERT_ComputeType {
    cuBERT_COMPUTE_FLOAT = 0,
    cuBERT_COMPUTE_HALF = 1
};

/* Which tensor cuBERT_compute copies out.   replaces: reference src/cuBERT.h:17-23 */
enum cuBERT_OutputType {
    cuBERT_LOGITS = 0,           /* [batch, num_labels]              */
    cuBERT_POOLED_OUTPUT = 1,    /* [batch, hidden]                  */
    cuBERT_SEQUENCE_OUTPUT = 2,  /* [batch, seq_length, hidden]      */
    cuBERT_EMBEDDING_OUTPUT = 3, /* [batch, seq_length, hidden]      */
    cuBERT_PROBS = 4             /* softmax(logits)                  */
};

#ifdef __cplusplus
/* Any subset of outputs in one call; NULL fields are skipped.  Field order is
 * part of the ABI (JNA maps it positionally).  replaces: reference src/cuBERT.h:66-72 */
struct cuBERT_Output {
    void *logits = nullptr;
    void *pooled_output = nullptr;
    void *sequence_output = nullptr;
    void *embedding_output = nullptr;
    void *probs = nullptr;
};
#else
typedef enum cuBERT_ComputeType cuBERT_ComputeType;
typedef enum cuBERT_OutputType cuBERT_OutputType;
typedef struct cuBERT_Output {
    void *logits;
    void *pooled_output;
    void *sequence_output;
    void *embedding_output;
    void *probs;
} cuBERT_Output;
#endif

/* replaces: reference src/cuBERT.h:25-28 */
void cuBERT_initialize();
void cuBERT_finalize();
int cuBERT_get_gpu_count();

/* Load a frozen TensorFlow GraphDef (.pb) and put one model replica on every
 * visible GPU.  hidden / intermediate / vocabulary sizes and num_labels come
 * from the tensor shapes in the file.       replaces: reference src/cuBERT.h:30-35 */
void *cuBERT_open(const char *model_file, int max_batch_size, int seq_length, int num_hidden_layers,
                  int num_attention_heads, cuBERT_ComputeType compute_type CUBERT_DEFAULT(cuBERT_COMPUTE_FLOAT));

/* One forward pass, one output.             replaces: reference src/cuBERT.h:37-44 */
void cuBERT_compute(void *model, int batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids,
                    void *output, cuBERT_OutputType output_type CUBERT_DEFAULT(cuBERT_LOGITS),
                    cuBERT_ComputeType compute_type CUBERT_DEFAULT(cuBERT_COMPUTE_FLOAT));

/* replaces: reference src/cuBERT.h:46-47 */
void cuBERT_close(void *model, cuBERT_ComputeType compute_type CUBERT_DEFAULT(cuBERT_COMPUTE_FLOAT));

/* WordPiece tokenizer + compute on raw text.  replaces: reference src/cuBERT.h:51-62 */
void *cuBERT_open_tokenizer(const char *vocab_file, int do_lower_case CUBERT_DEFAULT(1));
void cuBERT_close_tokenizer(void *tokenizer);
void cuBERT_tokenize_compute(void *model, void *tokenizer, int batch_size, const char **text_a,
                             const char **text_b, void *output,
                             cuBERT_OutputType output_type CUBERT_DEFAULT(cuBERT_LOGITS),
                             cuBERT_ComputeType compute_type CUBERT_DEFAULT(cuBERT_COMPUTE_FLOAT));

/* One forward pass, several outputs.  With output_to_float != 0 a half model
 * writes float arrays.                      replaces: reference src/cuBERT.h:78-85 */
void cuBERT_compute_m(void *model, int batch_size, int *input_ids, int8_t *input_mask, int8_t *segment_ids,
                      cuBERT_Output *output, cuBERT_ComputeType compute_type CUBERT_DEFAULT(cuBERT_COMPUTE_FLOAT),
                      int output_to_float CUBERT_DEFAULT(0));

/* replaces: reference src/cuBERT.h:87-94 */
void cuBERT_tokenize_compute_m(void *model, void *tokenizer, int batch_size, const char **text_a,
                               const char **text_b, cuBERT_Output *output,
                               cuBERT_ComputeType compute_type CUBERT_DEFAULT(cuBERT_COMPUTE_FLOAT),
                               int output_to_float CUBERT_DEFAULT(0));

#ifdef __cplusplus
}
#endif
#undef CUBERT_DEFAULT
#endif /* CUBERT_PUBLIC_API_H */
