// Streaming kernels: bias + GELU, bias + tanh, mean over the sequence axis and
// the plain embedding-row gather.  All are one read + one write per element
// with 16-byte accesses; arithmetic in fp32.

#include "cubert_kernels.h"
#include "activations.h"
#include "device_common.h"

namespace cubert {
namespace {

// The GELU functors (erf form, two polynomial variants) live in activations.h.
struct TanhOp {
    // reference: op_bert/BertPooler.cpp:13
    __device__ __forceinline__ float operator()(float x) const { return tanhf(x); }
};

// [rows, width] in place, y = f(x + bias[col]).  One workgroup per row, its threads walk the
// columns (16 bytes per thread per trip), so the bias index needs no division and consecutive
// workgroups stream consecutive memory.  Small workgroups with one or two loads in flight per
// thread measured fastest on this part (several rows per workgroup lost 10 % of the bandwidth).
// width must be a multiple of VEC.
template <typename T, typename Op, int VEC>
__global__ __launch_bounds__(kBlock) void bias_act_kernel(T *__restrict__ inout, const T *__restrict__ bias, int width) {
    T *row = inout + (size_t) blockIdx.x * width;
    Op op;
    for (int col = threadIdx.x * VEC; col < width; col += blockDim.x * VEC) {
        Vec<T, VEC> x = load_vec<T, VEC>(row + col);
        float b[VEC];
        if (bias != nullptr) {
            Vec<T, VEC> bv = load_vec<T, VEC>(bias + col);
#pragma unroll
            for (int i = 0; i < VEC; ++i) b[i] = to_f32(bv.v[i]);
        } else {
#pragma unroll
            for (int i = 0; i < VEC; ++i) b[i] = 0.f;
        }
        Vec<T, VEC> y;
#pragma unroll
        for (int i = 0; i < VEC; ++i) y.v[i] = from_f32<T>(op(to_f32(x.v[i]) + b[i]));
        store_vec<T, VEC>(row + col, y);
    }
}

// The same with the trip count known at compile time (width == TRIPS * blockDim.x * VEC): every load of the
// thread is issued before the first store, which the in-place loop above cannot do (the compiler must keep a
// trip's load behind the previous trip's store to the same array).
template <typename T, typename Op, int VEC, int TRIPS>
__global__ __launch_bounds__(kBlock) void bias_act_unrolled_kernel(T *__restrict__ inout, const T *__restrict__ bias,
                                                                   int width) {
    T *row = inout + (size_t) blockIdx.x * width;
    Op op;
    Vec<T, VEC> x[TRIPS], bv[TRIPS];
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) x[t] = load_vec<T, VEC>(row + (t * blockDim.x + threadIdx.x) * VEC);
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) {
        bv[t] = Vec<T, VEC>{};
        if (bias != nullptr) bv[t] = load_vec<T, VEC>(bias + (t * blockDim.x + threadIdx.x) * VEC);
    }
#pragma unroll
    for (int t = 0; t < TRIPS; ++t) {
        Vec<T, VEC> y;
#pragma unroll
        for (int i = 0; i < VEC; ++i) y.v[i] = from_f32<T>(op(to_f32(x[t].v[i]) + to_f32(bv[t].v[i])));
        store_vec<T, VEC>(row + (t * blockDim.x + threadIdx.x) * VEC, y);
    }
}

// Threads per workgroup so that the column walk has no ragged last trip when possible.
inline int pick_threads(int vectors_per_row) {
    for (int t = kBlock; t >= kWave; t -= kWave) {
        if (vectors_per_row % t == 0) return t;
    }
    return vectors_per_row < kBlock ? ((vectors_per_row + kWave - 1) / kWave) * kWave : kBlock;
}

template <typename T, typename Op>
int bias_act(T *inout, const T *bias, int rows, int width, void *stream) {
    if (rows < 0 || width <= 0 || !inout) return CUBERT_BAD_ARGUMENT;
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    constexpr int V = MaxVec<T>::value;
    if (width % V == 0 && is_aligned(inout, 16) && (bias == nullptr || is_aligned(bias, 16))) {
        const int threads = pick_threads(width / V);
        // measured inside the forward pass: fp32 rows of three trips gain 4 % from the unrolled form (batch 128,
        // seq 32: 17.3 -> 16.6 us); fp16 rows of two trips lose 3-7 % with it, so they keep the loop
        if (sizeof(T) == 4 && width == threads * V * 3) {
            return launch(bias_act_unrolled_kernel<T, Op, V, 3>, dim3(rows), dim3(threads), s, inout, bias, width);
        }
        return launch(bias_act_kernel<T, Op, V>, dim3(rows), dim3(threads), s, inout, bias, width);
    }
    return launch(bias_act_kernel<T, Op, 1>, dim3(rows), dim3(kBlock), s, inout, bias, width);
}

// out[b, c] = mean_s in[b, s, c].  grid = (column tiles, batch); the block's WAVES wavefronts split the
// sequence (each keeps four loads in flight), each lane keeps VEC channel sums, and the partial sums meet in
// LDS in wavefront order.  The launcher picks 8-byte vectors and 16 wavefronts for long sequences so that
// even a small batch puts a few hundred wavefronts on the chip (batch 32, seq 128, hidden 768: 96 workgroups
// of 16 wavefronts instead of 64 of 4).
template <typename T, int VEC, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void mean_pool_kernel(const T *__restrict__ in, T *__restrict__ out,
                                                                  int seq, int hidden) {
    __shared__ float partial[WAVES][kWave * VEC];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = wave_in_block();
    const int col = (blockIdx.x * kWave + lane) * VEC;
    const int b = blockIdx.y;
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    if (col < hidden) {
        const T *p = in + (size_t) b * seq * hidden + col;
        int s = wave;
        for (; s + 3 * WAVES < seq; s += 4 * WAVES) {
            Vec<T, VEC> v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = load_vec<T, VEC>(p + (size_t) (s + u * WAVES) * hidden);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[i] += to_f32(v[u].v[i]);
            }
        }
        for (; s < seq; s += WAVES) {
            Vec<T, VEC> v = load_vec<T, VEC>(p + (size_t) s * hidden);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += to_f32(v.v[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) partial[wave][lane * VEC + i] = acc[i];
    __syncthreads();
    if (wave == 0 && col < hidden) {
        Vec<T, VEC> o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            float t = partial[0][lane * VEC + i];
#pragma unroll
            for (int w = 1; w < WAVES; ++w) t += partial[w][lane * VEC + i];
            o.v[i] = from_f32<T>(t / (float) seq);
        }
        store_vec<T, VEC>(out + (size_t) b * hidden + col, o);
    }
}

template <typename T>
int mean_pool(const T *in, T *out, int batch, int seq, int hidden, void *stream) {
    if (batch < 0 || seq <= 0 || hidden <= 0 || !in || !out || batch > 65535) return CUBERT_BAD_ARGUMENT;
    if (batch == 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    constexpr int V = MaxVec<T>::value / 2;  // 8-byte vectors: twice the column tiles of 16-byte ones
    if (hidden % V == 0 && is_aligned(in, 16) && is_aligned(out, 16)) {
        dim3 grid((hidden / V + kWave - 1) / kWave, batch);
        if (seq >= 64) return launch(mean_pool_kernel<T, V, 16>, grid, dim3(16 * kWave), s, in, out, seq, hidden);
        return launch(mean_pool_kernel<T, V, 4>, grid, dim3(4 * kWave), s, in, out, seq, hidden);
    }
    dim3 grid((hidden + kWave - 1) / kWave, batch);
    return launch(mean_pool_kernel<T, 1, 4>, grid, dim3(4 * kWave), s, in, out, seq, hidden);
}

// out[i, :] = table[ids[i], :]; one wavefront per row.
template <typename T, typename Id, int VEC>
__global__ __launch_bounds__(kBlock) void gather_kernel(const Id *__restrict__ ids, int n, const T *__restrict__ table,
                                                        int width, T *__restrict__ out) {
    const int row = blockIdx.x * (kBlock / kWave) + wave_in_block();
    if (row >= n) return;
    const int lane = threadIdx.x & (kWave - 1);
    const T *src = table + (size_t) ids[row] * width;
    T *dst = out + (size_t) row * width;
    for (int col = lane * VEC; col < width; col += kWave * VEC) {
        store_vec<T, VEC>(dst + col, load_vec<T, VEC>(src + col));
    }
}

template <typename T, typename Id>
int gather(const Id *ids, int n, const T *table, int width, T *out, void *stream) {
    if (n < 0 || width <= 0 || !ids || !table || !out) return CUBERT_BAD_ARGUMENT;
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    constexpr int V = MaxVec<T>::value;
    dim3 grid((n + 3) / 4), block(kBlock);
    if (width % V == 0 && is_aligned(table, 16) && is_aligned(out, 16)) {
        return launch(gather_kernel<T, Id, V>, grid, block, s, ids, n, table, width, out);
    }
    return launch(gather_kernel<T, Id, 1>, grid, block, s, ids, n, table, width, out);
}

// The tail of a classification model in one launch, one workgroup per sequence:
//   pooled = tanh(pooled + pooler_bias)        (skipped when pooler_bias is null: pooled is final already)
//   logits = pooled W^T + out_bias             (W [labels, hidden] row-major; out_bias may be null)
//   probs  = softmax(logits)
// with few labels these are three launch-bound kernels otherwise (bias + tanh, a GEMM with a handful of output
// columns, a row softmax).  pooled and logits are rounded to the storage type before they are used further, as
// the separate kernels store them; the softmax divides by the sum in fp32 and multiplies by its reciprocal in
// fp16, as cubert_row_softmax_* does.
template <typename T>
__global__ __launch_bounds__(kBlock) void classifier_head_kernel(T *__restrict__ pooled, const T *__restrict__ pooler_bias,
                                                                 const T *__restrict__ weights,
                                                                 const T *__restrict__ out_bias, T *__restrict__ logits,
                                                                 T *__restrict__ probs, int hidden, int labels) {
    extern __shared__ float s_row[];  // [hidden] pooled row, then [labels] logits
    float *s_logit = s_row + hidden;
    T *row = pooled + (size_t) blockIdx.x * hidden;
    const int lane = threadIdx.x & (kWave - 1), wave = wave_in_block();
    // the weight row of this wavefront's first label is requested before anything else (rows of up to 1024
    // values; it comes from memory, cold, while the tanh below is computed)
    constexpr int kAhead = 16;
    float w_first[kAhead];
    const bool ahead = wave < labels && hidden <= kAhead * kWave;
#pragma unroll
    for (int t = 0; t < kAhead; ++t) {
        const int j = t * kWave + lane;
        w_first[t] = ahead && j < hidden ? to_f32(weights[(size_t) wave * hidden + j]) : 0.f;
    }
    for (int j = threadIdx.x; j < hidden; j += kBlock) {
        float v = to_f32(row[j]);
        if (pooler_bias != nullptr) {
            const T stored = from_f32<T>(TanhOp()(v + to_f32(pooler_bias[j])));
            row[j] = stored;
            v = to_f32(stored);
        }
        s_row[j] = v;
    }
    __syncthreads();
    for (int l = wave; l < labels; l += kBlock / kWave) {
        const T *w = weights + (size_t) l * hidden;
        float acc = 0.f;
        if (ahead && l == wave) {
#pragma unroll
            for (int t = 0; t < kAhead; ++t) {
                const int j = t * kWave + lane;
                acc += j < hidden ? s_row[j] * w_first[t] : 0.f;
            }
        } else {
            for (int j = lane; j < hidden; j += kWave) acc += s_row[j] * to_f32(w[j]);
        }
        acc = wave_sum(acc);
        if (lane == 0) {
            const T stored = from_f32<T>(acc + (out_bias != nullptr ? to_f32(out_bias[l]) : 0.f));
            logits[(size_t) blockIdx.x * labels + l] = stored;
            s_logit[l] = to_f32(stored);
        }
    }
    __syncthreads();
    if (wave == 0) {
        float mx = -3.402823466e+38f;
        for (int l = lane; l < labels; l += kWave) mx = fmaxf(mx, s_logit[l]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int l = lane; l < labels; l += kWave) sum += __expf(s_logit[l] - mx);
        sum = wave_sum(sum);
        const float inv = 1.f / sum;
        for (int l = lane; l < labels; l += kWave) {
            const float e = __expf(s_logit[l] - mx);
            probs[(size_t) blockIdx.x * labels + l] = from_f32<T>(sizeof(T) == 4 ? e / sum : e * inv);
        }
    }
}

template <typename T>
int classifier_head(T *pooled, const T *pooler_bias, const T *weights, const T *out_bias, T *logits, T *probs,
                    int batch, int hidden, int labels, void *stream) {
    if (batch < 0 || hidden <= 0 || labels <= 0 || !pooled || !weights || !logits || !probs) return CUBERT_BAD_ARGUMENT;
    if (batch == 0) return 0;
    // few labels only: a wavefront walks a whole weight row per label; beyond that a GEMM is the better tool
    const size_t lds = ((size_t) hidden + labels) * sizeof(float);
    if (labels > 64 || lds > 48 * 1024) return CUBERT_UNSUPPORTED;
    return launch_lds(classifier_head_kernel<T>, dim3(batch), dim3(kBlock), (unsigned) lds, (hipStream_t) stream, pooled,
                      pooler_bias, weights, out_bias, logits, probs, hidden, labels);
}

// out[c, r] = in[r, c] for a row-major [rows, cols] matrix: 32 x 32 tiles through LDS so that both the reads
// and the writes are contiguous runs.  Run once per weight matrix when a model is loaded.
template <typename T>
__global__ __launch_bounds__(kBlock) void transpose_kernel(const T *__restrict__ in, int rows, int cols,
                                                           T *__restrict__ out) {
    __shared__ T tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8 threads
    const int r0 = blockIdx.y * 32, c0 = blockIdx.x * 32;
#pragma unroll
    for (int j = ty; j < 32; j += 8) {
        if (r0 + j < rows && c0 + tx < cols) tile[j][tx] = in[(size_t) (r0 + j) * cols + c0 + tx];
    }
    __syncthreads();
#pragma unroll
    for (int j = ty; j < 32; j += 8) {
        if (c0 + j < cols && r0 + tx < rows) out[(size_t) (c0 + j) * rows + r0 + tx] = tile[tx][j];
    }
}

template <typename T>
int transpose(const T *in, int rows, int cols, T *out, void *stream) {
    if (rows < 0 || cols < 0 || !in || !out || in == out) return CUBERT_BAD_ARGUMENT;
    if (rows == 0 || cols == 0) return 0;
    dim3 grid((cols + 31) / 32, (rows + 31) / 32);
    if (grid.y > 65535) return CUBERT_UNSUPPORTED;
    return launch(transpose_kernel<T>, grid, dim3(kBlock), (hipStream_t) stream, in, rows, cols, out);
}

}  // namespace
}  // namespace cubert

using cubert::half_t;

extern "C" int cubert_bias_gelu_f32(float *inout, const float *bias, int rows, int width, void *stream) {
    return cubert::bias_act<float, cubert::GeluOp<float>>(inout, bias, rows, width, stream);
}
extern "C" int cubert_bias_gelu_f16(cubert_half *inout, const cubert_half *bias, int rows, int width, void *stream) {
    return cubert::bias_act<half_t, cubert::GeluOp<half_t>>((half_t *) inout, (const half_t *) bias, rows, width, stream);
}
extern "C" int cubert_bias_tanh_f32(float *inout, const float *bias, int rows, int width, void *stream) {
    return cubert::bias_act<float, cubert::TanhOp>(inout, bias, rows, width, stream);
}
extern "C" int cubert_bias_tanh_f16(cubert_half *inout, const cubert_half *bias, int rows, int width, void *stream) {
    return cubert::bias_act<half_t, cubert::TanhOp>((half_t *) inout, (const half_t *) bias, rows, width, stream);
}
extern "C" int cubert_mean_pool_f32(const float *in, float *out, int batch, int seq_length, int hidden, void *stream) {
    return cubert::mean_pool<float>(in, out, batch, seq_length, hidden, stream);
}
extern "C" int cubert_mean_pool_f16(const cubert_half *in, cubert_half *out, int batch, int seq_length, int hidden,
                                    void *stream) {
    return cubert::mean_pool<half_t>((const half_t *) in, (half_t *) out, batch, seq_length, hidden, stream);
}
extern "C" int cubert_gather_f32(const int32_t *ids, int n, const float *table, int width, float *out, void *stream) {
    return cubert::gather<float, int32_t>(ids, n, table, width, out, stream);
}
extern "C" int cubert_gather_f16(const int32_t *ids, int n, const cubert_half *table, int width, cubert_half *out,
                                 void *stream) {
    return cubert::gather<half_t, int32_t>(ids, n, (const half_t *) table, width, (half_t *) out, stream);
}
extern "C" int cubert_gather_i8_f32(const int8_t *ids, int n, const float *table, int width, float *out,
                                    void *stream) {
    return cubert::gather<float, int8_t>(ids, n, table, width, out, stream);
}
extern "C" int cubert_gather_i8_f16(const int8_t *ids, int n, const cubert_half *table, int width, cubert_half *out,
                                    void *stream) {
    return cubert::gather<half_t, int8_t>(ids, n, (const half_t *) table, width, (half_t *) out, stream);
}
extern "C" int cubert_transpose_f32(const float *in, int rows, int cols, float *out, void *stream) {
    return cubert::transpose<float>(in, rows, cols, out, stream);
}
extern "C" int cubert_transpose_f16(const cubert_half *in, int rows, int cols, cubert_half *out, void *stream) {
    return cubert::transpose<half_t>((const half_t *) in, rows, cols, (half_t *) out, stream);
}
extern "C" int cubert_classifier_head_f32(float *pooled, const float *pooler_bias, const float *weights,
                                          const float *out_bias, float *logits, float *probs, int batch, int hidden,
                                          int labels, void *stream) {
    return cubert::classifier_head<float>(pooled, pooler_bias, weights, out_bias, logits, probs, batch, hidden, labels,
                                          stream);
}
extern "C" int cubert_classifier_head_f16(cubert_half *pooled, const cubert_half *pooler_bias, const cubert_half *weights,
                                          const cubert_half *out_bias, cubert_half *logits, cubert_half *probs, int batch,
                                          int hidden, int labels, void *stream) {
    return cubert::classifier_head<half_t>((half_t *) pooled, (const half_t *) pooler_bias, (const half_t *) weights,
                                           (const half_t *) out_bias, (half_t *) logits, (half_t *) probs, batch, hidden,
                                           labels, stream);
}
