// Attention mask + scale + softmax over scores[batch, heads, seq, seq], and the
// small row softmax used for classifier probabilities.
//
// The reference builds a [batch, heads*seq, seq] tensor of 1.0/0.0 from the
// int8 input mask, copies it into the score buffer every layer, lets the QK
// GEMM compute alpha*QK + (-10000)*that, and then runs five softmax kernels
// (op_att/AttentionMask.cpp:41-54, AttentionSelf.cpp:58-60,99-108,
// op/Softmax.cu:104-115).  Here the int8 mask row of the batch element is read
// directly (seq bytes, cache resident), and one kernel does
//   s = score*scale + (mask==0 ? -10000 : 0);  p = exp(s - max) / sum
// with the row held in registers: the score tensor is read once and written
// once.  fp32 rows divide by the sum like the reference's CPU code
// (op/Softmax.cpp:32-35); fp16 rows multiply by its reciprocal.
//
// A row of seq elements is spread over LPR lanes (a power of two <= 64), each
// holding CH vectors of VEC elements, so short rows pack several to a
// wavefront: seq=32 fp32 -> 8 lanes per row, 8 rows per wavefront.  The mask
// bytes of a lane's columns are re-read per row (seq bytes per batch element,
// L1 resident).

#include "cubert_kernels.h"
#include "device_common.h"

namespace cubert {
namespace {

constexpr float kMaskedScore = -10000.0f;

template <typename T>
__device__ __forceinline__ float normalise(float e, float sum, float inv_sum);
template <>
__device__ __forceinline__ float normalise<float>(float e, float sum, float) { return e / sum; }
template <>
__device__ __forceinline__ float normalise<half_t>(float e, float, float inv_sum) { return e * inv_sum; }

// grid.x: blocks of rows inside one batch element, grid.y: batch element.  Every lane group
// handles one row (one or a few 16-byte loads per lane) and a workgroup is a single wavefront:
// the smallest unit of work per workgroup measured fastest inside the forward pass (64 threads
// vs 256: 108 vs 117 us at batch 64, seq 512; 40.9 vs 44.6 us at batch 256, seq 128).
template <typename T, int VEC, int LPR, int CH, int BLOCK>
__global__ __launch_bounds__(BLOCK) void mask_scale_softmax_kernel(T *__restrict__ scores,
                                                                   const int8_t *__restrict__ mask, float scale,
                                                                   int rows_per_batch) {
    constexpr int S = VEC * LPR * CH;
    constexpr int kGroups = BLOCK / LPR;
    const int group = threadIdx.x / LPR;
    const int gl = threadIdx.x % LPR;
    const int b = blockIdx.y;
    const int row = blockIdx.x * kGroups + group;
    if (row >= rows_per_batch) return;  // whole lane groups leave together
    T *p = scores + ((size_t) b * rows_per_batch + row) * S;

    Vec<T, VEC> raw[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) raw[c] = load_vec<T, VEC>(p + (c * LPR + gl) * VEC);

    float x[CH][VEC];
    float mx = -3.402823466e+38f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        if (mask != nullptr) {
            Vec<int8_t, VEC> m = load_vec<int8_t, VEC>(mask + (size_t) b * S + (c * LPR + gl) * VEC);
#pragma unroll
            for (int i = 0; i < VEC; ++i) x[c][i] = to_f32(raw[c].v[i]) * scale + (m.v[i] ? 0.f : kMaskedScore);
        } else {
#pragma unroll
            for (int i = 0; i < VEC; ++i) x[c][i] = to_f32(raw[c].v[i]) * scale;
        }
#pragma unroll
        for (int i = 0; i < VEC; ++i) mx = fmaxf(mx, x[c][i]);
    }
    mx = group_reduce<LPR>(mx, MaxOp());
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            x[c][i] = __expf(x[c][i] - mx);
            sum += x[c][i];
        }
    }
    sum = group_reduce<LPR>(sum, SumOp());
    const float inv = 1.f / sum;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        Vec<T, VEC> o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) o.v[i] = from_f32<T>(normalise<T>(x[c][i], sum, inv));
        store_vec<T, VEC>(p + (c * LPR + gl) * VEC, o);
    }
}

// Any row length: one wavefront per row, three strided passes over the row.
// `mask_row_div` = rows sharing one mask row (heads*seq), 0 when mask is null.
template <typename T>
__global__ __launch_bounds__(kBlock) void softmax_generic_kernel(const T *__restrict__ in, T *__restrict__ out,
                                                                 const int8_t *__restrict__ mask, float scale,
                                                                 int rows, int channel, int mask_row_div) {
    const int row = blockIdx.x * (kBlock / kWave) + wave_in_block();
    if (row >= rows) return;
    const int lane = threadIdx.x & (kWave - 1);
    const T *x = in + (size_t) row * channel;
    T *y = out + (size_t) row * channel;
    const int8_t *m = mask ? mask + (size_t) (row / mask_row_div) * channel : nullptr;

    float mx = -3.402823466e+38f;
    for (int j = lane; j < channel; j += kWave) {
        float s = to_f32(x[j]) * scale + ((m && !m[j]) ? kMaskedScore : 0.f);
        mx = fmaxf(mx, s);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int j = lane; j < channel; j += kWave) {
        float s = to_f32(x[j]) * scale + ((m && !m[j]) ? kMaskedScore : 0.f);
        sum += __expf(s - mx);
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int j = lane; j < channel; j += kWave) {
        float s = to_f32(x[j]) * scale + ((m && !m[j]) ? kMaskedScore : 0.f);
        y[j] = from_f32<T>(normalise<T>(__expf(s - mx), sum, inv));
    }
}

// Few, very short rows (classifier: channel = number of labels): one thread per row.
template <typename T>
__global__ __launch_bounds__(kBlock) void softmax_tiny_kernel(const T *__restrict__ in, T *__restrict__ out, int rows,
                                                              int channel) {
    const int row = blockIdx.x * kBlock + threadIdx.x;
    if (row >= rows) return;
    const T *x = in + (size_t) row * channel;
    T *y = out + (size_t) row * channel;
    float mx = -3.402823466e+38f;
    for (int j = 0; j < channel; ++j) mx = fmaxf(mx, to_f32(x[j]));
    float sum = 0.f;
    for (int j = 0; j < channel; ++j) sum += __expf(to_f32(x[j]) - mx);
    const float inv = 1.f / sum;
    for (int j = 0; j < channel; ++j) y[j] = from_f32<T>(normalise<T>(__expf(to_f32(x[j]) - mx), sum, inv));
}

template <typename T, int VEC, int LPR, int CH>
int launch_fast(T *scores, const int8_t *mask, float scale, int batch, int rows_per_batch, hipStream_t s) {
    constexpr int kThreads = kWave;
    constexpr int rows_per_block = kThreads / LPR;
    dim3 grid((rows_per_batch + rows_per_block - 1) / rows_per_block, batch), block(kThreads);
    return launch(mask_scale_softmax_kernel<T, VEC, LPR, CH, kThreads>, grid, block, s, scores, mask, scale,
                  rows_per_batch);
}

template <typename T>
int mask_scale_softmax(T *scores, const int8_t *mask, float scale, int batch, int heads, int seq, void *stream) {
    if (batch < 0 || heads <= 0 || seq <= 0 || !scores) return CUBERT_BAD_ARGUMENT;
    if (batch == 0) return 0;
    const long long rows_ll = (long long) batch * heads * seq;
    if (rows_ll > 0x7fffffffLL || batch > 65535) return CUBERT_BAD_ARGUMENT;
    hipStream_t s = (hipStream_t) stream;
    const int rpb = heads * seq;
    constexpr int V = MaxVec<T>::value;
    const bool aligned = is_aligned(scores, 16) && (mask == nullptr || is_aligned(mask, V)) && seq % V == 0;
    if (aligned) {
#define CUBERT_SM_CASE(NVEC, LPR, CH) \
    case NVEC: return launch_fast<T, V, LPR, CH>(scores, mask, scale, batch, rpb, s);
        switch (seq / V) {  // vectors per row
            CUBERT_SM_CASE(1, 1, 1)
            CUBERT_SM_CASE(2, 2, 1)
            CUBERT_SM_CASE(4, 4, 1)
            CUBERT_SM_CASE(8, 8, 1)
            CUBERT_SM_CASE(16, 16, 1)
            CUBERT_SM_CASE(32, 32, 1)
            CUBERT_SM_CASE(64, 64, 1)
            CUBERT_SM_CASE(128, 64, 2)
            CUBERT_SM_CASE(256, 64, 4)
            CUBERT_SM_CASE(12, 4, 3)
            CUBERT_SM_CASE(24, 8, 3)
            CUBERT_SM_CASE(48, 16, 3)   // seq 384 in fp16
            CUBERT_SM_CASE(96, 32, 3)   // seq 384 in fp32
            CUBERT_SM_CASE(192, 64, 3)
            default: break;
        }
#undef CUBERT_SM_CASE
    }
    const int rows = (int) rows_ll;
    dim3 grid((rows + 3) / 4), block(kBlock);
    return launch(softmax_generic_kernel<T>, grid, block, s, (const T *) scores, scores, mask, scale, rows, seq,
                  mask ? rpb : 0);
}

template <typename T>
int row_softmax(const T *in, T *out, int rows, int channel, void *stream) {
    if (rows < 0 || channel <= 0 || !in || !out) return CUBERT_BAD_ARGUMENT;
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    if (channel <= 16) {
        dim3 grid((rows + kBlock - 1) / kBlock), block(kBlock);
        return launch(softmax_tiny_kernel<T>, grid, block, s, in, out, rows, channel);
    }
    dim3 grid((rows + 3) / 4), block(kBlock);
    return launch(softmax_generic_kernel<T>, grid, block, s, in, out, (const int8_t *) nullptr, 1.0f, rows, channel, 0);
}

}  // namespace
}  // namespace cubert

using cubert::half_t;

extern "C" int cubert_mask_scale_softmax_f32(float *scores, const int8_t *mask, float scale, int batch, int heads,
                                             int seq_length, void *stream) {
    return cubert::mask_scale_softmax<float>(scores, mask, scale, batch, heads, seq_length, stream);
}

extern "C" int cubert_mask_scale_softmax_f16(cubert_half *scores, const int8_t *mask, float scale, int batch,
                                             int heads, int seq_length, void *stream) {
    return cubert::mask_scale_softmax<half_t>((half_t *) scores, mask, scale, batch, heads, seq_length, stream);
}

extern "C" int cubert_row_softmax_f32(const float *in, float *out, int rows, int channel, void *stream) {
    return cubert::row_softmax<float>(in, out, rows, channel, stream);
}

extern "C" int cubert_row_softmax_f16(const cubert_half *in, cubert_half *out, int rows, int channel, void *stream) {
    return cubert::row_softmax<half_t>((const half_t *) in, (half_t *) out, rows, channel, stream);
}
