// fp32 operands as sums of two fp16 numbers, for Dense layers of fp32 models computed on the fp16 matrix cores.
//
//   x = hi + lo + r,   hi = fp16(x),  lo = fp16(x - hi),  |r| <= 2^-22 |x|   (x - hi is exact in fp32)
//
// so  sum_k a_k w_k = sum_k (ah_k wh_k + ah_k wl_k + al_k wh_k) + O(2^-22) per product: the dropped al*wl term and
// the two r's are each below 2^-22 of the product, the size of the rounding of the fp32 accumulation that follows in
// either arithmetic.  The three sums are one GEMM over a reduction axis of three times the length: activation rows
// are stored [hi | hi | lo], weight rows [hi | lo | hi] (fp16), products accumulate in fp32 and the result is fp32.
// The fp16 matrix-core rate of this part is 16 times its fp32 rate, so the threefold GEMM is still several times
// faster (reference Dense: src/cuBERT/op/Dense.cpp:47-57, one fp32 GEMM).
//
// Range: fp16 holds |hi| <= 65504, and lo loses bits once it is subnormal (a scaled value below 2^-3 leaves an
// absolute error of up to 2^-25).  Both sides are therefore multiplied by a power of two before they are taken
// apart (`scale`, exact, taken out again by the GEMM's alpha): weights per matrix, so that the largest is in
// [512, 1024) and their size does not matter; activations by a fixed factor chosen by the caller (the host classes
// use 16: full accuracy for rows whose entries are of order 2^-7 to 2^12), clamped to the fp16 range beyond it.
// A value that had to be clamped (or is not a number) no longer equals its two terms: every kernel that writes
// two-term rows takes an `overflow` pointer (may be null) and stores 1 there when that happens -- an ordinary store by
// the lanes concerned, nothing otherwise -- so that the caller can recompute in fp32 instead of using a wrong product.

#include "cubert_kernels.h"
#include "activations.h"
#include "device_common.h"

namespace cubert {
namespace {

struct IdentityOp {
    __device__ __forceinline__ float operator()(float x) const { return x; }
};

// out[row] = [hi | hi | lo] (LO_IN_MIDDLE: [hi | lo | hi]) of scale * f(in[row] + bias), each part `width` halves.
// One workgroup per row, threads walk the columns 8 at a time: two 16-byte loads, three 16-byte stores.
template <typename Op, bool LO_IN_MIDDLE>
__global__ __launch_bounds__(kBlock) void split3_kernel(const float *__restrict__ in, const float *__restrict__ bias,
                                                         int width, float scale, half_t *__restrict__ out,
                                                         int *__restrict__ overflow) {
    const float *row = in + (size_t) blockIdx.x * width;
    half_t *dst = out + (size_t) blockIdx.x * 3 * width;
    Op op;
    bool over = false;
    for (int col = threadIdx.x * 8; col < width; col += blockDim.x * 8) {
        const Vec<float, 4> x0 = load_vec<float, 4>(row + col), x1 = load_vec<float, 4>(row + col + 4);
        Vec<float, 4> b0 = {}, b1 = {};
        if (bias != nullptr) {
            b0 = load_vec<float, 4>(bias + col);
            b1 = load_vec<float, 4>(bias + col + 4);
        }
        Vec<half_t, 8> hi, lo;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float y0 = op(x0.v[i] + b0.v[i]) * scale, y1 = op(x1.v[i] + b1.v[i]) * scale;
            split_two_terms(y0, hi.v[i], lo.v[i]);
            split_two_terms(y1, hi.v[4 + i], lo.v[4 + i]);
            over = over || two_term_overflow(y0) || two_term_overflow(y1);
        }
        store_vec<half_t, 8>(dst + col, hi);
        store_vec<half_t, 8>(dst + width + col, LO_IN_MIDDLE ? lo : hi);
        store_vec<half_t, 8>(dst + 2 * width + col, LO_IN_MIDDLE ? hi : lo);
    }
    if (over && overflow != nullptr) *overflow = 1;
}

// any width and alignment
template <typename Op, bool LO_IN_MIDDLE>
__global__ __launch_bounds__(kBlock) void split3_scalar_kernel(const float *__restrict__ in,
                                                                const float *__restrict__ bias, int width, float scale,
                                                                half_t *__restrict__ out, int *__restrict__ overflow) {
    const float *row = in + (size_t) blockIdx.x * width;
    half_t *dst = out + (size_t) blockIdx.x * 3 * width;
    Op op;
    bool over = false;
    for (int col = threadIdx.x; col < width; col += blockDim.x) {
        half_t hi, lo;
        const float y = op(row[col] + (bias != nullptr ? bias[col] : 0.f)) * scale;
        split_two_terms(y, hi, lo);
        over = over || two_term_overflow(y);
        dst[col] = hi;
        dst[width + col] = LO_IN_MIDDLE ? lo : hi;
        dst[2 * width + col] = LO_IN_MIDDLE ? hi : lo;
    }
    if (over && overflow != nullptr) *overflow = 1;
}

template <typename Op, bool LO_IN_MIDDLE>
int split3(const float *in, const float *bias, int rows, int width, float scale, half_t *out, int *overflow,
           void *stream) {
    if (rows < 0 || width <= 0 || !in || !out) return CUBERT_BAD_ARGUMENT;
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    if (width % 8 == 0 && is_aligned(in, 16) && is_aligned(out, 16) && (bias == nullptr || is_aligned(bias, 16))) {
        const int vectors = width / 8;
        const int threads = vectors >= kBlock ? kBlock : ((vectors + kWave - 1) / kWave) * kWave;
        return launch(split3_kernel<Op, LO_IN_MIDDLE>, dim3(rows), dim3(threads), s, in, bias, width, scale, out,
                      overflow);
    }
    return launch(split3_scalar_kernel<Op, LO_IN_MIDDLE>, dim3(rows), dim3(kBlock), s, in, bias, width, scale, out,
                  overflow);
}

}  // namespace
}  // namespace cubert

extern "C" int cubert_split3_f32(const float *in, int rows, int width, float scale, int lo_in_middle, cubert_half *out,
                                 int *overflow, void *stream) {
    using namespace cubert;
    return lo_in_middle ? split3<IdentityOp, true>(in, nullptr, rows, width, scale, (half_t *) out, overflow, stream)
                        : split3<IdentityOp, false>(in, nullptr, rows, width, scale, (half_t *) out, overflow, stream);
}

extern "C" int cubert_bias_gelu_split3_f32(const float *in, const float *bias, int rows, int width, float scale,
                                           cubert_half *out, int *overflow, void *stream) {
    using namespace cubert;
    return split3<GeluOp<float>, false>(in, bias, rows, width, scale, (half_t *) out, overflow, stream);
}
