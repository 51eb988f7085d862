// Row kernels that end in a LayerNorm: embedding gather + LayerNorm and
// bias + residual + LayerNorm.  One 64-lane wavefront owns one row of `hidden`
// elements; the row lives in registers between the statistics pass and the
// normalisation, so HBM sees each operand once (2 reads + 1 write per element
// for bias_res_ln, 1 gathered read + 1 write for embed_ln).
//
// Arithmetic follows the reference's CPU code (op/LayerNorm.cpp:20-41):
// sums of x and x*x in fp32, biased variance E[x^2] - mean^2, epsilon 1e-12
// inside the square root, out = beta + gamma * rstd * (x - mean).  The sums are
// tree-reduced across lanes instead of accumulated serially.  A variance that
// cancellation drives below zero is clamped to zero (the reference would take
// the square root of a negative number there).

#include <initializer_list>

#include "cubert_kernels.h"
#include "device_common.h"

namespace cubert {
namespace {

constexpr int kRowsPerBlock = kBlock / kWave;  // 4

__device__ __forceinline__ void ln_stats(float sum, float sumsq, int hidden, float &mean, float &rstd) {
    sum = wave_sum(sum);
    sumsq = wave_sum(sumsq);
    mean = sum / (float) hidden;
    float var = sumsq / (float) hidden - mean * mean;
    var = fmaxf(var, 0.f);
    rstd = 1.f / sqrtf(var + 1e-12f);
}

// One int8 at a wavefront-uniform index, read as the aligned 32-bit word that holds it: a scalar load like the
// one for a row's id, where a byte load would be a vector load whose latency the dependent row address waits for.
// (The word is the element's own aligned 4 bytes, so it cannot reach into an unmapped page.)
__device__ __forceinline__ int uniform_i8(const int8_t *__restrict__ p, int index) {
    const int8_t *at = p + index;
    const int within = (int) (reinterpret_cast<uintptr_t>(at) & 3);
    const uint32_t word = *reinterpret_cast<const uint32_t *>(at - within);
    return (int) (int8_t) (word >> (within * 8));
}

// ---- fast path: hidden == 64 * VEC * CHUNKS, everything 16-byte friendly ----

// Normalise the row held in x[][] and store it.  gamma/beta were loaded before
// the reduction so their latency overlaps it.
// With `split_row` the stored values, times split_scale, also go out as two-term fp16 rows [hi | hi | lo] (hi = fp16(y),
// lo = fp16(y - hi), clamped to the fp16 range), the token operand of a Dense GEMM on the fp16 matrix cores (see split.hip).
template <typename T, int VEC, int CHUNKS>
__device__ __forceinline__ void ln_finish(float (&x)[CHUNKS][VEC], float sum, float sumsq, const Vec<T, VEC> (&g)[CHUNKS],
                                          const Vec<T, VEC> (&b)[CHUNKS], T *__restrict__ out_row, int lane,
                                          half_t *__restrict__ split_row = nullptr, float split_scale = 1.f,
                                          int *__restrict__ overflow = nullptr) {
    constexpr int H = kWave * VEC * CHUNKS;
    float mean, rstd;
    ln_stats(sum, sumsq, H, mean, rstd);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        Vec<T, VEC> o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            o.v[i] = from_f32<T>(to_f32(b[c].v[i]) + (to_f32(g[c].v[i]) * rstd) * (x[c][i] - mean));
        }
        store_vec<T, VEC>(out_row + (c * kWave + lane) * VEC, o);
        if (split_row != nullptr) {  // (uniform)
            Vec<half_t, VEC> hi, lo;
            bool over = false;
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                const float y = to_f32(o.v[i]) * split_scale;
                split_two_terms(y, hi.v[i], lo.v[i]);
                over = over || two_term_overflow(y);
            }
            if (over && overflow != nullptr) *overflow = 1;  // the caller recomputes in fp32
            half_t *at = split_row + (c * kWave + lane) * VEC;
            store_vec<half_t, VEC>(at, hi);
            store_vec<half_t, VEC>(at + H, hi);
            store_vec<half_t, VEC>(at + 2 * H, lo);
        }
    }
}

template <typename T, int VEC, int CHUNKS, bool HAS_BIAS, bool SPLIT = false>
__global__ __launch_bounds__(kBlock) void bias_res_ln_kernel(T *__restrict__ inout, const T *__restrict__ residual,
                                                             const T *__restrict__ bias, const T *__restrict__ beta,
                                                             const T *__restrict__ gamma, int rows,
                                                             half_t *__restrict__ split_out, float split_scale,
                                                             int *__restrict__ overflow) {
    constexpr int H = kWave * VEC * CHUNKS;
    const int row = blockIdx.x * kRowsPerBlock + wave_in_block();
    if (row >= rows) return;
    const int lane = threadIdx.x & (kWave - 1);
    T *io = inout + (size_t) row * H;
    const T *res = residual + (size_t) row * H;

    // every load of the row is issued before the first use
    Vec<T, VEC> a[CHUNKS], r[CHUNKS], bi[CHUNKS], g[CHUNKS], be[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int col = (c * kWave + lane) * VEC;
        a[c] = load_vec<T, VEC>(io + col);
        r[c] = load_vec<T, VEC>(res + col);
    }
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int col = (c * kWave + lane) * VEC;
        if (HAS_BIAS) bi[c] = load_vec<T, VEC>(bias + col);
        g[c] = load_vec<T, VEC>(gamma + col);
        be[c] = load_vec<T, VEC>(beta + col);
    }
    float x[CHUNKS][VEC];
    float sum = 0.f, sumsq = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            // (gemm output + bias) + residual: the order the reference adds them in
            float v = to_f32(a[c].v[i]);
            if (HAS_BIAS) v += to_f32(bi[c].v[i]);
            v += to_f32(r[c].v[i]);
            x[c][i] = v;
            sum += v;
            sumsq += v * v;
        }
    }
    ln_finish<T, VEC, CHUNKS>(x, sum, sumsq, g, be, io, lane, SPLIT ? split_out + (size_t) row * 3 * H : nullptr,
                              split_scale, overflow);
}

// N consecutive floats (N = 2, 4 or 8) with 16-byte loads where N allows.
template <int N>
__device__ __forceinline__ void load_floats(const float *__restrict__ p, float (&out)[N]) {
    if constexpr (N <= 4) {
        const Vec<float, N> x = load_vec<float, N>(p);
#pragma unroll
        for (int i = 0; i < N; ++i) out[i] = x.v[i];
    } else {
        static_assert(N % 4 == 0, "whole 16-byte pieces");
#pragma unroll
        for (int q = 0; q < N / 4; ++q) {
            const Vec<float, 4> x = load_vec<float, 4>(p + q * 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) out[q * 4 + i] = x.v[i];
        }
    }
}

// bias + residual + LayerNorm of a Dense layer that the few-token GEMM left as K slices
// (partials[(slice * R + row) * pitch + col], fp32, R = rows rounded up to 32): the slices are added here, in slice
// order from 0.f, and the
// sum is rounded to the storage type before anything else happens to it -- the value the GEMM's own last workgroup
// would have stored -- so the result has the bits of GEMM followed by bias_res_ln.  At most 64 rows.
template <typename T, int VEC, int CHUNKS, bool HAS_BIAS>
__global__ __launch_bounds__(kBlock) void bias_res_ln_partials_kernel(T *__restrict__ out,
                                                                      const float *__restrict__ partials, int slices,
                                                                      int pitch, const T *__restrict__ residual,
                                                                      const T *__restrict__ bias,
                                                                      const T *__restrict__ beta,
                                                                      const T *__restrict__ gamma, int rows) {
    constexpr int H = kWave * VEC * CHUNKS;
    constexpr int kAhead = CHUNKS * VEC <= 12 ? 8 : 4;  // slices whose loads are in flight together
    const int row = blockIdx.x * (int) (blockDim.x / kWave) + wave_in_block();
    if (row >= rows) return;
    const int lane = threadIdx.x & (kWave - 1);
    const float *prow = partials + (size_t) row * pitch;
    const size_t slice_stride = (size_t) ((rows + 31) / 32 * 32) * pitch;  // whole blocks of 32 token rows per slice
    const T *res = residual + (size_t) row * H;

    Vec<T, VEC> r[CHUNKS], bi[CHUNKS], g[CHUNKS], be[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) r[c] = load_vec<T, VEC>(res + (c * kWave + lane) * VEC);
    float acc[CHUNKS][VEC];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[c][i] = 0.f;
    }
    for (int s0 = 0; s0 < slices; s0 += kAhead) {
        // a slice past the last one is read from slice 0 (a valid address, so the loads go out back to back) and
        // counted as zero
        float p[kAhead][CHUNKS][VEC];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int s = s0 + u < slices ? s0 + u : 0;
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) load_floats<VEC>(prow + s * slice_stride + (c * kWave + lane) * VEC, p[u][c]);
        }
        if (s0 == 0) {
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
                const int col = (c * kWave + lane) * VEC;
                if (HAS_BIAS) bi[c] = load_vec<T, VEC>(bias + col);
                g[c] = load_vec<T, VEC>(gamma + col);
                be[c] = load_vec<T, VEC>(beta + col);
            }
            // (requested here, with the slices: the compiler would otherwise move these loads to where the values are
            // used, behind the loop, one more memory latency at the end of the kernel)
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
                if (HAS_BIAS) pin_registers(bi[c]);
                pin_registers(g[c]);
                pin_registers(be[c]);
            }
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const bool inside = s0 + u < slices;
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
#pragma unroll
                for (int i = 0; i < VEC; ++i) acc[c][i] += u == 0 ? p[u][c][i] : keep_or_zero(p[u][c][i], inside);
            }
        }
    }
    float x[CHUNKS][VEC];
    float sum = 0.f, sumsq = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            float v = to_f32(from_f32<T>(acc[c][i]));  // what the GEMM would have stored
            if (HAS_BIAS) v += to_f32(bi[c].v[i]);
            v += to_f32(r[c].v[i]);
            x[c][i] = v;
            sum += v;
            sumsq += v * v;
        }
    }
    ln_finish<T, VEC, CHUNKS>(x, sum, sumsq, g, be, out + (size_t) row * H, lane);
}

template <typename T, int VEC, int CHUNKS>
__global__ __launch_bounds__(kBlock) void embed_ln_kernel(const int32_t *__restrict__ ids,
                                                          const int8_t *__restrict__ segments,
                                                          const T *__restrict__ word, const T *__restrict__ pos,
                                                          const T *__restrict__ type, const T *__restrict__ beta,
                                                          const T *__restrict__ gamma, T *__restrict__ out, int rows,
                                                          int seq_length) {
    constexpr int H = kWave * VEC * CHUNKS;
    const int row = blockIdx.x * kRowsPerBlock + wave_in_block();
    if (row >= rows) return;
    const int lane = threadIdx.x & (kWave - 1);
    // row is wavefront-uniform, so the id and the segment id arrive through scalar loads; the loads that do not
    // depend on them (position row, gamma, beta) are issued while those two are on their way
    const int id = ids[row];
    const int segment = uniform_i8(segments, row);
    const T *p = pos + (size_t) (row % seq_length) * H;

    Vec<T, VEC> a[CHUNKS], b[CHUNKS], d[CHUNKS], g[CHUNKS], be[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int col = (c * kWave + lane) * VEC;
        b[c] = load_vec<T, VEC>(p + col);
        g[c] = load_vec<T, VEC>(gamma + col);
        be[c] = load_vec<T, VEC>(beta + col);
    }
    asm volatile("" ::: "memory");
    const T *w = word + (size_t) id * H;
    const T *t = type + (size_t) segment * H;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int col = (c * kWave + lane) * VEC;
        a[c] = load_vec<T, VEC>(w + col);
        d[c] = load_vec<T, VEC>(t + col);
    }
    asm volatile("" ::: "memory");  // every load is issued before the first conversion
    float x[CHUNKS][VEC];
    float sum = 0.f, sumsq = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            // (word + position) + token type: the order the reference adds them in
            float v = (to_f32(a[c].v[i]) + to_f32(b[c].v[i])) + to_f32(d[c].v[i]);
            x[c][i] = v;
            sum += v;
            sumsq += v * v;
        }
    }
    ln_finish<T, VEC, CHUNKS>(x, sum, sumsq, g, be, out + (size_t) row * H, lane);
}

// ---- rows of 96 * VEC elements (768 halves, 384 floats): 1.5 wavefront-wide 16-byte vectors ----
// Padding such a row to two loads per lane would leave a quarter of the lanes idle, and splitting
// it into three 8-byte loads doubles the number of memory instructions.  Instead a wavefront takes
// TWO consecutive rows (3072 bytes) as three full 16-byte loads: load 0 is row 0, load 2 is row 1,
// load 1 is row 0 in lanes 0..31 and row 1 in lanes 32..63.  Each row still gets its own statistics
// (four wavefront reductions instead of two).  An odd last row is handled with the second row masked.
template <typename T, int VEC, bool EMBED, bool HAS_BIAS>
__global__ __launch_bounds__(kBlock) void ln_pair_kernel(T *__restrict__ inout, const T *__restrict__ residual,
                                                         const T *__restrict__ bias, const int32_t *__restrict__ ids,
                                                         const int8_t *__restrict__ segments,
                                                         const T *__restrict__ word, const T *__restrict__ pos,
                                                         const T *__restrict__ type, const T *__restrict__ beta,
                                                         const T *__restrict__ gamma, int rows, int seq_length) {
    constexpr int H = 96 * VEC;
    const int row0 = (blockIdx.x * kRowsPerBlock + wave_in_block()) * 2;
    if (row0 >= rows) return;
    const int lane = threadIdx.x & (kWave - 1);
    const bool has_second = row0 + 1 < rows;  // wavefront-uniform
    const bool upper = lane >= 32;            // in load 1 the upper half of the lanes belongs to the second row

    T *dst[1] = {inout + (size_t) row0 * H};
    Vec<T, VEC> a[3], b[3], c[3], g[3], be[3];
    int col[3];
    bool second[3], active[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        const int flat = (k * kWave + lane) * VEC;  // element offset inside the two-row span
        second[k] = k == 2 || (k == 1 && upper);
        col[k] = second[k] ? flat - H : flat;
        active[k] = !second[k] || has_second;
    }
    // Loads are unconditional (a lane whose row does not exist re-reads the first row and is masked out of the
    // sums and the stores below), so nothing stands between the loads of a wavefront.
    if (EMBED) {
        // Wavefront-uniform ids through scalar loads: both rows' ids in one 8-byte load where the pair is aligned
        // (row0 is even), the segment ids as the aligned words that hold them.  The loads that do not depend on
        // them (position rows, gamma, beta) are issued while the ids are on their way.
        const int row1 = has_second ? row0 + 1 : row0;
        int id0, id1;
        if (has_second && is_aligned(ids + row0, 8)) {
            const int2 both = *reinterpret_cast<const int2 *>(ids + row0);
            id0 = both.x;
            id1 = both.y;
        } else {
            id0 = ids[row0];
            id1 = ids[row1];
        }
        const int seg0 = uniform_i8(segments, row0), seg1 = uniform_i8(segments, row1);
        const T *pos0 = pos + (size_t) (row0 % seq_length) * H, *pos1 = pos + (size_t) (row1 % seq_length) * H;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            b[k] = load_vec<T, VEC>((second[k] ? pos1 : pos0) + col[k]);
            g[k] = load_vec<T, VEC>(gamma + col[k]);
            be[k] = load_vec<T, VEC>(beta + col[k]);
        }
        asm volatile("" ::: "memory");
        const T *word0 = word + (size_t) id0 * H, *word1 = word + (size_t) id1 * H;
        const T *type0 = type + (size_t) seg0 * H, *type1 = type + (size_t) seg1 * H;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            a[k] = load_vec<T, VEC>((second[k] ? word1 : word0) + col[k]);
            c[k] = load_vec<T, VEC>((second[k] ? type1 : type0) + col[k]);
        }
    } else {
        // the two rows are adjacent in memory: one base address, the offset inside the two-row span
        const T *gemm_out = inout + (size_t) row0 * H, *res = residual + (size_t) row0 * H;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const int at = active[k] ? (k * kWave + lane) * VEC : col[k];
            a[k] = load_vec<T, VEC>(gemm_out + at);
            c[k] = load_vec<T, VEC>(res + at);
        }
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            if (HAS_BIAS) b[k] = load_vec<T, VEC>(bias + col[k]);
            g[k] = load_vec<T, VEC>(gamma + col[k]);
            be[k] = load_vec<T, VEC>(beta + col[k]);
        }
    }
    // every load above is issued before the first conversion below (loads do not move across this point)
    asm volatile("" ::: "memory");
    float x[3][VEC], s[3], ss[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        s[k] = 0.f;
        ss[k] = 0.f;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            float v = to_f32(a[k].v[i]);
            if (EMBED || HAS_BIAS) v += to_f32(b[k].v[i]);  // (word + position) or (gemm output + bias) first
            v += to_f32(c[k].v[i]);
            x[k][i] = v;
            s[k] += v;
            ss[k] += v * v;
        }
        if (!active[k]) {
            s[k] = 0.f;
            ss[k] = 0.f;
        }
    }
    float mean[2], rstd[2];
    ln_stats(s[0] + (upper ? 0.f : s[1]), ss[0] + (upper ? 0.f : ss[1]), H, mean[0], rstd[0]);
    ln_stats(s[2] + (upper ? s[1] : 0.f), ss[2] + (upper ? ss[1] : 0.f), H, mean[1], rstd[1]);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        const float m = second[k] ? mean[1] : mean[0];
        const float r = second[k] ? rstd[1] : rstd[0];
        Vec<T, VEC> o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) o.v[i] = from_f32<T>(to_f32(be[k].v[i]) + (to_f32(g[k].v[i]) * r) * (x[k][i] - m));
        if (active[k]) store_vec<T, VEC>(dst[0] + (k * kWave + lane) * VEC, o);  // dst rows are adjacent too
    }
}

// ---- generic path: any hidden size, scalar accesses, operands read twice ----

template <typename T, bool EMBED>
__global__ __launch_bounds__(kBlock) void ln_generic_kernel(T *__restrict__ inout, const T *__restrict__ residual,
                                                            const T *__restrict__ bias,
                                                            const int32_t *__restrict__ ids,
                                                            const int8_t *__restrict__ segments,
                                                            const T *__restrict__ word, const T *__restrict__ pos,
                                                            const T *__restrict__ type, const T *__restrict__ beta,
                                                            const T *__restrict__ gamma, int rows, int hidden,
                                                            int seq_length) {
    const int row = blockIdx.x * kRowsPerBlock + wave_in_block();
    if (row >= rows) return;
    const int lane = threadIdx.x & (kWave - 1);
    const T *a, *b, *c;
    if (EMBED) {
        a = word + (size_t) ids[row] * hidden;
        b = pos + (size_t) (row % seq_length) * hidden;
        c = type + (size_t) segments[row] * hidden;
    } else {
        a = inout + (size_t) row * hidden;
        b = bias;  // may be null
        c = residual + (size_t) row * hidden;
    }
    T *o = inout + (size_t) row * hidden;

    float sum = 0.f, sumsq = 0.f;
    for (int j = lane; j < hidden; j += kWave) {
        float x = to_f32(a[j]);
        if (EMBED || b != nullptr) x += to_f32(b[j]);
        x += to_f32(c[j]);
        sum += x;
        sumsq += x * x;
    }
    float mean, rstd;
    ln_stats(sum, sumsq, hidden, mean, rstd);
    for (int j = lane; j < hidden; j += kWave) {
        float x = to_f32(a[j]);
        if (EMBED || b != nullptr) x += to_f32(b[j]);
        x += to_f32(c[j]);
        o[j] = from_f32<T>(to_f32(beta[j]) + (to_f32(gamma[j]) * rstd) * (x - mean));
    }
}

template <typename T>
bool vector_ok(int hidden, int vec, std::initializer_list<const void *> ptrs) {
    if (hidden % (kWave * vec) != 0) return false;
    for (const void *p : ptrs) {
        if (p != nullptr && !is_aligned(p, sizeof(T) * vec)) return false;
    }
    return true;
}

template <typename T>
int bias_res_ln(T *inout, const T *residual, const T *bias, const T *beta, const T *gamma, int rows, int hidden,
                void *stream) {
    if (rows < 0 || hidden <= 0 || !inout || !residual || !beta || !gamma) return CUBERT_BAD_ARGUMENT;
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    dim3 grid((rows + kRowsPerBlock - 1) / kRowsPerBlock), block(kBlock);
    constexpr int V = MaxVec<T>::value;  // 4 floats or 8 halves
    if (hidden == 96 * V && vector_ok<T>(2 * kWave * V, V, {inout, residual, bias, beta, gamma})) {
        dim3 pair_grid(((rows + 1) / 2 + kRowsPerBlock - 1) / kRowsPerBlock);
        if (bias != nullptr)
            return launch(ln_pair_kernel<T, V, false, true>, pair_grid, block, s, inout, residual, bias, nullptr, nullptr,
                          nullptr, nullptr, nullptr, beta, gamma, rows, 1);
        return launch(ln_pair_kernel<T, V, false, false>, pair_grid, block, s, inout, residual, bias, nullptr, nullptr,
                      nullptr, nullptr, nullptr, beta, gamma, rows, 1);
    }
#define CUBERT_LN_CASE(VEC, CHUNKS)                                                                      \
    if (hidden == kWave * VEC * CHUNKS && vector_ok<T>(hidden, VEC, {inout, residual, bias, beta, gamma})) { \
        if (bias != nullptr)                                                                             \
            return launch(bias_res_ln_kernel<T, VEC, CHUNKS, true>, grid, block, s, inout, residual, bias, beta, gamma, \
                          rows, nullptr, 1.f, nullptr);                                                  \
        return launch(bias_res_ln_kernel<T, VEC, CHUNKS, false>, grid, block, s, inout, residual, bias, beta, gamma, \
                      rows, nullptr, 1.f, nullptr);                                                      \
    }
    CUBERT_LN_CASE(V, 1)
    CUBERT_LN_CASE(V, 2)
    CUBERT_LN_CASE(V, 3)
    CUBERT_LN_CASE(V, 4)
    CUBERT_LN_CASE(V / 2, 1)
    CUBERT_LN_CASE(V / 2, 3)  // 768 halves = 64 lanes x 4 x 3
    CUBERT_LN_CASE(V / 2, 5)
    CUBERT_LN_CASE(V / 2, 7)
    CUBERT_LN_CASE(V, 5)
    CUBERT_LN_CASE(V, 6)
    CUBERT_LN_CASE(V, 8)
#undef CUBERT_LN_CASE
    return launch(ln_generic_kernel<T, false>, grid, block, s, inout, residual, bias, nullptr, nullptr, nullptr, nullptr,
                  nullptr, beta, gamma, rows, hidden, 1);
}

// bias + residual + LayerNorm reading the Dense output as the few-token GEMM's K slices; only the register-resident
// shapes of bias_res_ln, anything else is declined and nothing is launched.
template <typename T>
int bias_res_ln_partials(T *out, const float *partials, int slices, int pitch, const T *residual, const T *bias,
                         const T *beta, const T *gamma, int rows, int hidden, void *stream) {
    if (rows < 0 || hidden <= 0 || slices <= 0 || !out || !partials || !residual || !beta || !gamma) {
        return CUBERT_BAD_ARGUMENT;
    }
    if (rows > 64 || pitch < hidden || pitch % 4 != 0 || !is_aligned(partials, 16)) return CUBERT_UNSUPPORTED;
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    // a wavefront per workgroup: what a row waits for is its slices arriving, and a compute unit pulls them at a
    // fraction of what the memory system delivers, so the rows are spread over as many compute units as there are rows
    dim3 grid(rows), block(kWave);
    constexpr int V = MaxVec<T>::value;
#define CUBERT_LN_CASE(VEC, CHUNKS)                                                                              \
    if (hidden == kWave * VEC * CHUNKS && vector_ok<T>(hidden, VEC, {out, residual, bias, beta, gamma})) {       \
        if (bias != nullptr)                                                                                     \
            return launch(bias_res_ln_partials_kernel<T, VEC, CHUNKS, true>, grid, block, s, out, partials, slices, \
                          pitch, residual, bias, beta, gamma, rows);                                             \
        return launch(bias_res_ln_partials_kernel<T, VEC, CHUNKS, false>, grid, block, s, out, partials, slices, \
                      pitch, residual, bias, beta, gamma, rows);                                                 \
    }
    CUBERT_LN_CASE(V, 1)
    CUBERT_LN_CASE(V, 2)
    CUBERT_LN_CASE(V, 3)
    CUBERT_LN_CASE(V, 4)
    CUBERT_LN_CASE(V / 2, 1)
    CUBERT_LN_CASE(V / 2, 3)
    CUBERT_LN_CASE(V / 2, 5)
#undef CUBERT_LN_CASE
    return CUBERT_UNSUPPORTED;
}

// bias + residual + LayerNorm of fp32 rows, in place, and the result again as two-term fp16 rows in split_out
// [rows, 3 * hidden]; only the register-resident shapes (hidden = 256 k), anything else is declined.
int bias_res_ln_split3(float *inout, const float *residual, const float *bias, const float *beta, const float *gamma,
                       int rows, int hidden, float scale, half_t *split_out, int *overflow, void *stream) {
    if (rows < 0 || hidden <= 0 || !inout || !residual || !beta || !gamma || !split_out) return CUBERT_BAD_ARGUMENT;
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    dim3 grid((rows + kRowsPerBlock - 1) / kRowsPerBlock), block(kBlock);
    if (!is_aligned(split_out, 8)) return CUBERT_UNSUPPORTED;
#define CUBERT_LN_SPLIT_CASE(CHUNKS)                                                                                  \
    if (hidden == kWave * 4 * CHUNKS && vector_ok<float>(hidden, 4, {inout, residual, bias, beta, gamma})) {         \
        if (bias != nullptr)                                                                                          \
            return launch(bias_res_ln_kernel<float, 4, CHUNKS, true, true>, grid, block, s, inout, residual, bias, beta, \
                          gamma, rows, split_out, scale, overflow);                                                   \
        return launch(bias_res_ln_kernel<float, 4, CHUNKS, false, true>, grid, block, s, inout, residual, bias, beta,  \
                      gamma, rows, split_out, scale, overflow);                                                       \
    }
    CUBERT_LN_SPLIT_CASE(1)
    CUBERT_LN_SPLIT_CASE(2)
    CUBERT_LN_SPLIT_CASE(3)
    CUBERT_LN_SPLIT_CASE(4)
    CUBERT_LN_SPLIT_CASE(5)
    CUBERT_LN_SPLIT_CASE(6)
    CUBERT_LN_SPLIT_CASE(8)
#undef CUBERT_LN_SPLIT_CASE
    return CUBERT_UNSUPPORTED;
}

template <typename T>
int embed_ln(const int32_t *ids, const int8_t *segments, const T *word, const T *pos, const T *type, const T *beta,
             const T *gamma, T *out, int batch, int seq_length, int hidden, void *stream) {
    if (batch < 0 || seq_length <= 0 || hidden <= 0 || !ids || !segments || !word || !pos || !type || !beta ||
        !gamma || !out)
        return CUBERT_BAD_ARGUMENT;
    const long long rows_ll = (long long) batch * seq_length;
    if (rows_ll > 0x7fffffffLL) return CUBERT_BAD_ARGUMENT;
    const int rows = (int) rows_ll;
    if (rows == 0) return 0;
    hipStream_t s = (hipStream_t) stream;
    dim3 grid((rows + kRowsPerBlock - 1) / kRowsPerBlock), block(kBlock);
    constexpr int V = MaxVec<T>::value;
    if (hidden == 96 * V && vector_ok<T>(2 * kWave * V, V, {word, pos, type, beta, gamma, out})) {
        dim3 pair_grid(((rows + 1) / 2 + kRowsPerBlock - 1) / kRowsPerBlock);
        return launch(ln_pair_kernel<T, V, true, false>, pair_grid, block, s, out, nullptr, nullptr, ids, segments, word,
                      pos, type, beta, gamma, rows, seq_length);
    }
#define CUBERT_EMB_CASE(VEC, CHUNKS)                                                                       \
    if (hidden == kWave * VEC * CHUNKS && vector_ok<T>(hidden, VEC, {word, pos, type, beta, gamma, out})) { \
        return launch(embed_ln_kernel<T, VEC, CHUNKS>, grid, block, s, ids, segments, word, pos, type, beta, gamma, \
                      out, rows, seq_length);                                                              \
    }
    CUBERT_EMB_CASE(V, 1)
    CUBERT_EMB_CASE(V, 2)
    CUBERT_EMB_CASE(V, 3)
    CUBERT_EMB_CASE(V, 4)
    CUBERT_EMB_CASE(V / 2, 1)
    CUBERT_EMB_CASE(V / 2, 3)
    CUBERT_EMB_CASE(V / 2, 5)
    CUBERT_EMB_CASE(V / 2, 7)
    CUBERT_EMB_CASE(V, 5)
    CUBERT_EMB_CASE(V, 6)
    CUBERT_EMB_CASE(V, 8)
#undef CUBERT_EMB_CASE
    return launch(ln_generic_kernel<T, true>, grid, block, s, out, nullptr, nullptr, ids, segments, word, pos, type,
                  beta, gamma, rows, hidden, seq_length);
}

}  // namespace
}  // namespace cubert

using cubert::half_t;

extern "C" int cubert_bias_res_ln_f32(float *inout, const float *residual, const float *bias, const float *beta,
                                      const float *gamma, int rows, int hidden, void *stream) {
    return cubert::bias_res_ln<float>(inout, residual, bias, beta, gamma, rows, hidden, stream);
}

extern "C" int cubert_bias_res_ln_split3_f32(float *inout, const float *residual, const float *bias, const float *beta,
                                             const float *gamma, int rows, int hidden, float scale,
                                             cubert_half *split_out, int *overflow, void *stream) {
    return cubert::bias_res_ln_split3(inout, residual, bias, beta, gamma, rows, hidden, scale,
                                      (cubert::half_t *) split_out, overflow, stream);
}

extern "C" int cubert_bias_res_ln_f16(cubert_half *inout, const cubert_half *residual, const cubert_half *bias,
                                      const cubert_half *beta, const cubert_half *gamma, int rows, int hidden,
                                      void *stream) {
    return cubert::bias_res_ln<half_t>((half_t *) inout, (const half_t *) residual, (const half_t *) bias,
                                       (const half_t *) beta, (const half_t *) gamma, rows, hidden, stream);
}

extern "C" int cubert_bias_res_ln_partials_f32(float *out, const float *partials, int slices, int pitch,
                                               const float *residual, const float *bias, const float *beta,
                                               const float *gamma, int rows, int hidden, void *stream) {
    return cubert::bias_res_ln_partials<float>(out, partials, slices, pitch, residual, bias, beta, gamma, rows, hidden,
                                               stream);
}

extern "C" int cubert_bias_res_ln_partials_f16(cubert_half *out, const float *partials, int slices, int pitch,
                                               const cubert_half *residual, const cubert_half *bias,
                                               const cubert_half *beta, const cubert_half *gamma, int rows, int hidden,
                                               void *stream) {
    return cubert::bias_res_ln_partials<half_t>((half_t *) out, partials, slices, pitch, (const half_t *) residual,
                                                (const half_t *) bias, (const half_t *) beta, (const half_t *) gamma,
                                                rows, hidden, stream);
}

extern "C" int cubert_embed_ln_f32(const int32_t *ids, const int8_t *segments, const float *word, const float *pos,
                                   const float *type, const float *beta, const float *gamma, float *out, int batch,
                                   int seq_length, int hidden, void *stream) {
    return cubert::embed_ln<float>(ids, segments, word, pos, type, beta, gamma, out, batch, seq_length, hidden,
                                   stream);
}

extern "C" int cubert_embed_ln_f16(const int32_t *ids, const int8_t *segments, const cubert_half *word,
                                   const cubert_half *pos, const cubert_half *type, const cubert_half *beta,
                                   const cubert_half *gamma, cubert_half *out, int batch, int seq_length, int hidden,
                                   void *stream) {
    return cubert::embed_ln<half_t>(ids, segments, (const half_t *) word, (const half_t *) pos,
                                    (const half_t *) type, (const half_t *) beta, (const half_t *) gamma,
                                    (half_t *) out, batch, seq_length, hidden, stream);
}
