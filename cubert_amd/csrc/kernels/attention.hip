// The two attention contractions as single launches over every (batch, head) problem:
//   scores[b, a, q, k] = alpha * sum_j Q[b, q, a, j] * K[b, k, a, j]
//   ctx[b, q, a, j]    = sum_k P[b, a, q, k] * V[b, k, a, j]
// Q, K, V are column blocks of the packed projection output (row stride `ld`), scores / P are
// [batch, heads, seq, seq].  The (b, a) problems sit at two different strides (b: seq*ld, a: head
// size), which a strided-batched library GEMM cannot express, so the library path needs
// min(batch, heads) launches per contraction; here a problem is addressed from blockIdx.
//
// All kernels run on the matrix cores: a wavefront accumulates 32x32 tiles with
// v_mfma_f32_32x32x16_f16 (fp16 storage) or v_mfma_f32_32x32x2_f32 (fp32 storage), fp32 accumulation.
// An MFMA sums over its K slots in whatever order the operands name them, as long as A and B agree,
// so the two lane halves (hh = lane / 32) are given whatever split of the reduction axis makes their
// 16-byte operand fetches land where memory likes them.
//   * scores, seq < 128 (or wide head rows): one wavefront = 32 queries x 32..128 keys, operands straight
//     from global memory, no LDS.
//   * scores, seq >= 128: a workgroup owns a 128 x 128 tile; the 128 query rows and 128 key rows of the head
//     are loaded once with coalesced 16-byte loads (all issued before the first LDS write) and kept in LDS;
//     each wavefront computes a 64 x 64 sub-tile as 2 x 2 MFMA tiles with A = key rows, B = query rows, so a
//     lane ends up with 4 consecutive keys of one query; results are staged in LDS and leave as full rows.
//   * context: A = 32 rows of P from global memory (the big operand, read exactly once), B = V^T, staged
//     transposed in LDS once per workgroup ([head_size][seq + pad]) because an MFMA B operand needs
//     consecutive k for a fixed column and V is stored with consecutive columns.

#include <atomic>
#include <cstdlib>
#include <initializer_list>
#include <string>

#include "cubert_kernels.h"
#include "device_common.h"

namespace cubert {
namespace {

typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef float v16f32 __attribute__((ext_vector_type(16)));

// One accumulation step on a 32x32 tile from a 16-byte operand vector per lane.
template <typename T>
struct Mma;

template <>
struct Mma<half_t> {
    static constexpr int kVec = 8;  // 8 halves: one v_mfma_f32_32x32x16_f16
    static __device__ __forceinline__ void run(v16f32 &acc, const Vec<half_t, 8> &a, const Vec<half_t, 8> &b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8f16, a), __builtin_bit_cast(v8f16, b), acc, 0,
                                                     0, 0);
    }
};

template <>
struct Mma<float> {
    static constexpr int kVec = 4;  // 4 floats: four v_mfma_f32_32x32x2_f32
    static __device__ __forceinline__ void run(v16f32 &acc, const Vec<float, 4> &a, const Vec<float, 4> &b) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[i], b.v[i], acc, 0, 0, 0);
    }
};

// Accumulator register i of lane (r = lane % 32, hh = lane / 32) is element (row, col) of the tile:
__device__ __forceinline__ int acc_row(int i, int hh) { return (i >> 2) * 8 + hh * 4 + (i & 3); }

// Where the context goes when it is wanted in two-term form (fp32 models whose Dense layers run on the fp16 matrix
// cores): width = 0 means the ordinary store.
struct SplitOut {
    int width = 0;            // halves per part of a row [hi | hi | lo]
    float scale = 1.f;        // applied before the value is taken apart
    int *overflow = nullptr;  // set to 1 when a scaled value is outside the fp16 range (or not a number); may be null
};

// One element of the attention context.  split.width = 0: ctx[row, col] in the storage type.  split.width = W > 0
// (fp32 only): `ctx` is really a buffer of halves with rows [hi | hi | lo] of W each, the two-term form of
// split.scale * v that the Dense GEMM on the fp16 matrix cores reads (hi = fp16(.), lo = fp16(. - hi), clamped to
// the fp16 range; a value that had to be clamped raises split.overflow, and the caller recomputes in fp32).
// (SPLIT is a compile-time choice so that the plain kernels are exactly what they were without it.)
template <typename T, bool SPLIT>
__device__ __forceinline__ void store_context(T *ctx, int ld_ctx, size_t row, int col, float v, const SplitOut &split) {
    if constexpr (SPLIT) {
        // v as the plain kernel would store it: rounded to fp32 before it is taken apart (without this the compiler
        // fuses a product that made v into the subtraction below, and lo would belong to the unrounded value)
        asm volatile("" : "+v"(v));
        v *= split.scale;
        half_t *p = reinterpret_cast<half_t *>(ctx) + row * 3 * split.width + col;
        half_t hi, lo;
        split_two_terms(v, hi, lo);
        if (two_term_overflow(v) && split.overflow != nullptr) *split.overflow = 1;
        p[0] = hi;
        p[split.width] = hi;
        p[2 * split.width] = lo;
    } else {
        ctx[row * ld_ctx + col] = from_f32<T>(v);
    }
}

// grid = (seq / 32 query tiles, key super-tiles, batch * heads); a wavefront computes 32 queries x (32 * NT) keys.
template <typename T, int D, int NT>
__global__ __launch_bounds__(kBlock) void attention_scores_kernel(const T *__restrict__ q, const T *__restrict__ k,
                                                                  int ld, T *__restrict__ scores, float alpha, int seq,
                                                                  int heads) {
    constexpr int V = Mma<T>::kVec;
    constexpr int kSteps = D / 2 / V;
    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5;
    const int bh = blockIdx.z;
    const int b = bh / heads, h = bh - b * heads;
    const int q0 = blockIdx.x * 32;
    const int key0 = (blockIdx.y * (blockDim.x >> 6) + wave_in_block()) * (32 * NT);
    if (key0 >= seq) return;

    const size_t head_off = (size_t) h * D + hh * (D / 2);
    const T *q_row = q + ((size_t) b * seq + q0 + r) * ld + head_off;
    Vec<T, V> a[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; ++t) a[t] = load_vec<T, V>(q_row + t * V);

    v16f32 acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const T *k_row = k + ((size_t) b * seq + key0 + nt * 32 + r) * ld + head_off;
        Vec<T, V> bv[kSteps];
#pragma unroll
        for (int t = 0; t < kSteps; ++t) bv[t] = load_vec<T, V>(k_row + t * V);
        v16f32 c = {};
#pragma unroll
        for (int t = 0; t < kSteps; ++t) Mma<T>::run(c, a[t], bv[t]);
        acc[nt] = c;
    }

    // lane holds key column r of each tile and 16 query rows
    T *out = scores + ((size_t) bh * seq + q0) * seq + key0 + r;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            out[(size_t) acc_row(i, hh) * seq + nt * 32] = from_f32<T>(acc[nt][i] * alpha);
        }
    }
}

// grid = (ceil(seq / 128) query blocks, ceil(seq / 128) key blocks, batch * heads); 256 threads.
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void attention_scores_tiled_kernel(const T *__restrict__ q,
                                                                        const T *__restrict__ k, int ld,
                                                                        T *__restrict__ scores, float alpha, int seq,
                                                                        int heads) {
    constexpr int V = Mma<T>::kVec;
    constexpr int kSteps = D / (2 * V);
    constexpr int kPitch = D + V;                          // operand row pitch (+16 bytes: conflict-free 16-byte reads)
    constexpr int kOutPitch = 64 + 8 / (int) sizeof(T);    // staged output row pitch (+8 bytes)
    constexpr int kOperands = 2 * 128 * kPitch, kStage = 4 * 64 * kOutPitch;
    __shared__ __align__(16) T lds[kOperands > kStage ? kOperands : kStage];
    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5, wave = wave_in_block();
    const int bh = blockIdx.z;
    const int b = bh / heads, h = bh - b * heads;
    const int q0 = blockIdx.x * 128, k0 = blockIdx.y * 128;

    // rows 0..127 of the staging area are queries, 128..255 keys; rows past the sequence are zero
    constexpr int kVecPerRow = D / V;
    constexpr int kLoads = kVecPerRow;  // 256 rows * kVecPerRow vectors / 256 threads
    Vec<T, V> x[kLoads];
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int idx = threadIdx.x + u * kBlock;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        const bool is_key = row >= 128;
        const int src_row = (is_key ? k0 - 128 : q0) + row;
        x[u] = Vec<T, V>{};
        if (src_row < seq) {
            x[u] = load_vec<T, V>((is_key ? k : q) + ((size_t) b * seq + src_row) * ld + (size_t) h * D + c * V);
        }
    }
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int idx = threadIdx.x + u * kBlock;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        store_vec<T, V>(lds + row * kPitch + c * V, x[u]);
    }
    __syncthreads();

    const T *s_q = lds, *s_k = lds + 128 * kPitch;
    const int wq = wave >> 1, wk = wave & 1;
    v16f32 acc[2][2];  // [key tile][query tile]
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = v16f32{};
    }
#pragma unroll
    for (int t = 0; t < kSteps; ++t) {
        // reduction slot s of step t in lane half hh is head column t*2V + hh*V + s
        Vec<T, V> ak[2], bq[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            ak[i] = load_vec<T, V>(s_k + (wk * 64 + i * 32 + r) * kPitch + t * 2 * V + hh * V);
            bq[i] = load_vec<T, V>(s_q + (wq * 64 + i * 32 + r) * kPitch + t * 2 * V + hh * V);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) Mma<T>::run(acc[i][j], ak[i], bq[j]);
        }
    }
    __syncthreads();  // every wavefront is done with the operands: the space now stages the output

    // lane owns query j*32 + r and, per accumulator group g, keys i*32 + g*8 + hh*4 .. +3
    T *stage = lds + wave * 64 * kOutPitch;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                Vec<T, 4> o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o.v[e] = from_f32<T>(acc[i][j][g * 4 + e] * alpha);
                store_vec<T, 4>(stage + (j * 32 + r) * kOutPitch + i * 32 + g * 8 + hh * 4, o);
            }
        }
    }
    // The same wavefront reads back what it staged; LDS operations of one wavefront complete in order.
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
    constexpr int kChunks = 64 / V;        // 16-byte chunks per staged row
    constexpr int kRowsPerPass = kWave / kChunks;
    const int chunk = lane % kChunks, row_in = lane / kChunks;
    const int q_base = q0 + wq * 64, k_base = k0 + wk * 64;
    if (k_base + chunk * V < seq) {  // seq is a multiple of 32, so a chunk is all inside or all outside
#pragma unroll
        for (int pass = 0; pass < 64 / kRowsPerPass; ++pass) {
            const int row = row_in + kRowsPerPass * pass;
            if (q_base + row < seq) {
                store_vec<T, V>(scores + ((size_t) bh * seq + q_base + row) * seq + k_base + chunk * V,
                                load_vec<T, V>(stage + row * kOutPitch + chunk * V));
            }
        }
    }
}

// grid = (query-tile groups, batch * heads); dynamic LDS = D * (seq + pad) elements.
template <typename T, int D>
__global__ __launch_bounds__(kBlock) void attention_context_kernel(const T *__restrict__ probs, const T *__restrict__ v,
                                                                   int ld, T *__restrict__ ctx, int ld_ctx, int seq,
                                                                   int heads, int q_tiles_per_block) {
    extern __shared__ __align__(16) unsigned char smem[];
    T *vt = reinterpret_cast<T *>(smem);  // V^T: [D][pitch]
    constexpr int V = Mma<T>::kVec;
    constexpr int kColTiles = D / 32;
    constexpr int kPrefetch = 4;  // P vectors in flight per lane
    const int pitch = seq + V;    // +16 bytes: conflict-free 16-byte reads down a column of V^T
    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5;
    const int bh = blockIdx.y;
    const int b = bh / heads, h = bh - b * heads;

    // Stage V[b, :, h, :] transposed.  A thread takes one head column j and V consecutive keys: V element loads
    // (consecutive threads = consecutive j: coalesced), one 16-byte LDS write.
    const T *v_head = v + (size_t) b * seq * ld + (size_t) h * D;
    for (int idx = threadIdx.x; idx < (seq / V) * D; idx += blockDim.x) {
        const int j = idx % D, kg = idx / D;
        Vec<T, V> x;
#pragma unroll
        for (int i = 0; i < V; ++i) x.v[i] = v_head[(size_t) (kg * V + i) * ld + j];
        store_vec<T, V>(vt + j * pitch + kg * V, x);
    }
    __syncthreads();

    const int waves = blockDim.x >> 6;
    const int q_tiles = seq / 32;
    int qt_end = (blockIdx.x + 1) * q_tiles_per_block;
    if (qt_end > q_tiles) qt_end = q_tiles;
    const int steps = seq / (2 * V);  // reduction slot s of step t in lane half hh is key t*2V + hh*V + s
    for (int qt = blockIdx.x * q_tiles_per_block + wave_in_block(); qt < qt_end; qt += waves) {
        const T *p_row = probs + ((size_t) bh * seq + qt * 32 + r) * seq + hh * V;
        v16f32 acc[kColTiles];
#pragma unroll
        for (int jt = 0; jt < kColTiles; ++jt) acc[jt] = v16f32{};
        for (int t0 = 0; t0 < steps; t0 += kPrefetch) {
            Vec<T, V> a[kPrefetch];
#pragma unroll
            for (int u = 0; u < kPrefetch; ++u) {
                a[u] = Vec<T, V>{};
                if (t0 + u < steps) a[u] = load_vec<T, V>(p_row + (t0 + u) * 2 * V);
            }
#pragma unroll
            for (int u = 0; u < kPrefetch; ++u) {
                if (t0 + u < steps) {
#pragma unroll
                    for (int jt = 0; jt < kColTiles; ++jt) {
                        Mma<T>::run(acc[jt], a[u], load_vec<T, V>(vt + (jt * 32 + r) * pitch + (t0 + u) * 2 * V + hh * V));
                    }
                }
            }
        }
        // lane holds output column jt*32 + r and 16 query rows
        T *out = ctx + ((size_t) b * seq + qt * 32) * ld_ctx + (size_t) h * D + r;
#pragma unroll
        for (int jt = 0; jt < kColTiles; ++jt) {
#pragma unroll
            for (int i = 0; i < 16; ++i) out[(size_t) acc_row(i, hh) * ld_ctx + jt * 32] = from_f32<T>(acc[jt][i]);
        }
    }
}

// ---- whole attention core in one launch for short sequences (seq <= 128) ----
// ctx = softmax(alpha * Q K^T + mask) V per (batch, head) without the [batch, heads, seq, seq] tensor ever
// leaving the registers.  A workgroup owns one (batch, head) problem: its seq/32 wavefronts take 32 queries
// each and share K, V and the mask, staged once in LDS by coalesced loads that are all issued up front.
// The score tiles are computed transposed (A = key rows, B = query rows), so lane (r, hh) ends up with query
// r and 16 keys per key tile: the softmax statistics of a query are an in-lane reduction plus one exchange
// with lane r + 32.  The lane's probabilities are then exactly the A operand slots of the second contraction:
// a reduction slot may be any key as long as the B operand names the same key, so V is staged transposed
// ([head column][key]) with the keys permuted into slot order and a lane's B operand is one 16-byte LDS read.
// P never moves.  Scores stay in fp32 (the three-kernel path rounds them to the storage type when it stores
// them; the difference is within the fp16 storage tolerance), probabilities are rounded to the storage type as
// the matrix-core operand they are.
constexpr float kMaskedScore = -10000.0f;
constexpr float kLog2e = 1.4426950408889634f;

// A probability from its exponential: times the reciprocal of the row's sum (one division per query instead of one
// per score; at 128 sequences x 12 heads x 32 keys in fp32 the divisions were 0.7 us of a 12.4 us launch).  Within
// 1.5 units in the last place of the quotient the reference forms (src/cuBERT/op/Softmax.cpp:32-35).
template <typename T>
__device__ __forceinline__ float normalise_prob(float e, float, float inv_sum) {
    return e * inv_sum;
}

// LDS bytes of attention_fused_kernel<T, D, KT>: K rows, V^T rows (both padded by 16 bytes), additive mask.
template <typename T, int D, int KT>
constexpr size_t fused_lds_bytes() {
    constexpr int V = 16 / sizeof(T), S = KT * 32;
    return (size_t) S * (D + V) * sizeof(T) + (size_t) D * (S + V) * sizeof(T) + S * sizeof(float);
}

// grid = batch * heads workgroups of KT wavefronts; seq = 32 * KT.
template <typename T, int D, int KT, bool SPLIT>
__global__ __launch_bounds__(KT * kWave) void attention_fused_kernel(const T *__restrict__ q, const T *__restrict__ k,
                                                                     const T *__restrict__ v, int ld,
                                                                     const int8_t *__restrict__ mask,
                                                                     T *__restrict__ ctx, int ld_ctx, float alpha,
                                                                     int heads, SplitOut split) {
    constexpr int V = Mma<T>::kVec;
    constexpr int kSteps = D / 2 / V;
    constexpr int kColTiles = D / 32;
    constexpr int S = KT * 32;
    constexpr int kThreads = KT * kWave;
    constexpr int kPitchK = D + V;  // +16 bytes: conflict-free 16-byte reads down a column of rows
    constexpr int kPitchV = S + V;
    extern __shared__ __align__(16) unsigned char smem[];
    T *s_k = reinterpret_cast<T *>(smem);                 // [S][kPitchK]
    T *s_vt = s_k + S * kPitchK;                          // [D][kPitchV], keys in slot order
    float *s_mask = reinterpret_cast<float *>(s_vt + D * kPitchV);  // [S] additive mask

    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5;
    const int qt = wave_in_block();
    const int bh = blockIdx.x;
    const int b = bh / heads, h = bh - b * heads;
    const T *k_head = k + (size_t) b * S * ld + (size_t) h * D;
    const T *v_head = v + (size_t) b * S * ld + (size_t) h * D;

    // this wavefront's query operand, straight from memory: lane half hh takes head columns hh*D/2 .. +D/2
    const T *q_row = q + ((size_t) b * S + qt * 32 + r) * ld + (size_t) h * D + hh * (D / 2);
    Vec<T, V> qv[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; ++t) qv[t] = load_vec<T, V>(q_row + t * V);

    // K: S rows of D/V vectors.  V^T: for head column j and slot group (kt, u, half) the V keys
    // kt*32 + acc_row(u*V + e, half), e < V, go to positions kt*32 + u*2V + half*V + e of row j.
    constexpr int kVecPerRow = D / V;
    constexpr int kLoadsK = S * kVecPerRow / kThreads;    // = D / V / 2
    constexpr int kGroups = S / V;                        // slot groups per head column
    constexpr int kLoadsV = kGroups * D / kThreads;       // = D / V / 2
    Vec<T, V> kreg[kLoadsK], vreg[kLoadsV];
#pragma unroll
    for (int u = 0; u < kLoadsK; ++u) {
        const int idx = threadIdx.x + u * kThreads;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        kreg[u] = load_vec<T, V>(k_head + (size_t) row * ld + c * V);
    }
#pragma unroll
    for (int u = 0; u < kLoadsV; ++u) {
        const int idx = threadIdx.x + u * kThreads;
        const int j = idx % D, grp = idx / D;             // consecutive threads: consecutive columns (coalesced)
        const int kt = grp / (32 / V), in_tile = grp % (32 / V);
        const int run = in_tile >> 1, half = in_tile & 1;
#pragma unroll
        for (int e = 0; e < V; ++e) {
            vreg[u].v[e] = v_head[(size_t) (kt * 32 + acc_row(run * V + e, half)) * ld + j];
        }
    }
    for (int i = threadIdx.x; i < S; i += kThreads) {
        s_mask[i] = (mask != nullptr && !mask[(size_t) b * S + i]) ? kMaskedScore * kLog2e : 0.f;
    }
#pragma unroll
    for (int u = 0; u < kLoadsK; ++u) {
        const int idx = threadIdx.x + u * kThreads;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        store_vec<T, V>(s_k + row * kPitchK + c * V, kreg[u]);
    }
    __syncthreads();  // K and the mask are in LDS; the V loads are still in flight

    // scores^T[key, query]
    v16f32 p[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        v16f32 c = {};
#pragma unroll
        for (int t = 0; t < kSteps; ++t) {
            Mma<T>::run(c, load_vec<T, V>(s_k + (kt * 32 + r) * kPitchK + hh * (D / 2) + t * V), qv[t]);
        }
        p[kt] = c;
    }

    // register i of tile kt: key kt*32 + acc_row(i, hh), query qt*32 + r.  Scores are kept in units of log 2
    // (t = s * log2 e): scale, change of base and mask are one multiply-add, exp(s - max) one v_exp_f32.
    const float scale = alpha * kLog2e;
    float mx = -3.402823466e+38f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const Vec<float, 4> m = load_vec<float, 4>(s_mask + kt * 32 + g * 8 + hh * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float sc = fmaf(p[kt][g * 4 + e], scale, m.v[e]);
                p[kt][g * 4 + e] = sc;
                mx = fmaxf(mx, sc);
            }
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    float sum = 0.f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            p[kt][i] = __builtin_amdgcn_exp2f(p[kt][i] - mx);
            sum += p[kt][i];
        }
    }
    sum += __shfl_xor(sum, 32, kWave);
    const float inv = 1.f / sum;

    // V^T goes to LDS only now: its loads had the whole score and softmax phase to arrive
#pragma unroll
    for (int u = 0; u < kLoadsV; ++u) {
        const int idx = threadIdx.x + u * kThreads;
        const int j = idx % D, grp = idx / D;
        store_vec<T, V>(s_vt + j * kPitchV + grp * V, vreg[u]);
    }
    __syncthreads();

    // ctx[query, column]: A slots = this lane's probabilities, B = the same keys of V^T row (column) jt*32 + r
    v16f32 out[kColTiles];
#pragma unroll
    for (int jt = 0; jt < kColTiles; ++jt) out[jt] = v16f32{};
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int run = 0; run < 16 / V; ++run) {
            Vec<T, V> a;
#pragma unroll
            for (int e = 0; e < V; ++e) a.v[e] = from_f32<T>(normalise_prob<T>(p[kt][run * V + e], sum, inv));
#pragma unroll
            for (int jt = 0; jt < kColTiles; ++jt) {
                Mma<T>::run(out[jt], a,
                            load_vec<T, V>(s_vt + (jt * 32 + r) * kPitchV + kt * 32 + run * 2 * V + hh * V));
            }
        }
    }
    // lane holds output column jt*32 + r and 16 query rows
    const size_t first_row = (size_t) b * S + qt * 32;
#pragma unroll
    for (int jt = 0; jt < kColTiles; ++jt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            store_context<T, SPLIT>(ctx, ld_ctx, first_row + acc_row(i, hh), h * D + jt * 32 + r, out[jt][i], split);
        }
    }
}

// ---- the same for fp16 storage with the ordinary-instruction work cut down ----
// Counters on attention_fused_kernel<half> at 128 keys showed the vector ALU, not memory or the matrix cores, as its
// busiest unit: 13 ordinary instructions per score.  This variant computes the same thing with about 5:
//  * key tiles (32 keys) are classified from the mask row, read as 32-bit words with scalar loads: a tile whose keys
//    are all masked is left out of the arithmetic altogether when the sequence has an unmasked key -- a
//    masked key's exp is exactly 0 in fp32 there; a tile whose keys are all kept needs no mask term, so its maximum
//    is taken over the raw products and scale, change of base and the subtraction of the maximum are one
//    multiply-add in front of v_exp_f32; only tiles with kept and masked keys (at most one per sequence with a
//    prefix mask), and every tile of a sequence without any kept key (there the shift cancels, as in the
//    reference), take the general path of attention_fused_kernel;
//  * the row sums come out of the matrix cores: the unnormalised probabilities (rounded to fp16, the operand type)
//    are multiplied with a tile of ones next to V, which leaves every query's sum in the accumulator layout of the
//    context tiles, where the division by it is 32 multiplications per lane instead of 64 plus 64 additions;
//  * V is loaded like K, with coalesced 16-byte loads, and kept in LDS as it is in memory ([key][head column]); the
//    B operand of P V (8 keys of one head column per lane) is transposed on its way out of LDS by two
//    ds_read_b64_tr_b16 (gfx950): in a group of 16 lanes, lane i names 4 consecutive columns of row i / 4 at column
//    block i % 4 of a 4 x 16 patch, and lane j receives column j of the patch, rows 0..3.  (The general kernel
//    gathers V^T from memory with 32 two-byte loads per thread; that gather was measured to cost 6-16 us of 65-77
//    at 256 sequences x 16 heads x 128 keys.)  Rows of V are pitched so that the four rows of a patch fall on
//    different banks;
//  * the context tile leaves through LDS as full 128-byte row segments (4 stores per lane instead of 32 two-byte
//    ones).
// Needs the mask (if any) readable as words and ctx rows 16-byte aligned; the launcher falls back otherwise.
typedef _Float16 v4f16 __attribute__((ext_vector_type(4)));

// ds_read_b64_tr_b16: see the comment above for what arrives in which lane.
__device__ __forceinline__ v4f16 lds_read_transposed(const half_t *p) {
    typedef short v4i16 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4i16 lds_v4i16;
    return __builtin_bit_cast(v4f16, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4i16 *) p));
}

// Halves per row of V in LDS: the 32 lanes of a lane half read 4 rows x 64 bytes at once, which fall on different
// banks when the pitch is an odd multiple of 64 bytes (64 banks of 4 bytes).
template <int D>
constexpr int fused_half_v_pitch() {
    return ((D * 2 + 63) / 128 * 128 + 64) / 2;
}

// LDS bytes of attention_fused_half_kernel<D, KT>: K rows (padded by 16 bytes), V rows, additive mask.
template <int D, int KT>
constexpr size_t fused_half_lds_bytes() {
    constexpr int S = KT * 32;
    return (size_t) S * (D + 8) * 2 + (size_t) S * fused_half_v_pitch<D>() * 2 + S * sizeof(float);
}

template <int D, int KT>
__global__ __launch_bounds__(KT * kWave) void attention_fused_half_kernel(const half_t *__restrict__ q,
                                                                          const half_t *__restrict__ k,
                                                                          const half_t *__restrict__ v, int ld,
                                                                          const int8_t *__restrict__ mask,
                                                                          half_t *__restrict__ ctx, int ld_ctx,
                                                                          float alpha, int heads) {
    typedef half_t T;
    constexpr int V = 8;
    constexpr int kSteps = D / 2 / V;
    constexpr int kColTiles = D / 32;
    constexpr int S = KT * 32;
    constexpr int kThreads = KT * kWave;
    constexpr int kPitchK = D + V;
    constexpr int kPitchV = fused_half_v_pitch<D>();  // halves per row of V
    constexpr int kPitchOut = D + V;  // staged context rows: +16 bytes keeps rows 4 apart on different banks
    constexpr unsigned kAllTiles = (1u << KT) - 1u;
    extern __shared__ __align__(16) unsigned char smem[];
    T *s_k = reinterpret_cast<T *>(smem);                 // [S][kPitchK]; later the staged context tiles
    T *s_v = s_k + S * kPitchK;                           // [S][kPitchV], as in memory
    float *s_mask = reinterpret_cast<float *>(s_v + S * kPitchV);  // [S] additive mask

    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5;
    const int qt = wave_in_block();
    const int bh = blockIdx.x;
    const int b = bh / heads, h = bh - b * heads;
    const T *k_head = k + (size_t) b * S * ld + (size_t) h * D;
    const T *v_head = v + (size_t) b * S * ld + (size_t) h * D;

    const T *q_row = q + ((size_t) b * S + qt * 32 + r) * ld + (size_t) h * D + hh * (D / 2);
    Vec<T, V> qv[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; ++t) qv[t] = load_vec<T, V>(q_row + t * V);

    constexpr int kVecPerRow = D / V;
    constexpr int kLoads = S * kVecPerRow / kThreads;     // = D / V / 2 vectors per thread, for K and for V
    Vec<T, V> kreg[kLoads], vreg[kLoads];
    // (every tile is loaded, also those the mask will leave out: with at most 128 keys a workgroup's time is a
    // chain of latencies, and loads that wait for the mask words would add one more link to it)
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int idx = threadIdx.x + u * kThreads;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        kreg[u] = load_vec<T, V>(k_head + row * ld + c * V);
    }
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int idx = threadIdx.x + u * kThreads;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        vreg[u] = load_vec<T, V>(v_head + row * ld + c * V);
    }

    // bit kt of keep_any: tile kt has a kept key; of keep_all: all of its keys are kept (workgroup-uniform)
    unsigned keep_any = kAllTiles, keep_all = kAllTiles;
    if (mask != nullptr) {
        const uint32_t *words = reinterpret_cast<const uint32_t *>(mask + (size_t) b * S);
        keep_any = 0, keep_all = 0;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            uint32_t any = 0, every = 0x80808080u;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t w = words[kt * 8 + i];
                any |= w;
                every &= ((w & 0x7f7f7f7fu) + 0x7f7f7f7fu) | w;  // bit 7 of a byte: that byte is not zero
            }
            keep_any |= (any != 0 ? 1u : 0u) << kt;
            keep_all |= ((every & 0x80808080u) == 0x80808080u ? 1u : 0u) << kt;
        }
        if (keep_any == 0) keep_any = kAllTiles;  // no kept key at all: every tile, general path
    }
    if (!(alpha > 0.f)) keep_all = 0;             // the shortcut takes the maximum before scaling
    keep_any = __builtin_amdgcn_readfirstlane(keep_any);
    keep_all = __builtin_amdgcn_readfirstlane(keep_all);

    const bool general_tiles = (keep_any & ~keep_all) != 0;  // uniform
    if (general_tiles) {
        for (int i = threadIdx.x; i < S; i += kThreads) {
            s_mask[i] = !mask[(size_t) b * S + i] ? kMaskedScore * kLog2e : 0.f;  // (mask is not null here)
        }
    }
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int idx = threadIdx.x + u * kThreads;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        store_vec<T, V>(s_k + row * kPitchK + c * V, kreg[u]);
    }
    __syncthreads();  // K and the mask are in LDS; the V loads are still in flight

    // scores^T[key, query], in p[kt]: raw products for an all-kept tile, log2-unit masked scores for a general one
    const float scale = alpha * kLog2e;
    v16f32 p[KT];
    float mx = -3.402823466e+38f;
    // (The empty asm statements keep the workgroup-uniform tests below as branches: folded into selects, both sides
    // of each would be computed for every score.)
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        if ((keep_any >> kt) & 1u) {
            asm volatile("");
            v16f32 c = {};
#pragma unroll
            for (int t = 0; t < kSteps; ++t) {
                Mma<T>::run(c, load_vec<T, V>(s_k + (kt * 32 + r) * kPitchK + hh * (D / 2) + t * V), qv[t]);
            }
            if ((keep_all >> kt) & 1u) {
                asm volatile("");
                float raw = c[0];
#pragma unroll
                for (int i = 1; i < 16; ++i) raw = fmaxf(raw, c[i]);
                mx = fmaxf(mx, raw * scale);
            } else {
                asm volatile("");
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const Vec<float, 4> m = load_vec<float, 4>(s_mask + kt * 32 + g * 8 + hh * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float sc = fmaf(c[g * 4 + e], scale, m.v[e]);
                        c[g * 4 + e] = sc;
                        mx = fmaxf(mx, sc);
                    }
                }
            }
            p[kt] = c;
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float shift = -mx;

    // V goes to LDS only now: its loads had the whole score phase to arrive
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int idx = threadIdx.x + u * kThreads;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        store_vec<T, V>(s_v + row * kPitchV + c * V, vreg[u]);
    }
    __syncthreads();  // (also: every wavefront is done with K, whose space the context tiles use below)

    // ctx[query, column] and, in `total`, every query's sum of probabilities: A slots = this lane's unnormalised
    // probabilities, B = the same keys of column jt*32 + r of V, or ones.  The lane's slots of step (kt, run) are
    // keys kt*32 + run*16 + hh*4 + {0..3} and the same + 8: one transposing read each.  In its group of 16 lanes
    // (group g: columns (g & 1) * 16 .. + 15, lane half g >> 1), lane i names row i / 4 and column block i % 4.
    const int tr_group = lane >> 4, tr_i = lane & 15;
    const T *tr_base = s_v + ((tr_group >> 1) * 4 + (tr_i >> 2)) * kPitchV + (tr_group & 1) * 16 + (tr_i & 3) * 4;
    v16f32 out[kColTiles], total = {};
#pragma unroll
    for (int jt = 0; jt < kColTiles; ++jt) out[jt] = v16f32{};
    Vec<T, V> ones;
#pragma unroll
    for (int e = 0; e < V; ++e) ones.v[e] = (T) 1.f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        if (!((keep_any >> kt) & 1u)) continue;
        asm volatile("");
        Vec<T, V> a[16 / V];
        if ((keep_all >> kt) & 1u) {
            asm volatile("");
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                a[i / V].v[i % V] = from_f32<T>(__builtin_amdgcn_exp2f(fmaf(p[kt][i], scale, shift)));
            }
        } else {
            asm volatile("");
#pragma unroll
            for (int i = 0; i < 16; ++i) a[i / V].v[i % V] = from_f32<T>(__builtin_amdgcn_exp2f(p[kt][i] + shift));
        }
#pragma unroll
        for (int run = 0; run < 16 / V; ++run) {
#pragma unroll
            for (int jt = 0; jt < kColTiles; ++jt) {
                const T *at = tr_base + (kt * 32 + run * 16) * kPitchV + jt * 32;
                Vec<T, V> bv;
                const v4f16 lo = lds_read_transposed(at), hi = lds_read_transposed(at + 8 * kPitchV);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    bv.v[e] = lo[e];
                    bv.v[4 + e] = hi[e];
                }
                Mma<T>::run(out[jt], a[run], bv);
            }
            Mma<T>::run(total, a[run], ones);
        }
    }

    // lane holds output column jt*32 + r of 16 query rows and, in total[i], the sum of row acc_row(i, hh)
    T *stage = s_k + qt * 32 * kPitchOut;  // this wavefront's 32 x D tile
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float inv = __builtin_amdgcn_rcpf(total[i]);
#pragma unroll
        for (int jt = 0; jt < kColTiles; ++jt) {
            stage[acc_row(i, hh) * kPitchOut + jt * 32 + r] = from_f32<T>(out[jt][i] * inv);
        }
    }
    // the same wavefront reads back what it staged; LDS operations of one wavefront complete in order
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_wave_barrier();
    constexpr int kChunks = D / V;             // 16-byte chunks per row
    constexpr int kRowsPerPass = kWave / kChunks;
    const int chunk = lane % kChunks, row_in = lane / kChunks;
    T *dst = ctx + ((size_t) b * S + qt * 32) * ld_ctx + (size_t) h * D + chunk * V;
#pragma unroll
    for (int pass = 0; pass < 32 / kRowsPerPass; ++pass) {
        const int row = row_in + kRowsPerPass * pass;
        store_vec<T, V>(dst + row * ld_ctx, load_vec<T, V>(stage + row * kPitchOut + chunk * V));
    }
}

// ---- seq = 32, head size 64, few (batch, head) problems: four wavefronts per problem ----
// With fewer problems than compute units the one-wavefront kernel above is a chain of latencies: 32 dependent
// matrix instructions per contraction in fp32.  Here the four wavefronts of a workgroup split the work of one
// problem: each takes a quarter of the head columns of Q K^T (operands straight from memory, every element is
// used by one lane only), the four partial score tiles are added in wavefront order through LDS, every
// wavefront repeats the (cheap) softmax, and P V is split into (column tile, key half), the two key halves
// meeting in LDS again.  Same arithmetic and rounding as attention_fused_kernel, other summation order.
template <typename T, bool SPLIT>
__global__ __launch_bounds__(4 * kWave) void attention_small_kernel(const T *__restrict__ q, const T *__restrict__ k,
                                                                    const T *__restrict__ v, int ld,
                                                                    const int8_t *__restrict__ mask,
                                                                    T *__restrict__ ctx, int ld_ctx, float alpha,
                                                                    int heads, SplitOut split) {
    constexpr int D = 64, S = 32;
    constexpr int V = Mma<T>::kVec;
    constexpr int kSteps = D / 8 / V;  // operand vectors per lane and contraction: a quarter of D over two lane halves
    __shared__ float s_part[4][16 * kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5;
    const int w = wave_in_block();
    const int bh = blockIdx.x;
    const int b = bh / heads, h = bh - b * heads;
    const size_t row0 = (size_t) b * S;

    // every load of the wavefront is requested here
    const size_t d0 = (size_t) h * D + w * (D / 4) + hh * (D / 8);
    Vec<T, V> qv[kSteps], kv[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; ++t) {
        qv[t] = load_vec<T, V>(q + (row0 + r) * ld + d0 + t * V);
        kv[t] = load_vec<T, V>(k + (row0 + r) * ld + d0 + t * V);
    }
    const int jt = w & 1, kh = w >> 1;  // second contraction: output columns jt*32 .. +31, keys of registers kh*8 .. +7
    T vreg[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        vreg[i] = v[(row0 + acc_row(kh * 8 + i, hh)) * ld + (size_t) h * D + jt * 32 + r];
    }
    float add[16];  // additive mask of this lane's 16 keys, in units of log 2
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        uint32_t word = 0x01010101u;
        if (mask != nullptr) word = *reinterpret_cast<const uint32_t *>(mask + row0 + g * 8 + hh * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) add[g * 4 + e] = ((word >> (8 * e)) & 0xffu) ? 0.f : kMaskedScore * kLog2e;
    }

    v16f32 c = {};
#pragma unroll
    for (int t = 0; t < kSteps; ++t) Mma<T>::run(c, kv[t], qv[t]);  // scores^T[key, query] over this quarter of D
#pragma unroll
    for (int i = 0; i < 16; ++i) s_part[w][i * kWave + lane] = c[i];
    __syncthreads();
    float p[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        p[i] = ((s_part[0][i * kWave + lane] + s_part[1][i * kWave + lane]) + s_part[2][i * kWave + lane]) +
               s_part[3][i * kWave + lane];
    }

    // register i: key acc_row(i, hh), query r
    const float scale = alpha * kLog2e;
    float mx = -3.402823466e+38f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        p[i] = fmaf(p[i], scale, add[i]);
        mx = fmaxf(mx, p[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        p[i] = __builtin_amdgcn_exp2f(p[i] - mx);
        sum += p[i];
    }
    sum += __shfl_xor(sum, 32, kWave);
    const float inv = 1.f / sum;

    // ctx[query, jt*32 + r] over this wavefront's half of the keys
    v16f32 out = {};
#pragma unroll
    for (int run = 0; run < 8 / V; ++run) {
        Vec<T, V> a, bv;
#pragma unroll
        for (int e = 0; e < V; ++e) {
            a.v[e] = from_f32<T>(normalise_prob<T>(p[kh * 8 + run * V + e], sum, inv));
            bv.v[e] = vreg[run * V + e];
        }
        Mma<T>::run(out, a, bv);
    }
    __syncthreads();  // the score partials have been read by everyone
    if (kh == 1) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s_part[jt][i * kWave + lane] = out[i];
    }
    __syncthreads();
    if (kh == 0) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            store_context<T, SPLIT>(ctx, ld_ctx, (size_t) row0 + acc_row(i, hh), h * D + jt * 32 + r,
                             out[i] + s_part[jt][i * kWave + lane], split);
        }
    }
}

// ---- the same for longer sequences (128 < seq <= 512): online softmax over chunks of 64 keys ----
// The layout is that of attention_fused_kernel (a workgroup per (batch, head), a wavefront per 32 queries, K and
// slot-ordered V^T in LDS), but a lane cannot hold seq/2 scores, so the keys are walked in chunks: each chunk
// updates the query's running maximum m and sum l, rescales the context accumulators by exp(m_old - m_new) and
// adds exp(s - m_new) V.  The accumulators have queries along registers while m and l live in the lane of the
// query, so the per-query factors cross lanes through 128 bytes of wavefront-private LDS.  The result is divided
// by l once at the end (scores and probabilities are not rounded to the storage type one by one as the
// three-kernel path does; the difference is within the fp16 storage tolerance).
//
// Key tiles (32 keys) whose mask is zero throughout are left out altogether -- not loaded, not multiplied: a
// masked key's score is 10000 below every unmasked one of its query, its exp is exactly 0 in fp32, so it adds
// nothing to the sum or the context as long as the sequence has one unmasked key (a sequence without any keeps
// all its tiles: there the shift cancels and the softmax runs over the raw scores, as in the reference).  Every
// query row, padded or not, is still computed.  skip_masked_tiles = 0 (a mask that cannot be read as 32-bit
// words) computes all tiles.
template <typename T, int D, bool SPLIT>
__global__ __launch_bounds__(1024) void attention_flash_kernel(const T *__restrict__ q, const T *__restrict__ k,
                                                               const T *__restrict__ v, int ld,
                                                               const int8_t *__restrict__ mask, T *__restrict__ ctx,
                                                               int ld_ctx, float alpha, int heads, int seq,
                                                               int skip_masked_tiles, SplitOut split, const int *__restrict__ order) {
    constexpr int V = Mma<T>::kVec;
    constexpr int kSteps = D / 2 / V;
    constexpr int kColTiles = D / 32;
    constexpr int kChunk = 2;  // key tiles per step
    constexpr int kPitchK = D + V;
    const int S = seq, KT = seq / 32;
    const int threads = blockDim.x;  // = KT * 64
    const int pitch_v = S + V;
    extern __shared__ __align__(16) unsigned char smem[];
    T *s_k = reinterpret_cast<T *>(smem);                              // [S][kPitchK]
    T *s_vt = s_k + (size_t) S * kPitchK;                              // [D][pitch_v], keys in slot order
    float *s_mask = reinterpret_cast<float *>(s_vt + (size_t) D * pitch_v);  // [S] additive mask
    float *s_factor = s_mask + S;                                      // [KT][32] per-query factors

    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5;
    const int qt = wave_in_block();
    const int bh = blockIdx.x;
    const int rank = bh / heads, h = bh - rank * heads;
    const int b = order != nullptr ? order[rank] : rank;  // workgroup-uniform
    const T *k_head = k + (size_t) b * S * ld + (size_t) h * D;
    const T *v_head = v + (size_t) b * S * ld + (size_t) h * D;

    const T *q_row = q + ((size_t) b * S + qt * 32 + r) * ld + (size_t) h * D + hh * (D / 2);
    Vec<T, V> qv[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; ++t) qv[t] = load_vec<T, V>(q_row + t * V);

    // bit kt: key tile kt has an unmasked key (workgroup-uniform: scalar loads of the mask row as words)
    unsigned live = 0;
    if (mask != nullptr && skip_masked_tiles) {
        const uint32_t *words = reinterpret_cast<const uint32_t *>(mask + (size_t) b * S);
        for (int kt = 0; kt < KT; ++kt) {
            uint32_t any = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) any |= words[kt * 8 + i];
            live |= (any != 0 ? 1u : 0u) << kt;
        }
    }
    if (live == 0) live = KT >= 32 ? ~0u : (1u << KT) - 1u;
    live = __builtin_amdgcn_readfirstlane(live);

    constexpr int kVecPerRow = D / V;
    constexpr int kLoads = D / V / 2;  // vectors per thread for K, slot groups per thread for V^T
    Vec<T, V> kreg[kLoads], vreg[kLoads];
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        // (the 64 consecutive idx of a wavefront lie in one key tile, so the tests below are wavefront-uniform)
        const int idx = threadIdx.x + u * threads;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        kreg[u] = Vec<T, V>{};
        if ((live >> (row >> 5)) & 1u) kreg[u] = load_vec<T, V>(k_head + (size_t) row * ld + c * V);
    }
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int idx = threadIdx.x + u * threads;
        const int j = idx % D, grp = idx / D;
        const int kt = grp / (32 / V), in_tile = grp % (32 / V);
        const int run = in_tile >> 1, half = in_tile & 1;
        vreg[u] = Vec<T, V>{};
        if ((live >> kt) & 1u) {
#pragma unroll
            for (int e = 0; e < V; ++e) {
                vreg[u].v[e] = v_head[(size_t) (kt * 32 + acc_row(run * V + e, half)) * ld + j];
            }
        }
    }
    for (int i = threadIdx.x; i < S; i += threads) {
        s_mask[i] = (mask != nullptr && !mask[(size_t) b * S + i]) ? kMaskedScore * kLog2e : 0.f;
    }
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int idx = threadIdx.x + u * threads;
        const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;
        store_vec<T, V>(s_k + row * kPitchK + c * V, kreg[u]);
    }
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
        const int idx = threadIdx.x + u * threads;
        const int j = idx % D, grp = idx / D;
        store_vec<T, V>(s_vt + j * pitch_v + grp * V, vreg[u]);
    }
    __syncthreads();

    // Scores are kept in units of log 2 (t = s * log2 e), so that exp(s - m) is one v_exp_f32 of t - m_t and the
    // scale 1/sqrt(d) and the change of base are a single multiply-add with the mask.
    const float scale = alpha * kLog2e;
    float *factor = s_factor + qt * 32;  // private to this wavefront
    float m = -3.402823466e+38f, l = 0.f;
    v16f32 out[kColTiles];
#pragma unroll
    for (int jt = 0; jt < kColTiles; ++jt) out[jt] = v16f32{};

    bool first_chunk = true;
    for (unsigned todo = live; todo != 0;) {  // the live key tiles in ascending order, kChunk per step
        int tiles[kChunk];
#pragma unroll
        for (int cc = 0; cc < kChunk; ++cc) {
            tiles[cc] = -1;
            if (todo != 0) {
                tiles[cc] = __builtin_ctz(todo);
                todo &= todo - 1;
            }
        }
        v16f32 p[kChunk];
        float cm = -3.402823466e+38f;
#pragma unroll
        for (int cc = 0; cc < kChunk; ++cc) {
            const int kt = tiles[cc];
            v16f32 c = {};
            if (kt >= 0) {  // wavefront-uniform
#pragma unroll
                for (int t = 0; t < kSteps; ++t) {
                    Mma<T>::run(c, load_vec<T, V>(s_k + (kt * 32 + r) * kPitchK + hh * (D / 2) + t * V), qv[t]);
                }
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const Vec<float, 4> mk = load_vec<float, 4>(s_mask + kt * 32 + g * 8 + hh * 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float sc = fmaf(c[g * 4 + e], scale, mk.v[e]);
                        c[g * 4 + e] = sc;
                        cm = fmaxf(cm, sc);
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) c[i] = -3.402823466e+38f;  // exp(. - m) = 0
            }
            p[cc] = c;
        }
        cm = fmaxf(cm, __shfl_xor(cm, 32, kWave));
        const float m_new = fmaxf(m, cm);
        const float f = __builtin_amdgcn_exp2f(m - m_new);  // 0 in the first chunk (m = -max float); out is 0 there
        float part = 0.f;
#pragma unroll
        for (int cc = 0; cc < kChunk; ++cc) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                p[cc][i] = __builtin_amdgcn_exp2f(p[cc][i] - m_new);
                part += p[cc][i];
            }
        }
        part += __shfl_xor(part, 32, kWave);
        l = l * f + part;
        m = m_new;

        // rescale the accumulators: row i of a lane is query acc_row(i, hh), whose factor is in lane acc_row(i, hh)
        if (!first_chunk && __any(f != 1.f)) {  // wavefront-uniform: skipped when no query's maximum moved
            if (hh == 0) factor[r] = f;
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): LDS operations of one wavefront complete in order
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const Vec<float, 4> fr = load_vec<float, 4>(factor + g * 8 + hh * 4);
#pragma unroll
                for (int jt = 0; jt < kColTiles; ++jt) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) out[jt][g * 4 + e] *= fr.v[e];
                }
            }
            __builtin_amdgcn_wave_barrier();  // the reads above come before the next chunk's write
        }
        first_chunk = false;
#pragma unroll
        for (int cc = 0; cc < kChunk; ++cc) {
            const int kt = tiles[cc];
            if (kt >= 0) {
#pragma unroll
                for (int run = 0; run < 16 / V; ++run) {
                    Vec<T, V> a;
#pragma unroll
                    for (int e = 0; e < V; ++e) a.v[e] = from_f32<T>(p[cc][run * V + e]);
#pragma unroll
                    for (int jt = 0; jt < kColTiles; ++jt) {
                        Mma<T>::run(out[jt], a,
                                    load_vec<T, V>(s_vt + (jt * 32 + r) * pitch_v + kt * 32 + run * 2 * V + hh * V));
                    }
                }
            }
        }
    }

    // divide row (query) i by its sum
    if (hh == 0) factor[r] = 1.f / l;
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
    const size_t first_row = (size_t) b * S + qt * 32;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const Vec<float, 4> fr = load_vec<float, 4>(factor + g * 8 + hh * 4);
#pragma unroll
        for (int jt = 0; jt < kColTiles; ++jt) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                store_context<T, SPLIT>(ctx, ld_ctx, first_row + acc_row(g * 4 + e, hh), h * D + jt * 32 + r,
                                 out[jt][g * 4 + e] * fr.v[e], split);
            }
        }
    }
}

// ---- seq 512 with the keys staged a group at a time ----
// attention_flash_kernel loads K and V of the whole head before the first score is computed.  Here the 16 wavefronts
// of a workgroup walk the live key tiles in groups of G = 32 V / D tiles (4 for fp16, head size 64): load a group
// (one K vector and one V^T slot group per thread), barrier, online-softmax update from it, barrier, next group.  A
// compute unit still holds one such workgroup (128 registers per lane x 16 wavefronts fill its register files), but
// the arithmetic of the first group starts after a quarter of the loads, 40 KB of LDS are claimed instead of 148,
// and, since the LDS no longer grows with the sequence, fp32 fits as well.  Measured at batch 64, 12 heads, ~4 live
// tiles per sequence: 54.6 against 59.5 us; groups of 2 or 8 tiles are slower.  Arithmetic and rounding are those of
// attention_flash_kernel.
template <typename T, int D, bool SPLIT>
__global__ __launch_bounds__(1024) void attention_flash_grouped_kernel(
    const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v, int ld, const int8_t *__restrict__ mask,
    T *__restrict__ ctx, int ld_ctx, float alpha, int heads, int skip_masked_tiles, SplitOut split,
    const int *__restrict__ order, int order_has_records) {
    constexpr int V = Mma<T>::kVec;
    constexpr int kSteps = D / 2 / V;
    constexpr int kColTiles = D / 32;
    constexpr int kChunk = 2;                // key tiles per online-softmax step
    constexpr int G = 32 * V / D;            // key tiles per group
    constexpr int kThreads = 1024;
    constexpr int kSeq = 512;
    constexpr int kPitchK = D + V;
    constexpr int kPitchV = G * 32 + V;
    constexpr int kVecPerRow = D / V;
    constexpr int kLoads = G * 32 * kVecPerRow / kThreads;  // = 1: vectors per thread for K, slot groups for V^T
    static_assert(kLoads == 1, "one K vector and one V^T slot group per thread");
    constexpr int S = kSeq, KT = kSeq / 32;
    extern __shared__ __align__(16) unsigned char smem[];
    T *s_k = reinterpret_cast<T *>(smem);                                      // [G * 32][kPitchK]
    T *s_vt = s_k + G * 32 * kPitchK;                                          // [D][kPitchV], keys in slot order
    float *s_mask = reinterpret_cast<float *>(s_vt + D * kPitchV);             // [S] additive mask
    float *s_factor = s_mask + S;                                              // [16][32] per-query factors

    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5;
    const int wave = wave_in_block();
    const int bh = blockIdx.x;
    const int rank = bh / heads, h = bh - rank * heads;
    const int b = order != nullptr ? order[rank] : rank;  // workgroup-uniform
    const int qt = wave;
    const T *k_head = k + (size_t) b * S * ld + (size_t) h * D;
    const T *v_head = v + (size_t) b * S * ld + (size_t) h * D;

    const T *q_row = q + ((size_t) b * S + qt * 32 + r) * ld + (size_t) h * D + hh * (D / 2);
    Vec<T, V> qv[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; ++t) qv[t] = load_vec<T, V>(q_row + t * V);

    // The live key tiles (those with an unmasked key) as a list: n_live tile numbers in ascending order, 4 bits each.
    // With an order array that carries records (attention_order writes them) the list of this sequence is one scalar
    // load next to the one for `b`; otherwise it is made here from the mask row, read as words with scalar loads
    // (workgroup-uniform either way).
    int n_live = 0;
    unsigned long long tile_list = 0;
    if (order != nullptr && order_has_records && mask != nullptr && skip_masked_tiles) {
        const int batch = (int) gridDim.x / heads;
        const int *rec = order + 4 * (size_t) batch + 4 * (size_t) rank;
        n_live = rec[0];
        tile_list = (unsigned long long) (unsigned) rec[1] | ((unsigned long long) (unsigned) rec[2] << 32);
        if (n_live < 1 || n_live > KT) {  // not a record attention_order wrote: every tile, rather than a loop without end
            n_live = KT;
            tile_list = 0xfedcba9876543210ull;
        }
    } else {
        if (mask != nullptr && skip_masked_tiles) {
            const uint32_t *words = reinterpret_cast<const uint32_t *>(mask + (size_t) b * S);
            for (int kt = 0; kt < KT; ++kt) {
                uint32_t any = 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) any |= words[kt * 8 + i];
                if (any != 0) tile_list |= (unsigned long long) kt << (4 * n_live++);
            }
        }
        if (n_live == 0) {  // no mask, or no kept key at all: every tile
            n_live = KT;
            tile_list = 0xfedcba9876543210ull;
        }
    }
    n_live = __builtin_amdgcn_readfirstlane(n_live);
    tile_list = (unsigned long long) (unsigned) __builtin_amdgcn_readfirstlane((int) (unsigned) tile_list) |
                ((unsigned long long) (unsigned) __builtin_amdgcn_readfirstlane((int) (unsigned) (tile_list >> 32)) << 32);

    for (int i = threadIdx.x; i < S; i += kThreads) {
        s_mask[i] = (mask != nullptr && !mask[(size_t) b * S + i]) ? kMaskedScore * kLog2e : 0.f;
    }

    const float scale = alpha * kLog2e;
    float *factor = s_factor + wave * 32;  // private to this wavefront
    float m = -3.402823466e+38f, l = 0.f;
    v16f32 out[kColTiles];
#pragma unroll
    for (int jt = 0; jt < kColTiles; ++jt) out[jt] = v16f32{};
    bool first_chunk = true;

    for (int g0 = 0; g0 < n_live; g0 += G) {
        // the next group: the lowest G live tiles that are left
        const int in_group = n_live - g0 < G ? n_live - g0 : G;
        // tile of slot s of this group (wavefront-uniform: a wavefront's 64 vectors lie in one tile)
        auto tile_of = [&](int slot) { return (int) ((tile_list >> (4 * (g0 + slot))) & 15u); };
        Vec<T, V> kreg[kLoads], vreg[kLoads];
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int idx = threadIdx.x + u * kThreads;
            const int slot = idx / (32 * kVecPerRow), within = idx - slot * (32 * kVecPerRow);
            const int row = within / kVecPerRow, c = within - row * kVecPerRow;
            kreg[u] = Vec<T, V>{};
            if (slot < in_group) kreg[u] = load_vec<T, V>(k_head + (size_t) (tile_of(slot) * 32 + row) * ld + c * V);
        }
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int idx = threadIdx.x + u * kThreads;
            const int j = idx % D, grp = idx / D;               // grp: slot group of V keys, (32 / V) per tile
            const int slot = grp / (32 / V), in_tile = grp % (32 / V);
            const int run = in_tile >> 1, half = in_tile & 1;
            vreg[u] = Vec<T, V>{};
            if (slot < in_group) {
                const int kt = tile_of(slot);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    vreg[u].v[e] = v_head[(size_t) (kt * 32 + acc_row(run * V + e, half)) * ld + j];
                }
            }
        }
        __syncthreads();  // everyone is done with the previous group's tiles
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int idx = threadIdx.x + u * kThreads;
            const int row = idx / kVecPerRow, c = idx - row * kVecPerRow;  // row = slot * 32 + row in tile
            store_vec<T, V>(s_k + row * kPitchK + c * V, kreg[u]);
        }
#pragma unroll
        for (int u = 0; u < kLoads; ++u) {
            const int idx = threadIdx.x + u * kThreads;
            const int j = idx % D, grp = idx / D;
            store_vec<T, V>(s_vt + j * kPitchV + grp * V, vreg[u]);
        }
        __syncthreads();
        for (int s0 = 0; s0 < in_group; s0 += kChunk) {  // the group's tiles in ascending order, kChunk per step
            int tiles[kChunk], slots[kChunk];
#pragma unroll
            for (int cc = 0; cc < kChunk; ++cc) {
                const bool present = s0 + cc < in_group;
                tiles[cc] = present ? tile_of(s0 + cc) : -1;
                slots[cc] = present ? s0 + cc : 0;
            }
            v16f32 p[kChunk];
            float cm = -3.402823466e+38f;
#pragma unroll
            for (int cc = 0; cc < kChunk; ++cc) {
                v16f32 c = {};
                if (tiles[cc] >= 0) {  // wavefront-uniform
#pragma unroll
                    for (int t = 0; t < kSteps; ++t) {
                        Mma<T>::run(c, load_vec<T, V>(s_k + (slots[cc] * 32 + r) * kPitchK + hh * (D / 2) + t * V), qv[t]);
                    }
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const Vec<float, 4> mk = load_vec<float, 4>(s_mask + tiles[cc] * 32 + g * 8 + hh * 4);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float sc = fmaf(c[g * 4 + e], scale, mk.v[e]);
                            c[g * 4 + e] = sc;
                            cm = fmaxf(cm, sc);
                        }
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 16; ++i) c[i] = -3.402823466e+38f;  // exp(. - m) = 0
                }
                p[cc] = c;
            }
            cm = fmaxf(cm, __shfl_xor(cm, 32, kWave));
            const float m_new = fmaxf(m, cm);
            const float f = __builtin_amdgcn_exp2f(m - m_new);
            float part = 0.f;
#pragma unroll
            for (int cc = 0; cc < kChunk; ++cc) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    p[cc][i] = __builtin_amdgcn_exp2f(p[cc][i] - m_new);
                    part += p[cc][i];
                }
            }
            part += __shfl_xor(part, 32, kWave);
            l = l * f + part;
            m = m_new;
            if (!first_chunk && __any(f != 1.f)) {  // wavefront-uniform: skipped when no query's maximum moved
                if (hh == 0) factor[r] = f;
                __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): LDS operations of one wavefront complete in order
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const Vec<float, 4> fr = load_vec<float, 4>(factor + g * 8 + hh * 4);
#pragma unroll
                    for (int jt = 0; jt < kColTiles; ++jt) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) out[jt][g * 4 + e] *= fr.v[e];
                    }
                }
                __builtin_amdgcn_wave_barrier();  // the reads above come before the next chunk's write
            }
            first_chunk = false;
#pragma unroll
            for (int cc = 0; cc < kChunk; ++cc) {
                if (tiles[cc] >= 0) {
#pragma unroll
                    for (int run = 0; run < 16 / V; ++run) {
                        Vec<T, V> a;
#pragma unroll
                        for (int e = 0; e < V; ++e) a.v[e] = from_f32<T>(p[cc][run * V + e]);
#pragma unroll
                        for (int jt = 0; jt < kColTiles; ++jt) {
                            Mma<T>::run(out[jt], a,
                                        load_vec<T, V>(s_vt + (jt * 32 + r) * kPitchV + slots[cc] * 32 + run * 2 * V + hh * V));
                        }
                    }
                }
            }
        }
    }
    // divide row (query) i by its sum
    if (hh == 0) factor[r] = 1.f / l;
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
    const size_t first_row = (size_t) b * S + qt * 32;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const Vec<float, 4> fr = load_vec<float, 4>(factor + g * 8 + hh * 4);
#pragma unroll
        for (int jt = 0; jt < kColTiles; ++jt) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                store_context<T, SPLIT>(ctx, ld_ctx, first_row + acc_row(g * 4 + e, hh), h * D + jt * 32 + r,
                                        out[jt][g * 4 + e] * fr.v[e], split);
            }
        }
    }
}

// ---- longest sequences first ----
// The long-sequence kernels leave out key tiles without a kept key, so a workgroup's time goes with its sequence's
// number of live tiles, and a compute unit holds one such workgroup at a time.  Workgroups are handed out in index
// order: a long sequence that comes late in the batch starts late and the whole launch waits for it (measured at 64
// sequences x 12 heads x 512 keys, valid lengths 16 + Exp(96): 55.7 us in batch order, 44.0 us longest first).  This
// kernel writes the sequence indices by falling live-tile count (a counting sort in one workgroup); the attention
// kernels then take sequence order[blockIdx / heads].  Results do not depend on the order in any way.
constexpr int kOrderMaxBatch = 4096;

// order[0 .. batch): the sequence indices, most live tiles first.  order[4 * batch + 4 * i ...]: a record for the
// sequence at position i -- {number of live tiles, their tile numbers in ascending order 4 bits each (low word, high
// word), the live tiles as a bit mask} -- so that a long-sequence kernel gets its list of tiles with one scalar load
// instead of reading the mask row again.  8 * batch ints in all.
__global__ __launch_bounds__(kBlock) void attention_order_kernel(const int8_t *__restrict__ mask, int batch, int seq,
                                                                 int *__restrict__ order) {
    __shared__ unsigned char tiles_of[kOrderMaxBatch];
    __shared__ unsigned short bits_of[kOrderMaxBatch];
    __shared__ int bucket[20];  // [t]: sequences with t live tiles (t <= 16), then their first position
    const int key_tiles = seq / 32;
    if (threadIdx.x < 20) bucket[threadIdx.x] = 0;
    __syncthreads();
    for (int b = threadIdx.x; b < batch; b += kBlock) {
        const uint32_t *words = reinterpret_cast<const uint32_t *>(mask + (size_t) b * seq);
        int live = 0;
        unsigned bits = 0;
        for (int kt = 0; kt < key_tiles; ++kt) {
            uint32_t any = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) any |= words[kt * 8 + i];
            live += any != 0;
            bits |= (any != 0 ? 1u : 0u) << kt;
        }
        if (live == 0) {  // no kept key: the kernels compute every tile
            live = key_tiles;
            bits = (1u << key_tiles) - 1u;
        }
        tiles_of[b] = (unsigned char) live;
        bits_of[b] = (unsigned short) bits;
        atomicAdd(&bucket[live], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {  // first position of each count, largest count first
        int at = 0;
        for (int t = 16; t >= 0; --t) {
            const int n = bucket[t];
            bucket[t] = at;
            at += n;
        }
    }
    __syncthreads();
    for (int b = threadIdx.x; b < batch; b += kBlock) {
        const int at = atomicAdd(&bucket[tiles_of[b]], 1);
        order[at] = b;
        const unsigned bits = bits_of[b];
        unsigned long long list = 0;
        int n = 0;
        for (int kt = 0; kt < key_tiles; ++kt) {
            if ((bits >> kt) & 1u) list |= (unsigned long long) kt << (4 * n++);
        }
        int *rec = order + 4 * (size_t) batch + 4 * (size_t) at;
        rec[0] = n;
        rec[1] = (int) (unsigned) list;
        rec[2] = (int) (unsigned) (list >> 32);
        rec[3] = (int) bits;
    }
}

int attention_order(const int8_t *mask, int batch, int seq, int *order, void *stream) {
    if (!mask || !order || batch < 0 || seq <= 0) return CUBERT_BAD_ARGUMENT;
    if (batch == 0) return 0;
    if (seq % 32 != 0 || seq > 512 || batch > kOrderMaxBatch || !is_aligned(mask, 4) || !is_aligned(order, 16)) {
        return CUBERT_UNSUPPORTED;
    }
    return launch_untimed(attention_order_kernel, dim3(1), dim3(kBlock), 0u, (hipStream_t) stream, mask, batch, seq,
                          order);
}

template <typename T>
bool shapes_ok(int batch, int heads, int seq, int head_size, int ld, std::initializer_list<const void *> ptrs) {
    constexpr int V = Mma<T>::kVec;
    if (batch <= 0 || heads <= 0 || seq <= 0) return false;
    if (seq % 32 != 0 || (head_size != 32 && head_size != 64 && head_size != 128)) return false;
    if (ld % V != 0 || (long long) batch * heads > 65535) return false;
    for (const void *p : ptrs) {
        if (!is_aligned(p, 16)) return false;
    }
    return true;
}

// Kernels that ask for more than 48 KB of dynamic LDS need their limit raised once per device (the attribute
// belongs to the function on the current device).  One bit per device ordinal, set after a successful call.
template <typename Kernel>
bool allow_large_lds(Kernel kernel, std::atomic<unsigned long long> &done) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return false;
    const unsigned long long bit = 1ull << device;
    if (done.load(std::memory_order_acquire) & bit) return true;
    if (hipFuncSetAttribute((const void *) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) !=
        hipSuccess) {
        (void) hipGetLastError();
        return false;
    }
    done.fetch_or(bit, std::memory_order_release);
    return true;
}

template <typename T, int D>
int launch_scores(const T *q, const T *k, int ld, T *scores, float alpha, int batch, int heads, int seq,
                  hipStream_t s) {
    if constexpr (D * sizeof(T) <= 128) {  // a head row is at most one cache line: both operand tiles fit 64 KB of LDS
        if (seq >= 128) {
            dim3 grid((seq + 127) / 128, (seq + 127) / 128, batch * heads), block(kBlock);
            return launch(attention_scores_tiled_kernel<T, D>, grid, block, s, q, k, ld, scores, alpha, seq, heads);
        }
    }
    const int key_tiles = seq / 32;
    // keys per wavefront: up to 4 tiles (128 keys) while the grid still has enough workgroups
    const int nt = key_tiles % 4 == 0 && key_tiles >= 16 ? 4 : (key_tiles % 2 == 0 && key_tiles >= 8 ? 2 : 1);
    const int strips = key_tiles / nt;
    const int waves = strips >= 4 ? 4 : strips;
    dim3 grid(seq / 32, (strips + waves - 1) / waves, batch * heads), block(waves * kWave);
    if (nt == 4) return launch(attention_scores_kernel<T, D, 4>, grid, block, s, q, k, ld, scores, alpha, seq, heads);
    if (nt == 2) return launch(attention_scores_kernel<T, D, 2>, grid, block, s, q, k, ld, scores, alpha, seq, heads);
    return launch(attention_scores_kernel<T, D, 1>, grid, block, s, q, k, ld, scores, alpha, seq, heads);
}

template <typename T>
int attention_scores(const T *q, const T *k, int ld, T *scores, float alpha, int batch, int heads, int seq,
                     int head_size, void *stream) {
    if (!q || !k || !scores || batch < 0) return CUBERT_BAD_ARGUMENT;
    if (batch == 0) return 0;
    if (!shapes_ok<T>(batch, heads, seq, head_size, ld, {q, k, scores})) return CUBERT_UNSUPPORTED;
    hipStream_t s = (hipStream_t) stream;
    switch (head_size) {
        case 32: return launch_scores<T, 32>(q, k, ld, scores, alpha, batch, heads, seq, s);
        case 64: return launch_scores<T, 64>(q, k, ld, scores, alpha, batch, heads, seq, s);
        default: return launch_scores<T, 128>(q, k, ld, scores, alpha, batch, heads, seq, s);
    }
}

template <typename T, int D>
int launch_context(const T *probs, const T *v, int ld, T *ctx, int ld_ctx, int batch, int heads, int seq,
                   hipStream_t s) {
    const int q_tiles = seq / 32;
    const int waves = q_tiles >= 4 ? 4 : q_tiles;
    // query tiles per workgroup: more of them amortise the V^T staging, fewer give more workgroups
    const int per_block = q_tiles >= 16 ? 8 : waves;
    const size_t lds = (size_t) D * (seq + 16 / sizeof(T)) * sizeof(T);
    if (lds > 160 * 1024) return CUBERT_UNSUPPORTED;
    auto kernel = attention_context_kernel<T, D>;
    if (lds > 48 * 1024) {
        static std::atomic<unsigned long long> raised{0};  // per instantiation
        if (!allow_large_lds(kernel, raised)) return CUBERT_UNSUPPORTED;
    }
    dim3 grid((q_tiles + per_block - 1) / per_block, batch * heads), block(waves * kWave);
    return launch_lds(kernel, grid, block, (unsigned) lds, s, probs, v, ld, ctx, ld_ctx, seq, heads, per_block);
}

template <typename T>
int attention_context(const T *probs, const T *v, int ld, T *ctx, int ld_ctx, int batch, int heads, int seq,
                      int head_size, void *stream) {
    if (!probs || !v || !ctx || batch < 0) return CUBERT_BAD_ARGUMENT;
    if (batch == 0) return 0;
    if (!shapes_ok<T>(batch, heads, seq, head_size, ld, {probs, v}) || ld_ctx < heads * head_size) return CUBERT_UNSUPPORTED;
    hipStream_t s = (hipStream_t) stream;
    switch (head_size) {
        case 32: return launch_context<T, 32>(probs, v, ld, ctx, ld_ctx, batch, heads, seq, s);
        case 64: return launch_context<T, 64>(probs, v, ld, ctx, ld_ctx, batch, heads, seq, s);
        default: return launch_context<T, 128>(probs, v, ld, ctx, ld_ctx, batch, heads, seq, s);
    }
}

template <typename T, int D, int KT>
int launch_fused_kt(const T *q, const T *k, const T *v, int ld, const int8_t *mask, T *ctx, int ld_ctx, float alpha,
                    int batch, int heads, SplitOut split, hipStream_t s) {
    constexpr size_t lds = fused_lds_bytes<T, D, KT>();
    if (lds > 160 * 1024) return CUBERT_UNSUPPORTED;
    if constexpr (sizeof(T) == 4) {
        if (split.width > 0) {
            auto kernel = attention_fused_kernel<T, D, KT, true>;
            if (lds > 48 * 1024) {
                static std::atomic<unsigned long long> raised{0};  // per instantiation
                if (!allow_large_lds(kernel, raised)) return CUBERT_UNSUPPORTED;
            }
            return launch_lds(kernel, dim3(batch * heads), dim3(KT * kWave), (unsigned) lds, s, q, k, v, ld, mask,
                                  ctx, ld_ctx, alpha, heads, split);
        }
    }
    if (split.width > 0) return CUBERT_UNSUPPORTED;
    if constexpr (sizeof(T) == 2) {
        // CUBERT_ATTENTION_KERNEL=general / lean in the environment forces one of the two; by default the lean kernel
        // runs where the grid fills the chip several times over (measured at 128 keys, head size 64: 4096 workgroups
        // 65.6 -> 57.0 us) and the general one where a workgroup's own chain of latencies is what takes the time
        // (384 workgroups: 10.8 us against 11.3 with the lean kernel's extra pass through LDS on the way out).
        static const int forced = [] {
            const char *e = getenv("CUBERT_ATTENTION_KERNEL");
            return e == nullptr ? 0 : (std::string(e) == "general" ? 1 : (std::string(e) == "lean" ? 2 : 0));
        }();
        const bool lean = forced == 2 || (forced == 0 && batch * heads >= 1024);
        if (lean && (mask == nullptr || is_aligned(mask, 4)) && is_aligned(ctx, 16) && ld_ctx % 8 == 0) {
            auto kernel = attention_fused_half_kernel<D, KT>;
            constexpr size_t half_lds = fused_half_lds_bytes<D, KT>();
            if (half_lds > 48 * 1024) {
                static std::atomic<unsigned long long> raised{0};  // per instantiation
                if (!allow_large_lds(kernel, raised)) return CUBERT_UNSUPPORTED;
            }
            return launch_lds(kernel, dim3(batch * heads), dim3(KT * kWave), (unsigned) half_lds, s, q, k, v, ld,
                                  mask, ctx, ld_ctx, alpha, heads);
        }
    }
    auto kernel = attention_fused_kernel<T, D, KT, false>;
    if (lds > 48 * 1024) {
        static std::atomic<unsigned long long> raised{0};  // per instantiation
        if (!allow_large_lds(kernel, raised)) return CUBERT_UNSUPPORTED;
    }
    return launch_lds(kernel, dim3(batch * heads), dim3(KT * kWave), (unsigned) lds, s, q, k, v, ld, mask, ctx,
                          ld_ctx, alpha, heads, split);
}

template <typename T, int D>
int launch_fused(const T *q, const T *k, const T *v, int ld, const int8_t *mask, T *ctx, int ld_ctx, float alpha,
                 int batch, int heads, int seq, SplitOut split, hipStream_t s) {
    if constexpr (D == 64) {
        // split each problem over four wavefronts: a quarter of the dependent matrix instructions per wavefront
        // (12 problems 5.3 -> 4.7 us, 1536 problems 15.95 -> 15.0 us; not measured beyond)
        if (seq == 32 && batch * heads <= 2048 && (mask == nullptr || is_aligned(mask, 4))) {
            if constexpr (sizeof(T) == 4) {
                if (split.width > 0) {
                    return launch_lds(attention_small_kernel<T, true>, dim3(batch * heads), dim3(4 * kWave), 0u, s, q,
                                          k, v, ld, mask, ctx, ld_ctx, alpha, heads, split);
                }
            }
            if (split.width > 0) return CUBERT_UNSUPPORTED;
            return launch_lds(attention_small_kernel<T, false>, dim3(batch * heads), dim3(4 * kWave), 0u, s, q, k, v,
                                  ld, mask, ctx, ld_ctx, alpha, heads, split);
        }
    }
    switch (seq / 32) {
        case 1:
            return launch_fused_kt<T, D, 1>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, split, s);
        case 2:
            return launch_fused_kt<T, D, 2>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, split, s);
        case 3:
            return launch_fused_kt<T, D, 3>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, split, s);
        case 4:
            return launch_fused_kt<T, D, 4>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, split, s);
        default: return CUBERT_UNSUPPORTED;
    }
}

template <typename T, int D>
int launch_flash(const T *q, const T *k, const T *v, int ld, const int8_t *mask, T *ctx, int ld_ctx, float alpha,
                 int batch, int heads, int seq, SplitOut split, const int *order, hipStream_t s) {
    constexpr int V = 16 / sizeof(T);
    if (seq > 512) return CUBERT_UNSUPPORTED;  // a workgroup has at most 16 wavefronts
    const size_t lds = (size_t) seq * (D + V) * sizeof(T) + (size_t) D * (seq + V) * sizeof(T) +
                       2 * (size_t) seq * sizeof(float);
    const int skip_masked_tiles = mask != nullptr && is_aligned(mask, 4);  // seq is a multiple of 32
    static const bool whole_head = getenv("CUBERT_FLASH_WHOLE") != nullptr;
    if (seq == 512 && !whole_head) {
        constexpr int G = 32 * V / D;
        // CUBERT_FLASH_RECORDS=0 in the environment: the kernel reads the mask row itself instead of the order array's
        // records (for comparison)
        static const int use_records = [] {
            const char *e = std::getenv("CUBERT_FLASH_RECORDS");
            return e != nullptr && std::string(e) == "0" ? 0 : 1;
        }();
        const size_t grouped_lds = ((size_t) G * 32 * (D + V) + (size_t) D * (G * 32 + V)) * sizeof(T) +
                                   ((size_t) seq + 16 * 32) * sizeof(float);
        if constexpr (sizeof(T) == 4) {
            if (split.width > 0) {
                return launch_lds(attention_flash_grouped_kernel<T, D, true>, dim3(batch * heads), dim3(1024),
                                      (unsigned) grouped_lds, s, q, k, v, ld, mask, ctx, ld_ctx, alpha, heads,
                                      skip_masked_tiles, split, order, use_records);
            }
        }
        if (split.width > 0) return CUBERT_UNSUPPORTED;
        return launch_lds(attention_flash_grouped_kernel<T, D, false>, dim3(batch * heads), dim3(1024),
                              (unsigned) grouped_lds, s, q, k, v, ld, mask, ctx, ld_ctx, alpha, heads, skip_masked_tiles,
                              split, order, use_records);
    }
    if (lds > 160 * 1024) return CUBERT_UNSUPPORTED;
    if constexpr (sizeof(T) == 4) {
        if (split.width > 0) {
            auto kernel = attention_flash_kernel<T, D, true>;
            static std::atomic<unsigned long long> raised{0};  // per instantiation
            if (!allow_large_lds(kernel, raised)) return CUBERT_UNSUPPORTED;
            return launch_lds(kernel, dim3(batch * heads), dim3(seq / 32 * kWave), (unsigned) lds, s, q, k, v, ld,
                                  mask, ctx, ld_ctx, alpha, heads, seq, skip_masked_tiles, split, order);
        }
    }
    if (split.width > 0) return CUBERT_UNSUPPORTED;
    auto kernel = attention_flash_kernel<T, D, false>;
    static std::atomic<unsigned long long> raised{0};  // per instantiation
    if (!allow_large_lds(kernel, raised)) return CUBERT_UNSUPPORTED;
    return launch_lds(kernel, dim3(batch * heads), dim3(seq / 32 * kWave), (unsigned) lds, s, q, k, v, ld, mask,
                          ctx, ld_ctx, alpha, heads, seq, skip_masked_tiles, split, order);
}

template <typename T>
int attention_fused(const T *q, const T *k, const T *v, int ld, const int8_t *mask, T *ctx, int ld_ctx, float alpha,
                    int batch, int heads, int seq, int head_size, void *stream, SplitOut split = SplitOut(), const int *order = nullptr) {
    if (batch == 0 || heads == 0 || seq == 0) return 0;
    if (!q || !k || !v || !ctx || batch < 0 || heads < 0 || seq < 0 || head_size <= 0) return CUBERT_BAD_ARGUMENT;
    if (ld < heads * head_size) return CUBERT_BAD_ARGUMENT;
    if (!shapes_ok<T>(batch, heads, seq, head_size, ld, {q, k, v}) || ld_ctx < heads * head_size) {
        return CUBERT_UNSUPPORTED;
    }
    hipStream_t s = (hipStream_t) stream;
    if (seq > 128) {
        switch (head_size) {
            case 32:
                return launch_flash<T, 32>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, seq, split, order, s);
            case 64:
                return launch_flash<T, 64>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, seq, split, order, s);
            default: return CUBERT_UNSUPPORTED;  // head size 128 would spill the accumulators to scratch
        }
    }
    switch (head_size) {
        case 32:
            return launch_fused<T, 32>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, seq, split,
                                       s);
        case 64:
            return launch_fused<T, 64>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, seq, split,
                                       s);
        default:
            return launch_fused<T, 128>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, seq, split,
                                        s);
    }
}

}  // namespace
}  // namespace cubert

using cubert::half_t;

extern "C" int cubert_attention_scores_f32(const float *q, const float *k, int ld, float *scores, float alpha, int batch,
                                           int heads, int seq_length, int head_size, void *stream) {
    return cubert::attention_scores<float>(q, k, ld, scores, alpha, batch, heads, seq_length, head_size, stream);
}
extern "C" int cubert_attention_scores_f16(const cubert_half *q, const cubert_half *k, int ld, cubert_half *scores,
                                           float alpha, int batch, int heads, int seq_length, int head_size,
                                           void *stream) {
    return cubert::attention_scores<half_t>((const half_t *) q, (const half_t *) k, ld, (half_t *) scores, alpha, batch,
                                            heads, seq_length, head_size, stream);
}
extern "C" int cubert_attention_context_f32(const float *probs, const float *v, int ld, float *ctx, int ld_ctx, int batch,
                                            int heads, int seq_length, int head_size, void *stream) {
    return cubert::attention_context<float>(probs, v, ld, ctx, ld_ctx, batch, heads, seq_length, head_size, stream);
}
extern "C" int cubert_attention_context_f16(const cubert_half *probs, const cubert_half *v, int ld, cubert_half *ctx,
                                            int ld_ctx, int batch, int heads, int seq_length, int head_size,
                                            void *stream) {
    return cubert::attention_context<half_t>((const half_t *) probs, (const half_t *) v, ld, (half_t *) ctx, ld_ctx,
                                             batch, heads, seq_length, head_size, stream);
}

extern "C" int cubert_attention_fused_f32(const float *q, const float *k, const float *v, int ld, const int8_t *mask,
                                          float *ctx, int ld_ctx, float alpha, int batch, int heads, int seq_length,
                                          int head_size, void *stream) {
    return cubert::attention_fused<float>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, seq_length, head_size,
                                          stream);
}

extern "C" int cubert_attention_order(const int8_t *mask, int batch, int seq_length, int *order, void *stream) {
    return cubert::attention_order(mask, batch, seq_length, order, stream);
}

extern "C" int cubert_attention_fused_ordered_f32(const float *q, const float *k, const float *v, int ld,
                                                  const int8_t *mask, const int *order, float *ctx, int ld_ctx,
                                                  float alpha, int batch, int heads, int seq_length, int head_size,
                                                  void *stream) {
    return cubert::attention_fused<float>(q, k, v, ld, mask, ctx, ld_ctx, alpha, batch, heads, seq_length, head_size,
                                          stream, cubert::SplitOut(), order);
}

extern "C" int cubert_attention_fused_ordered_f16(const cubert_half *q, const cubert_half *k, const cubert_half *v, int ld,
                                                  const int8_t *mask, const int *order, cubert_half *ctx, int ld_ctx,
                                                  float alpha, int batch, int heads, int seq_length, int head_size,
                                                  void *stream) {
    return cubert::attention_fused<cubert::half_t>((const cubert::half_t *) q, (const cubert::half_t *) k,
                                                   (const cubert::half_t *) v, ld, mask, (cubert::half_t *) ctx,
                                                   ld_ctx, alpha, batch, heads, seq_length, head_size, stream, cubert::SplitOut(),
                                                   order);
}

extern "C" int cubert_attention_fused_split3_f32(const float *q, const float *k, const float *v, int ld,
                                                const int8_t *mask, float scale, cubert_half *split_ctx, float alpha,
                                                int batch, int heads, int seq_length, int head_size, int *overflow,
                                                void *stream) {
    if (split_ctx != nullptr && !cubert::is_aligned(split_ctx, 2)) return CUBERT_BAD_ARGUMENT;
    const int hidden = heads * head_size;
    return cubert::attention_fused<float>(q, k, v, ld, mask, reinterpret_cast<float *>(split_ctx), hidden, alpha, batch,
                                          heads, seq_length, head_size, stream, cubert::SplitOut{hidden, scale, overflow});
}

extern "C" int cubert_attention_fused_f16(const cubert_half *q, const cubert_half *k, const cubert_half *v, int ld,
                                          const int8_t *mask, cubert_half *ctx, int ld_ctx, float alpha, int batch,
                                          int heads, int seq_length, int head_size, void *stream) {
    return cubert::attention_fused<cubert::half_t>((const cubert::half_t *) q, (const cubert::half_t *) k,
                                                   (const cubert::half_t *) v, ld, mask, (cubert::half_t *) ctx,
                                                   ld_ctx, alpha, batch, heads, seq_length, head_size, stream);
}
