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

#include <initializer_list>

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
        static thread_local bool raised = false;  // per instantiation and thread; the call is cheap and idempotent
        if (!raised) {
            if (hipFuncSetAttribute((const void *) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) !=
                hipSuccess) {
                (void) hipGetLastError();
                return CUBERT_UNSUPPORTED;
            }
            raised = true;
        }
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
