// Batched GEMM over arrays of pointers:  C_z = alpha * op(A_z) * op(B_z) + beta * C_z  (column-major), z < batch.
// This is the interface the reference's attention contractions are written against (blas_gemm_batch,
// src/cuBERT/common.h:70-80; Att_Q_K and Att_QK_V hand it one pointer per (batch, head) problem,
// src/cuBERT/op_att/BatchMatMul.cpp:31-38,57-68).  The host classes here do not call it: their attention runs in the
// kernels of attention.hip.  It is kept for a host program that keeps the reference's BatchMatMul classes.
//
// Two kernels.  When M, N and K are multiples of 32 (every attention shape the one-launch kernels take) a wavefront
// computes one 32 x 32 tile of one problem on the matrix cores: per 32 reduction values both operand tiles go
// through the wavefront's own piece of LDS as [row][k] (whatever the transposes, the global loads walk the
// contiguous dimension; an operand whose rows are contiguous is transposed on its way into LDS), operands come back
// as 16-byte reads, and the tile of C leaves through LDS in runs along its contiguous dimension.  Any other shape: one workgroup
// computes a 64 x 64 tile of one problem with operand tiles of 16 reduction values staged in LDS as fp32, a thread
// owning a 4 x 4 block of the tile (plain fmaf, fp32 accumulation).  The problems of a BERT attention layer are
// small (seq x seq x head size), so a launch is bound by the number of problems, not by the tile arithmetic.

#include "cubert_kernels.h"
#include "device_common.h"

namespace cubert {
namespace {

constexpr int kTile = 64;    // rows and columns of C per workgroup
constexpr int kDepth = 16;   // reduction values per staging step
constexpr int kPitch = kTile + 4;

template <typename T>
__global__ __launch_bounds__(kBlock) void gemm_batch_kernel(int transA, int transB, int M, int N, int K, float alpha,
                                                            const T *const *__restrict__ A_array, int lda,
                                                            const T *const *__restrict__ B_array, int ldb, float beta,
                                                            T *const *__restrict__ C_array, int ldc, int batch) {
    __shared__ __align__(16) float s_a[kDepth][kPitch];  // [k][i]
    __shared__ __align__(16) float s_b[kDepth][kPitch];  // [k][j]
    const int t = threadIdx.x;
    const int i0 = blockIdx.x * kTile, j0 = blockIdx.y * kTile;
    const int ti = (t & 15) * 4, tj = (t >> 4) * 4;  // this thread's 4 x 4 block inside the tile
    for (int z = blockIdx.z; z < batch; z += gridDim.z) {
        const T *__restrict__ a = A_array[z];
        const T *__restrict__ b = B_array[z];
        T *__restrict__ c = C_array[z];
        float acc[4][4] = {};
        for (int k0 = 0; k0 < K; k0 += kDepth) {
            // A(i, k) is a[i + k * lda], or a[k + i * lda] when transposed; the 64 x 16 tile is 4 elements per thread
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int e = t + u * kBlock;
                const int i = transA ? e / kDepth : e % kTile, k = transA ? e % kDepth : e / kTile;
                float v = 0.f;
                if (i0 + i < M && k0 + k < K) {
                    v = to_f32(transA ? a[(size_t) (i0 + i) * lda + k0 + k] : a[(size_t) (k0 + k) * lda + i0 + i]);
                }
                s_a[k][i] = v;
            }
            // B(k, j) is b[k + j * ldb], or b[j + k * ldb] when transposed
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int e = t + u * kBlock;
                const int j = transB ? e % kTile : e / kDepth, k = transB ? e / kTile : e % kDepth;
                float v = 0.f;
                if (j0 + j < N && k0 + k < K) {
                    v = to_f32(transB ? b[(size_t) (k0 + k) * ldb + j0 + j] : b[(size_t) (j0 + j) * ldb + k0 + k]);
                }
                s_b[k][j] = v;
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < kDepth; ++k) {
                const Vec<float, 4> av = load_vec<float, 4>(&s_a[k][ti]);
                const Vec<float, 4> bv = load_vec<float, 4>(&s_b[k][tj]);
#pragma unroll
                for (int x = 0; x < 4; ++x) {
#pragma unroll
                    for (int y = 0; y < 4; ++y) acc[y][x] = fmaf(av.v[x], bv.v[y], acc[y][x]);
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int y = 0; y < 4; ++y) {
            const int j = j0 + tj + y;
            if (j >= N) continue;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int i = i0 + ti + x;
                if (i >= M) continue;
                T *at = c + (size_t) j * ldc + i;
                float v = alpha * acc[y][x];
                if (beta != 0.f) v += beta * to_f32(*at);  // beta = 0: C is not read (it may hold anything)
                *at = from_f32<T>(v);
            }
        }
    }
}

typedef float v16f32 __attribute__((ext_vector_type(16)));
typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));

// One accumulation step over V consecutive reduction values per lane half (8 halves: one v_mfma_f32_32x32x16_f16;
// 4 floats: four v_mfma_f32_32x32x2_f32).  A reduction slot may be any k as long as both operands agree.
__device__ __forceinline__ void mma_step(v16f32 &acc, const Vec<half_t, 8> &a, const Vec<half_t, 8> &b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8f16, a), __builtin_bit_cast(v8f16, b), acc, 0, 0, 0);
}
__device__ __forceinline__ void mma_step(v16f32 &acc, const Vec<float, 4> &a, const Vec<float, 4> &b) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[i], b.v[i], acc, 0, 0, 0);
}

// Accumulator register x of lane half hh belongs to this row of the first operand (column of C here).
__device__ __forceinline__ int acc_column(int x, int hh) { return (x >> 2) * 8 + hh * 4 + (x & 3); }

constexpr int kMmaTile = 32;   // rows, columns and reduction values per step of a wavefront's tile
constexpr int kMmaWaves = kBlock / kWave;

// A 32 (rows) x 32 (k) operand tile into LDS as tile[row][k].  k_contiguous: element (row, k) is src[k + row * ld];
// otherwise it is src[row + k * ld] and the vector loaded along the rows is scattered into a column.  `vector` (the
// same for all lanes): the tile's addresses are 16-byte aligned, else element loads.
template <typename T, int PITCH>
__device__ __forceinline__ void stage_tile(T *__restrict__ tile, const T *__restrict__ src, int ld, bool k_contiguous,
                                           bool vector, int lane) {
    constexpr int V = 16 / sizeof(T);
    constexpr int kVecPerRow = kMmaTile / V;
    constexpr int kPerLane = kMmaTile * kVecPerRow / kWave;
    Vec<T, V> x[kPerLane];
#pragma unroll
    for (int u = 0; u < kPerLane; ++u) {
        const int idx = lane + u * kWave;
        const int line = idx / kVecPerRow, c = idx - line * kVecPerRow;  // `line` runs along the strided dimension
        const T *at = src + (size_t) line * ld + c * V;
        if (vector) {
            x[u] = load_vec<T, V>(at);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) x[u].v[e] = at[e];
        }
    }
#pragma unroll
    for (int u = 0; u < kPerLane; ++u) {
        const int idx = lane + u * kWave;
        const int line = idx / kVecPerRow, c = idx - line * kVecPerRow;
        if (k_contiguous) {
            store_vec<T, V>(tile + line * PITCH + c * V, x[u]);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) tile[(c * V + e) * PITCH + line] = x[u].v[e];
        }
    }
}

// grid.x = ceil(batch * (M / 32) * (N / 32) / 4); a wavefront per 32 x 32 tile of C.
template <typename T>
__global__ __launch_bounds__(kBlock) void gemm_batch_mma_kernel(int transA, int transB, int M, int N, int K, float alpha,
                                                                const T *const *__restrict__ A_array, int lda,
                                                                const T *const *__restrict__ B_array, int ldb,
                                                                float beta, T *const *__restrict__ C_array, int ldc,
                                                                long long tiles) {
    constexpr int V = 16 / sizeof(T);
    constexpr int PITCH = kMmaTile + V;  // +16 bytes per row: 16-byte reads of 32 rows spread over the banks
    __shared__ __align__(16) T lds[kMmaWaves][2][kMmaTile * PITCH];
    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5, wave = wave_in_block();
    const int tiles_m = M / kMmaTile, tiles_n = N / kMmaTile;
    long long tile = (long long) blockIdx.x * kMmaWaves + wave;
    const bool live = tile < tiles;
    if (!live) tile = tiles - 1;  // keeps the workgroup's barriers matched; nothing is stored
    const int per_problem = tiles_m * tiles_n;
    const int z = (int) (tile / per_problem), in_problem = (int) (tile - (long long) z * per_problem);
    const int i0 = (in_problem % tiles_m) * kMmaTile, j0 = (in_problem / tiles_m) * kMmaTile;
    const T *__restrict__ a = A_array[z];
    const T *__restrict__ b = B_array[z];
    T *__restrict__ c = C_array[z];
    // op(A)(i, k) is a[i + k * lda], or a[k + i * lda] when transposed; op(B)(k, j) is b[k + j * ldb], or b[j + k * ldb]
    const bool a_k_contiguous = transA != 0, b_k_contiguous = transB == 0;
    const bool a_vector = is_aligned(a, 16) && (lda * sizeof(T)) % 16 == 0;
    const bool b_vector = is_aligned(b, 16) && (ldb * sizeof(T)) % 16 == 0;
    T *tile_a = lds[wave][0], *tile_b = lds[wave][1];

    v16f32 acc = {};
    for (int k0 = 0; k0 < K; k0 += kMmaTile) {
        const T *src_a = a_k_contiguous ? a + (size_t) i0 * lda + k0 : a + (size_t) k0 * lda + i0;
        const T *src_b = b_k_contiguous ? b + (size_t) j0 * ldb + k0 : b + (size_t) k0 * ldb + j0;
        stage_tile<T, PITCH>(tile_a, src_a, lda, a_k_contiguous, a_vector, lane);
        stage_tile<T, PITCH>(tile_b, src_b, ldb, b_k_contiguous, b_vector, lane);
        __syncthreads();
#pragma unroll
        for (int t = 0; t < kMmaTile / (2 * V); ++t) {
            // the first operand's rows become the accumulator's rows, the second operand's its columns: a lane ends
            // up with row i0 + r of C and 16 of the tile's columns
            const Vec<T, V> av = load_vec<T, V>(tile_a + r * PITCH + t * 2 * V + hh * V);
            const Vec<T, V> bv = load_vec<T, V>(tile_b + r * PITCH + t * 2 * V + hh * V);
            mma_step(acc, bv, av);
        }
        __syncthreads();  // the tiles are overwritten by the next step
    }
    // Through LDS (fp32, the wavefront's own piece, free after the last barrier) so that C leaves in runs along its
    // contiguous dimension: accumulator register g * 4 + e of lane (r, hh) is C(i0 + r, j0 + g * 8 + hh * 4 + e).
    constexpr int kStagePitch = kMmaTile + 4;
    static_assert(kStagePitch * kMmaTile * sizeof(float) <= 2 * kMmaTile * PITCH * sizeof(T), "stage fits the two tiles");
    float *stage = reinterpret_cast<float *>(lds[wave][0]);
#pragma unroll
    for (int x = 0; x < 16; ++x) stage[acc_column(x, hh) * kStagePitch + r] = alpha * acc[x];
    __syncthreads();
    if (!live) return;
    const bool c_vector = is_aligned(c, 4 * sizeof(T)) && ldc % 4 == 0;
#pragma unroll
    for (int u = 0; u < kMmaTile * kMmaTile / 4 / kWave; ++u) {
        const int idx = lane + u * kWave;
        const int j = idx / (kMmaTile / 4), i = (idx % (kMmaTile / 4)) * 4;
        const Vec<float, 4> v = load_vec<float, 4>(stage + j * kStagePitch + i);
        T *at = c + (size_t) (j0 + j) * ldc + i0 + i;
        Vec<T, 4> o;
        if (beta != 0.f) {  // beta = 0: C is not read (it may hold anything)
            if (c_vector) {
                o = load_vec<T, 4>(at);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) o.v[e] = at[e];
            }
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) o.v[e] = from_f32<T>(beta != 0.f ? v.v[e] + beta * to_f32(o.v[e]) : v.v[e]);
        if (c_vector) {
            store_vec<T, 4>(at, o);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) at[e] = o.v[e];
        }
    }
}

}  // namespace

template <typename T>
int gemm_batch(int transA, int transB, int M, int N, int K, float alpha, const T *const *A_array, int lda,
               const T *const *B_array, int ldb, float beta, T *const *C_array, int ldc, int batch,
               hipStream_t stream) {
    if (M < 0 || N < 0 || K < 0 || batch < 0) return CUBERT_BAD_ARGUMENT;
    if (M == 0 || N == 0 || batch == 0) return 0;
    if (!A_array || !B_array || !C_array) return CUBERT_BAD_ARGUMENT;
    if (lda < (transA ? K : M) || ldb < (transB ? N : K) || ldc < M) return CUBERT_BAD_ARGUMENT;
    if (M % kMmaTile == 0 && N % kMmaTile == 0 && K % kMmaTile == 0 && K > 0) {
        const long long tiles = (long long) batch * (M / kMmaTile) * (N / kMmaTile);
        const long long groups = (tiles + kMmaWaves - 1) / kMmaWaves;
        if (groups <= 0x7fffffffll) {
            return launch(gemm_batch_mma_kernel<T>, dim3((unsigned) groups), dim3(kBlock), stream, transA, transB, M, N,
                          K, alpha, A_array, lda, B_array, ldb, beta, C_array, ldc, tiles);
        }
    }
    const unsigned tiles_m = (unsigned) ((M + kTile - 1) / kTile), tiles_n = (unsigned) ((N + kTile - 1) / kTile);
    if (tiles_n > 65535u) return CUBERT_UNSUPPORTED;
    const dim3 grid(tiles_m, tiles_n, (unsigned) (batch < 65535 ? batch : 65535));
    return launch(gemm_batch_kernel<T>, grid, dim3(kBlock), stream, transA, transB, M, N, K, alpha, A_array, lda,
                  B_array, ldb, beta, C_array, ldc, batch);
}

template int gemm_batch<float>(int, int, int, int, int, float, const float *const *, int, const float *const *, int, float,
                               float *const *, int, int, hipStream_t);
template int gemm_batch<half_t>(int, int, int, int, int, float, const half_t *const *, int, const half_t *const *, int,
                                float, half_t *const *, int, int, hipStream_t);

}  // namespace cubert
