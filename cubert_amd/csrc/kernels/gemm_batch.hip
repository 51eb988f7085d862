// Batched GEMM over arrays of pointers:  C_z = alpha * op(A_z) * op(B_z) + beta * C_z  (column-major), z < batch.
// This is the interface the reference's attention contractions are written against (blas_gemm_batch,
// src/cuBERT/common.h:70-80; Att_Q_K and Att_QK_V hand it one pointer per (batch, head) problem,
// src/cuBERT/op_att/BatchMatMul.cpp:31-38,57-68).  The host classes here do not call it: their attention runs in the
// kernels of attention.hip.  It is kept for a host program that keeps the reference's BatchMatMul classes.
//
// One workgroup computes a 64 x 64 tile of one problem: operand tiles of 16 reduction values are staged in LDS
// as fp32 (whatever the transposes, the global loads walk the contiguous dimension), a thread owns a 4 x 4 block of
// the tile and accumulates in fp32.  The problems of a BERT attention layer are small (seq x seq x head size), so a
// launch is bound by the number of problems, not by the tile arithmetic.

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

}  // namespace

template <typename T>
int gemm_batch(int transA, int transB, int M, int N, int K, float alpha, const T *const *A_array, int lda,
               const T *const *B_array, int ldb, float beta, T *const *C_array, int ldc, int batch,
               hipStream_t stream) {
    if (M < 0 || N < 0 || K < 0 || batch < 0) return CUBERT_BAD_ARGUMENT;
    if (M == 0 || N == 0 || batch == 0) return 0;
    if (!A_array || !B_array || !C_array) return CUBERT_BAD_ARGUMENT;
    if (lda < (transA ? K : M) || ldb < (transB ? N : K) || ldc < M) return CUBERT_BAD_ARGUMENT;
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
