// Dense layer for a handful of tokens:  C[M, N] = alpha * A[M, K] * B[K, N] + bias  (column-major, no
// transposes) with N <= 64.  In the row-major picture of a Dense layer A is the weight matrix [in, out]
// (M = out features, K = in features), B the activations of N tokens and C their outputs.
//
// With so few tokens the GEMM is a single pass over the weights: every weight is used once per token and
// the work is bounded by how fast the weight matrix streams in, i.e. by how much of it is requested at
// once.  A library GEMM tiled for large N keeps few loads in flight here (a BERT-base forward pass at
// batch 1, seq 32 spends most of its time in such GEMMs at a few percent of the memory bandwidth).
//
// Decomposition: a workgroup of 16 wavefronts owns 32 output features and a slice of K (256 values per
// pass); each wavefront multiplies a [32 tokens x 16] block of B with a [16 x 32 features] block of A on
// the matrix cores (fp32: eight v_mfma_f32_32x32x2_f32; fp16: one v_mfma_f32_32x32x16_f16 on the operands as
// they are stored, a sixteenth of the matrix-core time, fp32 accumulation either way).  Every load of
// the wavefront is issued before the first MFMA.  The 16 partial tiles are summed through LDS in wavefront
// order.  When K is cut into several slices (grid.y > 1) each workgroup stores its partial tile to a
// workspace and the last workgroup to arrive for a feature block (ticket from an atomic counter) adds the
// slices in slice order, so the result does not depend on scheduling.
//
// That hand-over (partial tile written through, ticket, partial tiles read back) is 2 us of a 7-10 us kernel.
// gemm_skinny_partials leaves it out: every workgroup stores its partial tile and is done, and the kernel that
// consumes the Dense layer's output (bias + residual + LayerNorm) adds the slices in slice order while it loads its
// operand.

#include <cstdio>
#include <mutex>

#include "activations.h"
#include "cubert_kernels.h"
#include "device_common.h"

namespace cubert {
namespace {

typedef float v16f32 __attribute__((ext_vector_type(16)));

constexpr int kSkinnyWaves = 16;
constexpr int kSkinnyThreads = kSkinnyWaves * kWave;
constexpr int kSkinnyChunk = 16;  // reduction values a wavefront consumes per pass: 8 per lane half
constexpr int kSkinnyMaxTokens = 64;  // two blocks of 32 tokens per wavefront

// Accumulator register i of the lane half hh holds this row of a 32x32 MFMA result (column = lane % 32).
__device__ __forceinline__ int acc_row(int i, int hh) { return (i >> 2) * 8 + hh * 4 + (i & 3); }

typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));

// The 8 reduction values k = hh * 8 + t a lane (r, hh) brings to a chunk, of token r or of feature r, in the form the
// matrix instruction of the storage type takes them.
template <typename T>
struct ChunkOperand;
template <>
struct ChunkOperand<float> {
    float v[8];
    __device__ __forceinline__ void set(int t, float x) { v[t] = x; }
    __device__ __forceinline__ void loaded() {}
};
template <>
struct ChunkOperand<half_t> {
    v8f16 v;
    __device__ __forceinline__ void set(int t, half_t x) { v[t] = x; }
    // Counts as a use: every operand has been requested before the first MFMA.  (One short instruction per chunk:
    // nothing to gain from starting early, and left alone the compiler requests the last operand of a second pass
    // only after the first pass's MFMA, a second memory latency.)
    __device__ __forceinline__ void loaded() { asm volatile("" : "+v"(v)); }
};

// acc[token, feature] += sum over the 16 reduction values of a chunk
__device__ __forceinline__ void chunk_mma(v16f32 &acc, const ChunkOperand<float> &x, const ChunkOperand<float> &w) {
#pragma unroll
    for (int t = 0; t < 8; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(x.v[t], w.v[t], acc, 0, 0, 0);
}
__device__ __forceinline__ void chunk_mma(v16f32 &acc, const ChunkOperand<half_t> &x, const ChunkOperand<half_t> &w) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(x.v, w.v, acc, 0, 0, 0);
}

// Weights in the order the kernel consumes them: for feature block fb and chunk c (16 reduction values), lane
// (r, hh) finds its 8 operand values A[c*16 + hh*8 + t, fb*32 + r], t < 8, in 8 consecutive elements, so a
// workgroup's slice of the weights is one contiguous run (32 KB for fp32) read with 16-byte loads instead of
// 128-byte pieces at a stride of a weight row.  Features past M are stored as zeros.
template <typename T>
__global__ __launch_bounds__(kBlock) void gemm_skinny_pack_kernel(const T *__restrict__ A, int lda, int M, int chunks,
                                                                  T *__restrict__ packed, size_t total) {
    const size_t idx = (size_t) blockIdx.x * kBlock + threadIdx.x;
    if (idx >= total) return;
    const int t = (int) (idx % 8), lane = (int) ((idx / 8) % kWave);
    const size_t tile = idx / (8 * kWave);
    const int c = (int) (tile % chunks), fb = (int) (tile / chunks);
    const int r = lane & 31, hh = lane >> 5;
    const int k = c * kSkinnyChunk + hh * 8 + t, feature = fb * 32 + r;
    packed[idx] = feature < M ? A[(size_t) k * lda + feature] : from_f32<T>(0.f);
}

template <typename T, bool GELU, bool PACKED, int PASSES, int TB>
__global__ __launch_bounds__(kSkinnyThreads) void gemm_skinny_kernel(const T *__restrict__ A, int lda,
                                                                     const T *__restrict__ B, int ldb,
                                                                     const T *__restrict__ bias, T *__restrict__ C,
                                                                     int ldc, int M, int N, int K, float alpha,
                                                                     float *partials, int *counters,
                                                                     int chunks_per_slice, int leave_partials) {
    __shared__ float red[kSkinnyWaves][32 * 32];
    constexpr int V = 16 / sizeof(T);
    const int lane = threadIdx.x & (kWave - 1);
    const int r = lane & 31, hh = lane >> 5, wave = wave_in_block();
    const int m0 = blockIdx.x * 32;
    const int feature = m0 + r;
    const int chunks = K / kSkinnyChunk;
    const int c_begin = blockIdx.y * chunks_per_slice;
    const int c_end = c_begin + chunks_per_slice < chunks ? c_begin + chunks_per_slice : chunks;

    // TB blocks of 32 tokens: a wavefront multiplies its weights with each of them (the weights are loaded once)
    v16f32 acc[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) acc[tb] = v16f32{};
    for (int c0 = c_begin + wave; c0 < c_end; c0 += kSkinnyWaves * PASSES) {
        // reduction slot of MFMA t in lane half hh is k = c*16 + hh*8 + t: the token operand of a lane is 8
        // consecutive values of one row of B (vector loads), the weight operand one column of 8 rows of A.
        // The loads of all PASSES chunks are issued before the first MFMA; a chunk past the slice is read
        // from the wavefront's first chunk (a valid address, no branch around the loads) with its tokens zeroed.
        ChunkOperand<T> x[PASSES][TB], w[PASSES];
        const T zero = from_f32<T>(0.f);
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int c = c0 + p * kSkinnyWaves;
            const bool inside = c < c_end;
            const int kb = (inside ? c : c0) * kSkinnyChunk + hh * 8;
            // (token rows from N on read row N - 1 and count as zero, weight columns from M on read column M - 1 and
            // are never stored: no load stands under a branch, so the first pass can start while the second is on its way)
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) {
                const int row = tb * 32 + r;
#pragma unroll
                for (int u = 0; u < 8 / V; ++u) {
                    const Vec<T, V> xv = load_vec<T, V>(B + (size_t) (row < N ? row : N - 1) * ldb + kb + u * V);
#pragma unroll
                    for (int e = 0; e < V; ++e) x[p][tb].set(u * V + e, inside && row < N ? xv.v[e] : zero);
                }
            }
            if (PACKED) {
                const T *src = A + (((size_t) blockIdx.x * chunks + (inside ? c : c0)) * kWave + lane) * 8;
#pragma unroll
                for (int u = 0; u < 8 / V; ++u) {
                    const Vec<T, V> wv = load_vec<T, V>(src + u * V);
#pragma unroll
                    for (int e = 0; e < V; ++e) w[p].set(u * V + e, wv.v[e]);
                }
            } else {
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    w[p].set(t, A[(size_t) (kb + t) * lda + (feature < M ? feature : M - 1)]);
                }
            }
        }
        // nothing moves across this line: every load of the wavefront is requested before its first MFMA (the waits
        // are placed per operand afterwards, so a first pass still starts while the second is on its way)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            w[p].loaded();
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) x[p][tb].loaded();
        }
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
#pragma unroll
            for (int tb = 0; tb < TB; ++tb) chunk_mma(acc[tb], x[p][tb], w[p]);
        }
    }
    // lane holds C[feature = m0 + r, token = tb * 32 + acc_row(i, hh)]; one output element per thread and token block
    const int token = threadIdx.x >> 5, f = threadIdx.x & 31;
    float sum[TB];
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
        if (tb > 0) __syncthreads();  // the sums of the block before have been read
#pragma unroll
        for (int i = 0; i < 16; ++i) red[wave][acc_row(i, hh) * 32 + r] = acc[tb][i];
        __syncthreads();
        sum[tb] = 0.f;
#pragma unroll
        for (int w = 0; w < kSkinnyWaves; ++w) sum[tb] += red[w][threadIdx.x];
    }
    const int slices = gridDim.y;
    const size_t pitch = (size_t) gridDim.x * 32;  // features, padded to whole blocks
    if (leave_partials) {  // (uniform) the consumer adds the slices: partials[slice][token][feature], all TB * 32 rows
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            partials[((size_t) (blockIdx.y * TB + tb) * 32 + token) * pitch + m0 + f] = sum[tb];
        }
        return;
    }
    if (slices > 1) {
        // The L2 caches of the chip's dies are not coherent with each other, and a device-scope fence would
        // write back / invalidate a whole L2 per call.  Instead every access that crosses workgroups is a
        // relaxed device-scope atomic: such stores write through, such loads read past the die-local cache,
        // and a store has reached the coherent level once the wavefront's store counter has drained.
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            __hip_atomic_store(&partials[((size_t) (blockIdx.y * TB + tb) * 32 + token) * pitch + m0 + f], sum[tb],
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wavefront's partial sums are written
        __syncthreads();                     // ... and so are the other wavefronts' (and red[] is free)
        int *ticket = reinterpret_cast<int *>(&red[0][0]);
        if (threadIdx.x == 0) {
            *ticket = __hip_atomic_fetch_add(&counters[blockIdx.x], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (*ticket != slices - 1) return;
        // last workgroup of this feature block: every slice's partial tile is complete
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            sum[tb] = 0.f;
            for (int s0 = 0; s0 < slices; s0 += 16) {  // up to 16 loads in flight, added in slice order
                float p[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    p[u] = s0 + u < slices
                               ? __hip_atomic_load(&partials[((size_t) ((s0 + u) * TB + tb) * 32 + token) * pitch + m0 + f],
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                               : 0.f;
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) sum[tb] += p[u];
            }
        }
        if (threadIdx.x == 0) {  // ready for the next launch
            __hip_atomic_store(&counters[blockIdx.x], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if (m0 + f < M) {
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            if (tb * 32 + token >= N) break;
            float v = alpha * sum[tb];
            if (bias != nullptr) v += to_f32(bias[m0 + f]);
            if (GELU) v = GeluOp<T>()(v);
            C[(size_t) (tb * 32 + token) * ldc + m0 + f] = from_f32<T>(v);
        }
    }
}

}  // namespace

// How a problem is cut: feature blocks, K slices and the chunks of 16 reduction values per slice.
struct SkinnyPlan {
    int blocks = 0, slices = 0, chunks_per_slice = 0, token_blocks = 0;
};

// Every check gemm_skinny makes and the cut it would launch with; launches nothing.  Returns 0, CUBERT_BAD_ARGUMENT or
// CUBERT_UNSUPPORTED exactly as gemm_skinny does for the same arguments.
template <typename T>
int gemm_skinny_plan(int M, int N, int K, const T *A, int lda, int packed, const T *B, int ldb, int ldc, int activation,
                     size_t partial_floats, int n_counters, SkinnyPlan *plan) {
    if (activation != 0 && activation != 1) return CUBERT_BAD_ARGUMENT;
    if (M <= 0 || N <= 0 || N > kSkinnyMaxTokens || K <= 0 || K % kSkinnyChunk != 0) return CUBERT_UNSUPPORTED;
    if ((!packed && lda < M) || ldb < K || ldc < M) return CUBERT_BAD_ARGUMENT;
    if (packed && !is_aligned(A, 16)) return CUBERT_BAD_ARGUMENT;
    if (!is_aligned(B, 16) || (ldb * sizeof(T)) % 16 != 0) return CUBERT_UNSUPPORTED;
    const int blocks = (M + 31) / 32;
    const int chunks = K / kSkinnyChunk;
    const int token_blocks = (N + 31) / 32;
    // One pass (16 reduction values) per wavefront, unless that makes more workgroups than the chip has compute
    // units: a second round of workgroups costs more than a second pass of every wavefront (measured at
    // 768 x 3072 and 3072 x 768: 10.3 -> 9.5 us), while fewer, longer workgroups lose where one round is enough
    // (768 x 768: 6.4 -> 8.1 us).  Not for 2-byte weights in the plain layout, whose 2-byte loads make the
    // second pass expensive (10.1 -> 11.5 us).  More passes still when the workspace cannot hold that many slices.
    constexpr int kComputeUnits = 256;
    int chunks_per_slice = kSkinnyWaves;
    int slices = (chunks + chunks_per_slice - 1) / chunks_per_slice;
    // With two token blocks of 4-byte operands the matrix-core time per pass doubles and outweighs both (768 x 3072 at
    // 64 tokens: two passes 17.0 us, one 15.1 us; 2-byte operands, whose MFMAs are short, keep two: 8.0 against 8.7 us).
    if (slices > 1 && (long long) slices * blocks > kComputeUnits && (packed || sizeof(T) == 4) &&
        !(sizeof(T) == 4 && token_blocks > 1)) {
        chunks_per_slice = 2 * kSkinnyWaves;
        slices = (chunks + chunks_per_slice - 1) / chunks_per_slice;
    }
    while (slices > 1 && (size_t) slices * token_blocks * 32 * blocks * 32 > partial_floats) {
        chunks_per_slice += kSkinnyWaves;
        slices = (chunks + chunks_per_slice - 1) / chunks_per_slice;
    }
    if (blocks > 65535 || slices > 65535 || (slices > 1 && blocks > n_counters)) return CUBERT_UNSUPPORTED;
    plan->blocks = blocks, plan->slices = slices, plan->chunks_per_slice = chunks_per_slice;
    plan->token_blocks = token_blocks;
    return 0;
}

// Launches the kernel when the problem fits it, else returns CUBERT_UNSUPPORTED and launches nothing.
// activation: 0 = none, 1 = erf-form GELU applied to alpha * A B + bias (the BertIntermediate layer).
// `partials` holds partial_floats floats, `counters` n_counters ints that are zero between launches.
// packed != 0: A is the output of gemm_skinny_pack for the same M and K (lda is ignored).
template <typename T>
int gemm_skinny(int M, int N, int K, float alpha, const T *A, int lda, int packed, const T *B, int ldb, T *C, int ldc,
                const T *bias, int activation, float *partials, size_t partial_floats, int *counters,
                int n_counters, hipStream_t stream) {
    SkinnyPlan plan;
    const int rc = gemm_skinny_plan<T>(M, N, K, A, lda, packed, B, ldb, ldc, activation, partial_floats, n_counters, &plan);
    if (rc) return rc;
    const int blocks = plan.blocks, slices = plan.slices, chunks_per_slice = plan.chunks_per_slice;
    const dim3 grid(blocks, slices), block(kSkinnyThreads);
#define CUBERT_SKINNY_LAUNCH_TB(GELU, PACKED, PASSES, TB)                                                            \
    return launch(gemm_skinny_kernel<T, GELU, PACKED, PASSES, TB>, grid, block, stream, A, lda, B, ldb, bias, C, ldc, M, \
                  N, K, alpha, partials, counters, chunks_per_slice, 0)
#define CUBERT_SKINNY_LAUNCH(GELU, PACKED)                                                                           \
    do {                                                                                                             \
        if (plan.token_blocks == 1) {                                                                                \
            if (chunks_per_slice == kSkinnyWaves) CUBERT_SKINNY_LAUNCH_TB(GELU, PACKED, 1, 1);                       \
            CUBERT_SKINNY_LAUNCH_TB(GELU, PACKED, 2, 1);                                                             \
        }                                                                                                            \
        if (chunks_per_slice == kSkinnyWaves) CUBERT_SKINNY_LAUNCH_TB(GELU, PACKED, 1, 2);                           \
        CUBERT_SKINNY_LAUNCH_TB(GELU, PACKED, 2, 2);                                                                 \
    } while (0)
    if (activation == 1) {
        if (packed) CUBERT_SKINNY_LAUNCH(true, true);
        CUBERT_SKINNY_LAUNCH(true, false);
    }
    if (packed) CUBERT_SKINNY_LAUNCH(false, true);
    CUBERT_SKINNY_LAUNCH(false, false);
#undef CUBERT_SKINNY_LAUNCH_TB
#undef CUBERT_SKINNY_LAUNCH
}

// The same product left as partial tiles: partials[(slice * 32 + token) * pitch + feature] holds slice `slice` of
// sum_k A[k, feature] B[k, token] for all 32 token rows (rows from N on are zero), *slices and *pitch say how many
// and how wide.  No alpha, bias or activation: the consumer adds the slices in slice order (0.f + p0 + p1 + ...) and
// goes on from there, which is what gemm_skinny's last workgroup does.  The cut is gemm_skinny's, or a finer one
// (below), so the sum agrees with gemm_skinny's result up to the order of the additions.  Nothing is launched when
// the problem does not fit.
template <typename T>
int gemm_skinny_partials(int M, int N, int K, const T *A, int lda, int packed, const T *B, int ldb, float *partials,
                         size_t partial_floats, int *slices_out, int *pitch_out, hipStream_t stream) {
    if (!A || !B || !partials || !slices_out || !pitch_out) return CUBERT_BAD_ARGUMENT;
    SkinnyPlan plan;
    const int rc = gemm_skinny_plan<T>(M, N, K, A, lda, packed, B, ldb, M, 0, partial_floats, 0x7fffffff, &plan);
    if (rc) return rc;
    // More slices cost this kernel nothing (it adds none of them), and a matrix with few feature blocks streams faster
    // when more compute units pull on it: such a reduction is cut thinner than a pass of 16 chunks, up to about 192
    // workgroups.  Measured at 768 x 768 (24 feature blocks) inside a forward pass: 3 slices of 16 chunks 7.2 us, 6 of 8
    // and 8 of 6 6.5 us; 12 of 4 no better, and whoever adds the slices reads more of them.
    constexpr int kThinTarget = 192;
    if (plan.chunks_per_slice == kSkinnyWaves && plan.blocks * plan.slices < kThinTarget) {
        const int chunks = K / kSkinnyChunk;
        const int want = kThinTarget / plan.blocks;
        int thin = (chunks + want - 1) / want;
        const size_t tile = (size_t) plan.token_blocks * 32 * plan.blocks * 32;  // floats per slice
        while (thin < kSkinnyWaves && (size_t) ((chunks + thin - 1) / thin) * tile > partial_floats) ++thin;  // what fits
        if (thin >= 1 && thin < kSkinnyWaves) {
            plan.chunks_per_slice = thin;
            plan.slices = (chunks + thin - 1) / thin;
        }
    }
    if ((size_t) plan.slices * plan.token_blocks * 32 * plan.blocks * 32 > partial_floats) return CUBERT_UNSUPPORTED;
    const int chunks_per_slice = plan.chunks_per_slice;
    const dim3 grid(plan.blocks, plan.slices), block(kSkinnyThreads);
    *slices_out = plan.slices;
    *pitch_out = plan.blocks * 32;
    const T *no_bias = nullptr;
    T *no_output = nullptr;
    int *no_counters = nullptr;
#define CUBERT_SKINNY_PARTIALS(PACKED, PASSES, TB)                                                                   \
    return launch(gemm_skinny_kernel<T, false, PACKED, PASSES, TB>, grid, block, stream, A, lda, B, ldb, no_bias,    \
                  no_output, M, M, N, K, 1.f, partials, no_counters, chunks_per_slice, 1)
#define CUBERT_SKINNY_PARTIALS_TB(TB)                                                                                \
    do {                                                                                                             \
        if (chunks_per_slice <= kSkinnyWaves) {                                                                      \
            if (packed) CUBERT_SKINNY_PARTIALS(true, 1, TB);                                                         \
            CUBERT_SKINNY_PARTIALS(false, 1, TB);                                                                    \
        }                                                                                                            \
        if (packed) CUBERT_SKINNY_PARTIALS(true, 2, TB);                                                             \
        CUBERT_SKINNY_PARTIALS(false, 2, TB);                                                                        \
    } while (0)
    if (plan.token_blocks == 1) CUBERT_SKINNY_PARTIALS_TB(1);
    CUBERT_SKINNY_PARTIALS_TB(2);
#undef CUBERT_SKINNY_PARTIALS_TB
#undef CUBERT_SKINNY_PARTIALS
}

// Elements of the packed form of an [K, M] weight matrix.
size_t gemm_skinny_packed_elements(int M, int K) { return (size_t) ((M + 31) / 32) * 32 * (size_t) K; }

template <typename T>
int gemm_skinny_pack(const T *A, int lda, int M, int K, T *packed, hipStream_t stream) {
    if (!A || !packed || M <= 0 || K <= 0 || lda < M) return CUBERT_BAD_ARGUMENT;
    if (K % kSkinnyChunk != 0 || !is_aligned(packed, 16)) return CUBERT_UNSUPPORTED;
    const size_t total = gemm_skinny_packed_elements(M, K);
    const size_t blocks = (total + kBlock - 1) / kBlock;
    if (blocks > 0x7fffffffull) return CUBERT_UNSUPPORTED;
    return launch(gemm_skinny_pack_kernel<T>, dim3((unsigned) blocks), dim3(kBlock), stream, A, lda, M,
                  K / kSkinnyChunk, packed, total);
}

// ---- the same kernel for callers that cannot allocate ---------------------------------------------------
// The split-K partial tiles and the arrival counters of cubert_gemm_skinny_noalloc_f32 live in this array, which is
// part of the library's device image: each GPU the library runs on holds its own copy (4 MiB + 16 KiB) at its own
// address until the process ends.  In host code the array's name is only a stand-in for the symbol; the device
// address comes from hipGetSymbolAddress, once per device, and only that pointer is handed to kernels.
namespace {

constexpr size_t kNoAllocPartialFloats = 1u << 20;  // as many as a BLAS context's workspace: same K slices, same sums
constexpr int kNoAllocCounters = 4096;
constexpr size_t kNoAllocBytes = kNoAllocPartialFloats * sizeof(float) + kNoAllocCounters * sizeof(int);
constexpr int kNoAllocMaxDevices = 64;

// (`used`: no kernel names the array, every kernel receives its address as an argument)
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kNoAllocBytes];

std::mutex g_noalloc_mutex;
void *g_noalloc_scratch[kNoAllocMaxDevices];  // per device: address of that device's copy of `scratch`, once known

__global__ __launch_bounds__(kBlock) void zero_ints_kernel(int *p, int n) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = 0;
}

// Address of the current device's copy of the array (looked up on the first call per device).
int noalloc_scratch(unsigned char **out) {
    int device = -1;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return (int) e;
    if (device < 0 || device >= kNoAllocMaxDevices) {
        fprintf(stderr, "cubert_gemm_skinny_noalloc_f32: device %d is outside the %d devices it keeps scratch addresses for\n",
                device, kNoAllocMaxDevices);
        return CUBERT_BAD_ARGUMENT;
    }
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    if (g_noalloc_scratch[device] == nullptr) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            fprintf(stderr, "cubert_gemm_skinny_noalloc_f32: hipGetSymbolAddress failed on device %d: %s\n", device,
                    hipGetErrorString(e));
            return e != hipSuccess ? (int) e : CUBERT_BAD_ARGUMENT;
        }
        g_noalloc_scratch[device] = ptr;
    }
    *out = static_cast<unsigned char *>(g_noalloc_scratch[device]);
    return 0;
}

}  // namespace

int gemm_skinny_noalloc_f32(int M, int N, int K, float alpha, const float *A, int lda, const float *B, int ldb, float *C,
                            int ldc, const float *bias, int activation, hipStream_t stream) {
    if (!A || !B || !C) return CUBERT_BAD_ARGUMENT;
    if (M > CUBERT_GEMM_SKINNY_NOALLOC_MAX_M || K > CUBERT_GEMM_SKINNY_NOALLOC_MAX_K) {
        fprintf(stderr,
                "cubert_gemm_skinny_noalloc_f32: M = %d, K = %d is beyond what its fixed scratch array is sized for "
                "(M <= %d output features, K <= %d); use cubert_gemm_skinny_f32 with a BLAS context\n",
                M, K, CUBERT_GEMM_SKINNY_NOALLOC_MAX_M, CUBERT_GEMM_SKINNY_NOALLOC_MAX_K);
        return CUBERT_TOO_LARGE;
    }
    unsigned char *base = nullptr;
    const int rc = noalloc_scratch(&base);
    if (rc) return rc;
    float *partials = reinterpret_cast<float *>(base);
    int *counters = reinterpret_cast<int *>(base + kNoAllocPartialFloats * sizeof(float));
    // Every argument and shape check first: a call that is refused has launched nothing (a caller that is capturing
    // a graph records no stray node), exactly as cubert_gemm_skinny_f32.
    SkinnyPlan plan;
    const int refused = gemm_skinny_plan<float>(M, N, K, A, lda, 0, B, ldb, ldc, activation, kNoAllocPartialFloats,
                                                kNoAllocCounters, &plan);
    if (refused) return refused;
    // The array keeps what the last call left in it.  The partial tiles are written before they are read; the
    // counters must start at zero, so the ones this launch can touch are cleared first, on the same stream, by a
    // kernel (not a memset node, which a caller's graph capture would record).
    if (plan.slices > 1) {
        const int e = launch_untimed(zero_ints_kernel, dim3((plan.blocks + kBlock - 1) / kBlock), dim3(kBlock), 0, stream,
                                     counters, plan.blocks);
        if (e) return e;
    }
    return gemm_skinny<float>(M, N, K, alpha, A, lda, 0, B, ldb, C, ldc, bias, activation, partials,
                              kNoAllocPartialFloats, counters, kNoAllocCounters, stream);
}

template int gemm_skinny<float>(int, int, int, float, const float *, int, int, const float *, int, float *, int,
                                const float *, int, float *, size_t, int *, int, hipStream_t);
template int gemm_skinny<half_t>(int, int, int, float, const half_t *, int, int, const half_t *, int, half_t *, int,
                                 const half_t *, int, float *, size_t, int *, int, hipStream_t);
template int gemm_skinny_partials<float>(int, int, int, const float *, int, int, const float *, int, float *, size_t, int *,
                                         int *, hipStream_t);
template int gemm_skinny_partials<half_t>(int, int, int, const half_t *, int, int, const half_t *, int, float *, size_t,
                                          int *, int *, hipStream_t);
template int gemm_skinny_pack<float>(const float *, int, int, int, float *, hipStream_t);
template int gemm_skinny_pack<half_t>(const half_t *, int, int, int, half_t *, hipStream_t);

}  // namespace cubert
