// Device runtime of the library: memory, copies, streams and GEMM.
// The only translation unit that talks to the HIP runtime API and hipBLASLt
// (the layer kernels launch through hipLaunchKernelGGL in their own files).
//
// GEMMs use hipBLASLt with fp32 accumulation (HIPBLAS_COMPUTE_32F) for both
// storage types; plans (descriptor + layouts + the algorithm the heuristic
// ranks first) are cached per shape in the BLAS context, so a steady-state call
// is one hipblasLtMatmul.

#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

#include "cubert_kernels.h"
#include "device_common.h"

namespace cubert {
// kernels/gemm_skinny.hip
template <typename T>
int gemm_skinny(int M, int N, int K, float alpha, const T *A, int lda, int packed, const T *B, int ldb, T *C, int ldc,
                const T *bias, int activation, float *partials, size_t partial_floats, int *counters,
                int n_counters, hipStream_t stream);
size_t gemm_skinny_packed_elements(int M, int K);
int gemm_skinny_noalloc_f32(int M, int N, int K, float alpha, const float *A, int lda, const float *B, int ldb, float *C,
                            int ldc, const float *bias, int activation, hipStream_t stream);
template <typename T>
int gemm_skinny_pack(const T *A, int lda, int M, int K, T *packed, hipStream_t stream);
template <typename T>
int gemm_skinny_partials(int M, int N, int K, const T *A, int lda, int packed, const T *B, int ldb, float *partials,
                         size_t partial_floats, int *slices, int *pitch, hipStream_t stream);
// kernels/gemm_batch.hip
template <typename T>
int gemm_batch(int transA, int transB, int M, int N, int K, float alpha, const T *const *A_array, int lda,
               const T *const *B_array, int ldb, float beta, T *const *C_array, int ldc, int batch, hipStream_t stream);

LaunchTiming &pending_launch_timing() {
    static thread_local LaunchTiming pending;
    return pending;
}
}  // namespace cubert

namespace {

inline int hip_rc(hipError_t e) { return e == hipSuccess ? 0 : (int) e; }

hipMemcpyKind copy_kind(int kind) {
    switch (kind) {
        case 1: return hipMemcpyHostToDevice;
        case 2: return hipMemcpyDeviceToHost;
        case 3: return hipMemcpyDeviceToDevice;
        case 0: return hipMemcpyHostToHost;
        default: return hipMemcpyDefault;
    }
}

constexpr size_t kWorkspaceBytes = 64u << 20;
constexpr int kMaxCandidates = 32;
// scratch of the few-token GEMM kernel: partial tiles (fp32) and one arrival counter per feature block
constexpr size_t kSkinnyPartialFloats = 1u << 20;
constexpr int kSkinnyCounters = 4096;

struct GemmKey {
    int type;  // 0 = f32, 1 = f16, 2 = f16 operands with an f32 result
    int transA, transB, M, N, K, lda, ldb, ldc, batch;
    long long strideA, strideB, strideC;
    bool bias;
    bool beta_zero;
    bool operator<(const GemmKey &o) const {
        return std::tie(type, transA, transB, M, N, K, lda, ldb, ldc, batch, strideA, strideB, strideC, bias, beta_zero) <
               std::tie(o.type, o.transA, o.transB, o.M, o.N, o.K, o.lda, o.ldb, o.ldc, o.batch, o.strideA, o.strideB,
                        o.strideC, o.bias, o.beta_zero);
    }
};

struct GemmPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t a = nullptr, b = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;
    bool ok = false;  // false: hipBLASLt has no algorithm for this shape, the plain kernel runs instead
    // what the heuristic returned, best first by its own ranking; `algo` is one of them
    std::vector<hipblasLtMatmulHeuristicResult_t> candidates;
    bool tuned = false;  // `algo` was chosen by timing (or timing does not apply to this plan)
};

struct BlasContext {
    hipblasLtHandle_t lt = nullptr;
    hipStream_t stream = nullptr;
    void *workspace = nullptr;
    hipEvent_t tune_start = nullptr, tune_stop = nullptr;  // created on first use
    float *skinny_partials = nullptr;
    int *skinny_counters = nullptr;  // zero between launches (the kernel resets what it counted)
    std::map<GemmKey, GemmPlan> plans;
    std::mutex mutex;
    bool used = false;  // something was launched on `stream` since it was set
};

#define LT_TRY(call)                                                                                      \
    do {                                                                                                  \
        hipblasStatus_t st_ = (call);                                                                     \
        if (st_ != HIPBLAS_STATUS_SUCCESS) {                                                              \
            fprintf(stderr, "hipBLASLt error %d at %s:%d: %s\n", (int) st_, __FILE__, __LINE__, #call);   \
            return 1000 + (int) st_;                                                                      \
        }                                                                                                 \
    } while (0)

int make_layout(hipblasLtMatrixLayout_t *out, hipDataType type, int rows, int cols, int ld, int batch,
                long long stride) {
    LT_TRY(hipblasLtMatrixLayoutCreate(out, type, (uint64_t) rows, (uint64_t) cols, (int64_t) ld));
    if (batch > 1) {
        int32_t bc = batch;
        int64_t st = stride;
        LT_TRY(hipblasLtMatrixLayoutSetAttribute(*out, HIPBLASLT_MATRIX_LAYOUT_BATCH_COUNT, &bc, sizeof bc));
        LT_TRY(hipblasLtMatrixLayoutSetAttribute(*out, HIPBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET, &st, sizeof st));
    }
    return 0;
}

int build_plan(BlasContext *ctx, const GemmKey &k, GemmPlan *plan) {
    const hipDataType type = k.type == 0 ? HIP_R_32F : HIP_R_16F;        // of A and B
    const hipDataType out_type = k.type == 1 ? HIP_R_16F : HIP_R_32F;    // of C and the bias
    LT_TRY(hipblasLtMatmulDescCreate(&plan->desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
    hipblasOperation_t ta = k.transA ? HIPBLAS_OP_T : HIPBLAS_OP_N, tb = k.transB ? HIPBLAS_OP_T : HIPBLAS_OP_N;
    LT_TRY(hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof ta));
    LT_TRY(hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof tb));
    if (k.bias) {
        hipblasLtEpilogue_t ep = HIPBLASLT_EPILOGUE_BIAS;
        LT_TRY(hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &ep, sizeof ep));
        int32_t bt = (int32_t) out_type;
        LT_TRY(hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof bt));
        // the heuristic wants a bias pointer to be present; the real one is set per call
        const void *dummy = ctx->workspace;
        LT_TRY(hipblasLtMatmulDescSetAttribute(plan->desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &dummy, sizeof dummy));
    }
    int rc;
    if ((rc = make_layout(&plan->a, type, k.transA ? k.K : k.M, k.transA ? k.M : k.K, k.lda, k.batch, k.strideA))) return rc;
    if ((rc = make_layout(&plan->b, type, k.transB ? k.N : k.K, k.transB ? k.K : k.N, k.ldb, k.batch, k.strideB))) return rc;
    if ((rc = make_layout(&plan->c, out_type, k.M, k.N, k.ldc, k.batch, k.strideC))) return rc;

    hipblasLtMatmulPreference_t pref;
    LT_TRY(hipblasLtMatmulPreferenceCreate(&pref));
    uint64_t ws = kWorkspaceBytes;
    LT_TRY(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof ws));
    hipblasLtMatmulHeuristicResult_t found[kMaxCandidates];
    int n = 0;
    hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(ctx->lt, plan->desc, plan->a, plan->b, plan->c, plan->c, pref,
                                                         kMaxCandidates, found, &n);
    hipblasLtMatmulPreferenceDestroy(pref);
    if (st != HIPBLAS_STATUS_SUCCESS || n == 0) {
        if (getenv("CUBERT_VERBOSE")) {
            fprintf(stderr,
                    "hipBLASLt: no algorithm for gemm type=%d trans=%d%d M=%d N=%d K=%d lda=%d ldb=%d ldc=%d batch=%d "
                    "bias=%d (status %d); using the plain kernel\n",
                    k.type, k.transA, k.transB, k.M, k.N, k.K, k.lda, k.ldb, k.ldc, k.batch, (int) k.bias, (int) st);
        }
        plan->ok = false;
        return 0;
    }
    plan->algo = found[0].algo;
    plan->workspace = found[0].workspaceSize;
    plan->candidates.assign(found, found + n);
    plan->ok = true;
    return 0;
}

// ---- choosing among the heuristic's candidates by timing -------------------------------------------------
// The heuristic ranks algorithms without knowing the data; on this part the matrix cores are power limited and
// the ranking moves with the operand values (measured on the Dense shapes of batch 128 x seq 32 fp32 and of
// BERT-large batch 256 x seq 128 fp16 with random operands: its first choice is 7-18 % slower than the best of
// its 32 candidates).  So the first call of a large enough GEMM shape times every candidate on the caller's
// own operands (beta = 0 only: the output is simply overwritten each time) and keeps the fastest (with a margin of
// 3 % a candidate that is 3 % faster was taken in some runs and not in others, and the forward pass of batch 64 x
// seq 512 landed at 7.26 or 7.41 ms accordingly; with two timing passes and a margin of 1 % it is 7.25-7.29 ms).  The choice
// is remembered per shape for the whole process, so that every context computes a shape the same way.
// CUBERT_GEMM_TUNE=0 in the environment keeps the heuristic's first choice.  (The reference exposes the same
// decision as its GEMM_ALGO_* environment variables, src/cuBERT/common.cpp:106-160.)

constexpr double kTuneMinFlops = 1e9;
// fp32 operands are timed from much smaller shapes on (forward pass of BERT-base fp32 at seq 32 with against without,
// two alternating runs on one box: batch 4 0.740 / 0.757 ms, batch 6 0.791 / 0.898, batch 8 0.887 / 0.943, batch 16
// 1.110 / 1.184, batch 32 1.71-1.75 / 1.829; batch 3 equal).  The same for fp16 operands loses more often than it
// wins (batch 4 0.565 / 0.546 ms, batch 6 0.56-0.59 / 0.54-0.56, batch 8 0.56-0.58 / 0.55), so they keep the limits.
constexpr double kTuneMinFlopsF32 = 5e7;
constexpr float kTuneMinCallMsF32 = 0.004f;
constexpr int kTuneRuns = 8;
constexpr int kTunePasses = 2;
constexpr float kTuneMinGain = 0.99f;  // leave the heuristic's first choice unless another is at least 1 % faster
// A shape whose first choice takes less than this per call keeps it: what a call that short costs inside a layer is
// set by the kernels around it (launch gaps, what they left in the caches), which a burst of identical calls does
// not show.  Measured, forward pass with against without the timing on one box, three runs each: batch 32 x seq 128
// fp16 (calls of 22 us) 1.454-1.481 against 1.434 ms; batch 64 x seq 512 fp16 (109 us) 7.19-7.20 against 7.34 ms;
// batch 128 x seq 32 fp32 (102 us) 5.47-5.50 against 5.59-5.61 ms; BERT-large batch 256 x seq 128 fp16 (159 us) equal.
constexpr float kTuneMinCallMs = 0.05f;

bool tuning_enabled() {
    static const bool on = [] {
        const char *v = getenv("CUBERT_GEMM_TUNE");
        return v == nullptr || std::string(v) != "0";
    }();
    return on;
}

std::mutex &tuned_mutex() {
    static std::mutex m;
    return m;
}
std::map<GemmKey, int> &tuned_ranks() {
    static std::map<GemmKey, int> ranks;
    return ranks;
}

void tune_plan(BlasContext *ctx, const GemmKey &k, GemmPlan &p, float alpha, const void *A, const void *B, void *C) {
    p.tuned = true;
    const double flops = 2.0 * k.M * k.N * k.K * k.batch;
    const bool f32 = k.type == 0;
    if (!tuning_enabled() || !k.beta_zero || p.candidates.size() < 2 || flops < (f32 ? kTuneMinFlopsF32 : kTuneMinFlops)) {
        return;
    }
    {
        std::lock_guard<std::mutex> lock(tuned_mutex());
        auto it = tuned_ranks().find(k);
        if (it != tuned_ranks().end()) {
            if (it->second < (int) p.candidates.size()) {
                p.algo = p.candidates[it->second].algo;
                p.workspace = p.candidates[it->second].workspaceSize;
            }
            return;
        }
    }
    if (ctx->tune_start == nullptr) {
        if (hipEventCreate(&ctx->tune_start) != hipSuccess || hipEventCreate(&ctx->tune_stop) != hipSuccess) {
            (void) hipGetLastError();
            return;
        }
    }
    const float beta = 0.f;
    // Two passes over the candidates, each candidate judged by the faster of its two bursts: the chip's clocks move
    // while the timing runs, and a candidate timed once during a slow spell would lose to a worse one.
    std::vector<float> fastest(p.candidates.size(), 0.f);
    for (int pass = 0; pass < kTunePasses; ++pass) {
        for (int i = 0; i < (int) p.candidates.size(); ++i) {
            if (pass > 0 && fastest[i] == 0.f) continue;  // failed in the first pass
            hipblasLtMatmulAlgo_t *algo = &p.candidates[i].algo;
            bool ok = true;
            if (pass == 0) {  // warm-up, also a check
                ok = hipblasLtMatmul(ctx->lt, p.desc, &alpha, A, p.a, B, p.b, &beta, C, p.c, C, p.c, algo, ctx->workspace,
                                     kWorkspaceBytes, ctx->stream) == HIPBLAS_STATUS_SUCCESS;
                if (!ok) continue;
            }
            if (hipEventRecord(ctx->tune_start, ctx->stream) != hipSuccess) return;
            for (int r = 0; r < kTuneRuns && ok; ++r) {
                ok = hipblasLtMatmul(ctx->lt, p.desc, &alpha, A, p.a, B, p.b, &beta, C, p.c, C, p.c, algo, ctx->workspace,
                                     kWorkspaceBytes, ctx->stream) == HIPBLAS_STATUS_SUCCESS;
            }
            float ms = 0.f;
            if (hipEventRecord(ctx->tune_stop, ctx->stream) != hipSuccess ||
                hipEventSynchronize(ctx->tune_stop) != hipSuccess ||
                hipEventElapsedTime(&ms, ctx->tune_start, ctx->tune_stop) != hipSuccess) {
                (void) hipGetLastError();
                return;
            }
            if (!ok) {
                fastest[i] = 0.f;
                continue;
            }
            if (fastest[i] == 0.f || ms < fastest[i]) fastest[i] = ms;
            if (pass == 0 && i == 0 && ms < (f32 ? kTuneMinCallMsF32 : kTuneMinCallMs) * kTuneRuns) {
                std::lock_guard<std::mutex> lock(tuned_mutex());
                tuned_ranks()[k] = 0;
                return;
            }
        }
    }
    int best = 0;
    float best_ms = 0.f;
    const float first_ms = fastest[0];
    for (int i = 0; i < (int) p.candidates.size(); ++i) {
        if (fastest[i] > 0.f && (best_ms == 0.f || fastest[i] < best_ms)) {
            best_ms = fastest[i];
            best = i;
        }
    }
    if (best_ms == 0.f) return;
    if (first_ms > 0.f && best_ms > kTuneMinGain * first_ms) {  // within the noise of the timing: the heuristic's choice stays
        best = 0;
        best_ms = first_ms;
    }
    p.algo = p.candidates[best].algo;
    p.workspace = p.candidates[best].workspaceSize;
    {
        std::lock_guard<std::mutex> lock(tuned_mutex());
        tuned_ranks()[k] = best;
    }
    if (getenv("CUBERT_VERBOSE")) {
        fprintf(stderr, "hipBLASLt: gemm type=%d trans=%d%d M=%d N=%d K=%d batch=%d bias=%d: candidate %d of %d, %.1f us\n",
                k.type, k.transA, k.transB, k.M, k.N, k.K, k.batch, (int) k.bias, best, (int) p.candidates.size(),
                best_ms * 1e3 / kTuneRuns);
    }
}

// Plain one-thread-per-output GEMM (fp32 accumulation, k ascending).  Used for shapes hipBLASLt has no
// algorithm for (tiny or oddly aligned operands) and, with CUBERT_GEMM=naive in the environment, for all
// of them, which gives an independent check of the hipBLASLt call convention.
template <typename T, typename TC = T>
__global__ void naive_gemm_kernel(int transA, int transB, int M, int N, int K, float alpha, const T *__restrict__ A,
                                  int lda, long long strideA, const T *__restrict__ B, int ldb, long long strideB,
                                  float beta, TC *__restrict__ C, int ldc, long long strideC, int batch,
                                  const TC *__restrict__ bias) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const int j = blockIdx.y * blockDim.y + threadIdx.y;
    if (i >= M || j >= N) return;
    for (int z = blockIdx.z; z < batch; z += gridDim.z) {
        const T *a = A + z * strideA;
        const T *b = B + z * strideB;
        TC *c = C + z * strideC;
        float acc = 0.f;
        for (int k = 0; k < K; ++k) {
            const float av = (float) (transA ? a[k + (size_t) i * lda] : a[i + (size_t) k * lda]);
            const float bv = (float) (transB ? b[j + (size_t) k * ldb] : b[k + (size_t) j * ldb]);
            acc += av * bv;
        }
        float v = alpha * acc;
        if (beta != 0.f) v += beta * (float) c[i + (size_t) j * ldc];
        if (bias != nullptr) v += (float) bias[i];
        c[i + (size_t) j * ldc] = (TC) v;
    }
}

int run_naive_gemm(hipStream_t stream, int type, int transA, int transB, int M, int N, int K, float alpha,
                   const void *A, int lda, long long strideA, const void *B, int ldb, long long strideB, float beta,
                   void *C, int ldc, long long strideC, int batch, const void *bias) {
    dim3 block(16, 16), grid((M + 15) / 16, (N + 15) / 16, batch < 65535 ? batch : 65535);
    if (grid.y > 65535) return CUBERT_BAD_ARGUMENT;
    if (type == 0) {
        hipLaunchKernelGGL(naive_gemm_kernel<float>, grid, block, 0, stream, transA, transB, M, N, K, alpha,
                           (const float *) A, lda, strideA, (const float *) B, ldb, strideB, beta, (float *) C, ldc,
                           strideC, batch, (const float *) bias);
    } else if (type == 1) {
        hipLaunchKernelGGL(naive_gemm_kernel<_Float16>, grid, block, 0, stream, transA, transB, M, N, K, alpha,
                           (const _Float16 *) A, lda, strideA, (const _Float16 *) B, ldb, strideB, beta,
                           (_Float16 *) C, ldc, strideC, batch, (const _Float16 *) bias);
    } else {
        hipLaunchKernelGGL((naive_gemm_kernel<_Float16, float>), grid, block, 0, stream, transA, transB, M, N, K, alpha,
                           (const _Float16 *) A, lda, strideA, (const _Float16 *) B, ldb, strideB, beta, (float *) C,
                           ldc, strideC, batch, (const float *) bias);
    }
    return hip_rc(hipGetLastError());
}

bool gemm_mode_is(const char *mode) {
    const char *v = getenv("CUBERT_GEMM");
    return v != nullptr && std::string(v) == mode;
}

bool force_naive_gemm() {
    static const bool forced = gemm_mode_is("naive");
    return forced;
}

// CUBERT_GEMM=library sends every GEMM to hipBLASLt, also those the few-token kernel would take.
bool library_gemm_only() {
    static const bool forced = gemm_mode_is("library");
    return forced;
}

int run_skinny(BlasContext *ctx, int type, int M, int N, int K, float alpha, const void *A, int lda, const void *B,
               int ldb, void *C, int ldc, const void *bias, int activation, int packed = 0) {
    if (type == 0) {
        return cubert::gemm_skinny<float>(M, N, K, alpha, (const float *) A, lda, packed, (const float *) B, ldb, (float *) C,
                                          ldc, (const float *) bias, activation, ctx->skinny_partials,
                                          kSkinnyPartialFloats, ctx->skinny_counters, kSkinnyCounters, ctx->stream);
    }
    return cubert::gemm_skinny<cubert::half_t>(M, N, K, alpha, (const cubert::half_t *) A, lda, packed,
                                               (const cubert::half_t *) B, ldb, (cubert::half_t *) C, ldc,
                                               (const cubert::half_t *) bias, activation, ctx->skinny_partials,
                                               kSkinnyPartialFloats, ctx->skinny_counters, kSkinnyCounters,
                                               ctx->stream);
}

// The same for the entry points that reach the kernel directly: one launch at a time per context.
int run_skinny_locked(BlasContext *ctx, int type, int M, int N, int K, float alpha, const void *A, int lda,
                      const void *B, int ldb, void *C, int ldc, const void *bias, int activation, int packed = 0) {
    std::lock_guard<std::mutex> lock(ctx->mutex);
    ctx->used = true;
    return run_skinny(ctx, type, M, N, K, alpha, A, lda, B, ldb, C, ldc, bias, activation, packed);
}

int run_gemm(void *handle, int type, int transA, int transB, int M, int N, int K, float alpha, const void *A, int lda,
             long long strideA, const void *B, int ldb, long long strideB, float beta, void *C, int ldc,
             long long strideC, int batch, const void *bias) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx || !A || !B || !C || M < 0 || N < 0 || K < 0 || batch < 0) return CUBERT_BAD_ARGUMENT;
    if (M == 0 || N == 0 || batch == 0) return 0;
    GemmKey key{type, transA, transB, M, N, K, lda, ldb, ldc, batch, strideA, strideB, strideC, bias != nullptr,
                beta == 0.f};
    // one launch at a time per context: the stream it launches on (cubert_blas_set_stream changes it under the same
    // lock), the plan cache, and the few-token kernel's partial tiles and counters
    std::lock_guard<std::mutex> lock(ctx->mutex);
    ctx->used = true;
    if (force_naive_gemm()) {
        return run_naive_gemm(ctx->stream, type, transA, transB, M, N, K, alpha, A, lda, strideA, B, ldb, strideB,
                              beta, C, ldc, strideC, batch, bias);
    }
    if (type != 2 && !transA && !transB && batch == 1 && beta == 0.f && N <= 32 && !library_gemm_only()) {
        const int rc = run_skinny(ctx, type, M, N, K, alpha, A, lda, B, ldb, C, ldc, bias, 0);
        if (rc != CUBERT_UNSUPPORTED) return rc;
    }
    auto it = ctx->plans.find(key);
    if (it == ctx->plans.end()) {
        GemmPlan plan;
        int rc = build_plan(ctx, key, &plan);
        if (rc) return rc;
        it = ctx->plans.emplace(key, plan).first;
    }
    GemmPlan &p = it->second;
    if (!p.ok) {
        return run_naive_gemm(ctx->stream, type, transA, transB, M, N, K, alpha, A, lda, strideA, B, ldb, strideB,
                              beta, C, ldc, strideC, batch, bias);
    }
    if (bias) {
        LT_TRY(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof bias));
    }
    if (!p.tuned) tune_plan(ctx, key, p, alpha, A, B, C);
    LT_TRY(hipblasLtMatmul(ctx->lt, p.desc, &alpha, A, p.a, B, p.b, &beta, C, p.c, C, p.c, &p.algo, ctx->workspace,
                           kWorkspaceBytes, ctx->stream));
    return 0;
}

}  // namespace

extern "C" {

int cubert_get_gpu_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void) hipGetLastError();
        return 0;
    }
    return n;
}

int cubert_set_gpu(int device) { return hip_rc(hipSetDevice(device)); }

int cubert_gpu_info(int device) {
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return (int) e;
    fprintf(stderr, "Found device %d: %s (%s), %d compute units, %.1f GiB, memory clock %d kHz, pci bus %d\n", device,
            prop.name, prop.gcnArchName, prop.multiProcessorCount, prop.totalGlobalMem / 1073741824.0,
            prop.memoryClockRate, prop.pciBusID);
    return 0;
}

void *cubert_malloc(size_t size) {
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, size ? size : 1);
    if (e != hipSuccess) {
        size_t free_b = 0, total_b = 0;
        (void) hipMemGetInfo(&free_b, &total_b);
        fprintf(stderr, "HIP %s. Tried to allocate %zu (%zu total; %zu free)\n", hipGetErrorString(e), size, total_b,
                free_b);
        return nullptr;
    }
    return p;
}

int cubert_free(void *ptr) { return ptr ? hip_rc(hipFree(ptr)) : 0; }

int cubert_mem_info(size_t *free_bytes, size_t *total_bytes) {
    size_t free_b = 0, total_b = 0;
    const hipError_t e = hipMemGetInfo(&free_b, &total_b);
    if (e != hipSuccess) return (int) e;
    if (free_bytes != nullptr) *free_bytes = free_b;
    if (total_bytes != nullptr) *total_bytes = total_b;
    return 0;
}

int cubert_memcpy(void *dst, const void *src, size_t n, int kind) {
    if (n == 0) return 0;
    return hip_rc(hipMemcpy(dst, src, n, copy_kind(kind)));
}

int cubert_memcpy_async(void *dst, const void *src, size_t n, int kind, void *stream) {
    if (n == 0) return 0;
    return hip_rc(hipMemcpyAsync(dst, src, n, copy_kind(kind), (hipStream_t) stream));
}

void *cubert_stream_create(void) {
    hipStream_t s = nullptr;
    if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess) return nullptr;
    return s;
}

int cubert_stream_destroy(void *stream) { return stream ? hip_rc(hipStreamDestroy((hipStream_t) stream)) : 0; }

int cubert_stream_synchronize(void *stream) { return hip_rc(hipStreamSynchronize((hipStream_t) stream)); }

void *cubert_event_create(void) {
    // Device-scope release: recording the event does not write the caches back to memory, which keeps
    // the marker cheap and leaves the cache state of the timed kernels as it would be without timing.
    hipEvent_t e = nullptr;
    if (hipEventCreateWithFlags(&e, hipEventReleaseToDevice) != hipSuccess) return nullptr;
    return e;
}

void *cubert_malloc_host(size_t size) {
    void *p = nullptr;
    if (hipHostMalloc(&p, size, hipHostMallocDefault) != hipSuccess) {
        (void) hipGetLastError();
        return nullptr;
    }
    return p;
}

int cubert_free_host(void *ptr) { return ptr ? hip_rc(hipHostFree(ptr)) : 0; }

int cubert_event_synchronize(void *event) { return hip_rc(hipEventSynchronize((hipEvent_t) event)); }

int cubert_event_destroy(void *event) { return event ? hip_rc(hipEventDestroy((hipEvent_t) event)) : 0; }

int cubert_event_record(void *event, void *stream) { return hip_rc(hipEventRecord((hipEvent_t) event, (hipStream_t) stream)); }

int cubert_time_next_launch(void *start_event, void *stop_event) {
    cubert::LaunchTiming &t = cubert::pending_launch_timing();
    t.start = (hipEvent_t) start_event;
    t.stop = (hipEvent_t) stop_event;
    return 0;
}

int cubert_event_elapsed_ms(void *start, void *stop, float *ms) {
    return hip_rc(hipEventElapsedTime(ms, (hipEvent_t) start, (hipEvent_t) stop));
}

void *cubert_blas_create(void) {
    BlasContext *ctx = new BlasContext();
    if (hipblasLtCreate(&ctx->lt) != HIPBLAS_STATUS_SUCCESS) {
        delete ctx;
        return nullptr;
    }
    if (hipMalloc(&ctx->workspace, kWorkspaceBytes) != hipSuccess ||
        hipMalloc((void **) &ctx->skinny_partials, kSkinnyPartialFloats * sizeof(float)) != hipSuccess ||
        hipMalloc((void **) &ctx->skinny_counters, kSkinnyCounters * sizeof(int)) != hipSuccess ||
        hipMemset(ctx->skinny_counters, 0, kSkinnyCounters * sizeof(int)) != hipSuccess) {
        (void) hipFree(ctx->workspace);
        (void) hipFree(ctx->skinny_partials);
        (void) hipFree(ctx->skinny_counters);
        hipblasLtDestroy(ctx->lt);
        delete ctx;
        return nullptr;
    }
    return ctx;
}

int cubert_blas_destroy(void *handle) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx) return 0;
    for (auto &kv : ctx->plans) {
        GemmPlan &p = kv.second;
        if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
        if (p.b) hipblasLtMatrixLayoutDestroy(p.b);
        if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
        if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
    }
    (void) hipFree(ctx->workspace);
    (void) hipFree(ctx->skinny_partials);
    (void) hipFree(ctx->skinny_counters);
    if (ctx->tune_start) (void) hipEventDestroy(ctx->tune_start);
    if (ctx->tune_stop) (void) hipEventDestroy(ctx->tune_stop);
    hipblasLtDestroy(ctx->lt);
    delete ctx;
    return 0;
}

int cubert_blas_set_stream(void *handle, void *stream) {
    if (!handle) return CUBERT_BAD_ARGUMENT;
    BlasContext *ctx = (BlasContext *) handle;
    std::lock_guard<std::mutex> lock(ctx->mutex);
    if (ctx->stream != (hipStream_t) stream && ctx->used) {
        // launches on the old stream may still be using the context's workspaces: let them finish before the
        // next launch, on the new stream, reuses them
        const int rc = hip_rc(hipStreamSynchronize(ctx->stream));
        if (rc) return rc;
        ctx->used = false;
    }
    ctx->stream = (hipStream_t) stream;
    return 0;
}

void *cubert_blas_get_stream(void *handle) { return handle ? (void *) ((BlasContext *) handle)->stream : nullptr; }

int cubert_gemm_f32(void *handle, int transA, int transB, int M, int N, int K, float alpha, const float *A, int lda,
                    const float *B, int ldb, float beta, float *C, int ldc, const float *bias) {
    return run_gemm(handle, 0, transA, transB, M, N, K, alpha, A, lda, 0, B, ldb, 0, beta, C, ldc, 0, 1, bias);
}

int cubert_gemm_f16(void *handle, int transA, int transB, int M, int N, int K, float alpha, const cubert_half *A,
                    int lda, const cubert_half *B, int ldb, float beta, cubert_half *C, int ldc,
                    const cubert_half *bias) {
    return run_gemm(handle, 1, transA, transB, M, N, K, alpha, A, lda, 0, B, ldb, 0, beta, C, ldc, 0, 1, bias);
}

int cubert_gemm_f16_f32(void *handle, int transA, int transB, int M, int N, int K, float alpha, const cubert_half *A,
                        int lda, const cubert_half *B, int ldb, float beta, float *C, int ldc, const float *bias) {
    return run_gemm(handle, 2, transA, transB, M, N, K, alpha, A, lda, 0, B, ldb, 0, beta, C, ldc, 0, 1, bias);
}

int cubert_gemm_skinny_f32(void *handle, int M, int N, int K, float alpha, const float *A, int lda, const float *B,
                           int ldb, float *C, int ldc, const float *bias, int activation) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx || !A || !B || !C) return CUBERT_BAD_ARGUMENT;
    if (library_gemm_only() || force_naive_gemm()) return CUBERT_UNSUPPORTED;
    return run_skinny_locked(ctx, 0, M, N, K, alpha, A, lda, B, ldb, C, ldc, bias, activation);
}

int cubert_gemm_skinny_f16(void *handle, int M, int N, int K, float alpha, const cubert_half *A, int lda,
                           const cubert_half *B, int ldb, cubert_half *C, int ldc, const cubert_half *bias,
                           int activation) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx || !A || !B || !C) return CUBERT_BAD_ARGUMENT;
    if (library_gemm_only() || force_naive_gemm()) return CUBERT_UNSUPPORTED;
    return run_skinny_locked(ctx, 1, M, N, K, alpha, A, lda, B, ldb, C, ldc, bias, activation);
}

int cubert_gemm_skinny_noalloc_f32(void *stream, int M, int N, int K, float alpha, const float *A, int lda,
                                   const float *B, int ldb, float *C, int ldc, const float *bias, int activation) {
    if (!A || !B || !C) return CUBERT_BAD_ARGUMENT;
    if (library_gemm_only() || force_naive_gemm()) return CUBERT_UNSUPPORTED;  // as cubert_gemm_skinny_f32
    return cubert::gemm_skinny_noalloc_f32(M, N, K, alpha, A, lda, B, ldb, C, ldc, bias, activation,
                                           (hipStream_t) stream);
}

size_t cubert_gemm_skinny_packed_elements(int M, int K) { return cubert::gemm_skinny_packed_elements(M, K); }

int cubert_gemm_skinny_pack_f32(void *handle, const float *A, int lda, int M, int K, float *packed) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx) return CUBERT_BAD_ARGUMENT;
    return cubert::gemm_skinny_pack<float>(A, lda, M, K, packed, ctx->stream);
}

int cubert_gemm_skinny_pack_f16(void *handle, const cubert_half *A, int lda, int M, int K, cubert_half *packed) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx) return CUBERT_BAD_ARGUMENT;
    return cubert::gemm_skinny_pack<cubert::half_t>((const cubert::half_t *) A, lda, M, K, (cubert::half_t *) packed,
                                                    ctx->stream);
}

int cubert_gemm_skinny_packed_f32(void *handle, int M, int N, int K, float alpha, const float *packedA, const float *B,
                                  int ldb, float *C, int ldc, const float *bias, int activation) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx || !packedA || !B || !C) return CUBERT_BAD_ARGUMENT;
    if (library_gemm_only() || force_naive_gemm()) return CUBERT_UNSUPPORTED;
    return run_skinny_locked(ctx, 0, M, N, K, alpha, packedA, 0, B, ldb, C, ldc, bias, activation, 1);
}

int cubert_gemm_skinny_packed_f16(void *handle, int M, int N, int K, float alpha, const cubert_half *packedA,
                                  const cubert_half *B, int ldb, cubert_half *C, int ldc, const cubert_half *bias,
                                  int activation) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx || !packedA || !B || !C) return CUBERT_BAD_ARGUMENT;
    if (library_gemm_only() || force_naive_gemm()) return CUBERT_UNSUPPORTED;
    return run_skinny_locked(ctx, 1, M, N, K, alpha, packedA, 0, B, ldb, C, ldc, bias, activation, 1);
}

int cubert_gemm_skinny_partials_f32(void *handle, int M, int N, int K, const float *A, int lda, int packed,
                                    const float *B, int ldb, float *partials, size_t partial_floats, int *slices,
                                    int *pitch) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx || !A || !B || !partials || !slices || !pitch) return CUBERT_BAD_ARGUMENT;
    if (library_gemm_only() || force_naive_gemm()) return CUBERT_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(ctx->mutex);
    ctx->used = true;
    return cubert::gemm_skinny_partials<float>(M, N, K, A, lda, packed, B, ldb, partials, partial_floats, slices, pitch,
                                               ctx->stream);
}

int cubert_gemm_skinny_partials_f16(void *handle, int M, int N, int K, const cubert_half *A, int lda, int packed,
                                    const cubert_half *B, int ldb, float *partials, size_t partial_floats, int *slices,
                                    int *pitch) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx || !A || !B || !partials || !slices || !pitch) return CUBERT_BAD_ARGUMENT;
    if (library_gemm_only() || force_naive_gemm()) return CUBERT_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(ctx->mutex);
    ctx->used = true;
    return cubert::gemm_skinny_partials<cubert::half_t>(M, N, K, (const cubert::half_t *) A, lda, packed,
                                                        (const cubert::half_t *) B, ldb, partials, partial_floats,
                                                        slices, pitch, ctx->stream);
}

int cubert_gemm_strided_batch_f32(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                                  const float *A, int lda, long long strideA, const float *B, int ldb,
                                  long long strideB, float beta, float *C, int ldc, long long strideC,
                                  int batch_count) {
    return run_gemm(handle, 0, transA, transB, M, N, K, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC,
                    batch_count, nullptr);
}

int cubert_gemm_strided_batch_f16(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                                  const cubert_half *A, int lda, long long strideA, const cubert_half *B, int ldb,
                                  long long strideB, float beta, cubert_half *C, int ldc, long long strideC,
                                  int batch_count) {
    return run_gemm(handle, 1, transA, transB, M, N, K, alpha, A, lda, strideA, B, ldb, strideB, beta, C, ldc, strideC,
                    batch_count, nullptr);
}

int cubert_gemm_batch_f32(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                          const float *const *A_array, int lda, const float *const *B_array, int ldb, float beta,
                          float *const *C_array, int ldc, int batch_count) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx) return CUBERT_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ctx->mutex);
    ctx->used = true;
    return cubert::gemm_batch<float>(transA, transB, M, N, K, alpha, A_array, lda, B_array, ldb, beta, C_array, ldc,
                                     batch_count, ctx->stream);
}

int cubert_gemm_batch_f16(void *handle, int transA, int transB, int M, int N, int K, float alpha,
                          const cubert_half *const *A_array, int lda, const cubert_half *const *B_array, int ldb,
                          float beta, cubert_half *const *C_array, int ldc, int batch_count) {
    BlasContext *ctx = (BlasContext *) handle;
    if (!ctx) return CUBERT_BAD_ARGUMENT;
    std::lock_guard<std::mutex> lock(ctx->mutex);
    ctx->used = true;
    return cubert::gemm_batch<cubert::half_t>(transA, transB, M, N, K, alpha, (const cubert::half_t *const *) A_array,
                                              lda, (const cubert::half_t *const *) B_array, ldb, beta,
                                              (cubert::half_t *const *) C_array, ldc, batch_count, ctx->stream);
}

}  // extern "C"
