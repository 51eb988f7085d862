// Shared device helpers for the gfx950 layer kernels: 16-byte vector access,
// storage <-> fp32 conversion and cross-lane reductions for 64-wide wavefronts.
#pragma once

#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cubert {

constexpr int kWave = 64;        // CDNA wavefront width
constexpr int kBlock = 256;      // threads per workgroup used by every kernel here (4 wavefronts)

typedef _Float16 half_t;         // IEEE binary16 storage type

// N consecutive elements moved with one memory instruction (N * sizeof(T) <= 16 bytes).
template <typename T, int N>
struct alignas(sizeof(T) * N) Vec {
    T v[N];
};

template <typename T, int N>
__device__ __forceinline__ Vec<T, N> load_vec(const T *p) {
    return *reinterpret_cast<const Vec<T, N> *>(p);
}

template <typename T, int N>
__device__ __forceinline__ void store_vec(T *p, const Vec<T, N> &x) {
    *reinterpret_cast<Vec<T, N> *>(p) = x;
}

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(half_t x) { return (float) x; }

template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <>
__device__ __forceinline__ half_t from_f32<half_t>(float x) { return (half_t) x; }  // round to nearest even

// An fp32 value as the sum of two fp16 numbers, hi = fp16(x) and lo = fp16(x - hi) (x - hi is exact in fp32), both
// clamped to the fp16 range: the operand form of the fp32 Dense layers that run on the fp16 matrix cores.
__device__ __forceinline__ void split_two_terms(float x, half_t &hi, half_t &lo) {
    constexpr float kMax = 65504.f;
    hi = (half_t) fminf(fmaxf(x, -kMax), kMax);
    lo = (half_t) fminf(fmaxf(x - (float) hi, -kMax), kMax);
}

// Whether split_two_terms had to clamp x (or x is not a number): the two terms then do not add up to x, and whoever
// consumes them must be told (the kernels that write two-term rows raise a flag the caller looks at).
__device__ __forceinline__ bool two_term_overflow(float x) { return !(fabsf(x) <= 65504.f); }

// x when keep, +0.f otherwise, as a bit operation: a select between a loaded value and zero invites the compiler to
// put the load itself under a branch, where it is waited for on the spot.
__device__ __forceinline__ float keep_or_zero(float x, bool keep) {
    return __builtin_bit_cast(float, __builtin_bit_cast(unsigned, x) & (keep ? 0xffffffffu : 0u));
}

// An empty statement that counts as a use and a redefinition of x (whole 32-bit registers).  Such statements keep
// their order among themselves, and a loaded value has to have arrived before one that names it: a way to make the
// compiler request a load early instead of where its value is first needed.
template <typename X>
__device__ __forceinline__ void pin_registers(X &x) {
    static_assert(sizeof(X) % 4 == 0, "whole registers");
    unsigned words[sizeof(X) / 4];
    __builtin_memcpy(words, &x, sizeof(X));
#pragma unroll
    for (unsigned i = 0; i < sizeof(X) / 4; ++i) asm volatile("" : "+v"(words[i]));
    __builtin_memcpy(&x, words, sizeof(X));
}

// Widest vector (in elements) that is at most 16 bytes.
template <typename T>
struct MaxVec {
    static constexpr int value = 16 / sizeof(T);
};

// ---- cross-lane exchange -------------------------------------------------
// DPP moves data between lanes of a row of 16 in the same instruction slot as
// an ALU op; 32- and 64-lane steps go through the LDS crossbar (ds_bpermute).

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    int i = __builtin_bit_cast(int, v);
    i = __builtin_amdgcn_update_dpp(i, i, CTRL, 0xf, 0xf, false);
    return __builtin_bit_cast(float, i);
}

constexpr int kDppQuadXor1 = 0xB1;       // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;       // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141; // lane i <- lane 7-i within each 8 lanes
constexpr int kDppRowMirror = 0x140;     // lane i <- lane 15-i within each 16 lanes

struct SumOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct MaxOp {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

// All-reduce over aligned groups of LANES consecutive lanes (LANES = 1..64, a
// power of two).  Every lane of a group ends up with the group's result.
template <int LANES, typename Op>
__device__ __forceinline__ float group_reduce(float v, Op op) {
    static_assert(LANES >= 1 && LANES <= 64 && (LANES & (LANES - 1)) == 0, "LANES must be a power of two");
    if (LANES >= 2) v = op(v, dpp_move<kDppQuadXor1>(v));
    if (LANES >= 4) v = op(v, dpp_move<kDppQuadXor2>(v));
    if (LANES >= 8) v = op(v, dpp_move<kDppRowHalfMirror>(v));
    if (LANES >= 16) v = op(v, dpp_move<kDppRowMirror>(v));
    if (LANES >= 32) v = op(v, __shfl_xor(v, 16, kWave));
    if (LANES >= 64) v = op(v, __shfl_xor(v, 32, kWave));
    return v;
}

__device__ __forceinline__ float wave_sum(float v) { return group_reduce<kWave>(v, SumOp()); }
__device__ __forceinline__ float wave_max(float v) { return group_reduce<kWave>(v, MaxOp()); }

// Wavefront index inside the workgroup as a scalar (SGPR) value, so that
// addresses derived from it use scalar arithmetic and scalar loads.
__device__ __forceinline__ int wave_in_block() {
    return __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
}

__host__ __device__ __forceinline__ bool is_aligned(const void *p, size_t bytes) {
    return (reinterpret_cast<uintptr_t>(p) & (bytes - 1)) == 0;
}

// ---- launching ------------------------------------------------------------
// A caller may ask (cubert_time_next_launch) for the next kernel launched from
// its thread to carry a pair of events that receive the kernel's own start and
// stop timestamps (the dispatch packet's, not those of separate marker packets
// around it), so a single launch inside a forward pass can be timed exactly.

struct LaunchTiming {
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
};
LaunchTiming &pending_launch_timing();  // thread-local; defined in runtime.hip

template <typename... Params, typename... Args>
inline int launch_lds(void (*kernel)(Params...), dim3 grid, dim3 block, unsigned lds_bytes, hipStream_t stream,
                      Args... args) {
    LaunchTiming &t = pending_launch_timing();
    if (t.start != nullptr) {
        hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, t.start, t.stop, 0, static_cast<Params>(args)...);
        t = LaunchTiming();
    } else {
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, static_cast<Params>(args)...);
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int) e;
}

// A launch that never carries timing events (the pending pair, if any, stays pending for the next launch()).
template <typename... Params, typename... Args>
inline int launch_untimed(void (*kernel)(Params...), dim3 grid, dim3 block, unsigned lds_bytes, hipStream_t stream,
                          Args... args) {
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, static_cast<Params>(args)...);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int) e;
}

template <typename... Params, typename... Args>
inline int launch(void (*kernel)(Params...), dim3 grid, dim3 block, hipStream_t stream, Args... args) {
    return launch_lds(kernel, grid, block, 0u, stream, args...);
}

}  // namespace cubert
