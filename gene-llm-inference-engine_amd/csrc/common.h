// Shared declarations of the gfx950 kernel library: element types, error reporting, wave helpers.
//
// Every entry point is `extern "C"`, takes raw device pointers and a HIP stream, checks on the host
// that the operand shapes fit what its kernel assumes, launches, and returns 0 or a negative code
// whose text `gi_last_error()` gives.  Nothing here allocates device memory.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define GI_API extern "C" __attribute__((visibility("default")))

enum GiDtype : int { GI_F32 = 0, GI_BF16 = 1 };

typedef uint16_t bf16_t;   // storage of a bfloat16: the high half of a float

// Records the message and returns -1 (defined in elementwise.hip).
int gi_fail(const char* fmt, ...);

// Compute units of the current device (defined in elementwise.hip).
GI_API int gi_compute_units();

#define GI_REQUIRE(cond, ...)                  \
    do {                                       \
        if (!(cond)) return gi_fail(__VA_ARGS__); \
    } while (0)

#define GI_CHECK_LAUNCH(name)                                                        \
    do {                                                                             \
        hipError_t e_ = hipGetLastError();                                           \
        if (e_ != hipSuccess) return gi_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); \
    } while (0)

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// Round to nearest, ties to even; NaN stays NaN.  gfx950 converts in hardware (v_cvt_pk_bf16_f32).
typedef __bf16 gi_bf16x2 __attribute__((ext_vector_type(2)));
typedef float gi_floatx2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
    const gi_floatx2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, gi_bf16x2));
}
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return (bf16_t)(f32x2_to_bf16x2(f, 0.f) & 0xffffu); }

__device__ __forceinline__ float load_f32(const float* p, size_t i) { return p[i]; }
__device__ __forceinline__ float load_f32(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }
__device__ __forceinline__ void store_f32(float* p, size_t i, float v) { p[i] = v; }
__device__ __forceinline__ void store_f32(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

// A workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() also waits for every load
// from global memory the wave has in flight, which undoes a prefetch into registers; use this one where the
// barrier orders LDS reads and writes and nothing else.
__device__ __forceinline__ void barrier_lds() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Butterfly reductions over the 64 lanes of a wave: every lane ends with the same value, and the
// order of the additions is fixed by the lane numbers alone.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Sum over a workgroup of `NT` threads (a multiple of 64, at most 1024); `red` holds NT/64 floats of LDS.
// All threads get the result; the order of additions depends on NT only.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < NT / 64; ++w) t += red[w];
    return t;
}
