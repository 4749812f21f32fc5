// What this chip gives code of this library's kind, measured rather than quoted: the rate at which a plain kernel
// streams memory, and the rate at which a loop of bfloat16 matrix instructions runs with nothing else to do.  The
// benchmark reports its kernels against these beside the published peaks (the reference does the same with a copy
// bandwidth of its own, bench/bench_main.cpp:204-211).
#include "common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// Every thread walks the buffer in strides of the grid, U 16-byte loads in flight; with `dst` it stores what it read, without it
// folds it into one word per thread (so that the loads cannot be dropped).
template <int U>
__global__ __launch_bounds__(256) void stream_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16, uint32_t* __restrict__ sink) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t fold = 0;
    for (; i + (U - 1) * stride < n16; i += U * stride) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (dst) dst[i + u * stride] = v[u];
            else fold ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
        }
    }
    for (; i < n16; i += stride) {
        const uint4 a = src[i];
        if (dst) dst[i] = a; else fold ^= a.x ^ a.y ^ a.z ^ a.w;
    }
    if (!dst) sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = fold;
}

constexpr int MFMA_CHAINS = 8;              // independent sums per wave: the matrix unit never waits for a result

__global__ __launch_bounds__(256) void mfma_loop_kernel(int iters, float* __restrict__ sink) {
    bf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = (__bf16)(float)((threadIdx.x + i) & 3);
        b[i] = (__bf16)(float)((threadIdx.x * 3 + i) & 1);
    }
    floatx16 acc[MFMA_CHAINS];
#pragma unroll
    for (int c = 0; c < MFMA_CHAINS; ++c) acc[c] = floatx16{};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int c = 0; c < MFMA_CHAINS; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
    }
    float total = 0.f;
#pragma unroll
    for (int c = 0; c < MFMA_CHAINS; ++c)
#pragma unroll
        for (int v = 0; v < 16; ++v) total += acc[c][v];
    sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = total;
}

}  // namespace

// Streams `bytes` (a multiple of 16) from `src`, into `dst` if that is given (a copy: `bytes` read and as many written)
// or nowhere (a read), with `in_flight` (4, 8 or 16) loads of 16 bytes a thread.  `sink` takes one word per thread of a read:
// n_blocks * 256 words.
GI_API int gi_probe_stream(const void* src, void* dst, long bytes, void* sink, int n_blocks, int in_flight, hipStream_t stream) {
    GI_REQUIRE(src != nullptr && bytes > 0 && bytes % 16 == 0 && n_blocks > 0, "probe_stream: bad arguments (bytes %ld, blocks %d)", bytes, n_blocks);
    GI_REQUIRE(in_flight == 4 || in_flight == 8 || in_flight == 16, "probe_stream: %d loads in flight (4, 8 or 16)", in_flight);
    GI_REQUIRE(((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0, "probe_stream: buffers must be 16-byte aligned");
    GI_REQUIRE(dst != nullptr || sink != nullptr, "probe_stream: a read needs a sink of n_blocks * 256 words");
    if (in_flight == 4) stream_kernel<4><<<n_blocks, 256, 0, stream>>>((const uint4*)src, (uint4*)dst, (size_t)bytes / 16, (uint32_t*)sink);
    else if (in_flight == 8) stream_kernel<8><<<n_blocks, 256, 0, stream>>>((const uint4*)src, (uint4*)dst, (size_t)bytes / 16, (uint32_t*)sink);
    else stream_kernel<16><<<n_blocks, 256, 0, stream>>>((const uint4*)src, (uint4*)dst, (size_t)bytes / 16, (uint32_t*)sink);
    GI_CHECK_LAUNCH("probe_stream");
    return 0;
}

// n_blocks workgroups of four waves run `iters` rounds of 8 independent v_mfma_f32_32x32x16_bf16 each:
// n_blocks * 4 * iters * 8 * 32768 floating-point operations in all.  `sink`: n_blocks * 256 floats.
GI_API int gi_probe_mfma(int iters, float* sink, int n_blocks, hipStream_t stream) {
    GI_REQUIRE(iters > 0 && n_blocks > 0 && sink != nullptr, "probe_mfma: bad arguments");
    mfma_loop_kernel<<<n_blocks, 256, 0, stream>>>(iters, sink);
    GI_CHECK_LAUNCH("probe_mfma");
    return 0;
}

GI_API long gi_probe_mfma_flops(int iters, int n_blocks) { return (long)n_blocks * 4 * iters * MFMA_CHAINS * 32768L; }
