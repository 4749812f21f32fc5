// Sampling on the device from rows of 32-bit logits: greedy (arg max, lowest index among equal
// maxima) and temperature sampling by the inverse distribution function with a given uniform
// number per row.  Rules as the reference's host sampler states them
// (src/sampler/sampler.cpp:54-80, 119-128): p_i = exp((l_i - max) / T) in 32-bit, sums in 64-bit,
// tokens walked in index order, the first with r = u * total < cumulative sum wins, the last
// token if rounding lets none win.
#include "common.h"

namespace {

constexpr int NT = 1024;

// Arg max in two stages so that a few rows still fill the chip: stage one takes runs of CHUNK
// logits (one workgroup each), stage two the winners of a row.  Among equal values the lowest index
// wins at every comparison, so the result is the lowest index of the maximum.
constexpr int CHUNK = 4096;

__device__ __forceinline__ void better(float& bv, int& bi, float ov, int oi) {
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
}

__global__ __launch_bounds__(256) void argmax_chunks_kernel(const float* __restrict__ logits, float* __restrict__ part_v, int* __restrict__ part_i,
                                                            int vocab, long stride, int n_chunks) {
    __shared__ float sv[4];
    __shared__ int si[4];
    const float* row = logits + (size_t)blockIdx.y * stride;
    const int begin = blockIdx.x * CHUNK, end = min(vocab, begin + CHUNK);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = begin + threadIdx.x; i < end; i += 256) {
        const float v = row[i];
        if (v > bv || bi == 0x7fffffff) { bv = v; bi = i; }      // ascending i: strict > keeps the lowest index
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) better(bv, bi, __shfl_xor(bv, off, 64), __shfl_xor(bi, off, 64));
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w) better(bv, bi, sv[w], si[w]);
        part_v[(size_t)blockIdx.y * n_chunks + blockIdx.x] = bv;
        part_i[(size_t)blockIdx.y * n_chunks + blockIdx.x] = bi;
    }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ part_v, const int* __restrict__ part_i, int* __restrict__ out,
                                                          int n_chunks) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int c = threadIdx.x; c < n_chunks; c += 64) better(bv, bi, part_v[(size_t)blockIdx.x * n_chunks + c], part_i[(size_t)blockIdx.x * n_chunks + c]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) better(bv, bi, __shfl_xor(bv, off, 64), __shfl_xor(bi, off, 64));
    if (threadIdx.x == 0) out[blockIdx.x] = bi;
}

// Each thread owns a contiguous run of tokens, so that cumulative sums follow index order.
__global__ __launch_bounds__(NT) void sample_temperature_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                                const float* __restrict__ uniform, int* __restrict__ out, int vocab,
                                                                long stride) {
    __shared__ float red_f[NT / 64];
    __shared__ double run_start[NT];
    __shared__ double total_s;
    __shared__ int winner;
    const float* row = logits + (size_t)blockIdx.x * stride;
    const float temp = temperature[blockIdx.x];
    const int tid = threadIdx.x;

    float mx = -INFINITY;
    for (int i = tid; i < vocab; i += NT) mx = fmaxf(mx, row[i]);
    mx = wave_max(mx);
    if ((tid & 63) == 0) red_f[tid >> 6] = mx;
    __syncthreads();
    mx = red_f[0];
    for (int w = 1; w < NT / 64; ++w) mx = fmaxf(mx, red_f[w]);

    const int per = (vocab + NT - 1) / NT;
    const int begin = min(vocab, tid * per), end = min(vocab, begin + per);
    double mine = 0.0;
    for (int i = begin; i < end; ++i) mine += (double)expf((row[i] - mx) / temp);
    run_start[tid] = mine;
    if (tid == 0) winner = vocab - 1;       // if rounding lets no token win, the last one does
    __syncthreads();
    if (tid == 0) {                         // prefix sums of the 1024 run totals, in index order
        double c = 0.0;
        for (int i = 0; i < NT; ++i) {
            const double s = run_start[i];
            run_start[i] = c;
            c += s;
        }
        total_s = c;
    }
    __syncthreads();
    // The reference normalises p by a 32-bit 1/sum before it draws; the draw compares u * sum(p) with
    // cumulative p, which is the same comparison scaled by a constant, so it is made on the
    // unnormalised values here.
    const double r = (double)uniform[blockIdx.x] * total_s;
    const double start = run_start[tid];
    const double stop = (tid == NT - 1) ? total_s : run_start[tid + 1];
    if (begin < end && r >= start && r < stop) {
        double c = start;
        int pick = -1;
        for (int i = begin; i < end; ++i) {
            c += (double)expf((row[i] - mx) / temp);
            if (r < c) { pick = i; break; }
        }
        // Rounding may leave r just beyond this run's last partial sum: the next token in index order wins.
        winner = pick >= 0 ? pick : min(end, vocab - 1);
    }
    __syncthreads();
    if (tid == 0) out[blockIdx.x] = winner;
}

}  // namespace

// Chunks per row, so that the caller can size the scratch: n_rows * chunks floats and as many ints.
GI_API int gi_argmax_chunks(int vocab) { return (vocab + CHUNK - 1) / CHUNK; }

GI_API int gi_argmax(const float* logits, int* out, float* part_v, int* part_i, int n_rows, int vocab, long stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_rows <= 65535 && vocab > 0 && stride >= vocab, "argmax: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    GI_REQUIRE(part_v != nullptr && part_i != nullptr, "argmax: scratch is missing");
    const int n_chunks = gi_argmax_chunks(vocab);
    argmax_chunks_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, part_v, part_i, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("argmax (chunks)");
    argmax_final_kernel<<<n_rows, 64, 0, stream>>>(part_v, part_i, out, n_chunks);
    GI_CHECK_LAUNCH("argmax (final)");
    return 0;
}

GI_API int gi_sample_temperature(const float* logits, const float* temperature, const float* uniform, int* out, int n_rows, int vocab,
                                 long stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && vocab > 0 && stride >= vocab, "sample_temperature: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    sample_temperature_kernel<<<n_rows, NT, 0, stream>>>(logits, temperature, uniform, out, vocab, stride);
    GI_CHECK_LAUNCH("sample_temperature");
    return 0;
}
