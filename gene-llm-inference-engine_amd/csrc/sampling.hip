// Sampling on the device from rows of 32-bit logits: greedy (arg max, lowest index among equal
// maxima) and temperature sampling by the inverse distribution function with a given uniform
// number per row.  Rules as the reference's host sampler states them
// (src/sampler/sampler.cpp:54-80, 119-128): p_i = exp((l_i - max) / T) in 32-bit, sums in 64-bit,
// tokens walked in index order, the first with r = u * total < cumulative sum wins, the last
// token if rounding lets none win.
#include "common.h"

namespace {

constexpr int NT = 1024;

__global__ __launch_bounds__(NT) void argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int vocab, long stride) {
    __shared__ float best_v[NT / 64];
    __shared__ int best_i[NT / 64];
    const float* row = logits + (size_t)blockIdx.x * stride;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += NT) {
        const float v = row[i];
        if (v > bv || bi == 0x7fffffff) { bv = v; bi = i; }      // ascending i: strict > keeps the lowest index
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) { best_v[wave] = bv; best_i[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < NT / 64; ++w)
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) { bv = best_v[w]; bi = best_i[w]; }
        out[blockIdx.x] = bi;
    }
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

GI_API int gi_argmax(const float* logits, int* out, int n_rows, int vocab, long stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && vocab > 0 && stride >= vocab, "argmax: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    argmax_kernel<<<n_rows, NT, 0, stream>>>(logits, out, vocab, stride);
    GI_CHECK_LAUNCH("argmax");
    return 0;
}

GI_API int gi_sample_temperature(const float* logits, const float* temperature, const float* uniform, int* out, int n_rows, int vocab,
                                 long stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && vocab > 0 && stride >= vocab, "sample_temperature: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    sample_temperature_kernel<<<n_rows, NT, 0, stream>>>(logits, temperature, uniform, out, vocab, stride);
    GI_CHECK_LAUNCH("sample_temperature");
    return 0;
}
