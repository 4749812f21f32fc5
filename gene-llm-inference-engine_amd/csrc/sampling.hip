// Sampling on the device from rows of 32-bit logits: greedy (arg max, lowest index among equal
// maxima) and temperature sampling by the inverse distribution function with a given uniform
// number per row.  Rules as the reference's host sampler states them
// (src/sampler/sampler.cpp:54-80, 119-128): p_i = exp((l_i - max) / T) in 32-bit, sums in 64-bit,
// tokens walked in index order, the first with r = u * total < cumulative sum wins, the last
// token if rounding lets none win.  (The 64-bit sums are taken in a tree, not one by one: the draw
// can differ from the reference's only where r falls within rounding of a boundary.)
#include "common.h"
#include "geneinfer_no_alloc.h"

#include <mutex>

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

// Temperature sampling in three stages, so that a few rows still fill the chip: the maxima of runs of
// CHUNK logits (one workgroup each); with the row's maximum known, the runs' sums of p = exp((l - max) / T)
// in 64-bit; then one workgroup per row finds the run that holds r = u * total (runs in index order),
// gives each of its threads 16 consecutive tokens of that run, finds the thread by a prefix sum, and that
// thread walks its tokens one by one.  Cumulative sums follow index order up to the rounding of 64-bit sums.
__global__ __launch_bounds__(256) void chunk_max_kernel(const float* __restrict__ logits, float* __restrict__ part_m, int vocab, long stride,
                                                        int n_chunks) {
    __shared__ float red[4];
    const float* row = logits + (size_t)blockIdx.y * stride;
    const int begin = blockIdx.x * CHUNK, end = min(vocab, begin + CHUNK);
    float mx = -INFINITY;
    for (int i = begin + threadIdx.x; i < end; i += 256) mx = fmaxf(mx, row[i]);
    mx = wave_max(mx);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
    __syncthreads();
    if (threadIdx.x == 0) part_m[(size_t)blockIdx.y * n_chunks + blockIdx.x] = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
}

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float row_max(const float* __restrict__ part_m, int n_chunks) {       // the same value in every thread
    float mx = -INFINITY;
    for (int c = 0; c < n_chunks; ++c) mx = fmaxf(mx, part_m[c]);
    return mx;
}

__global__ __launch_bounds__(256) void chunk_sum_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                        const float* __restrict__ part_m, double* __restrict__ part_s, int vocab,
                                                        long stride, int n_chunks) {
    __shared__ double red[4];
    const float* row = logits + (size_t)blockIdx.y * stride;
    const float temp = temperature[blockIdx.y], mx = row_max(part_m + (size_t)blockIdx.y * n_chunks, n_chunks);
    const int begin = blockIdx.x * CHUNK, end = min(vocab, begin + CHUNK);
    double sum = 0.0;
    for (int i = begin + threadIdx.x; i < end; i += 256) sum += (double)expf((row[i] - mx) / temp);
    sum = wave_sum_f64(sum);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) part_s[(size_t)blockIdx.y * n_chunks + blockIdx.x] = ((red[0] + red[1]) + red[2]) + red[3];
}

constexpr int RUN = CHUNK / 256;            // tokens a thread of the last stage owns

__global__ __launch_bounds__(256) void sample_pick_kernel(const float* __restrict__ logits, const float* __restrict__ temperature,
                                                          const float* __restrict__ uniform, const float* __restrict__ part_m,
                                                          const double* __restrict__ part_s, int* __restrict__ out, int vocab, long stride,
                                                          int n_chunks) {
    __shared__ double wave_total[4];
    __shared__ int winner;
    const float* row = logits + (size_t)blockIdx.x * stride;
    const float temp = temperature[blockIdx.x], mx = row_max(part_m + (size_t)blockIdx.x * n_chunks, n_chunks);
    const double* sums = part_s + (size_t)blockIdx.x * n_chunks;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // The reference normalises p by a 32-bit 1/sum before it draws; the draw compares u * sum(p) with
    // cumulative p, which is the same comparison scaled by a constant, so it is made on the
    // unnormalised values here.
    double total = 0.0;
    for (int c = 0; c < n_chunks; ++c) total += sums[c];
    const double r = (double)uniform[blockIdx.x] * total;
    int chunk = n_chunks - 1;                // the run that holds r (the last one if rounding lets none hold it)
    double before = 0.0;
    for (int c = 0; c < n_chunks - 1; ++c) {
        if (r < before + sums[c]) { chunk = c; break; }
        before += sums[c];
    }
    const int begin = chunk * CHUNK, end = min(vocab, begin + CHUNK);
    const int lo = min(end, begin + tid * RUN), hi = min(end, lo + RUN);
    double mine = 0.0;
    for (int i = lo; i < hi; ++i) mine += (double)expf((row[i] - mx) / temp);
    double c = mine;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {                  // inclusive prefix sum over the lanes of a wave
        const double below = __shfl_up(c, off, 64);
        if (lane >= off) c += below;
    }
    if (lane == 63) wave_total[wave] = c;
    if (tid == 0) winner = min(end, vocab - 1);              // if rounding leaves r beyond the run: the next token in index order
    __syncthreads();
    for (int w = 0; w < wave; ++w) before += wave_total[w];
    const double run_stop = before + c, run_start = run_stop - mine;
    if (lo < hi && r >= run_start && r < run_stop) {          // at most one thread
        double walk = run_start;
        int pick = min(hi, vocab - 1);
        for (int i = lo; i < hi; ++i) {
            walk += (double)expf((row[i] - mx) / temp);
            if (r < walk) { pick = i; break; }
        }
        winner = pick;
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

// part_m: n_rows * gi_argmax_chunks(vocab) floats, part_s: as many doubles.
GI_API int gi_sample_temperature(const float* logits, const float* temperature, const float* uniform, int* out, float* part_m, double* part_s,
                                 int n_rows, int vocab, long stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_rows <= 65535 && vocab > 0 && stride >= vocab, "sample_temperature: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    GI_REQUIRE(part_m != nullptr && part_s != nullptr, "sample_temperature: scratch is missing");
    const int n_chunks = gi_argmax_chunks(vocab);
    chunk_max_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, part_m, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("sample_temperature (maxima)");
    chunk_sum_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, temperature, part_m, part_s, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("sample_temperature (sums)");
    sample_pick_kernel<<<n_rows, 256, 0, stream>>>(logits, temperature, uniform, part_m, part_s, out, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("sample_temperature (pick)");
    return 0;
}

// ------------------------------------------------------------------ arg max without a scratch argument
// The partial results of gi_argmax's first stage live in a static array in device memory instead of memory the caller
// brings.  In host code the array's name is only a handle for hipGetSymbolAddress: every GPU holds its own copy at its
// own address, which is asked for once per device and kept; kernels, and anything else on the host that needs the
// memory, get that address.
static __device__ __align__(256) unsigned char scratch[GI_NO_ALLOC_ARGMAX_MAX_PARTS * (sizeof(float) + sizeof(int))];

namespace {
constexpr int MAX_DEVICES = 64;
void* g_scratch_of_device[MAX_DEVICES] = {};
std::mutex g_scratch_mutex;

// This GPU's copy of `scratch` (the current device's), or nullptr with the error recorded.
void* scratch_of_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
        gi_fail("no_alloc: no current HIP device (or more than %d devices)", MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_of_device[dev] == nullptr) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            gi_fail("no_alloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_of_device[dev] = ptr;
    }
    return g_scratch_of_device[dev];
}
}  // namespace

GI_API int gi_no_alloc_prepare(void) { return scratch_of_current_device() != nullptr ? 0 : -1; }

GI_API int gi_argmax_no_alloc(const float* logits, int* out, int n_rows, int vocab, long stride, hipStream_t stream) {
    GI_REQUIRE(logits != nullptr && out != nullptr, "argmax_no_alloc: logits and out must be given");
    GI_REQUIRE(n_rows > 0 && n_rows <= 65535 && vocab > 0 && stride >= vocab, "argmax_no_alloc: bad sizes (rows %d, vocab %d, stride %ld)", n_rows, vocab, stride);
    const int n_chunks = gi_argmax_chunks(vocab);
    GI_REQUIRE((long)n_rows * n_chunks <= GI_NO_ALLOC_ARGMAX_MAX_PARTS,
               "argmax_no_alloc: %d rows x %d runs of %d logits need %ld partial results, the static scratch holds %d; use gi_argmax with scratch of your own",
               n_rows, n_chunks, CHUNK, (long)n_rows * n_chunks, GI_NO_ALLOC_ARGMAX_MAX_PARTS);
    unsigned char* ptr = (unsigned char*)scratch_of_current_device();
    if (ptr == nullptr) return -1;
    float* part_v = (float*)ptr;
    int* part_i = (int*)(ptr + (size_t)GI_NO_ALLOC_ARGMAX_MAX_PARTS * sizeof(float));
    argmax_chunks_kernel<<<dim3(n_chunks, n_rows), 256, 0, stream>>>(logits, part_v, part_i, vocab, stride, n_chunks);
    GI_CHECK_LAUNCH("argmax_no_alloc (chunks)");
    argmax_final_kernel<<<n_rows, 64, 0, stream>>>(part_v, part_i, out, n_chunks);
    GI_CHECK_LAUNCH("argmax_no_alloc (final)");
    return 0;
}
