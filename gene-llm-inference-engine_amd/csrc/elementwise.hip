// Row-wise kernels around the matrix products: token embedding, RMS norm, rotary angles,
// rotation + cache write, SiLU gating, row gather.  All arithmetic is 32-bit (angles 64-bit);
// only what is loaded or stored may be bfloat16.
#include "common.h"

#include <stdarg.h>
#include <stdio.h>

static thread_local char g_error[512] = "";

int gi_fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return -1;
}

GI_API const char* gi_last_error() { return g_error; }

// Compute units of the current device, asked for once per device; where no device answers, those of an MI355X.  Dispatch
// rules that speak of "one round of workgroups" or "three quarters of the chip" are stated in terms of this number.
GI_API int gi_compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return 256;
    }
    int n = __atomic_load_n(&cached[dev], __ATOMIC_RELAXED);
    if (n > 0) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        n = 256;
    }
    __atomic_store_n(&cached[dev], n, __ATOMIC_RELAXED);
    return n;
}

GI_API int gi_device_arch(char* out, int cap) {
    hipDeviceProp_t p;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&p, dev) != hipSuccess) return gi_fail("no HIP device");
    snprintf(out, cap, "%s", p.gcnArchName);
    return 0;
}

// ------------------------------------------------------------------------------------- embedding
// x[t, :] = table[tokens[t], :], widened to 32-bit.  Reference: src/gpu/device_kernels.inc:37-51.
template <typename TT>
__global__ void embed_kernel(const TT* __restrict__ table, const int* __restrict__ tokens, float* __restrict__ x, int dim) {
    const int t = blockIdx.x;
    const TT* row = table + (size_t)tokens[t] * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) x[(size_t)t * dim + d] = load_f32(row, d);
}

GI_API int gi_embed(const void* table, int table_dtype, const int* tokens, float* x, int n_rows, int dim, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0, "embed: n_rows %d and dim %d must be positive", n_rows, dim);
    if (table_dtype == GI_F32)
        embed_kernel<float><<<n_rows, 256, 0, stream>>>((const float*)table, tokens, x, dim);
    else if (table_dtype == GI_BF16)
        embed_kernel<bf16_t><<<n_rows, 256, 0, stream>>>((const bf16_t*)table, tokens, x, dim);
    else
        return gi_fail("embed: unknown table dtype %d", table_dtype);
    GI_CHECK_LAUNCH("embed");
    return 0;
}

// The same for a step of a few rows whose first norm the product behind it finishes (see the products' `NormIn`): beside x the
// row goes out times the norm's weights in bfloat16, and its sum of squares as one number.
template <typename TT>
__global__ __launch_bounds__(256) void embed_handing_kernel(const TT* __restrict__ table, const int* __restrict__ tokens, float* __restrict__ x, int dim,
                                                            const float* __restrict__ g, bf16_t* __restrict__ scaled, float* __restrict__ squares) {
    __shared__ float red[4];
    const int t = blockIdx.x;
    const TT* row = table + (size_t)tokens[t] * dim;
    float sum = 0.f;
    if (dim % 4 == 0 && (((uintptr_t)table | (uintptr_t)x | (uintptr_t)g | (uintptr_t)scaled) & 15) == 0) {      // four neighbouring channels a thread
        for (int d = threadIdx.x * 4; d < dim; d += 1024) {
            float v[4];
            if constexpr (sizeof(TT) == 2) {
                const uint2 raw = *reinterpret_cast<const uint2*>(row + d);
                v[0] = __uint_as_float(raw.x << 16); v[1] = __uint_as_float(raw.x & 0xffff0000u);
                v[2] = __uint_as_float(raw.y << 16); v[3] = __uint_as_float(raw.y & 0xffff0000u);
            } else {
                const float4 raw = *reinterpret_cast<const float4*>(row + d);
                v[0] = raw.x; v[1] = raw.y; v[2] = raw.z; v[3] = raw.w;
            }
            const float4 gd = *reinterpret_cast<const float4*>(g + d);
            *reinterpret_cast<float4*>(x + (size_t)t * dim + d) = float4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<uint2*>(scaled + (size_t)t * dim + d) = uint2{f32x2_to_bf16x2(gd.x * v[0], gd.y * v[1]), f32x2_to_bf16x2(gd.z * v[2], gd.w * v[3])};
            sum += (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
        }
    } else {
        for (int d = threadIdx.x; d < dim; d += 256) {
            const float v = load_f32(row, d);
            x[(size_t)t * dim + d] = v;
            scaled[(size_t)t * dim + d] = f32_to_bf16(g[d] * v);
            sum = fmaf(v, v, sum);
        }
    }
    sum = block_sum<256>(sum, red);
    if (threadIdx.x == 0) squares[t] = sum;
}

GI_API int gi_embed_handing(const void* table, int table_dtype, const int* tokens, float* x, int n_rows, int dim, const float* g, void* scaled,
                            float* squares, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && g != nullptr && scaled != nullptr && squares != nullptr, "embed: n_rows %d and dim %d must be positive, and the norm's operands given", n_rows, dim);
    if (table_dtype == GI_F32)
        embed_handing_kernel<float><<<n_rows, 256, 0, stream>>>((const float*)table, tokens, x, dim, g, (bf16_t*)scaled, squares);
    else if (table_dtype == GI_BF16)
        embed_handing_kernel<bf16_t><<<n_rows, 256, 0, stream>>>((const bf16_t*)table, tokens, x, dim, g, (bf16_t*)scaled, squares);
    else
        return gi_fail("embed: unknown table dtype %d", table_dtype);
    GI_CHECK_LAUNCH("embed");
    return 0;
}

// -------------------------------------------------------------------------------------- RMS norm
// out = w * (x * rsqrt(mean(x^2) + eps)), one workgroup per row; the sum of squares is taken in
// 32-bit in an order that depends on the row's length only.  Reference: src/kernels/kernels.cpp:72-83.
template <typename TW, typename TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const TW* __restrict__ w, TO* __restrict__ out, int dim, float eps,
                               size_t x_stride, size_t out_stride) {
    __shared__ float red[4];
    const float* xr = x + (size_t)blockIdx.x * x_stride;
    TO* orow = out + (size_t)blockIdx.x * out_stride;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) ss = fmaf(xr[d], xr[d], ss);
    ss = block_sum<256>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += 256) store_f32(orow, d, load_f32(w, d) * (scale * xr[d]));
}

// The same for rows whose length is a multiple of 4 and at most 4096, 16-byte aligned: every thread
// loads its (at most four) groups of four values at once and keeps them for the second pass, so the
// kernel waits for memory once.  `rows` (optional) gathers the input rows.
__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) { *reinterpret_cast<float4*>(p) = float4{a, b, c, d}; }
__device__ __forceinline__ void store4(bf16_t* p, float a, float b, float c, float d) {
    *reinterpret_cast<uint2*>(p) = uint2{(uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16), (uint32_t)f32_to_bf16(c) | ((uint32_t)f32_to_bf16(d) << 16)};
}
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    return float4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u)};
}

template <typename TW, typename TO>
__global__ __launch_bounds__(256) void rmsnorm_fast_kernel(const float* __restrict__ x, const int* __restrict__ rows, const TW* __restrict__ w,
                                                          TO* __restrict__ out, int dim, float eps, size_t x_stride, size_t out_stride) {
    __shared__ float red[4];
    const float* xr = x + (size_t)(rows ? rows[blockIdx.x] : blockIdx.x) * x_stride;
    TO* orow = out + (size_t)blockIdx.x * out_stride;
    const int n4 = dim / 4;
    float4 v[4], wv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = threadIdx.x + 256 * i;
        v[i] = c < n4 ? load4(xr + 4 * c) : float4{0.f, 0.f, 0.f, 0.f};
        wv[i] = c < n4 ? load4(w + 4 * c) : float4{0.f, 0.f, 0.f, 0.f};
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        ss = fmaf(v[i].x, v[i].x, ss); ss = fmaf(v[i].y, v[i].y, ss); ss = fmaf(v[i].z, v[i].z, ss); ss = fmaf(v[i].w, v[i].w, ss);
    }
    ss = block_sum<256>(ss, red);
    const float scale = 1.0f / sqrtf(ss / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = threadIdx.x + 256 * i;
        if (c < n4) store4(orow + 4 * c, wv[i].x * (scale * v[i].x), wv[i].y * (scale * v[i].y), wv[i].z * (scale * v[i].z), wv[i].w * (scale * v[i].w));
    }
}

// rows != nullptr: out[i] = norm(x[rows[i]]) (needs the fast kernel's conditions: dim a multiple of 4, at most 4096, aligned rows).
GI_API int gi_rmsnorm(const float* x, const int* rows, const void* w, int w_dtype, void* out, int out_dtype, int n_rows, int dim, float eps,
                      long x_stride, long out_stride, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0, "rmsnorm: n_rows %d and dim %d must be positive", n_rows, dim);
    GI_REQUIRE(x_stride >= dim && out_stride >= dim, "rmsnorm: row strides must be at least dim");
    const bool fast = dim % 4 == 0 && dim <= 4096 && x_stride % 4 == 0 && out_stride % 4 == 0 && ((uintptr_t)x & 15) == 0 &&
                      ((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 15) == 0;
    GI_REQUIRE(rows == nullptr || fast, "rmsnorm: gathering rows needs a row length that is a multiple of 4 and at most 4096, and aligned operands");
#define LAUNCH(TW, TO)                                                                                                                   \
    do {                                                                                                                                 \
        if (fast) rmsnorm_fast_kernel<TW, TO><<<n_rows, 256, 0, stream>>>(x, rows, (const TW*)w, (TO*)out, dim, eps, (size_t)x_stride, (size_t)out_stride); \
        else rmsnorm_kernel<TW, TO><<<n_rows, 256, 0, stream>>>(x, (const TW*)w, (TO*)out, dim, eps, (size_t)x_stride, (size_t)out_stride);              \
    } while (0)
    if (w_dtype == GI_F32 && out_dtype == GI_F32) LAUNCH(float, float);
    else if (w_dtype == GI_F32 && out_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else if (w_dtype == GI_BF16 && out_dtype == GI_F32) LAUNCH(bf16_t, float);
    else if (w_dtype == GI_BF16 && out_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else return gi_fail("rmsnorm: unknown dtypes %d, %d", w_dtype, out_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("rmsnorm");
    return 0;
}

// -------------------------------------------------------------------------------- rotary angles
// cos and sin of pos * f_k for every row, the angle taken in 64-bit: a 32-bit angle loses digits
// at large positions (reference: src/kernels/kernels.cpp:145-161).
__global__ void rope_cos_sin_kernel(const int* __restrict__ pos, const double* __restrict__ inv_freq, float* __restrict__ cos_out,
                                    float* __restrict__ sin_out, int n_rows, int half) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_rows * half) return;
    const double a = (double)pos[i / half] * inv_freq[i % half];
    cos_out[i] = (float)cos(a);
    sin_out[i] = (float)sin(a);
}

GI_API int gi_rope_cos_sin(const int* pos, const double* inv_freq, float* cos_out, float* sin_out, int n_rows, int half,
                           hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && half > 0, "rope_cos_sin: n_rows %d and half %d must be positive", n_rows, half);
    const int n = n_rows * half;
    rope_cos_sin_kernel<<<(n + 255) / 256, 256, 0, stream>>>(pos, inv_freq, cos_out, sin_out, n_rows, half);
    GI_CHECK_LAUNCH("rope_cos_sin");
    return 0;
}

// ---------------------------------------------------------------- rotation and cache write, fused
// For row t at position pos[t] of the request in slot[t]:
//   q heads are rotated and written to q_out [n_rows, n_heads*hd];
//   k heads are rotated and, with the v heads as they are, written into the page
//   table[slot[t]][pos / page_size] at place pos % page_size.
// Pairs are (k, k + hd/2): a' = a*cos - b*sin, b' = a*sin + b*cos (src/kernels/kernels.cpp:165-180).
// Cache of one layer: per page the keys [kv_head][place][hd], then the values transposed
// [kv_head][hd][place] (so that consecutive positions of one value channel are contiguous, which is
// what the matrix instructions of the attention kernels load).  cos == nullptr means no rotation.
// k == nullptr means the layer reads another layer's cache and writes none.
template <typename TQ, typename TC>
__global__ void rope_store_kernel(const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v, long ldq, long ldk,
                                  long ldv, const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int* __restrict__ pos,
                                  const int* __restrict__ slot, const int* __restrict__ table, int table_stride, TQ* __restrict__ q_out,
                                  TC* __restrict__ cache, long page_stride, int page_size, int n_heads, int n_kv, int hd) {
    // One thread per pair: items 0 .. n_heads*half-1 are query pairs, the rest key pairs (which also carry the two values).
    const int t = blockIdx.x, half = hd / 2;
    const int i = blockIdx.y * blockDim.x + threadIdx.x;
    const int n_q_items = n_heads * half, n_k_items = k ? n_kv * half : 0;
    if (i >= n_q_items + n_k_items) return;
    const bool is_q = i < n_q_items;
    const int j = is_q ? i : i - n_q_items, h = j / half, kk = j % half;
    const float cc = cos_t ? cos_t[(size_t)t * half + kk] : 1.f, ss = sin_t ? sin_t[(size_t)t * half + kk] : 0.f;
    if (is_q) {
        const float a = q[(size_t)t * ldq + h * hd + kk], b = q[(size_t)t * ldq + h * hd + kk + half];
        store_f32(q_out, (size_t)t * n_heads * hd + h * hd + kk, a * cc - b * ss);
        store_f32(q_out, (size_t)t * n_heads * hd + h * hd + kk + half, a * ss + b * cc);
        return;
    }
    const float a = k[(size_t)t * ldk + h * hd + kk], b = k[(size_t)t * ldk + h * hd + kk + half];
    const float va = v[(size_t)t * ldv + h * hd + kk], vb = v[(size_t)t * ldv + h * hd + kk + half];
    const int p = pos[t];
    const long page = table[(size_t)slot[t] * table_stride + p / page_size];
    const int place = p % page_size;
    TC* kbase = cache + page * page_stride;
    TC* vbase = kbase + (size_t)n_kv * page_size * hd;
    const size_t o = ((size_t)h * page_size + place) * hd;
    store_f32(kbase, o + kk, a * cc - b * ss);
    store_f32(kbase, o + kk + half, a * ss + b * cc);
    store_f32(vbase, ((size_t)h * hd + kk) * page_size + place, va);
    store_f32(vbase, ((size_t)h * hd + kk + half) * page_size + place, vb);
}

GI_API int gi_rope_store(const float* q, const float* k, const float* v, long ldq, long ldk, long ldv, const float* cos_t,
                         const float* sin_t, const int* pos, const int* slot, const int* table, int table_stride, void* q_out,
                         int q_dtype, void* cache, int cache_dtype, long page_stride, int page_size, int n_rows, int n_heads,
                         int n_kv, int hd, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_kv > 0 && hd > 0 && hd % 2 == 0, "rope_store: bad sizes (rows %d heads %d kv %d hd %d)",
               n_rows, n_heads, n_kv, hd);
    GI_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "rope_store: cos and sin must both be given or both be absent");
    GI_REQUIRE(k == nullptr || (v != nullptr && cache != nullptr && table != nullptr && page_size > 0 &&
                                page_stride >= 2L * n_kv * page_size * hd),
               "rope_store: cache write needs v, a cache, a table and a page stride of at least 2*n_kv*page_size*hd");
    const int items = (n_heads + (k ? n_kv : 0)) * (hd / 2);
    dim3 grid(n_rows, (items + 255) / 256);
    GI_REQUIRE(grid.y <= 65535, "rope_store: too many heads");
#define LAUNCH(TQ, TC)                                                                                                       \
    rope_store_kernel<TQ, TC><<<grid, 256, 0, stream>>>(q, k, v, ldq, ldk, ldv, cos_t, sin_t, pos, slot, table, table_stride, \
                                                          (TQ*)q_out, (TC*)cache, page_stride, page_size, n_heads, n_kv, hd)
    if (q_dtype == GI_F32 && cache_dtype == GI_F32) LAUNCH(float, float);
    else if (q_dtype == GI_BF16 && cache_dtype == GI_BF16) LAUNCH(bf16_t, bf16_t);
    else if (q_dtype == GI_F32 && cache_dtype == GI_BF16) LAUNCH(float, bf16_t);
    else if (q_dtype == GI_BF16 && cache_dtype == GI_F32) LAUNCH(bf16_t, float);
    else return gi_fail("rope_store: unknown dtypes %d, %d", q_dtype, cache_dtype);
#undef LAUNCH
    GI_CHECK_LAUNCH("rope_store");
    return 0;
}

// ------------------------------------------------------------------------------------ SiLU gate
// h[t, i] = silu(gu[t, i]) * gu[t, inter + i], silu(g) = g * (1 / (1 + exp(-g)))
// (src/gpu/device_kernels.inc:460-469).  gu is the product with the stacked [gate; up] matrix.
template <typename TO>
__global__ void silu_mul_kernel(const float* __restrict__ gu, TO* __restrict__ h, int inter, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / inter, c = i % inter;
    const float g = gu[t * 2 * inter + c], u = gu[t * 2 * inter + inter + c];
    store_f32(h, i, (g * (1.0f / (1.0f + expf(-g)))) * u);
}

GI_API int gi_silu_mul(const float* gate_up, void* h, int h_dtype, int n_rows, int inter, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && inter > 0, "silu_mul: n_rows %d and inter %d must be positive", n_rows, inter);
    const size_t n = (size_t)n_rows * inter;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (h_dtype == GI_F32) silu_mul_kernel<float><<<blocks, 256, 0, stream>>>(gate_up, (float*)h, inter, n);
    else if (h_dtype == GI_BF16) silu_mul_kernel<bf16_t><<<blocks, 256, 0, stream>>>(gate_up, (bf16_t*)h, inter, n);
    else return gi_fail("silu_mul: unknown dtype %d", h_dtype);
    GI_CHECK_LAUNCH("silu_mul");
    return 0;
}

// ----------------------------------------------------------------------------------- row gather
// out[i, :] = x[rows[i], :] (the rows whose logits are wanted; src/gpu/gpu_transformer.cpp:441).
__global__ void gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ rows, float* __restrict__ out, int dim) {
    const float* src = x + (size_t)rows[blockIdx.x] * dim;
    for (int d = threadIdx.x; d < dim; d += blockDim.x) out[(size_t)blockIdx.x * dim + d] = src[d];
}

GI_API int gi_gather_rows(const float* x, const int* rows, float* out, int n_out, int dim, hipStream_t stream) {
    GI_REQUIRE(n_out > 0 && dim > 0, "gather_rows: n_out %d and dim %d must be positive", n_out, dim);
    gather_rows_kernel<<<n_out, 256, 0, stream>>>(x, rows, out, dim);
    GI_CHECK_LAUNCH("gather_rows");
    return 0;
}

// ------------------------------------------------------------------------------- row transforms
// In place over float32 rows [n_rows, dim] with row stride `stride`: x <- x * factor, or x <- cap * tanh(x / cap).
template <bool CAP>
__global__ void rows_in_place_kernel(float* __restrict__ x, int dim, long stride, float c) {
    float* row = x + (size_t)blockIdx.x * stride;
    for (int d = blockIdx.y * blockDim.x + threadIdx.x; d < dim; d += gridDim.y * blockDim.x) row[d] = CAP ? c * tanhf(row[d] / c) : row[d] * c;
}

GI_API int gi_scale_rows(float* x, int n_rows, int dim, long stride, float factor, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && stride >= dim, "scale_rows: bad sizes (rows %d, dim %d, stride %ld)", n_rows, dim, stride);
    rows_in_place_kernel<false><<<dim3(n_rows, min(64, (dim + 1023) / 1024)), 256, 0, stream>>>(x, dim, stride, factor);
    GI_CHECK_LAUNCH("scale_rows");
    return 0;
}

GI_API int gi_softcap_rows(float* x, int n_rows, int dim, long stride, float cap, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && dim > 0 && stride >= dim, "softcap_rows: bad sizes (rows %d, dim %d, stride %ld)", n_rows, dim, stride);
    GI_REQUIRE(cap > 0.f, "softcap_rows: the cap %g must be positive", (double)cap);
    rows_in_place_kernel<true><<<dim3(n_rows, min(64, (dim + 1023) / 1024)), 256, 0, stream>>>(x, dim, stride, cap);
    GI_CHECK_LAUNCH("softcap_rows");
    return 0;
}

// ------------------------------------------------------------------------------- random weights
// out[i] = offset + scale * z_i with z_i a standard normal number that is a function of (key, i) alone, so that a model's random
// weights can be re-made anywhere from the seed and the tensors' names (the key is made of both on the host):
//   r  = mix(key + (i + 1) * 0x9E3779B97F4A7C15)      mix: the splitmix64 finaliser
//   u1 = ((r >> 40) + 1) / 2^24  in (0, 1],  u2 = ((r >> 8) & 0xFFFFFF) / 2^24  in [0, 1)
//   z  = sqrt(-2 ln u1) * cos(2 pi u2)                 in 64-bit; offset + scale * z is rounded to 32-bit, then to the storage type
__device__ __forceinline__ uint64_t splitmix_finish(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

template <typename T>
__global__ __launch_bounds__(256) void random_normal_kernel(T* __restrict__ out, size_t n, uint64_t key, double offset, double scale) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const uint64_t r = splitmix_finish(key + (uint64_t)(i + 1) * 0x9E3779B97F4A7C15ull);
        const double u1 = (double)((r >> 40) + 1) * (1.0 / 16777216.0), u2 = (double)((r >> 8) & 0xFFFFFFull) * (1.0 / 16777216.0);
        const double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
        store_f32(out, i, (float)(offset + scale * z));
    }
}

GI_API int gi_random_normal(void* out, int dtype, long n, unsigned long long key, double offset, double scale, hipStream_t stream) {
    GI_REQUIRE(out != nullptr && n > 0, "random_normal: bad arguments (n %ld)", n);
    const unsigned grid = (unsigned)min((n + 255) / 256, (long)gi_compute_units() * 16);
    if (dtype == GI_F32) random_normal_kernel<float><<<grid, 256, 0, stream>>>((float*)out, (size_t)n, key, offset, scale);
    else if (dtype == GI_BF16) random_normal_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, (size_t)n, key, offset, scale);
    else return gi_fail("random_normal: unknown dtype %d", dtype);
    GI_CHECK_LAUNCH("random_normal");
    return 0;
}
