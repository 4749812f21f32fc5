// Causal attention of single rows over a paged key/value cache, in true 32-bit arithmetic.
//
// One wave per (row, query head).  Row t of the request in slot[t] at position pos[t] sees the
// keys at positions lo .. pos[t] of its own request, lo = max(0, pos - window + 1) with a window
// and 0 without; query head h uses key/value head h / (n_heads / n_kv).  Scores are scaled by
// 1/sqrt(hd) after the dot product, softmax is taken with a running maximum over tiles of 64
// keys, and the weighted sum of the values follows in position order
// (src/model/transformer.cpp:228-255, src/gpu/device_kernels.inc:377-449).  The softmax's
// denominator is a 64-bit sum, as the reference's (src/kernels/kernels.cpp:95-100): a 32-bit
// running sum over tens of thousands of keys loses digits that every output of the head then lacks.
// The order of every sum depends on (pos, window, hd) only, so a row's result has the same bits
// whatever else is in the batch and whichever pages hold its request.
//
// Cache of one layer: per page the keys [kv_head][place][hd], then the values transposed
// [kv_head][hd][place]; table[slot][i] is the page of positions i*page_size .. (i+1)*page_size - 1.
#include "common.h"

namespace {

constexpr int MAX_HD = 256;

template <typename TQ, typename TC, typename TO>
__global__ __launch_bounds__(64) void attention_exact_kernel(const TQ* __restrict__ q, const TC* __restrict__ cache, TO* __restrict__ out,
                                                            const int* __restrict__ pos, const int* __restrict__ slot,
                                                            const int* __restrict__ table, int table_stride, long page_stride,
                                                            int page_size, int n_heads, int n_kv, int hd, int window, float scale) {
    __shared__ float q_s[MAX_HD];
    __shared__ float p_s[64];
    __shared__ long v_off[64];
    const int lane = threadIdx.x;
    const int t = blockIdx.x / n_heads, h = blockIdx.x % n_heads, g = h / (n_heads / n_kv);
    const int p_row = pos[t];
    const int* tab = table + (size_t)slot[t] * table_stride;
    const int lo = (window > 0 && p_row - window + 1 > 0) ? p_row - window + 1 : 0;
    for (int d = lane; d < hd; d += 64) q_s[d] = load_f32(q, (size_t)t * n_heads * hd + h * hd + d);
    __syncthreads();

    const long v_plane = (long)n_kv * page_size * hd;   // from a page's keys to its values
    float m = -INFINITY;
    double l = 0.0;
    float acc[MAX_HD / 64] = {};
    for (int j0 = lo; j0 <= p_row; j0 += 64) {
        const int j = j0 + lane;
        const bool valid = j <= p_row;
        float s = -INFINITY;
        long off = 0, voff = 0;
        if (valid) {
            const long page = (long)tab[j / page_size] * page_stride;
            off = page + ((long)g * page_size + j % page_size) * hd;
            voff = page + v_plane + (long)g * hd * page_size + j % page_size;
            float dot = 0.f;
            for (int d = 0; d < hd; ++d) dot = fmaf(q_s[d], load_f32(cache, off + d), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m - m_new);      // 0 at the first tile (m = -inf)
        l = l * (double)corr + (double)wave_sum(p);
        m = m_new;
        __syncthreads();                         // the previous tile's p_s and v_off have been read
        p_s[lane] = p;
        v_off[lane] = voff;
        __syncthreads();
        const int n_here = min(64, p_row - j0 + 1);
#pragma unroll
        for (int i = 0; i < MAX_HD / 64; ++i) acc[i] *= corr;
        for (int jj = 0; jj < n_here; ++jj) {
            const float pj = p_s[jj];
            const long vo = v_off[jj];
#pragma unroll
            for (int i = 0; i < MAX_HD / 64; ++i) {
                const int d = lane + 64 * i;
                if (d < hd) acc[i] = fmaf(pj, load_f32(cache, vo + (long)d * page_size), acc[i]);
            }
        }
    }
    const float inv = 1.0f / (float)l;
#pragma unroll
    for (int i = 0; i < MAX_HD / 64; ++i) {
        const int d = lane + 64 * i;
        if (d < hd) store_f32(out, (size_t)t * n_heads * hd + h * hd + d, acc[i] * inv);
    }
}

}  // namespace

GI_API int gi_attention_exact_max_head_size() { return MAX_HD; }

GI_API int gi_attention_exact(const void* q, int q_dtype, const void* cache, int cache_dtype, void* out, int out_dtype, const int* pos,
                              const int* slot, const int* table, int table_stride, long page_stride, int page_size, int n_rows,
                              int n_heads, int n_kv, int hd, int window, float scale, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention_exact: bad head counts (%d rows, %d heads, %d kv heads)",
               n_rows, n_heads, n_kv);
    GI_REQUIRE(hd > 0 && hd <= MAX_HD, "attention_exact: head size %d is outside 1..%d", hd, MAX_HD);
    GI_REQUIRE(page_size > 0 && page_stride >= 2L * n_kv * page_size * hd, "attention_exact: page stride %ld too small", page_stride);
    GI_REQUIRE((long)n_rows * n_heads < 2147483647L, "attention_exact: too many (row, head) pairs");
    const unsigned grid = (unsigned)(n_rows * n_heads);
#define GO(TQ, TC, TO)                                                                                                          \
    attention_exact_kernel<TQ, TC, TO><<<grid, 64, 0, stream>>>((const TQ*)q, (const TC*)cache, (TO*)out, pos, slot, table, table_stride, \
                                                                page_stride, page_size, n_heads, n_kv, hd, window, scale)
    if (q_dtype == GI_F32 && cache_dtype == GI_F32 && out_dtype == GI_F32) GO(float, float, float);
    else if (q_dtype == GI_BF16 && cache_dtype == GI_BF16 && out_dtype == GI_BF16) GO(bf16_t, bf16_t, bf16_t);
    else return gi_fail("attention_exact: dtypes (%d, %d, %d) must be all float32 or all bfloat16", q_dtype, cache_dtype, out_dtype);
#undef GO
    GI_CHECK_LAUNCH("attention_exact");
    return 0;
}
