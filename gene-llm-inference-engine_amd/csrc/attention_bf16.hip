// Causal attention over the paged bfloat16 cache on the matrix cores: one kernel for portions of
// prompts (many query rows of one request), one for single decoded rows.
//
// Cache of one layer, per page: keys [kv_head][place][HD], then values transposed
// [kv_head][HD][place].  Page sizes must be multiples of 16.  Scores are scaled after the dot
// product; softmax runs in 32-bit with a running maximum; probabilities are rounded to bfloat16
// for the product with the values, their sum is kept unrounded.
//
// Both kernels use the freedom that a matrix instruction sums over its k index in any order as
// long as both operands assign k to lanes in the same way: probabilities stay in the registers
// in which the score product left them, and the value operand is loaded to match.
#include "common.h"
#include <type_traits>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint4 load16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ uint2 load8(const bf16_t* p) { return *reinterpret_cast<const uint2*>(p); }
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }
__device__ __forceinline__ uint32_t pack2(float a, float b) { return f32x2_to_bf16x2(a, b); }
// e^x as 2^(x * log2 e): one multiply and the hardware's exp2.
constexpr float LOG2E = 1.4426950408889634f;
__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// =========================================================================================== prompt
// Workgroup: PAIR row tiles of one request (up to 32 * NW consecutive rows each), one query head.
// 32 rows belong to two waves: each takes one half (32 positions) of every tile of 64 keys and
// keeps its own running maximum, sum and output, which meet in LDS at the end.  That way a row's
// walk over the keys, a chain of dependent steps (products, maximum, exponentials, products),
// is shared by two waves that fill each other's waits.
// With PAIR = 2 a late tile of a prompt shares its workgroup with an early one: the two walk the
// keys together from the first position on, the early tile's waves stop where their rows end, and
// every workgroup of a prompt has about the same number of keys to visit (tile i sees i + 1 tiles
// of keys; a workgroup per tile would leave the chip waiting for the last ones).
// Keys and values come in tiles of 64 positions through LDS, staged once for all waves.  The
// score product is taken transposed, S^T[kv][q] = K * Q^T, so that each lane owns one query row
// (column lane%32) and the softmax statistics of a row live in one lane (and its partner lane^32);
// the output is accumulated transposed as well, O^T[d][q] = V^T * P^T.
//
// tiles[i] = {first row in the step, number of rows, position of the first row, request slot};
// workgroup w takes tiles[PAIR * w .. PAIR * w + PAIR), of one request (a tile of 0 rows fills a pair).
constexpr int KV_TILE = 64;
// The running maximum a row's exponentials are taken against need not be the true one: any m gives the same O / l as long as
// nothing overflows.  So m follows the scores only when one of a wave's rows has risen above it by more than this (in units of
// log2 e: e^(s - m) then stays under 2^8, nothing for 32-bit sums, and bfloat16 keeps its relative precision at every size),
// and the rescaling of everything gathered so far, a third of a tile's vector instructions, leaves the common path: with the
// true maximum some row of 32 has a new one in most tiles.  The first keys a row sees always set it (-inf + slack = -inf).
constexpr float MAX_SLACK = 8.0f;

template <int HD, int NW, int PAIR>
__global__ __launch_bounds__(128 * NW * PAIR) void attention_prompt_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache,
                                                                          bf16_t* __restrict__ out, const int4* __restrict__ tiles,
                                                                          const int* __restrict__ table, int table_stride, long page_stride,
                                                                          int page_size, int n_heads, int n_kv, int window, float scale,
                                                                          int n_splits, const int* __restrict__ tile_first, float* __restrict__ part) {
    constexpr int NT = 128 * NW * PAIR;         // threads
    constexpr int K_STRIDE = HD + 8;            // bf16 elements; 16-byte reads of 32 rows hit distinct banks
    constexpr int V_STRIDE = KV_TILE + 4;       // 8-byte reads of 32 rows hit distinct banks
    constexpr int QSTEPS = HD / 16, DT = HD / 32;
    constexpr int K_PIECES = KV_TILE * HD / 8;              // 16-byte pieces of a tile of keys; the values have as many
    constexpr int PP = (2 * K_PIECES + NT - 1) / NT;        // pieces per thread and tile
    constexpr int K_BYTES = KV_TILE * K_STRIDE * 2, V_BYTES = HD * V_STRIDE * 2;
    constexpr int MERGE_STRIDE = HD + 3;                    // floats per row in the final exchange: {m, l, O[HD]}, odd against bank conflicts
    static_assert(NW * 32 * MERGE_STRIDE * 4 <= 2 * (K_BYTES + V_BYTES), "the final exchange of one row tile must fit in the key and value tiles' memory");
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * (K_BYTES + V_BYTES)];     // two tiles: one is read while the next is written
    auto keys_of = [&](int b) { return reinterpret_cast<bf16_t*>(lds + b * (K_BYTES + V_BYTES)); };
    auto values_of = [&](int b) { return reinterpret_cast<bf16_t*>(lds + b * (K_BYTES + V_BYTES) + K_BYTES); };

    // With few tiles the keys are shared out over n_splits workgroups (grid x = groups of tiles * splits); each writes
    // an unnormalised partial result {m, l, O} per row, as the decode kernel's splits do, for the same combine kernel.
    const int group = gridDim.x / n_splits - 1 - blockIdx.x / n_splits, split = blockIdx.x % n_splits;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ks = wave & 1;                                    // which half of every key tile
    const int half = PAIR == 2 ? (wave >> 1) / NW : 0, wv = (wave >> 1) - half * NW;
    const int4 tile_a = tiles[PAIR * group];
    const int4 tile_b = PAIR == 2 ? tiles[PAIR * group + PAIR - 1] : int4{0, 0, 0, 0};
    const int4 tile = half ? tile_b : tile_a;
    const int row0 = tile.x, n_rows = tile.y, pos0 = tile.z, slot = tile_a.w;
    const int head = blockIdx.y, g = head / (n_heads / n_kv);
    const int col = lane & 31, hf = lane >> 5;
    const int* tab = table + (size_t)slot * table_stride;

    const int my_row = wv * 32 + col;                           // this lane's query row within its tile
    const bool row_ok = my_row < n_rows;
    const int my_pos = row_ok ? pos0 + my_row : -1;
    const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
    const int wave_last = pos0 + min(n_rows, wv * 32 + 32) - 1;         // the last position this wave's rows see
    const bool wave_ok = wv * 32 < n_rows;
    const bool wave_full = wv * 32 + 32 <= n_rows;
    const int wave_first = wave_full ? pos0 + wv * 32 : -1;             // keys up to here are seen by every row of the wave (none if rows are missing)
    const int wave_lo_max = window > 0 ? max(0, wave_last - window + 1) : 0;      // ... and keys from here on
    const int wave_lo_min = window > 0 ? max(0, pos0 + wv * 32 - window + 1) : 0; // no row of the wave sees a key before this one
    const float scale2 = scale * LOG2E;

    bf16x8 qreg[QSTEPS];
#pragma unroll
    for (int s = 0; s < QSTEPS; ++s) {
        uint4 v = {0, 0, 0, 0};
        if (row_ok) v = load16(q + ((size_t)(row0 + my_row) * n_heads + head) * HD + 16 * s + 8 * hf);
        qreg[s] = as_bf16x8(v);
    }
    floatx16 o[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) o[i] = floatx16{};
    float m = -INFINITY, l = 0.f;               // l: this lane's share of the sum (its partner lane^32 holds the rest)

    // the keys the workgroup walks: from the first one any of its rows sees to the last
    auto lowest = [&](const int4 t) { return (window > 0 && t.z - window + 1 > 0) ? t.z - window + 1 : 0; };
    int last_pos = tile_a.z + tile_a.y - 1, first_lo = lowest(tile_a);
    if (PAIR == 2 && tile_b.y > 0) {
        last_pos = max(last_pos, tile_b.z + tile_b.y - 1);
        first_lo = min(first_lo, lowest(tile_b));
    }
    const long v_plane = (long)n_kv * page_size * HD;
    // this workgroup's share of the key tiles [first_lo, last_pos]: whole tiles of 64, the same number for every split
    const int range_first = first_lo & ~(KV_TILE - 1);
    const int per_split = ((last_pos - range_first) / KV_TILE + n_splits) / n_splits * KV_TILE;
    const int kv_first = range_first + split * per_split, my_last = min(last_pos, kv_first + per_split - 1);

    // A tile of 64 key positions travels global memory -> registers -> LDS in 16-byte pieces, keys first, then the
    // values (stored transposed in the cache: HD rows of positions); a wave takes 64 consecutive pieces at a time.
    // For head sizes 32, 64 and 128 those 64 pieces lie in one page (they cover 16, 8 or 4 key rows, or 64 value
    // rows of 8 or 16 positions, and pages hold multiples of 16 positions): the page number, the place in the page
    // and the address of the page are then the same for the whole wave and worked out by the scalar unit, and a lane
    // only adds an offset that never changes.  Other head sizes look their pages up lane by lane.
    constexpr bool ONE_PAGE = HD == 32 || HD == 64 || HD == 128;
    const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
    auto page_index = [&](int kv) { return page_shift >= 0 ? kv >> page_shift : kv / page_size; };
    auto place_of = [&](int kv) { return page_shift >= 0 ? kv & (page_size - 1) : kv % page_size; };
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    __builtin_assume(wave_u >= 0 && wave_u < NT / 64);
    int kv_off[PP], per_place[PP], in_lds[PP], page[PP];
    unsigned in_page[PP];                       // elements from the start of the page's keys (or values) at place 0
    bool has[PP], is_key[PP];
    constexpr int DEPTH = PP == 1 ? 3 : 2;      // tiles on their way from the cache's memory, in registers (their number is paid in waves per compute unit)
    uint4 reg[DEPTH][PP];
#pragma unroll
    for (int i = 0; i < PP; ++i) {
        const int e0 = ONE_PAGE ? 64 * (wave_u + (NT / 64) * i) : tid + NT * i, e = ONE_PAGE ? e0 + lane : e0;      // e0: what the lookups go by
        has[i] = e0 < 2 * K_PIECES;
        is_key[i] = e0 < K_PIECES;
        if (is_key[i]) {                                      // keys: 64 rows of HD
            const int r = e / (HD / 8), c = (e % (HD / 8)) * 8, r0 = e0 / (HD / 8);
            kv_off[i] = r0;
            in_page[i] = g * page_size * HD + c + (r - r0) * HD;
            per_place[i] = HD;
            in_lds[i] = r * K_STRIDE + c;
        } else {                                              // values: HD rows of 64 positions, 8 positions a piece
            const int ev = e - K_PIECES, d = ev % HD, c = (ev / HD) * 8, c0 = ((e0 - K_PIECES) / HD) * 8;
            kv_off[i] = c0;
            in_page[i] = (g * HD + d) * page_size + (c - c0);
            per_place[i] = 1;
            in_lds[i] = d * V_STRIDE + c;
        }
    }
    auto fetch_pages = [&](int kv0) {
#pragma unroll
        for (int i = 0; i < PP; ++i) page[i] = (has[i] && kv0 + kv_off[i] <= my_last) ? tab[page_index(kv0 + kv_off[i])] : -1;
    };
    // Positions beyond the last one (or before a window) have no page (-1).  Their loads go to a page the request
    // does hold instead of being skipped, so that every tile issues the same loads and the count of loads in flight
    // is known where a tile's registers are waited for; what they bring is finite, and those keys are masked.
    const int held_page = tab[page_index(max(my_last, 0))];
    auto fetch = [&](int kv0, uint4* to) {      // with the pages that fetch_pages(kv0) brought
#pragma unroll
        for (int i = 0; i < PP; ++i) {
            if (!has[i]) continue;
            const int pg = page[i] >= 0 ? page[i] : held_page;
            const bf16_t* at_place = cache + (long)pg * page_stride + (is_key[i] ? 0 : v_plane) + place_of(kv0 + kv_off[i]) * per_place[i];
            to[i] = *reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(at_place) + (size_t)(2u * in_page[i]));
        }
    };
    auto stash = [&](const uint4* from, bf16_t* Ks, bf16_t* Vs) {
#pragma unroll
        for (int i = 0; i < PP; ++i) {
            if (!has[i]) continue;
            if (is_key[i]) {
                *reinterpret_cast<uint4*>(&Ks[in_lds[i]]) = from[i];
            } else {
                uint2* dst = reinterpret_cast<uint2*>(&Vs[in_lds[i]]);
                dst[0] = uint2{from[i].x, from[i].y};
                dst[1] = uint2{from[i].z, from[i].w};
            }
        }
    };

    // Tile t of the keys waits in LDS buffer t % 2 while the products of tile t - 1 run.  Its loads were issued
    // DEPTH tiles earlier (the products of a tile take less time than a load that misses the cache) into register
    // set t % DEPTH, and the page numbers they need one tile before that.  One barrier a tile: it orders this tile's
    // reads before the write after next, and the next tile's write before its reads.
    fetch_pages(kv_first);
    fetch(kv_first, reg[0]);
    fetch_pages(kv_first + KV_TILE);            // beyond the last position: no lookups, and no loads then
    stash(reg[0], keys_of(0), values_of(0));
    // (the queries are named here so that their loads are waited for once, with the first tile's, and the waits
    // inside the loop count the tiles' loads only)
#pragma unroll
    for (int k = 0; k < QSTEPS; ++k) asm volatile("" ::"v"(qreg[k]));
#pragma unroll
    for (int d = 1; d <= DEPTH; ++d) {
        fetch(kv_first + d * KV_TILE, reg[d % DEPTH]);
        fetch_pages(kv_first + (d + 1) * KV_TILE);
    }
    barrier_lds();
    int buf = 0, kv0 = kv_first;
    while (kv0 <= my_last) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d, kv0 += KV_TILE, buf ^= 1) {      // the tile in LDS is number d (mod DEPTH), the next one sits in set (d + 1) % DEPTH
        if (kv0 > my_last) break;
        // (also for the last tiles, where nothing more is to come: a tile without loads would leave the number of
        // loads in flight unknown to the compiler, which then waits for all of them)
        stash(reg[(d + 1) % DEPTH], keys_of(buf ^ 1), values_of(buf ^ 1));
        fetch(kv0 + (1 + DEPTH) * KV_TILE, reg[(d + 1) % DEPTH]);
        fetch_pages(kv0 + (2 + DEPTH) * KV_TILE);
        const int kv_base = kv0 + 32 * ks;                              // this wave's half of the tile
        if (wave_ok && kv_base <= wave_last && kv_base + 32 > wave_lo_min) {      // else: no row of this wave sees a key of it
            const bf16_t* Ks = keys_of(buf);
            const bf16_t* Vs = values_of(buf);
            floatx16 s = floatx16{};
#pragma unroll
            for (int k = 0; k < QSTEPS; ++k) {
                const bf16x8 a = as_bf16x8(*reinterpret_cast<const uint4*>(&Ks[(32 * ks + col) * K_STRIDE + 16 * k + 8 * hf]));
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[k], s, 0, 0, 0);
            }
            // element v of s: key position kv_base + 8*(v/4) + 4*hf + v%4, query row `col`.  Scores are kept
            // in units of log2 e (scale2 = scale * log2 e), so that e^(s - m) is one exp2.
            const bool inside = kv_base + 31 <= wave_first && kv_base >= wave_lo_max;     // every key here is seen by every row of the wave
            float mx = -INFINITY;
            if (inside) {
#pragma unroll
                for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[v]);
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int kv = kv_base + 8 * (v / 4) + 4 * hf + (v & 3);
                    s[v] = (kv <= my_pos && kv >= my_lo) ? s[v] : -INFINITY;
                    mx = fmaxf(mx, s[v]);
                }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * scale2;             // scale2 > 0: the maximum of the scaled scores
            const float m_new = fmaxf(m, mx);
            if (__any(m_new > m + MAX_SLACK)) {                           // some row's maximum rose by much: rescale what was gathered so far
                const float corr = exp2_fast(m - ((m_new == -INFINITY) ? 0.f : m_new));
                l *= corr;
#pragma unroll
                for (int i = 0; i < DT; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) o[i][v] *= corr;
                m = m_new;
            }
            const float m_use = (m == -INFINITY) ? 0.f : m;              // a row that has seen nothing yet
            float sum = 0.f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                s[v] = exp2_fast(fmaf(s[v], scale2, -m_use));
                sum += s[v];
            }
            l += sum;
#pragma unroll
            for (int t = 0; t < 2; ++t) {                                 // two groups of 16 key positions
                const uint4 pb = {pack2(s[8 * t], s[8 * t + 1]), pack2(s[8 * t + 2], s[8 * t + 3]), pack2(s[8 * t + 4], s[8 * t + 5]),
                                  pack2(s[8 * t + 6], s[8 * t + 7])};
                // slot e of this lane is key position 32*ks + 16*t + 8*(e/4) + 4*hf + e%4 of the tile
#pragma unroll
                for (int i = 0; i < DT; ++i) {
                    const bf16_t* vrow = &Vs[(32 * i + col) * V_STRIDE + 32 * ks + 16 * t + 4 * hf];
                    const uint2 lo = *reinterpret_cast<const uint2*>(vrow), hi = *reinterpret_cast<const uint2*>(vrow + 8);
                    o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(uint4{lo.x, lo.y, hi.x, hi.y}), as_bf16x8(pb), o[i], 0, 0, 0);
                }
            }
        }
        barrier_lds();                          // not __syncthreads(): the loads of the tiles to come stay in flight
      }
    }
    l += __shfl_xor(l, 32, 64);                                // both lanes of a row used the same maxima: their sums add up

    // The two waves of 32 rows meet: the wave of the second key halves leaves {m, l, O} in LDS (the key tiles are
    // done with), the other one adds it to its own and writes the rows out.  One row tile at a time.
    float* xch = reinterpret_cast<float*>(lds) + (size_t)(wv * 32 + col) * MERGE_STRIDE;
#pragma unroll
    for (int pass = 0; pass < PAIR; ++pass) {
        if (pass > 0) __syncthreads();
        if (half == pass && ks == 1 && row_ok) {
            if (hf == 0) {
                xch[0] = m;
                xch[1] = l;
            }
#pragma unroll
            for (int i = 0; i < DT; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) xch[2 + 32 * i + 8 * (v / 4) + 4 * hf + (v & 3)] = o[i][v];
        }
        __syncthreads();
        if (half == pass && ks == 0 && row_ok) {
            const float m1 = xch[0], l1 = xch[1];
            const float m_all = fmaxf(m, m1);
            const float w0 = (m == -INFINITY) ? 0.f : exp2_fast(m - m_all), w1 = (m1 == -INFINITY) ? 0.f : exp2_fast(m1 - m_all);
            l = l * w0 + l1 * w1;
            m = m_all;
#pragma unroll
            for (int i = 0; i < DT; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[i][v] = o[i][v] * w0 + xch[2 + 32 * i + 8 * (v / 4) + 4 * hf + (v & 3)] * w1;
        }
    }
    if (!row_ok || ks != 0) return;
    if (n_splits > 1) {                                       // part[row of the split tiles][head][split] = {m, l, O[HD]}
        float* dst = part + (((size_t)(tile_first[PAIR * group + half] + my_row) * n_heads + head) * n_splits + split) * (HD + 2);
        if (hf == 0) {
            dst[0] = m;
            dst[1] = l;
        }
#pragma unroll
        for (int i = 0; i < DT; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) dst[2 + 32 * i + 8 * (v / 4) + 4 * hf + (v & 3)] = o[i][v];
        return;
    }
    const float inv = 1.0f / l;
    bf16_t* orow = out + ((size_t)(row0 + my_row) * n_heads + head) * HD;
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {                                  // element v: channel 32*i + 8*(v/4) + 4*hf + v%4
            const int d = 32 * i + 8 * v4 + 4 * hf;
            *reinterpret_cast<uint2*>(orow + d) = uint2{pack2(o[i][4 * v4] * inv, o[i][4 * v4 + 1] * inv),
                                                        pack2(o[i][4 * v4 + 2] * inv, o[i][4 * v4 + 3] * inv)};
        }
}

// ------------------------------------------------------------------------------------- prompt, wide
// The same attention for head sizes 64 and 128 with another division of the work: a wave owns 32 rows and takes whole
// tiles of 64 keys, a workgroup of NW waves owns one row tile, and a compute unit holds several workgroups that do not wait
// for each other (two at head size 128, three at 64): where the kernel above ties all waves of a compute unit to one barrier
// per tile, so that they load together and then multiply together, here a wave multiplies while its neighbours on the SIMD,
// of other workgroups, load or exponentiate.  Nothing is merged at the end, a row's statistics stay in its two lanes.
//
// Key and value tiles go from the cache straight into LDS (global_load_lds_dwordx4: lane l of a load lands at the load's
// LDS address + 16 l, whatever it read), two stages: the loads of tile t + 1 are issued at the start of the step that
// multiplies tile t and waited for at its end, before the barrier.  LDS rows are not padded (a load cannot pad); instead
// the 16-byte chunk c of a row lies at chunk position c ^ f(row), so that the 16 lanes a clock serves, which read one
// chunk column of 16 consecutive rows, hit 16 different bank groups: for the keys f(r) = r % 16 at 256 bytes a row
// (128 channels), (r / 2) % 8 at 128 bytes.  The values (transposed in the cache: per channel, a page's positions) lie in LDS as
// [group of 16 positions][channel][2 chunks of 8 positions], with the two chunks swapped for channels with (d / 8) % 2 = 1.
// A wave-wide load so covers 4 or 8 key rows or 32 channels of one group of 16 positions, which lie in one page (pages hold
// multiples of 16): the page's address and the place in it are worked out by the scalar unit, and a lane adds an offset
// that never changes.
//
// The rows of a key tile are taken in another order by the score product: row i of the matrix instruction reads key
// pi(i) = 16 (i / 16) + 8 ((i / 4) % 2) + 4 ((i / 8) % 2) + i % 4 of its 32, so that the 8 scores a lane holds for the
// next product's k index are 8 consecutive keys, and the value operand is one 16-byte read (8 positions of a channel).
template <int HD, int NW>
__global__ __launch_bounds__(64 * NW, HD == 128 ? 2 : 3) void attention_prompt_wide_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ cache,
                                                                       bf16_t* __restrict__ out, const int4* __restrict__ tiles,
                                                                       const int* __restrict__ table, int table_stride, long page_stride,
                                                                       int page_size, int n_heads, int n_kv, int window, float scale,
                                                                       int n_splits, const int* __restrict__ tile_first, float* __restrict__ part,
                                                                       int list_order) {
    static_assert(HD == 128 || HD == 64, "the chunk swizzle is made for key rows of 256 or 128 bytes");
    constexpr int QSTEPS = HD / 16, DT = HD / 32;
    constexpr int K_BYTES = KV_TILE * HD * 2, V_BYTES = HD * KV_TILE * 2, STAGE = K_BYTES + V_BYTES;
    constexpr int CK = HD / 8;                               // 16-byte chunks of a key row
    constexpr int K_LOADS = K_BYTES / 1024, V_LOADS = V_BYTES / 1024, LOADS = (K_LOADS + V_LOADS) / NW;      // wave-wide loads of 1 KB: per tile, per wave
    static_assert((K_LOADS + V_LOADS) % NW == 0 && K_LOADS % LOADS == 0, "a wave's loads are all keys or all values");
    static_assert(LOADS % (16 / (64 / CK)) == 0, "a wave's loads begin with a group's first rows");
    __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * STAGE];

    // Workgroups start in the order of their numbers, heads fastest: the long walks (late tiles) of all heads first, so that the
    // short ones fill the end.  A plain list runs from early tiles to late ones and is taken backwards; a list of pairs names a
    // late tile, an early one, the next later one, the next earlier one, ...: first its late tiles in their order, then its early
    // ones backwards.
    const int n_groups = gridDim.y / n_splits, turn = blockIdx.y / n_splits, split = blockIdx.y % n_splits;
    const int group = !list_order ? n_groups - 1 - turn : turn < n_groups / 2 ? 2 * turn : 2 * (n_groups - 1 - turn) + 1;
    const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int4 tile = tiles[group];
    const int row0 = tile.x, n_rows = tile.y, pos0 = tile.z, slot = tile.w;
    if (n_rows == 0) return;                                  // (a tile that only fills a pair)
    const int head = blockIdx.x, g = head / (n_heads / n_kv);
    const int col = lane & 31, hf = lane >> 5;
    const int* tab = table + (size_t)slot * table_stride;

    const int my_row = wv * 32 + col;
    const bool row_ok = my_row < n_rows;
    const int my_pos = row_ok ? pos0 + my_row : -1;
    const int my_lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
    const int wave_last = pos0 + min(n_rows, wv * 32 + 32) - 1;
    const bool wave_ok = wv * 32 < n_rows;
    const bool wave_full = wv * 32 + 32 <= n_rows;
    const int wave_first = wave_full ? pos0 + wv * 32 : -1;
    const int wave_lo_max = window > 0 ? max(0, wave_last - window + 1) : 0;
    const int wave_lo_min = window > 0 ? max(0, pos0 + wv * 32 - window + 1) : 0;
    const float scale2 = scale * LOG2E;

    bf16x8 qreg[QSTEPS];
#pragma unroll
    for (int s = 0; s < QSTEPS; ++s) {
        uint4 v = {0, 0, 0, 0};
        if (row_ok) v = load16(q + ((size_t)(row0 + my_row) * n_heads + head) * HD + 16 * s + 8 * hf);
        qreg[s] = as_bf16x8(v);
    }
    floatx16 o[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) o[i] = floatx16{};
    float m = -INFINITY, l = 0.f;

    const int last_pos = pos0 + n_rows - 1;
    const int first_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
    const int range_first = first_lo & ~(KV_TILE - 1);
    const int per_split = ((last_pos - range_first) / KV_TILE + n_splits) / n_splits * KV_TILE;
    const int kv_first = range_first + split * per_split, my_last = min(last_pos, kv_first + per_split - 1);
    const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
    auto page_index = [&](int kv) { return page_shift >= 0 ? kv >> page_shift : kv / page_size; };
    auto place_of = [&](int kv) { return page_shift >= 0 ? kv & (page_size - 1) : kv % page_size; };
    const int held_page = tab[page_index(max(my_last, 0))];   // stands in where a position has no page (beyond the end, before a window): finite, and masked
    const long v_plane = (long)n_kv * page_size * HD;

    // What this wave loads of every tile: LOADS loads of 1 KB, all of the keys' part or all of the values' part.
    // Keys: load n covers rows n * 64 / CK ..; lane l brings chunk (l % CK) ^ f(row) of row first + l / CK.
    // Values: load n covers group n / (HD / 32) of 16 positions and 32 channels; lane l brings chunk (l % 2) ^ ((d / 8) % 2) of channel d = first + l / 2.
    const bool loads_keys = wv * LOADS < K_LOADS;
    // Bytes from the group's place 0 in the page's keys (or values) to what this lane brings.  The key loads of a group of 16
    // positions differ in which of its rows they cover (KP loads a group, and the swizzle goes by the row): one offset each.
    // The value loads of a group differ in their 32 channels only, which the scalar unit adds to the page's address.
    constexpr int KP = 16 / (64 / CK);
    unsigned lane_off[KP];
#pragma unroll
    for (int j = 0; j < KP; ++j) {
        if (loads_keys) {
            const int r = j * (64 / CK) + lane / CK, c = (lane % CK) ^ (HD == 128 ? (r & 15) : ((r >> 1) & 7));      // (row within its group of 16)
            lane_off[j] = 2u * (unsigned)((g * page_size + r) * HD + 8 * c);
        } else {                                              // (the same for every j)
            const int d = lane / 2, h = (lane & 1) ^ ((d >> 3) & 1);
            lane_off[j] = 2u * (unsigned)((g * HD + d) * page_size + 8 * h);
        }
    }
    typedef __attribute__((address_space(3))) unsigned char* lds_ptr_t;
    const unsigned lds_base = (unsigned)(size_t)(lds_ptr_t)lds;      // the tiles' offset in LDS
    // A tile's four groups of 16 positions: lanes 0 .. 3 work out one group's page and place in it each (a division, if the page
    // size is no power of two, and a load: once a tile, by the vector unit), and the loads read them from those lanes.
    auto look_up = [&](int kv0, int& pages_v, int& places_v) {
        const int kv = kv0 + 16 * (lane & 3), index = page_index(kv);
        const int pg = kv <= my_last ? tab[index] : -1;
        pages_v = pg >= 0 ? pg : held_page;
        places_v = kv - index * page_size;
    };
    auto send_for = [&](int pages_v, int places_v, int stage) {      // the loads of a tile into `stage`, with what look_up gave for it
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int n = wv * LOADS + i;
            const int grp = loads_keys ? (n * (64 / CK)) >> 4 : (n - K_LOADS) / (HD / 32);      // which 16 positions of the tile (the same for the wave)
            const int pg = __builtin_amdgcn_readlane(pages_v, grp), place = __builtin_amdgcn_readlane(places_v, grp);
            const bf16_t* base = cache + (long)pg * page_stride +
                                 (loads_keys ? (long)place * HD : v_plane + place + (long)((n - K_LOADS) % (HD / 32)) * 32 * page_size);
            const unsigned dst = __builtin_amdgcn_readfirstlane(lds_base + stage * STAGE + n * 1024);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(lane_off[i % KP]), "s"(base) : "memory", "m0");
        }
    };
    auto landed_barrier = [&]() {                             // this wave's loads have landed; then everybody's, and everybody has read the other stage
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    };

    int pages_v, places_v;
    look_up(kv_first, pages_v, places_v);
    send_for(pages_v, places_v, 0);
    look_up(kv_first + KV_TILE, pages_v, places_v);
    landed_barrier();
    int stage = 0;
    for (int kv0 = kv_first; kv0 <= my_last; kv0 += KV_TILE, stage ^= 1) {
        // The loads of the next tile first (also behind the last one: they bring a held page's keys into the stage nobody reads any
        // more).  A wave that issues such a load is held while the memory pipeline takes it, some 200 clocks each here; issuing
        // them behind the matrix instructions of the scores, or half of them there and half behind those of the values, or all
        // at the end of the step, was 2 to 8 % slower than here, where they have the whole step to land.
        const bool active = wave_ok && kv0 <= wave_last && kv0 + KV_TILE > wave_lo_min;      // else: no row of this wave sees a key of the tile
        const unsigned char* Ks = lds + stage * STAGE;
        const unsigned char* Vs = Ks + K_BYTES;
        send_for(pages_v, places_v, stage ^ 1);
        look_up(kv0 + 2 * KV_TILE, pages_v, places_v);
        if (active) {
            floatx16 s[2] = {floatx16{}, floatx16{}};
            // scores of the tile's two halves of 32 keys: two chains of matrix instructions that do not wait for each other
            const int pi = (col & 16) | ((col & 4) << 1) | ((col & 8) >> 1) | (col & 3);       // the key this lane's row of the product reads
#pragma unroll
            for (int k = 0; k < QSTEPS; ++k) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int r = 32 * h + pi, c = (2 * k + hf) ^ (HD == 128 ? (r & 15) : ((r >> 1) & 7));
                    const bf16x8 a = as_bf16x8(*reinterpret_cast<const uint4*>(Ks + r * (HD * 2) + 16 * c));
                    s[h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[k], s[h], 0, 0, 0);
                }
            }
            // element v of s[h]: key kv0 + 32 h + 16 (v / 8) + 8 hf + v % 8, query row `col`; in units of log2 e after scale2
            // (keys some row of the wave does not see are masked where they stand, before the part that every tile walks)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int kv_base = kv0 + 32 * h;
                if (!(kv_base + 31 <= wave_first && kv_base >= wave_lo_max)) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int kv = kv_base + 16 * (v / 8) + 8 * hf + (v & 7);
                        s[h][v] = (kv <= my_pos && kv >= my_lo) ? s[h][v] : -INFINITY;
                    }
                }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[h][v]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64)) * scale2;
            const float m_new = fmaxf(m, mx);
            if (__any(m_new > m + MAX_SLACK)) {
                const float corr = exp2_fast(m - ((m_new == -INFINITY) ? 0.f : m_new));
                l *= corr;
#pragma unroll
                for (int i = 0; i < DT; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) o[i][v] *= corr;
                m = m_new;
            }
            const float m_use = (m == -INFINITY) ? 0.f : m;
            float sum = 0.f;
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    s[h][v] = exp2_fast(fmaf(s[h][v], scale2, -m_use));
                    sum += s[h][v];
                }
            l += sum;
#pragma unroll
            for (int t = 0; t < 4; ++t) {                     // four groups of 16 keys: slot e of this lane is key 16 t + 8 hf + e
                const floatx16& sh = s[t >> 1];
                const int e0 = 8 * (t & 1);
                const uint4 pb = {pack2(sh[e0], sh[e0 + 1]), pack2(sh[e0 + 2], sh[e0 + 3]), pack2(sh[e0 + 4], sh[e0 + 5]), pack2(sh[e0 + 6], sh[e0 + 7])};
#pragma unroll
                for (int i = 0; i < DT; ++i) {
                    const int d = 32 * i + col;
                    const bf16x8 a = as_bf16x8(*reinterpret_cast<const uint4*>(Vs + (t * HD + d) * 32 + 16 * (hf ^ ((d >> 3) & 1))));
                    o[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, as_bf16x8(pb), o[i], 0, 0, 0);
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this wave's reads of the stage are done before anybody overwrites it
        landed_barrier();
    }
    l += __shfl_xor(l, 32, 64);
    if (!row_ok) return;
    if (n_splits > 1) {                                       // part[row of the split tiles][head][split] = {m, l, O[HD]}
        float* dst = part + (((size_t)(tile_first[group] + my_row) * n_heads + head) * n_splits + split) * (HD + 2);
        if (hf == 0) {
            dst[0] = m;
            dst[1] = l;
        }
#pragma unroll
        for (int i = 0; i < DT; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) dst[2 + 32 * i + 8 * (v / 4) + 4 * hf + (v & 3)] = o[i][v];
        return;
    }
    const float inv = 1.0f / l;
    bf16_t* orow = out + ((size_t)(row0 + my_row) * n_heads + head) * HD;
#pragma unroll
    for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {                      // element v: channel 32*i + 8*(v/4) + 4*hf + v%4
            const int d = 32 * i + 8 * v4 + 4 * hf;
            *reinterpret_cast<uint2*>(orow + d) = uint2{pack2(o[i][4 * v4] * inv, o[i][4 * v4 + 1] * inv),
                                                        pack2(o[i][4 * v4 + 2] * inv, o[i][4 * v4 + 3] * inv)};
        }
}

// =========================================================================================== decode
// One workgroup per (row, key/value head, query-head group of up to 16, split of the context); its
// waves cut the split's range further, one piece each.  Keys and values stream from global memory
// straight into the operands of v_mfma_f32_16x16x32_bf16.  Scores: S[kv][head] = K * Q^T, 16 key
// positions at a time; output O^T[d][head] = V^T * P^T, 32 key positions at a time.  Lane
// (r = lane%16, q4 = lane/16) owns query head r of the group: its softmax statistics and its
// columns of S and O^T.  The waves' unnormalised results {m, l, O} meet in LDS and are merged in
// wave order; with one split the workgroup writes the attention output itself, otherwise it writes
// one partial result to `part` and the combine kernel merges the splits.
//
// FUSED: the queries, keys and values come unrotated in 32-bit, as the input product left them.
// Every wave rotates its own queries.  The row's own key and value are not in the cache yet: the
// wave whose piece ends at the row's position rotates the key, puts key and value into its
// operands in place of what the cache holds there, and writes both to the row's page for later
// steps (one store per element, by the first query-head group).
template <int HD>
struct DecodeShape {                                      // waves a workgroup may have, by the registers a wave needs
    static constexpr int MAX_WAVES = HD <= 128 ? 8 : 4;
};

// Channels c .. c+7 of a head and their partners in the other half, as loaded (`src` points at the head's channel 0), and the
// cosines and sines of their angles, which the row's queries and its key share: the loads are issued early and the rotation is
// taken when the values are needed.
struct Pairs8 {
    float4 a[2], b[2];
};
struct Angles8 {
    float4 cs[2], sn[2];
    bool low;
};
__device__ __forceinline__ Angles8 load_angles8(const float* __restrict__ cos_row, const float* __restrict__ sin_row, int c, int half) {
    Angles8 u;
    u.low = c < half;
    const int cl = u.low ? c : c - half;
#pragma unroll
    for (int h4 = 0; h4 < 2; ++h4) {
        u.cs[h4] = cos_row ? *reinterpret_cast<const float4*>(cos_row + cl + 4 * h4) : float4{1.f, 1.f, 1.f, 1.f};
        u.sn[h4] = sin_row ? *reinterpret_cast<const float4*>(sin_row + cl + 4 * h4) : float4{0.f, 0.f, 0.f, 0.f};
    }
    return u;
}
__device__ __forceinline__ Pairs8 load_pairs8(const float* __restrict__ src, int c, int half) {
    Pairs8 u;
    const int cl = c < half ? c : c - half;
#pragma unroll
    for (int h4 = 0; h4 < 2; ++h4) {
        u.a[h4] = *reinterpret_cast<const float4*>(src + cl + 4 * h4);
        u.b[h4] = *reinterpret_cast<const float4*>(src + cl + half + 4 * h4);
    }
    return u;
}
__device__ __forceinline__ float rotate1(bool low, float a, float b, float c, float s) { return low ? a * c - b * s : a * s + b * c; }
__device__ __forceinline__ uint4 rotated8(const Pairs8& p, const Angles8& u) {
    uint32_t w[4];
#pragma unroll
    for (int h4 = 0; h4 < 2; ++h4) {
        w[2 * h4] = pack2(rotate1(u.low, p.a[h4].x, p.b[h4].x, u.cs[h4].x, u.sn[h4].x), rotate1(u.low, p.a[h4].y, p.b[h4].y, u.cs[h4].y, u.sn[h4].y));
        w[2 * h4 + 1] = pack2(rotate1(u.low, p.a[h4].z, p.b[h4].z, u.cs[h4].z, u.sn[h4].z), rotate1(u.low, p.a[h4].w, p.b[h4].w, u.cs[h4].w, u.sn[h4].w));
    }
    return uint4{w[0], w[1], w[2], w[3]};
}

template <int HD, bool FUSED>
__global__ __launch_bounds__(64 * DecodeShape<HD>::MAX_WAVES) void attention_decode_kernel(
    const bf16_t* __restrict__ q, const float* __restrict__ qf, const float* __restrict__ kf, const float* __restrict__ vf, long ldq, long ldk,
    long ldv, const float* __restrict__ cos_t, const float* __restrict__ sin_t, bf16_t* __restrict__ cache, float* __restrict__ part,
    bf16_t* __restrict__ out, const int* __restrict__ rows, const int* __restrict__ pos, const int* __restrict__ slots,
    const int* __restrict__ table, int table_stride, long page_stride, int page_size, int n_heads, int n_kv, int window, float scale,
    int n_splits, int gh) {
    constexpr int KSTEPS = HD / 32, DT = HD / 16;
    extern __shared__ float merged[];                        // [wave][gh][HD + 2]
    const int group = n_heads / n_kv, hg_per_kv = (group + 15) / 16;
    const int row = rows ? rows[blockIdx.x] : blockIdx.x, g = blockIdx.y / hg_per_kv, hg = blockIdx.y % hg_per_kv, split = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), n_waves = blockDim.x >> 6;
    const int r = lane & 15, q4 = lane >> 4;
    const int head_in_group = hg * 16 + r;
    const bool head_ok = head_in_group < group;
    const int head = g * group + head_in_group;
    // The unrotated queries depend on the row alone: their loads go out first, ahead of the chain
    // position -> page table -> keys.
    [[maybe_unused]] Pairs8 q_raw[KSTEPS];
    [[maybe_unused]] Angles8 angles[KSTEPS];
    if constexpr (FUSED) {
        // (every lane asks for its queries, a lane without a head for the group's first head's: what it brings is dropped; with a
        // load that some lanes skip the compiler waits for all loads in flight at the first use of any)
        if (cos_t != nullptr && sin_t != nullptr) {
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) angles[s] = load_angles8(cos_t + (size_t)row * (HD / 2), sin_t + (size_t)row * (HD / 2), 32 * s + 8 * q4, HD / 2);
        } else {
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) angles[s] = load_angles8(nullptr, nullptr, 32 * s + 8 * q4, HD / 2);
        }
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) q_raw[s] = load_pairs8(qf + (size_t)row * ldq + (size_t)(head_ok ? head : g * group) * HD, 32 * s + 8 * q4, HD / 2);
    }
    const int my_pos = pos[row];
    const int lo = (window > 0 && my_pos - window + 1 > 0) ? my_pos - window + 1 : 0;
    const int* tab = table + (size_t)__builtin_amdgcn_readfirstlane(slots[row]) * table_stride;
    // every row cuts its own range into pieces (multiples of 32), one per wave of every split; short rows leave later pieces empty
    const int n_pieces = n_splits * n_waves, piece = split * n_waves + wave;
    const int span = my_pos + 1 - (lo & ~31);
    const int piece_len = (((span + n_pieces - 1) / n_pieces) + 31) & ~31;
    const int begin = (lo & ~31) + piece * piece_len, end = min(my_pos + 1, begin + piece_len);
    const int page_shift = (page_size & (page_size - 1)) == 0 ? __builtin_ctz(page_size) : -1;
    auto page_index = [&](int kv) { return page_shift >= 0 ? kv >> page_shift : kv / page_size; };
    auto place_of = [&](int kv) { return page_shift >= 0 ? kv & (page_size - 1) : kv % page_size; };
    const float scale2 = scale * LOG2E;            // scores are kept in units of log2 e: e^(s - m) is one exp2
    const long v_plane = (long)n_kv * page_size * HD;
    const bf16_t* kbase = cache + (long)g * page_size * HD;
    const bf16_t* vbase = cache + v_plane + (long)g * HD * page_size;

    const bool has_own = FUSED && kf != nullptr && begin < end && end == my_pos + 1;     // this wave's piece holds the row's own position

    // Loads run ahead of the products: the keys of the next 32 positions and the values of these 32
    // are requested before the scores of these 32 are taken.  An address beyond the row's own range
    // is clamped into it; what it brings is masked below.
    // A tile's 32 positions are two blocks of 16, each within one page (pages hold a multiple of 16 positions), so the two page
    // numbers of a tile are the same for the whole wave: they come through the scalar unit, a tile ahead of the keys that need them
    // (a page number fetched per lane is a vector load like the keys and values, and those come back in the order they were asked
    // for: waiting for it meant waiting for every key and value requested before it, several round trips to memory per tile).
    const int first_page = page_index(lo), last_page = page_index(my_pos);
    auto pages_of = [&](int kv0, int (&pg)[2]) {
#pragma unroll
        for (int t = 0; t < 2; ++t) pg[t] = tab[__builtin_amdgcn_readfirstlane(min(max(page_index(kv0 + 16 * t), first_page), last_page))];
    };
    uint4 k_a[2][KSTEPS], k_b[2][KSTEPS];
    auto load_keys = [&](int kv0, const int (&pg)[2], uint4 (&dst)[2][KSTEPS]) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int kv = min(max(kv0 + 16 * t + r, lo), my_pos);
            const bf16_t* krow = kbase + (long)pg[t] * page_stride + (long)place_of(kv) * HD + 8 * q4;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) dst[t][ks] = load16(krow + 32 * ks);
        }
    };
    // The values of a tile are asked for behind the products of the tile before it (the first tile's behind its keys), into the
    // registers those products have just read.  Slot e of a lane in the value product is key position kv0 + 16*(e/4) + 4*q4 + e%4.
    uint2 vx[DT], vy[DT];
    auto load_values = [&](int kv0, const int (&pg)[2]) {
        const int kva = min(max(kv0 + 4 * q4, lo & ~3), my_pos & ~3), kvb = min(max(kv0 + 16 + 4 * q4, lo & ~3), my_pos & ~3);
        const bf16_t* va = vbase + (long)pg[0] * page_stride + place_of(kva) + (long)r * page_size;
        const bf16_t* vb = vbase + (long)pg[1] * page_stride + place_of(kvb) + (long)r * page_size;
#pragma unroll
        for (int i = 0; i < DT; ++i) {
            vx[i] = load8(va + (long)(16 * i) * page_size);
            vy[i] = load8(vb + (long)(16 * i) * page_size);
        }
    };
    int pg_cur[2] = {0, 0}, pg_nxt[2] = {0, 0};
    if (begin < end) {
        pages_of(begin, pg_cur);
        pages_of(begin + 32, pg_nxt);
        load_keys(begin, pg_cur, k_a);
        load_values(begin, pg_cur);
    }

    bf16x8 qreg[KSTEPS];
    uint4 own_key[KSTEPS];
    bf16_t own_value[DT];
    if constexpr (FUSED) {
        // The row's own key and value (for the one wave whose piece ends at the row's position) are asked for when the first keys
        // are on their way and rotated behind the queries: at heads of 128 channels queries, key and angles at once are 200
        // registers a lane, which halves the waves a compute unit holds.
        [[maybe_unused]] Pairs8 k_raw[KSTEPS];
        [[maybe_unused]] float v_raw[DT];
        if (has_own) {
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) k_raw[ks] = load_pairs8(kf + (size_t)row * ldk + (size_t)g * HD, 32 * ks + 8 * q4, HD / 2);
#pragma unroll
            for (int i = 0; i < DT; ++i) v_raw[i] = vf[(size_t)row * ldv + (size_t)g * HD + 16 * i + r];
        }
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) qreg[s] = as_bf16x8(head_ok ? rotated8(q_raw[s], angles[s]) : uint4{0, 0, 0, 0});
        if (has_own) {
            bf16_t* page = cache + (long)tab[page_index(my_pos)] * page_stride;
            const int place = place_of(my_pos);
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                own_key[ks] = rotated8(k_raw[ks], angles[ks]);
                if (r == 0 && hg == 0)
                    *reinterpret_cast<uint4*>(page + (long)g * page_size * HD + (long)place * HD + 32 * ks + 8 * q4) = own_key[ks];
            }
#pragma unroll
            for (int i = 0; i < DT; ++i) {
                own_value[i] = f32_to_bf16(v_raw[i]);
                if ((i & 3) == q4 && hg == 0) page[v_plane + ((long)g * HD + 16 * i + r) * page_size + place] = own_value[i];
            }
        }
    } else {
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
            uint4 v = {0, 0, 0, 0};
            if (head_ok) v = load16(q + ((size_t)row * n_heads + head) * HD + 32 * s + 8 * q4);
            qreg[s] = as_bf16x8(v);
        }
    }

    floatx4 o[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) o[i] = floatx4{};
    float m = -INFINITY, l = 0.f;
    // One tile of 32 positions: its keys lie in `k_use`; with a tile behind it (NEXT), that tile's keys are requested into `k_fill`
    // and the page numbers of the tile after that through the scalar unit; behind its products that tile's values.  No load of
    // a tile is skipped by a lane or by a condition inside it, so the compiler counts the loads in flight: the scores wait for
    // this tile's keys alone, the output's products for its values alone.
    auto tile = [&](int kv0, auto next, uint4 (&k_use)[2][KSTEPS], uint4 (&k_fill)[2][KSTEPS]) __attribute__((always_inline)) {
        constexpr bool NEXT = decltype(next)::value;
        int pg_far[2] = {0, 0};
        if constexpr (NEXT) pages_of(kv0 + 64, pg_far);
        if constexpr (NEXT) load_keys(kv0 + 32, pg_nxt, k_fill);
        if constexpr (FUSED && !NEXT) {
            if (has_own) {                                // the last tile of the piece: the row's own key and value go in
                const int off = my_pos - kv0;             // 0 .. 31
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    if ((off >> 4) == t && (off & 15) == r) {
#pragma unroll
                        for (int ks = 0; ks < KSTEPS; ++ks) k_use[t][ks] = own_key[ks];
                    }
                if (((off & 15) >> 2) == q4) {
                    const int e = off & 3;
                    const bool second = (off >> 4) != 0;
#pragma unroll
                    for (int i = 0; i < DT; ++i) {
                        const uint2 had = second ? vy[i] : vx[i];
                        const uint32_t val = own_value[i];
                        const uint32_t x = e == 0 ? (had.x & 0xffff0000u) | val : e == 1 ? (had.x & 0x0000ffffu) | (val << 16) : had.x;
                        const uint32_t y = e == 2 ? (had.y & 0xffff0000u) | val : e == 3 ? (had.y & 0x0000ffffu) | (val << 16) : had.y;
                        vx[i] = second ? vx[i] : uint2{x, y};
                        vy[i] = second ? uint2{x, y} : vy[i];
                    }
                }
            }
        }

        floatx4 s[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            s[t] = floatx4{};
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(k_use[t][ks]), qreg[ks], s[t], 0, 0, 0);
        }
        // element v of s[t]: key position kv0 + 16*t + 4*q4 + v, query head r
        float mx = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int kv = kv0 + 16 * t + 4 * q4 + v;
                s[t][v] = (kv >= lo && kv < end) ? s[t][v] * scale2 : -INFINITY;
                mx = fmaxf(mx, s[t][v]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m, mx);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float corr = exp2_fast(m - m_use);
        float sum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                s[t][v] = exp2_fast(s[t][v] - m_use);
                sum += s[t][v];
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        l = l * corr + sum;
        m = m_new;
        const uint4 pb = {pack2(s[0][0], s[0][1]), pack2(s[0][2], s[0][3]), pack2(s[1][0], s[1][1]), pack2(s[1][2], s[1][3])};
#pragma unroll
        for (int i = 0; i < DT; ++i) {
#pragma unroll
            for (int v = 0; v < 4; ++v) o[i][v] *= corr;
            o[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(uint4{vx[i].x, vx[i].y, vy[i].x, vy[i].y}), as_bf16x8(pb), o[i], 0, 0, 0);
        }
        if constexpr (NEXT) {
            load_values(kv0 + 32, pg_nxt);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                pg_cur[t] = pg_nxt[t];
                pg_nxt[t] = pg_far[t];
            }
        }
    };
    // The two key buffers take turns; the piece's last tile has nothing behind it.
    int kv0 = begin;
    for (; kv0 + 64 < end; kv0 += 64) {
        tile(kv0, std::true_type{}, k_a, k_b);
        tile(kv0 + 32, std::true_type{}, k_b, k_a);
    }
    if (kv0 + 32 < end) {
        tile(kv0, std::true_type{}, k_a, k_b);
        tile(kv0 + 32, std::false_type{}, k_b, k_a);
    } else if (kv0 < end) {
        tile(kv0, std::false_type{}, k_a, k_b);
    }

    // The waves' results meet in LDS: element v of o[i] is channel 16*i + 4*q4 + v of query head r.
    if (r < gh) {
        float* mine = merged + ((size_t)wave * gh + r) * (HD + 2);
        if (q4 == 0) {
            mine[0] = m;
            mine[1] = l;
        }
#pragma unroll
        for (int i = 0; i < DT; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) mine[2 + 16 * i + 4 * q4 + v] = o[i][v];
    }
    __syncthreads();
    for (int e = threadIdx.x; e < gh * HD; e += blockDim.x) {
        const int hh = e / HD, d = e % HD;
        if (hg * 16 + hh >= group) continue;
        const int out_head = g * group + hg * 16 + hh;
        const float* first = merged + (size_t)hh * (HD + 2);
        const size_t wave_stride = (size_t)gh * (HD + 2);
        float big = -INFINITY;
        for (int w = 0; w < n_waves; ++w) big = fmaxf(big, first[w * wave_stride]);
        float denom = 0.f, acc = 0.f;
        for (int w = 0; w < n_waves; ++w) {                  // in wave order
            const float mw = first[w * wave_stride];
            const float weight = (mw == -INFINITY) ? 0.f : exp2_fast(mw - big);
            denom = fmaf(weight, first[w * wave_stride + 1], denom);
            acc = fmaf(weight, first[w * wave_stride + 2 + d], acc);
        }
        if (n_splits == 1) {
            out[((size_t)row * n_heads + out_head) * HD + d] = f32_to_bf16(acc / denom);
        } else {                                             // part[row_index][head][split] = {m, l, O[HD]}
            float* dst = part + (((size_t)blockIdx.x * n_heads + out_head) * n_splits + split) * (HD + 2);
            if (d == 0) {
                dst[0] = big;
                dst[1] = denom;
            }
            dst[2 + d] = acc;
        }
    }
}

// Merges the splits of one (row, head): out = sum_s e^(m_s - M) O_s / sum_s e^(m_s - M) l_s, the sums
// taken in split order.  One wave: lane s first fetches split s's {m, l} (all splits at once), then
// lane d adds channel d over the splits with the weights read from LDS.
constexpr int MAX_SPLITS = 256;

__global__ __launch_bounds__(64) void attention_decode_combine_kernel(const float* __restrict__ part, bf16_t* __restrict__ out,
                                                                     const int* __restrict__ rows, int n_heads, int hd, int n_splits) {
    __shared__ float weight[MAX_SPLITS], weighted_l[MAX_SPLITS];
    constexpr int EARLY = 8;                                 // splits whose channels are asked for together with the splits' {m, l}
    const int idx = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const float* src = part + ((size_t)idx * n_heads + head) * n_splits * (hd + 2);
    // Every lane issues every load (a split or channel beyond the end is clamped into the range and not used), and the first
    // channels do not wait for the weights: one round trip to memory for up to EARLY splits, not two.
    float mine_m[MAX_SPLITS / 64], mine_l[MAX_SPLITS / 64];
#pragma unroll
    for (int i = 0; i < MAX_SPLITS / 64; ++i) {
        const int s = min(lane + 64 * i, n_splits - 1);
        mine_m[i] = src[(size_t)s * (hd + 2)];
        mine_l[i] = src[(size_t)s * (hd + 2) + 1];
    }
    float early[2][EARLY];                                   // channels lane and lane + 64 (heads of up to 128 channels)
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int s = 0; s < EARLY; ++s) early[c][s] = src[(size_t)min(s, n_splits - 1) * (hd + 2) + 2 + min(lane + 64 * c, hd - 1)];
    float big = -INFINITY;
#pragma unroll
    for (int i = 0; i < MAX_SPLITS / 64; ++i) {
        if (lane + 64 * i >= n_splits) { mine_m[i] = -INFINITY; mine_l[i] = 0.f; }
        big = fmaxf(big, mine_m[i]);
    }
    big = wave_max(big);
#pragma unroll
    for (int i = 0; i < MAX_SPLITS / 64; ++i) {
        const int s = lane + 64 * i;
        if (s < n_splits) {
            const float w = (mine_m[i] == -INFINITY) ? 0.f : exp2_fast(mine_m[i] - big);      // the splits' maxima are in units of log2 e
            weight[s] = w;
            weighted_l[s] = w * mine_l[i];
        }
    }
    __syncthreads();
    float denom = 0.f;
    for (int s = 0; s < n_splits; ++s) denom += weighted_l[s];
    const float inv = 1.0f / denom;
    const int n_early = min(n_splits, EARLY);
    for (int d = lane, c = 0; d < hd; d += 64, ++c) {
        float acc = 0.f;
        if (c < 2) {
#pragma unroll
            for (int s = 0; s < EARLY; ++s)
                if (s < n_early) acc = fmaf(weight[s], c == 0 ? early[0][s] : early[1][s], acc);
        }
#pragma unroll 8
        for (int s = c < 2 ? n_early : 0; s < n_splits; ++s) acc = fmaf(weight[s], src[(size_t)s * (hd + 2) + 2 + d], acc);
        out[((size_t)(rows ? rows[idx] : idx) * n_heads + head) * hd + d] = f32_to_bf16(acc * inv);
    }
}

}  // namespace

GI_API int gi_attention_bf16_supports(int hd, int page_size, int prompt) {
    if (page_size % 16 != 0) return 0;
    if (prompt) return hd == 32 || hd == 64 || hd == 96 || hd == 128;
    return hd == 32 || hd == 64 || hd == 96 || hd == 128 || hd == 256;
}

// tiles hold at most `rows_per_tile` rows each (64 or 128).  `paired` != 0: tiles 2w and 2w + 1 belong to one request
// and share workgroup w (a late tile of a prompt beside an early one; a tile of 0 rows fills a pair).  n_splits > 1:
// the keys of a workgroup's tiles are shared out over that many workgroups; `tile_first[i]` is the number of rows in
// the tiles before tile i, `rows` lists the tiles' rows in that order (n_rows of them), `part` has room for
// n_rows * n_heads * n_splits * (hd + 2) floats.
GI_API int gi_attention_prompt_bf16(const void* q, const void* cache, void* out, const int* tiles, int n_tiles, int rows_per_tile, int paired,
                                    const int* table, int table_stride, long page_stride, int page_size, int n_heads, int n_kv, int hd,
                                    int window, float scale, int n_splits, const int* tile_first, const int* rows, int n_rows, float* part,
                                    long part_floats, hipStream_t stream) {
    GI_REQUIRE(rows_per_tile == 64 || rows_per_tile == 128, "attention_prompt: tiles of %d rows are not supported (64 or 128)", rows_per_tile);
    GI_REQUIRE(n_tiles > 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention_prompt: bad counts (%d tiles, %d heads, %d kv heads)",
               n_tiles, n_heads, n_kv);
    GI_REQUIRE(gi_attention_bf16_supports(hd, page_size, 1), "attention_prompt: head size %d with page size %d is not supported", hd, page_size);
    GI_REQUIRE(page_stride >= 2L * n_kv * page_size * hd && page_stride % 8 == 0, "attention_prompt: bad page stride %ld", page_stride);
    GI_REQUIRE(n_heads <= 65535, "attention_prompt: too many heads");
    GI_REQUIRE(n_splits >= 1 && n_splits <= MAX_SPLITS, "attention_prompt: the number of splits %d is outside 1..%d", n_splits, MAX_SPLITS);
    GI_REQUIRE(n_splits == 1 || (tile_first && rows && part && n_rows > 0 && part_floats >= (long)n_rows * n_heads * n_splits * (hd + 2)),
               "attention_prompt: splitting needs the tiles' row offsets, their rows and scratch for the partial results");
    GI_REQUIRE(!paired || n_tiles % 2 == 0, "attention_prompt: %d tiles cannot go in pairs", n_tiles);
    // Two tiles share a workgroup of 1024 threads up to head size 64; larger heads need more registers than such a
    // workgroup leaves a thread, and take the same list tile by tile (a filling tile of 0 rows then does nothing).
    // Head size 128 takes the wide kernel (measured at 8,192 rows: 726 against 1,577 us a layer of 32 heads).  At head size 64 the
    // first kernel's pairs of tiles are the better balance while they fit the chip in one round (a workgroup of 16 waves a compute
    // unit: 2,048 rows of 32 heads take 56 against 61 us) and where few tiles share their keys out; beyond one round its time
    // doubles at once and the wide kernel's many small workgroups win (2,560 rows: 68 against 100 us; 8,192: 360 against 572).
    const bool one_round = (long)(paired ? n_tiles / 2 : n_tiles) * n_heads <= gi_compute_units();
    if (hd == 128 || (hd == 64 && n_splits == 1 && !one_round)) {
        GI_REQUIRE((long)n_tiles * n_splits <= 65535, "attention_prompt: %d tiles in %d splits are too many for one launch", n_tiles, n_splits);
        dim3 wgrid(n_heads, n_tiles * n_splits);
#define WIDE(HD, NW)                                                                                                                    \
    attention_prompt_wide_kernel<HD, NW><<<wgrid, 64 * NW, 0, stream>>>((const bf16_t*)q, (const bf16_t*)cache, (bf16_t*)out, (const int4*)tiles, table, \
                                                                       table_stride, page_stride, page_size, n_heads, n_kv, window, scale, n_splits, \
                                                                       tile_first, part, paired ? 1 : 0)
        if (hd == 64) { if (rows_per_tile == 64) WIDE(64, 2); else WIDE(64, 4); }
        else WIDE(128, 4);      // (tiles of 64 rows too: two of its waves then only load; a workgroup of two waves would need 16 loads a wave and more registers than two to a SIMD leave)
#undef WIDE
        GI_CHECK_LAUNCH("attention_prompt (wide)");
        if (n_splits > 1) {
            dim3 cgrid(n_rows, n_heads);
            attention_decode_combine_kernel<<<cgrid, 64, 0, stream>>>(part, (bf16_t*)out, rows, n_heads, hd, n_splits);
            GI_CHECK_LAUNCH("attention_prompt (combine)");
        }
        return 0;
    }
    const bool pairs = paired && hd <= 64;
    dim3 grid((pairs ? n_tiles / 2 : n_tiles) * n_splits, n_heads);
#define GO_(HD, NW, PAIR)                                                                                                               \
    attention_prompt_kernel<HD, NW, PAIR><<<grid, 128 * NW * PAIR, 0, stream>>>((const bf16_t*)q, (const bf16_t*)cache, (bf16_t*)out, (const int4*)tiles, \
                                                                                table, table_stride, page_stride, page_size, n_heads, n_kv, window, \
                                                                                scale, n_splits, tile_first, part)
#define GO(HD)                                                                                                                          \
    do {                                                                                                                                \
        if (rows_per_tile == 64) { if (pairs) GO_(HD, 2, (HD <= 64 ? 2 : 1)); else GO_(HD, 2, 1); }                                     \
        else { if (pairs) GO_(HD, 4, (HD <= 64 ? 2 : 1)); else GO_(HD, 4, 1); }                                                         \
    } while (0)
    if (hd == 32) GO(32); else if (hd == 64) GO(64); else if (hd == 96) GO(96); else GO(128);
#undef GO
#undef GO_
    GI_CHECK_LAUNCH("attention_prompt");
    if (n_splits > 1) {
        dim3 cgrid(n_rows, n_heads);
        attention_decode_combine_kernel<<<cgrid, 64, 0, stream>>>(part, (bf16_t*)out, rows, n_heads, hd, n_splits);
        GI_CHECK_LAUNCH("attention_prompt (combine)");
    }
    return 0;
}


// Waves a workgroup of the decode kernel may have for this head size.
GI_API int gi_attention_decode_max_waves(int hd) { return hd <= 128 ? 8 : 4; }

// LDS a workgroup of the decode kernel asks for: what its waves' results need, and at least so much that a compute unit holds no
// more than 16 of the kernel's waves (of 160 KB: with 20 waves a unit, which the registers allow at heads of 64 channels, contexts
// cut over several workgroups took 2 to 4 % longer a step at 40 to 72 rows).
static size_t decode_lds_bytes(int hd, int n_waves, int gh) {
    const size_t need = (size_t)n_waves * gh * (hd + 2) * sizeof(float);
    const size_t floor_ = (size_t)(160.0 * 1024.0 / (16.0 / n_waves + 0.5));
    return need > floor_ ? need : (floor_ < 64 * 1024 ? floor_ : 64 * 1024);
}

// Workgroups of `n_waves` waves of the decode kernel that a compute unit holds at once (by the kernel's registers and its LDS for
// `gh` query heads per key/value head, at most 16), as the runtime works it out; 0 if it cannot say.  The cut of the context
// over workgroups is chosen by it: workgroups beyond what the chip holds run as a second round.
GI_API int gi_attention_decode_workgroups_per_unit(int hd, int fused, int n_waves, int gh) {
    if (n_waves < 1 || n_waves > gi_attention_decode_max_waves(hd) || gh < 1 || gh > 16) return 0;
    const size_t lds = decode_lds_bytes(hd, n_waves, gh);
    int n = 0;
    hipError_t e = hipErrorInvalidValue;
#define ASK2(HD, FUSED_) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, (const void*)attention_decode_kernel<HD, FUSED_>, 64 * n_waves, lds)
#define ASK(HD) do { if (fused) ASK2(HD, true); else ASK2(HD, false); } while (0)
    if (hd == 32) ASK(32); else if (hd == 64) ASK(64); else if (hd == 96) ASK(96); else if (hd == 128) ASK(128); else if (hd == 256) ASK(256);
#undef ASK
#undef ASK2
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

// Rows `rows[0 .. n_rows)` of the step (`rows` null: rows 0 .. n_rows-1), one new position each.  Either `q` holds their rotated
// queries in bfloat16 and the cache already holds their keys and values, or (`qf` given) `qf`,
// `kf`, `vf` hold the unrotated 32-bit products, `cos_t`/`sin_t` the rotation (or null for none),
// and the kernel rotates, attends and writes the new keys and values to the cache itself (`kf`
// null: the pages belong to another layer and hold them already).  `n_waves` pieces per workgroup,
// `n_splits` workgroups per row and head group; `part` is needed for n_splits > 1.
GI_API int gi_attention_decode_bf16(const void* q, const float* qf, const float* kf, const float* vf, long ldq, long ldk, long ldv,
                                    const float* cos_t, const float* sin_t, void* cache, void* out, float* part, long part_floats,
                                    const int* rows, int n_rows, const int* pos, const int* slots, const int* table, int table_stride,
                                    long page_stride, int page_size, int n_heads, int n_kv, int hd, int window, float scale, int n_splits,
                                    int n_waves, hipStream_t stream) {
    GI_REQUIRE(n_rows > 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attention_decode: bad counts (%d rows, %d heads, %d kv heads)",
               n_rows, n_heads, n_kv);
    GI_REQUIRE(gi_attention_bf16_supports(hd, page_size, 0), "attention_decode: head size %d with page size %d is not supported", hd, page_size);
    GI_REQUIRE(page_stride >= 2L * n_kv * page_size * hd && page_stride % 8 == 0, "attention_decode: bad page stride %ld", page_stride);
    GI_REQUIRE(n_splits >= 1 && n_splits <= MAX_SPLITS, "attention_decode: the number of splits %d is outside 1..%d", n_splits, MAX_SPLITS);
    GI_REQUIRE(n_waves >= 1 && n_waves <= gi_attention_decode_max_waves(hd), "attention_decode: %d waves per workgroup are outside 1..%d",
               n_waves, gi_attention_decode_max_waves(hd));
    GI_REQUIRE(n_splits == 1 || (part != nullptr && part_floats >= (long)n_rows * n_heads * n_splits * (hd + 2)), "attention_decode: scratch too small");
    GI_REQUIRE((q != nullptr) != (qf != nullptr), "attention_decode: give either rotated bfloat16 queries or the unrotated 32-bit products");
    if (qf) {
        GI_REQUIRE((kf == nullptr) == (vf == nullptr), "attention_decode: keys and values come together");
        GI_REQUIRE((cos_t == nullptr) == (sin_t == nullptr), "attention_decode: cos and sin must both be given or both be absent");
        GI_REQUIRE(ldq % 4 == 0 && ((uintptr_t)qf & 15) == 0 && (!kf || (ldk % 4 == 0 && ((uintptr_t)kf & 15) == 0)) &&
                       (!cos_t || ((((uintptr_t)cos_t | (uintptr_t)sin_t) & 15) == 0)),
                   "attention_decode: the 32-bit inputs must be 16-byte aligned with row strides that are multiples of 4");
        GI_REQUIRE(ldq >= (long)n_heads * hd && (!kf || (ldk >= (long)n_kv * hd && ldv >= (long)n_kv * hd)), "attention_decode: row strides too small");
    }
    const int group = n_heads / n_kv, hg = (group + 15) / 16, gh = group < 16 ? group : 16;
    GI_REQUIRE(n_kv * hg <= 65535, "attention_decode: too many heads");
    size_t lds = (size_t)n_waves * gh * (hd + 2) * sizeof(float);
    while (lds > 64 * 1024 && n_waves > 1) {                  // many wide heads: fewer waves so that their results fit
        n_waves /= 2;
        lds = (size_t)n_waves * gh * (hd + 2) * sizeof(float);
    }
    GI_REQUIRE(lds <= 64 * 1024, "attention_decode: %d heads of size %d per key/value head do not fit", gh, hd);
    lds = decode_lds_bytes(hd, n_waves, gh);
    dim3 grid(n_rows, n_kv * hg, n_splits);
#define GO2(HD, FUSED_)                                                                                                                    \
    attention_decode_kernel<HD, FUSED_><<<grid, 64 * n_waves, lds, stream>>>((const bf16_t*)q, qf, kf, vf, ldq, ldk, ldv, cos_t, sin_t,   \
                                                                             (bf16_t*)cache, part, (bf16_t*)out, rows, pos, slots, table, \
                                                                             table_stride, page_stride, page_size, n_heads, n_kv, window,  \
                                                                             scale, n_splits, gh)
#define GO(HD)                    \
    do {                          \
        if (qf) GO2(HD, true);    \
        else GO2(HD, false);      \
    } while (0)
    if (hd == 32) GO(32); else if (hd == 64) GO(64); else if (hd == 96) GO(96); else if (hd == 128) GO(128); else GO(256);
#undef GO
#undef GO2
    GI_CHECK_LAUNCH("attention_decode");
    if (n_splits > 1) {
        dim3 cgrid(n_rows, n_heads);
        attention_decode_combine_kernel<<<cgrid, 64, 0, stream>>>(part, (bf16_t*)out, rows, n_heads, hd, n_splits);
        GI_CHECK_LAUNCH("attention_decode (combine)");
    }
    return 0;
}
