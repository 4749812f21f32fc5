// C[m, n] (=|+=) sum_k A[m, k] * W[n, k] with bfloat16 operands on the matrix cores, 32-bit sums.
//
// Both operands are row-major with k contiguous, so each lane's operand of a matrix instruction is
// one 16-byte load of 8 consecutive k.  Five kernels:
//
//   pingpong  large prompt-sized products (256 x 256 tiles for most of the compute units): operands loaded
//           from global memory straight into two LDS stages; the workgroup's eight waves form two
//           groups that take turns at reading LDS and at the matrix instructions.
//   piped   the other products of 128 rows or more (K a multiple of 64): tiles of 128 x 128,
//           operands loaded from global memory straight into a ring of LDS stages, several
//           blocks of k in flight; v_mfma_f32_32x32x16_bf16.
//   tiled   the other shapes above 64 rows: a BM x 128 tile of C per workgroup of 4 waves,
//           operands staged through registers into LDS in k-blocks of 64.
//   skinny  up to 128 rows of A: weights stream from HBM straight into registers and are used
//           once, activations go through LDS; v_mfma_f32_16x16x32_bf16.  Wide outputs are
//           finished by the workgroup that sees all of k; for narrow ones k is split over
//           workgroups and the partial sums are added in a fixed order by a second kernel.
//   slim    at most 16 rows of A (decode): a workgroup of 8 waves owns 16 (or 2 x 16) weight
//           rows, its waves take interleaved blocks of k and add their sums through LDS in a
//           fixed order, so one launch does the whole product and its epilogue.
//
// The "gated" epilogue serves SwiGLU: the weight is [gate; up] interleaved in groups of 16 rows
// (16 gate rows, the 16 up rows of the same outputs, and so on), and the output column c of a
// pair of groups is silu(gate_c) * up_c, stored as bfloat16: the stacked product never reaches
// memory.
//
// Requirements (checked on the host): K a multiple of 8, rows of A and W 16-byte aligned.  The
// output is float32 (stored or added onto what is there) or bfloat16 (stored).
#include "common.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

enum Epilogue : int { EPI_STORE_F32 = 0, EPI_ADD_F32 = 1, EPI_STORE_BF16 = 2, EPI_GATED_BF16 = 3, EPI_QKV_ROPE = 4 };

__device__ __forceinline__ float silu_gate(float g, float u) { return (g * (1.0f / (1.0f + expf(-g)))) * u; }
// The same with the hardware's exp2 and reciprocal (each within a unit or two in the last place of 32 bits): for results
// that are rounded to bfloat16's 8 bits at once.  The exact form above costs some thirty vector instructions a value,
// which in a prompt-sized product's epilogue is a tenth of the kernel.
__device__ __forceinline__ float silu_gate_fast(float g, float u) {
    return (g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.4426950408889634f))) * u;
}

__device__ __forceinline__ uint4 load16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }

template <int EPI>
__device__ __forceinline__ void write_out(void* C, size_t o, float v) {
    if constexpr (EPI == EPI_STORE_F32) ((float*)C)[o] = v;
    else if constexpr (EPI == EPI_ADD_F32) ((float*)C)[o] += v;
    else ((bf16_t*)C)[o] = f32_to_bf16(v);
}

// ----------------------------------------------------------------- an RMS norm between two products of a few rows
// The norm of a row x is g * x * r with r = rsqrt(mean(x^2) + eps), and r, one number a row, commutes with the product that reads
// the normed row.  A product that adds onto the rows x also writes g * x of the sums it has just made, in bfloat16, and what its
// columns give to the sum of squares of every row, one number per row and piece of the row (`NormOut`); the product that reads
// those rows multiplies its results by r, which it gets from those numbers, added in a fixed order (`NormIn`).  No kernel for
// the norm, no second pass over the rows.
struct NormOut {                 // for a product that adds onto x: all null if it does not hand the norm on
    const float* g;              // the norm's weights [N]
    bf16_t* scaled;              // out: g * x, [M, ld]
    long ld;
    float* squares;              // out: [M, parts]
};
struct NormIn {                  // for a product whose rows A are g * x without r: squares null if they are ready-made rows
    const float* squares;        // [M, parts]
    int parts;
    float eps;
    int dim;                     // r = rsqrt(sum / dim + eps)
};

// Where an attention layer wants the sums of its q/k/v product (columns: n_heads * hd queries, n_kv * hd keys, n_kv * hd values):
// queries rotated into q_out, keys rotated and values as they are into the page table[slot][pos / page_size] at place
// pos % page_size (pairs (i, i + hd/2): a' = a cos - b sin, b' = a sin + b cos; the page's layout as the attention kernels read
// it: keys [kv_head][place][hd], then values [kv_head][hd][place]).
struct RopeStore {
    const float* cos_t;          // [M, hd/2], or null with sin_t: no rotation
    const float* sin_t;
    const int* pos;              // [M]
    const int* slot;             // [M]
    const int* table;
    int table_stride;
    bf16_t* q_out;               // [M, n_heads * hd]
    bf16_t* cache;
    long page_stride;
    int page_size, n_heads, n_kv, hd;
};


constexpr int PIPED_MAX_PARTS = 64;            // pieces of a row's sum of squares that a kernel for more than 128 rows reads

// r = rsqrt(mean square + eps) of the `rows` rows from `first` on into `scales` (LDS), by a workgroup of NT threads; rows
// beyond M get 1.  The caller puts a barrier before the use.
template <int NT>
__device__ __forceinline__ void tile_row_scales(float* scales, const NormIn& n, int first, int rows, int M) {
    for (int row = threadIdx.x; row < rows; row += NT) {
        float sum = 0.f;
        if (first + row < M)
            for (int p = 0; p < n.parts; ++p) sum += n.squares[(size_t)(first + row) * n.parts + p];
        scales[row] = first + row < M ? 1.0f / sqrtf(sum / (float)n.dim + n.eps) : 1.0f;
    }
}

// The factor of one row: rsqrt(mean square + eps) from the pieces of its sum of squares, added in their order.  The first eight
// pieces are asked for at once, by every lane (an index beyond the pieces is clamped and what it brings not added): a caller can
// ask early (`row_pieces`) and finish where the factor is needed (`row_scale_from`), with its other loads in flight in between.
struct RowPieces {
    float v[8];
};
__device__ __forceinline__ RowPieces row_pieces(const NormIn& n, int row) {
    RowPieces r;
    const float* pieces = n.squares + (size_t)row * n.parts;
#pragma unroll
    for (int u = 0; u < 8; ++u) r.v[u] = pieces[min(u, n.parts - 1)];
    return r;
}
__device__ __forceinline__ float row_scale_from(const NormIn& n, int row, const RowPieces& r) {
    float sum = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < n.parts) sum += r.v[u];
    for (int p = 8; p < n.parts; ++p) sum += n.squares[(size_t)row * n.parts + p];
    return 1.0f / sqrtf(sum / (float)n.dim + n.eps);
}
__device__ __forceinline__ float row_scale_of(const NormIn& n, int row) { return row_scale_from(n, row, row_pieces(n, row)); }

// Where the rows of a tile of 128 go in the cache: per row the page's offset and the place in the page, and per group of
// eight rows whether they are eight consecutive positions of one request that begin at a multiple of eight (rows of a prompt).
struct TilePlaces {
    long page[128];              // page * page_stride
    int place[128];
    int run[16];
};

// Filled by the workgroup's first 128 threads (each row's page is two loads that depend on each other: done once per row here,
// not once per piece of a row); the caller puts a barrier before the use.
__device__ __forceinline__ void tile_places(TilePlaces& t, int m0, int M, const RopeStore& rs) {
    const int row = threadIdx.x;
    if (row >= 128) return;
    const int m = min(m0 + row, M - 1), p = rs.pos[m], slot = rs.slot[m];
    t.page[row] = (long)rs.table[(size_t)slot * rs.table_stride + p / rs.page_size] * rs.page_stride;
    t.place[row] = p % rs.page_size;
    // the eight lanes of a group agree on the first row's slot and position
    const int first = row & ~7, p0 = __shfl(p, first & 63, 64), slot0 = __shfl(slot, first & 63, 64);
    const bool fits = m0 + row < M && slot == slot0 && p == p0 + (row & 7);
    const unsigned long long all = __ballot(fits);
    if ((row & 7) == 0) t.run[row >> 3] = ((all >> (row & 63)) & 0xffull) == 0xffull && p % 8 == 0 && rs.page_size % 8 == 0;
}

// A tile of 128 x 128 sums of a q/k/v product, row-major in LDS, goes where `RopeStore` says.  Whole heads lie inside the
// tile (hd divides 128, the tile starts at a multiple of 128 columns), so the other half of every pair is in LDS too.  Queries
// and keys: a thread takes four pairs of a row at a time, whose two halves leave as 8-byte pieces of contiguous rows; the
// cosines and sines of four such items are asked for at once.  Values are stored transposed in their pages ([hd][place]),
// so they are taken column by column, eight rows at a time: where those are a run of eight positions (`TilePlaces`), they
// leave as one 16-byte piece, otherwise one by one.
template <int NT>
__device__ __forceinline__ void qkv_tile_rope_store(const float* tile, const TilePlaces& at, int m0, int n0, int M, int N, const RopeStore& rs) {
    const int a_dim = rs.n_heads * rs.hd, kv_dim = rs.n_kv * rs.hd, half = rs.hd / 2;
    if (n0 < a_dim + kv_dim && rs.cos_t != nullptr) {
        // An item is four pairs (i, i + hd/2) of a row: two pieces of four columns, hd/2 apart, that share their cosines and sines.
        constexpr int BATCH = 4;
        const int per_head = rs.hd / 8;                                          // items of a head; 16 items a row of the tile
        for (int e0 = threadIdx.x; e0 < 128 * 16; e0 += NT * BATCH) {
            float4 cc[BATCH], ss[BATCH];
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                const int e = min(e0 + b * NT, 128 * 16 - 1), m = min(m0 + (e >> 4), M - 1), kq = (e & 15) % per_head;
                cc[b] = *reinterpret_cast<const float4*>(rs.cos_t + (size_t)m * half + kq * 4);
                ss[b] = *reinterpret_cast<const float4*>(rs.sin_t + (size_t)m * half + kq * 4);
            }
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                const int e = e0 + b * NT, row = e >> 4, item = e & 15, m = m0 + row;
                const int c_lo = (item / per_head) * rs.hd + (item % per_head) * 4, col = n0 + c_lo;      // in the tile; in the product
                if (e >= 128 * 16 || m >= M || col >= a_dim + kv_dim) continue;
                const float4 a = *reinterpret_cast<const float4*>(tile + row * 128 + c_lo);
                const float4 o = *reinterpret_cast<const float4*>(tile + row * 128 + c_lo + half);
                const uint2 lo = {f32x2_to_bf16x2(a.x * cc[b].x - o.x * ss[b].x, a.y * cc[b].y - o.y * ss[b].y),
                                  f32x2_to_bf16x2(a.z * cc[b].z - o.z * ss[b].z, a.w * cc[b].w - o.w * ss[b].w)};
                const uint2 hi = {f32x2_to_bf16x2(a.x * ss[b].x + o.x * cc[b].x, a.y * ss[b].y + o.y * cc[b].y),
                                  f32x2_to_bf16x2(a.z * ss[b].z + o.z * cc[b].z, a.w * ss[b].w + o.w * cc[b].w)};
                const bool key = col >= a_dim;
                const int c = key ? col - a_dim : col;                           // the column among the queries, or the keys
                bf16_t* dst = key ? rs.cache + at.page[row] + ((size_t)(c / rs.hd) * rs.page_size + at.place[row]) * rs.hd + c % rs.hd
                                  : rs.q_out + (size_t)m * a_dim + c;
                *reinterpret_cast<uint2*>(dst) = lo;
                *reinterpret_cast<uint2*>(dst + half) = hi;
            }
        }
    } else if (n0 < a_dim + kv_dim) {                                            // no rotation: the sums as they are
        for (int e = threadIdx.x; e < 128 * 32; e += NT) {
            const int row = e >> 5, c4 = (e & 31) * 4, m = m0 + row, col = n0 + c4;
            if (m >= M || col >= a_dim + kv_dim) continue;
            const float4 v = *reinterpret_cast<const float4*>(tile + row * 128 + c4);
            const uint2 packed = {f32x2_to_bf16x2(v.x, v.y), f32x2_to_bf16x2(v.z, v.w)};
            const bool key = col >= a_dim;
            const int c = key ? col - a_dim : col;
            bf16_t* dst = key ? rs.cache + at.page[row] + ((size_t)(c / rs.hd) * rs.page_size + at.place[row]) * rs.hd + c % rs.hd
                              : rs.q_out + (size_t)m * a_dim + c;
            *reinterpret_cast<uint2*>(dst) = packed;
        }
    }
    if (n0 + 128 > a_dim + kv_dim) {
        const size_t v_plane = (size_t)rs.n_kv * rs.page_size * rs.hd;           // from a page's keys to its values
        const bool aligned = ((uintptr_t)rs.cache & 15) == 0 && rs.page_stride % 8 == 0;
        for (int e = threadIdx.x; e < 16 * 128; e += NT) {
            const int rows = (e >> 7) * 8, c1 = e & 127, m = m0 + rows, col = n0 + c1;
            if (m >= M || col >= N || col < a_dim + kv_dim) continue;
            const size_t c = (size_t)(col - a_dim - kv_dim) * rs.page_size;     // (h * hd + kk) * page_size
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = tile[(rows + i) * 128 + c1];
            if (aligned && at.run[e >> 7]) {
                const uint4 packed = {f32x2_to_bf16x2(v[0], v[1]), f32x2_to_bf16x2(v[2], v[3]), f32x2_to_bf16x2(v[4], v[5]), f32x2_to_bf16x2(v[6], v[7])};
                *reinterpret_cast<uint4*>(rs.cache + at.page[rows] + v_plane + c + at.place[rows]) = packed;
            } else {
                const int last = min(7, M - 1 - m);
                for (int i = 0; i <= last; ++i) rs.cache[at.page[rows + i] + v_plane + c + at.place[rows + i]] = f32_to_bf16(v[i]);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------ tiled
constexpr int BN = 128, BK = 64, LDS_STRIDE = BK + 8;     // +8 bf16 (16 bytes) of padding: conflict-free 16-byte reads

template <int BM, int EPI>
__global__ __launch_bounds__(256) void gemm_bf16_tiled_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ C,
                                                             int M, int N, int K, long lda, long ldw, long ldc) {
    constexpr int WM = BM / 2;                 // rows of a wave's tile (waves sit 2 x 2)
    constexpr int TM = WM / 32, TN = 2;        // 32x32 tiles per wave
    constexpr int A_CHUNKS = BM * BK / 8 / 256, W_CHUNKS = BN * BK / 8 / 256;   // 16-byte chunks per thread
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) bf16_t Ws[BN * LDS_STRIDE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * 64;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = floatx16{};

    uint4 a_reg[A_CHUNKS], w_reg[W_CHUNKS];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int c = 0; c < A_CHUNKS; ++c) {
            const int e = tid + 256 * c, row = e / (BK / 8), kc = (e % (BK / 8)) * 8;
            const int m = m0 + row, k = k0 + kc;
            a_reg[c] = (m < M && k < K) ? load16(A + (size_t)m * lda + k) : uint4{0, 0, 0, 0};
        }
#pragma unroll
        for (int c = 0; c < W_CHUNKS; ++c) {
            const int e = tid + 256 * c, row = e / (BK / 8), kc = (e % (BK / 8)) * 8;
            const int n = n0 + row, k = k0 + kc;
            w_reg[c] = (n < N && k < K) ? load16(W + (size_t)n * ldw + k) : uint4{0, 0, 0, 0};
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int c = 0; c < A_CHUNKS; ++c) {
            const int e = tid + 256 * c, row = e / (BK / 8), kc = (e % (BK / 8)) * 8;
            *reinterpret_cast<uint4*>(&As[row * LDS_STRIDE + kc]) = a_reg[c];
        }
#pragma unroll
        for (int c = 0; c < W_CHUNKS; ++c) {
            const int e = tid + 256 * c, row = e / (BK / 8), kc = (e % (BK / 8)) * 8;
            *reinterpret_cast<uint4*>(&Ws[row * LDS_STRIDE + kc]) = w_reg[c];
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < K; k0 += BK) {
        __syncthreads();                       // everyone has finished reading the previous block
        stash();
        __syncthreads();
        if (k0 + BK < K) fetch(k0 + BK);       // in flight while the products below run
        const int r = lane & 31, kq = (lane >> 5) * 8;
#pragma unroll
        for (int ks = 0; ks < BK; ks += 16) {
            bf16x8 a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = as_bf16x8(*reinterpret_cast<const uint4*>(&As[(wm + i * 32 + r) * LDS_STRIDE + ks + kq]));
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = as_bf16x8(*reinterpret_cast<const uint4*>(&Ws[(wn + j * 32 + r) * LDS_STRIDE + ks + kq]));
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    }
    // Element v of a lane's 32x32 result: row 8*(v/4) + 4*(lane/32) + v%4, column lane%32.
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v & 3);
                const int n = n0 + wn + j * 32 + (lane & 31);
                if constexpr (EPI == EPI_GATED_BF16) {
                    // columns 32b .. 32b+15 are gates, 32b+16 .. 32b+31 the ups of outputs 16b .. 16b+15
                    const float up = __shfl_xor(acc[i][j][v], 16, 64);
                    if ((lane & 16) == 0 && m < M && n < N)
                        ((bf16_t*)C)[(size_t)m * ldc + (n >> 5) * 16 + (lane & 15)] = f32_to_bf16(silu_gate(acc[i][j][v], up));
                } else {
                    if (m < M && n < N) write_out<EPI>(C, (size_t)m * ldc + n, acc[i][j][v]);
                }
            }
}

// ------------------------------------------------------------------------------------------ piped
// The same product for large shapes, with the operands going from global memory straight into LDS
// (global_load_lds_dwordx4: no registers in between) through a ring of blocks of 64 k, so that
// several blocks are in flight while one is multiplied.  Workgroup: 4 waves (2 x 2), a tile of
// BM x BN; a wave owns (BM/2) x (BN/2).  A stage holds BM rows of A, then BN rows of W, 128 bytes
// (a cache line) each; a wave-wide load fills 8 rows.  The 16-byte chunk c of row `row` lies at
// chunk position c ^ ((row >> 1) & 7): the loads write LDS contiguously, and the 16-byte reads
// of 16 consecutive rows (what one clock serves: 64 banks of 4 bytes) hit 16 different slots,
// without padding (a load cannot pad).  Needs K % 64 == 0; rows beyond M or N are read from the
// last valid row and their results are dropped.  With few tiles, k is split over the grid's z: each
// workgroup then writes the sums of its share to its own [M, N] slab of 32-bit partial results, and the
// reduce kernel below adds the slabs in order and applies the epilogue.
constexpr int PK = 64;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int EPI>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void gemm_bf16_piped_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ C,
                                                             int M, int N, int K, long lda, long ldw, long ldc, int k_per_split,
                                                             long split_stride, NormIn norm_in, RopeStore rope, NormOut norm_out) {
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
    constexpr int ROWS = BM + BN, STAGE_BYTES = ROWS * 128, LOADS = ROWS / 8 / (WAVES_M * WAVES_N);      // loads per wave and stage
    static_assert(ROWS % (8 * WAVES_M * WAVES_N) == 0, "the rows of a stage must divide among the waves' loads");
    static_assert(STAGES >= 2 && STAGES <= 4, "the counted waits below cover 2 to 4 stages");
    extern __shared__ __attribute__((aligned(16))) unsigned char ring[];               // STAGES * STAGE_BYTES
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    const bf16_t* src[LOADS];                  // this lane's source of each of its wave's loads, at k = 0
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int row = (wave * LOADS + i) * 8 + (lane >> 3), c = (lane & 7) ^ ((row >> 1) & 7);
        src[i] = row < BM ? A + (size_t)min(m0 + row, M - 1) * lda + 8 * c : W + (size_t)min(n0 + row - BM, N - 1) * ldw + 8 * c;
        src[i] += (size_t)blockIdx.z * k_per_split;           // this workgroup's share of k (all of it without a split)
    }
    if (split_stride) C = (float*)C + (size_t)blockIdx.z * split_stride;       // ... and its own partial result
    // The loads are written as assembly so that the compiler does not see them: it would otherwise wait for all of
    // them before every read of LDS and at every barrier, and nothing would stay in flight.  What orders them against
    // the reads is below: the counted wait, then the barrier.
    const unsigned ring_base = (unsigned)(size_t)(lds_ptr_t)ring;
    auto issue = [&](int slot, int k0) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const unsigned dst = __builtin_amdgcn_readfirstlane(ring_base + slot * STAGE_BYTES + (wave * LOADS + i) * 1024);   // the wave's 1 KB; lane l lands at + 16 l
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(dst), "v"(src[i] + k0) : "memory", "m0");
        }
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = floatx16{};

    const int n_k = min(K - (int)blockIdx.z * k_per_split, k_per_split) / PK;
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < n_k) issue(s, s * PK);
    const int r = lane & 31, swz = (r >> 1) & 7;
    const unsigned char* a_rows = ring + (wm + r) * 128;
    const unsigned char* b_rows = ring + (BM + wn + r) * 128;
    for (int it = 0; it < n_k; ++it) {
        // this wave's part of block `it` has landed when at most the loads of the blocks after it are outstanding
        const int ahead = min(n_k - 1 - it, STAGES - 2);
        if (ahead >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LOADS) : "memory");
        else if (ahead == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();          // everyone's part has landed, and everyone has finished block it-1
        asm volatile("" ::: "memory");
        if (it + STAGES - 1 < n_k) issue((it + STAGES - 1) % STAGES, (it + STAGES - 1) * PK);      // into the slot of block it-1
        const int stage_off = (it % STAGES) * STAGE_BYTES;
        // operands of the next 16 k are read while the products of these 16 run
        bf16x8 a[2][TM], b[2][TN];
        auto read_operands = [&](int ks, bf16x8* av, bf16x8* bv) {
            const int chunk = (((ks >> 3) + (lane >> 5)) ^ swz) * 16;
#pragma unroll
            for (int i = 0; i < TM; ++i) av[i] = as_bf16x8(*reinterpret_cast<const uint4*>(a_rows + stage_off + i * 32 * 128 + chunk));
#pragma unroll
            for (int j = 0; j < TN; ++j) bv[j] = as_bf16x8(*reinterpret_cast<const uint4*>(b_rows + stage_off + j * 32 * 128 + chunk));
        };
        read_operands(0, a[0], b[0]);
#pragma unroll
        for (int step = 0; step < PK / 16; ++step) {
            if (step + 1 < PK / 16) read_operands(16 * (step + 1), a[(step + 1) & 1], b[(step + 1) & 1]);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[step & 1][i], b[step & 1][j], acc[i][j], 0, 0, 0);
        }
    }
    // Element v of a lane's 32x32 result: row 8*(v/4) + 4*(lane/32) + v%4, column lane%32.
    if constexpr (EPI == EPI_QKV_ROPE) {
        // The sums of a q/k/v product do not go out as they are: the tile is laid into LDS (the ring is free once everyone has
        // read the last block), scaled by a norm handed on if there is one, and leaves rotated, queries to their rows, keys and
        // values to their pages.
        static_assert(BM == 128 && BN == 128 && STAGES * STAGE_BYTES >= 128 * 128 * 4, "the tile in LDS is 128 x 128 floats");
        __shared__ float row_scale[128];
        __shared__ TilePlaces places;
        const bool scaled_rows = norm_in.squares != nullptr;
        if (scaled_rows) tile_row_scales<64 * WAVES_M * WAVES_N>(row_scale, norm_in, m0, 128, M);
        if (n0 + 128 > rope.n_heads * rope.hd) tile_places(places, m0, M, rope);       // (a tile of queries alone needs no pages)
        __syncthreads();
        float* tile = reinterpret_cast<float*>(ring);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = wm + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v & 3);
                    tile[row * 128 + wn + j * 32 + (lane & 31)] = scaled_rows ? acc[i][j][v] * row_scale[row] : acc[i][j][v];
                }
        __syncthreads();
        qkv_tile_rope_store<64 * WAVES_M * WAVES_N>(tile, places, m0, n0, M, N, rope);
        return;
    }
    if constexpr (EPI == EPI_ADD_F32 && BM == 128 && BN == 128 && STAGES * STAGE_BYTES >= 128 * 128 * 4) {
        if (norm_out.scaled != nullptr) {
            // The sums go onto 32-bit rows whose next reader is a norm: the tile is laid into LDS (the ring is free once everyone
            // has read the last block) and leaves row by row, 32 threads a row with four columns each: the rows' new values, the
            // same times the norm's weights in bfloat16, and the tile's piece of every row's sum of squares (N is a multiple of 128).
            constexpr int NT = 64 * WAVES_M * WAVES_N, PASSES = 128 / (NT / 32);
            // What the sums are added onto is asked for first, all of a thread's rows at once (a row beyond M is clamped and not
            // written): read row by row behind the tile, it was a round trip to memory a row, eight in a row at the end of the kernel.
            const int c4 = (tid & 31) * 4;
            const float4 g = *reinterpret_cast<const float4*>(norm_out.g + n0 + c4);
            float4 old[PASSES];
#pragma unroll
            for (int it = 0; it < PASSES; ++it)
                old[it] = *reinterpret_cast<const float4*>((const float*)C + (size_t)min(m0 + (tid >> 5) + it * (NT / 32), M - 1) * ldc + n0 + c4);
            __syncthreads();
            float* tile = reinterpret_cast<float*>(ring);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        tile[(wm + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v & 3)) * 128 + wn + j * 32 + (lane & 31)] = acc[i][j][v];
            __syncthreads();
#pragma unroll
            for (int it = 0; it < PASSES; ++it) {
                const int row = (tid >> 5) + it * (NT / 32), m = m0 + row;
                float square = 0.f;
                if (m < M) {
                    const float4 t = *reinterpret_cast<const float4*>(tile + row * 128 + c4);
                    float4* at = reinterpret_cast<float4*>((float*)C + (size_t)m * ldc + n0 + c4);
                    float4 x = old[it];
                    x.x += t.x; x.y += t.y; x.z += t.z; x.w += t.w;
                    *at = x;
                    *reinterpret_cast<uint2*>(norm_out.scaled + (size_t)m * norm_out.ld + n0 + c4) =
                        uint2{f32x2_to_bf16x2(g.x * x.x, g.y * x.y), f32x2_to_bf16x2(g.z * x.z, g.w * x.w)};
                    square = x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
                }
#pragma unroll
                for (int off = 16; off > 0; off >>= 1) square += __shfl_xor(square, off, 64);
                if ((tid & 31) == 0 && m < M) norm_out.squares[(size_t)m * gridDim.x + blockIdx.x] = square;
            }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm + i * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v & 3);
                const int n = n0 + wn + j * 32 + (lane & 31);
                if constexpr (EPI == EPI_GATED_BF16) {
                    const float up = __shfl_xor(acc[i][j][v], 16, 64);
                    if ((lane & 16) == 0 && m < M && n < N)
                        ((bf16_t*)C)[(size_t)m * ldc + (n >> 5) * 16 + (lane & 15)] = f32_to_bf16(silu_gate(acc[i][j][v], up));
                } else if constexpr (EPI != EPI_QKV_ROPE) {
                    if (m < M && n < N) write_out<EPI>(C, (size_t)m * ldc + n, acc[i][j][v]);
                }
            }
}

// --------------------------------------------------------------------------------------- pingpong
// A 256 x 256 tile and two LDS stages of 64 k, filled straight from global memory like the piped kernel's, with another
// order of work inside the workgroup.  Its eight waves form two groups of four, and a compute unit's four SIMDs hold
// one wave of each group.  A group alternates between a phase R in which it reads the operands of a block's 64 k from
// LDS into registers (and issues loads that refill the stages) and a phase M in which it does nothing but matrix
// instructions on them; a workgroup barrier ends every phase, and one group runs a barrier behind the other, so at any
// time one group reads while the other multiplies: on every SIMD the matrix unit always has a wave that has its
// operands at hand, instead of two waves that read together and then multiply together.
//
//   barrier number      0        1        2        3        4
//   group 0:    R(0)  |  M(0)  |  R(1)  |  M(1)  |  R(2)  | ...
//   group 1:          |  R(0)  |  M(0)  |  R(1)  |  M(1)  | ...        R(b), M(b): the phases of block b
//
// Every wave passes the same number of barriers: group 1's one ahead is matched by one more of group 0 at the end.
// Who loads which rows of which block when is said where the loads are set up, below.  Measured (cycle stamps per
// phase): M takes 1,080 clocks for its 32 matrix instructions, R 500 for its 24 reads plus what its 8 loads take to
// issue, which is what bounds the interval between two barriers (1,700 clocks); a load costs the wave that issues it
// 23 clocks when nothing else runs and 70 to 140 here, wherever in the two phases it is put.
template <int BN, int EPI>
__global__ __launch_bounds__(512) void gemm_bf16_pingpong_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ C,
                                                                int M, int N, int K, long lda, long ldw, long ldc, NormIn norm_in) {
    static_assert(BN == 256, "the sharing of the loads below is written for 256 x 256 tiles");
    constexpr int BM = 256, WAVES = 8, WM = 64, WN = BN / 2, TM = WM / 32, TN = WN / 32;
    constexpr int ROWS = BM + BN, STAGE_BYTES = ROWS * 128, LOADS = ROWS / 8 / WAVES;      // a wave-wide load fills 8 rows of 128 bytes
    extern __shared__ __attribute__((aligned(16))) unsigned char ring[];               // 2 * STAGE_BYTES
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), group = wave >> 2;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;

    // Row `row` of a stage (0 .. 255: rows of A, 256 .. 511: rows of W): where this lane's 16 bytes of it lie, in bytes from the
    // tile's first row of A or of W at k = 0.  The piece c of a row lies at piece position c ^ ((row >> 1) & 7): see the piped kernel.
    // A load's address is a scalar base (the tile's first row, advanced by the block's k) plus this offset, so that issuing one
    // needs no vector instruction: those wait behind a matrix instruction that is under way.
    const bf16_t* a_tile = A + (size_t)m0 * lda;
    const bf16_t* w_tile = W + (size_t)n0 * ldw;
    auto source = [&](int row) -> unsigned {
        const int c = (lane & 7) ^ ((row >> 1) & 7);
        return row < BM ? (unsigned)(((size_t)min(row, M - 1 - m0) * lda + 8 * c) * 2) : (unsigned)(((size_t)min(row - BM, N - 1 - n0) * ldw + 8 * c) * 2);
    };
    const unsigned ring_base = (unsigned)(size_t)(lds_ptr_t)ring;
    auto load_rows = [&](unsigned from, int first_row, int block) {                  // 8 rows from `first_row` (the same for the wave) of block `block`
        const unsigned dst = ring_base + (block & 1) * STAGE_BYTES + first_row * 128;
        const bf16_t* base = (first_row < BM ? a_tile : w_tile) + block * PK;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(from), "s"(base) : "memory", "m0");
    };
    // What a wave loads, 8 loads of 1 KB a block.  The memory pipeline takes such a load every 23 clocks or so, 64 of them a block:
    // three quarters of the time the block's matrix instructions take; and a wave that issues one is held for as long as the loads
    // of its workgroup that are ahead of it take, with its next instructions behind it.  So the loads are issued by the group that
    // reads, behind its reads of LDS (while it would wait for those and then for the other group's matrix instructions anyway), and
    // they are spread evenly over the block's two barrier intervals.  Which rows can be loaded when follows from who reads them:
    //   group 0 reads the first 128 rows of A and all of W, in the first interval of a block; group 1 the last 128 rows of A and all of W, in the second.
    //   group 0, R(b):  the rows of W of block b + 1           (their stage fell free at the barrier before, when group 1 had read block b - 1)
    //   group 1, R(b):  the first 128 rows of A of block b + 2 (group 0 has just read those of block b) and the last 128 of block b + 1
    // Every wave waits for its own loads at the end of its M phase; the rows are read two barriers later or more.
    const int turn = wave & 3;
    const int first_row = group == 0 ? BM + turn * 64 : turn * 32;                     // of the wave's load 0; group 1's loads 4 .. 7 lie 128 rows further
    auto row_of = [&](int i) { return first_row + (group == 0 ? 8 * i : 8 * (i & 3) + 128 * (i >> 2)); };
    unsigned src[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) src[i] = source(row_of(i) + (lane >> 3));
    const int n_k = K / PK;
    auto load_one = [&](int i, int block) {                                         // this wave's load i during R(block)
        const int of_block = group == 0 ? block + 1 : (i < 4 ? block + 2 : block + 1);
        if (of_block < n_k) load_rows(src[i], row_of(i), of_block);
    };
    auto phase_barrier = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = floatx16{};

    // to begin with: all of block 0, and the first 128 rows of A of block 1 (which the R phase before block 0 would have sent for)
#pragma unroll
    for (int i = 0; i < LOADS; ++i) load_rows(source((wave * LOADS + i) * 8 + (lane >> 3)), (wave * LOADS + i) * 8, 0);
    if (n_k > 1) {
#pragma unroll
        for (int i = 0; i < 2; ++i) load_rows(source((wave * 2 + i) * 8 + (lane >> 3)), (wave * 2 + i) * 8, 1);
    }
    // With a norm handed on (the gated product: the rows of A are g * x, and the results lack the rows' rsqrt(mean square + eps)),
    // the tile's 256 rows' factors are worked out once, a thread a row (16-byte reads of the row's pieces where they allow it: a lane
    // that asked for its rows' pieces one by one cost the kernel 18 us at 16 pieces), and wait in LDS for the epilogue (asked for behind the first block's loads; the
    // barriers of the loop lie between this write and the epilogue's reads).
    __shared__ float row_scale[EPI == EPI_GATED_BF16 ? BM : 1];
    if constexpr (EPI == EPI_GATED_BF16) {
        if (norm_in.squares != nullptr) {
            if (tid < BM) {
                const float* pieces = norm_in.squares + (size_t)min(m0 + tid, M - 1) * norm_in.parts;
                float sum = 0.f;
                if ((norm_in.parts & 3) == 0 && ((uintptr_t)norm_in.squares & 15) == 0) {
                    for (int p = 0; p < norm_in.parts; p += 4) {
                        const float4 v = *reinterpret_cast<const float4*>(pieces + p);
                        sum += v.x; sum += v.y; sum += v.z; sum += v.w;
                    }
                } else {
                    for (int p = 0; p < norm_in.parts; ++p) sum += pieces[p];
                }
                row_scale[tid] = 1.0f / sqrtf(sum / (float)norm_in.dim + norm_in.eps);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    phase_barrier();
    if (group == 1) phase_barrier();            // group 1 runs one barrier behind group 0's phases

    const int r = lane & 31, swz = (r >> 1) & 7;
    const unsigned char* a_rows = ring + (wm + r) * 128;
    const unsigned char* b_rows = ring + (BM + wn + r) * 128;
    for (int block = 0; block < n_k; ++block) {
        const int stage_off = (block & 1) * STAGE_BYTES;
        // ---- R: the operands of the block's 64 k into registers, and behind the reads this wave's loads
        // (two of the group's waves send their loads first and read then, two the other way round: the memory pipeline is at work
        // from the start of the interval, and nobody's reads wait behind everybody's loads)
        bf16x8 a[PK / 16][TM], b[PK / 16][TN];
        if (turn & 1) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) load_one(i, block);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int step = 0; step < PK / 16; ++step) {
            const int chunk = ((2 * step + (lane >> 5)) ^ swz) * 16;
#pragma unroll
            for (int i = 0; i < TM; ++i) a[step][i] = as_bf16x8(*reinterpret_cast<const uint4*>(a_rows + stage_off + i * 32 * 128 + chunk));
#pragma unroll
            for (int j = 0; j < TN; ++j) b[step][j] = as_bf16x8(*reinterpret_cast<const uint4*>(b_rows + stage_off + j * 32 * 128 + chunk));
        }
        __builtin_amdgcn_sched_barrier(0);
        if (!(turn & 1)) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) load_one(i, block);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                          // the reads are done before anyone may refill the stage
        phase_barrier();
        // ---- M: nothing but matrix instructions
#pragma unroll
        for (int step = 0; step < PK / 16; ++step)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[step][j], a[step][i], acc[i][j], 0, 0, 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                            // what this wave sent for during R has landed
        phase_barrier();
    }
    if (group == 0) phase_barrier();
    // The weights were the first operand: a lane's 32x32 result holds row (of A) m = lane%32 and, as element v, column
    // (row of W) n = 8*(v/4) + 4*(lane/32) + v%4, four neighbouring columns at a time.  The results leave through LDS
    // (the ring is free now: every wave has passed the barrier behind its last read), 128 bytes of 64 rows at a time
    // in a part of it that is this wave's own, so that every store instruction writes whole cache lines: eight rows of
    // 128 bytes instead of 32 pieces of 16 or 32 bytes.  Rows lie 144 bytes apart in LDS (16 consecutive rows then
    // start in 16 different groups of banks, for the 8- and 16-byte writes as for the 16-byte reads).
    constexpr int STAGE_ROW = 144;
    unsigned char* mine = ring + wave * (WM * STAGE_ROW);
    const int frow = lane >> 3, fchunk = lane & 7;                                 // the flush: lane -> (row within 8, 16-byte piece of 128)
    if constexpr (EPI == EPI_GATED_BF16) {
        // columns 32b .. 32b+15 are gates, 32b+16 .. 32b+31 the ups of outputs 16b .. 16b+15: element v beside element v + 8.
        // The wave's WN columns become WN/2 outputs: 2 * WN/2 bytes a row, flushed 64 outputs (128 bytes) at a time.
        static_assert(WN % 128 == 0, "the gated flush takes 64 outputs at a time");
#pragma unroll
        for (int part = 0; part < WN / 128; ++part) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    const int j = 4 * part + jj;
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        const float rs = norm_in.squares != nullptr ? row_scale[wm + i * 32 + (lane & 31)] : 1.0f;
                        const uint2 packed = {f32x2_to_bf16x2(silu_gate_fast(acc[i][j][4 * q] * rs, acc[i][j][4 * q + 8] * rs), silu_gate_fast(acc[i][j][4 * q + 1] * rs, acc[i][j][4 * q + 9] * rs)),
                                              f32x2_to_bf16x2(silu_gate_fast(acc[i][j][4 * q + 2] * rs, acc[i][j][4 * q + 10] * rs), silu_gate_fast(acc[i][j][4 * q + 3] * rs, acc[i][j][4 * q + 11] * rs))};
                        *reinterpret_cast<uint2*>(mine + (i * 32 + (lane & 31)) * STAGE_ROW + (jj * 16 + 8 * q + 4 * (lane >> 5)) * 2) = packed;
                    }
                }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int it = 0; it < WM / 8; ++it) {
                const int row = it * 8 + frow, m = m0 + wm + row, c = (n0 + wn) / 2 + part * 64 + fchunk * 8;      // output column
                const uint4 v = *reinterpret_cast<const uint4*>(mine + row * STAGE_ROW + fchunk * 16);
                if (m < M && c + 7 < N / 2 && (ldc & 7) == 0) *reinterpret_cast<uint4*>((bf16_t*)C + (size_t)m * ldc + c) = v;
                else if (m < M) {
                    const bf16_t* e = reinterpret_cast<const bf16_t*>(&v);
#pragma unroll
                    for (int x = 0; x < 8; ++x)
                        if (c + x < N / 2) ((bf16_t*)C)[(size_t)m * ldc + c + x] = e[x];
                }
            }
        }
    } else if constexpr (EPI == EPI_STORE_BF16) {
#pragma unroll
        for (int part = 0; part < TN / 2; ++part) {                                // 64 columns = 128 bytes a row at a time
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const floatx16& t = acc[i][2 * part + jj];
                        *reinterpret_cast<uint2*>(mine + (i * 32 + (lane & 31)) * STAGE_ROW + (jj * 32 + 8 * q + 4 * (lane >> 5)) * 2) =
                            uint2{f32x2_to_bf16x2(t[4 * q], t[4 * q + 1]), f32x2_to_bf16x2(t[4 * q + 2], t[4 * q + 3])};
                    }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int it = 0; it < WM / 8; ++it) {
                const int row = it * 8 + frow, m = m0 + wm + row, c = n0 + wn + part * 64 + fchunk * 8;
                const uint4 v = *reinterpret_cast<const uint4*>(mine + row * STAGE_ROW + fchunk * 16);
                if (m < M && c + 7 < N && (ldc & 7) == 0) *reinterpret_cast<uint4*>((bf16_t*)C + (size_t)m * ldc + c) = v;
                else if (m < M) {
                    const bf16_t* e = reinterpret_cast<const bf16_t*>(&v);
#pragma unroll
                    for (int x = 0; x < 8; ++x)
                        if (c + x < N) ((bf16_t*)C)[(size_t)m * ldc + c + x] = e[x];
                }
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < TN; ++j) {                                             // 32 columns = 128 bytes a row at a time
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<float4*>(mine + (i * 32 + (lane & 31)) * STAGE_ROW + (8 * q + 4 * (lane >> 5)) * 4) =
                        float4{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int it = 0; it < WM / 8; ++it) {
                const int row = it * 8 + frow, m = m0 + wm + row, c = n0 + wn + j * 32 + fchunk * 4;
                float4 v = *reinterpret_cast<const float4*>(mine + row * STAGE_ROW + fchunk * 16);
                if (m >= M) continue;
                float* dst = (float*)C + (size_t)m * ldc + c;
                if (c + 3 < N && (ldc & 3) == 0 && (((uintptr_t)C) & 15) == 0) {
                    if constexpr (EPI == EPI_ADD_F32) {
                        const float4 old = *reinterpret_cast<const float4*>(dst);
                        v.x += old.x; v.y += old.y; v.z += old.z; v.w += old.w;
                    }
                    *reinterpret_cast<float4*>(dst) = v;
                } else {
                    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                    for (int x = 0; x < 4; ++x)
                        if (c + x < N) write_out<EPI>(C, (size_t)m * ldc + c + x, e[x]);
                }
            }
        }
    }
}

// ----------------------------------------------------------------------------------------- skinny
// Workgroup: 8 waves = 4 strips of 16 weight rows x 2 halves of each 256-wide block of k; the
// workgroup covers 64 weight rows and the k range [k_begin, k_end) of its grid row.  Weights stream
// from HBM straight into registers, two blocks ahead of their use: for the j-th product of a
// block, lane (r = lane%16, q = lane/16) holds k0 + 128*half + 32j + 8q .. +8 of weight row r, so
// the four lanes of a row read 64 contiguous bytes per load.  The activations of a block go
// through LDS (they are shared by the strips) and are fetched into registers one block ahead.
// Cycle stamps of a workgroup's blocks (64 rows, gate/up: 5,300 clocks a block) showed a wait for every load in flight where the
// block's activations are stored into LDS (the weights asked for one block earlier included: the compiler counts loads exactly
// only if none of them is skipped by a lane or a block) and the products waiting for one LDS read each (1,250 clocks for 16
// products); with every load issued by everyone, barriers that wait for LDS only and the reads one product ahead: 850 clocks for
// the products, gate/up 21.4 -> 18.8 us at 17 rows, 25.5 -> 23.1 at 64, the decode step 2 to 3 % shorter at 17 to 128 rows.
// (Up to four tiles of rows the kernel stays within 128 registers, two workgroups a compute unit.)
// The halves' sums meet in LDS.  PARTIAL: the sums of the k range go to P[split][M][N] and a
// second kernel adds the splits in order; otherwise the workgroup saw all of k and writes the
// result with its epilogue itself.
constexpr int SK = 128;                               // k per product group of a wave (4 products of 32)
constexpr int SKINNY_MAX_ROWS = 128;                  // rows of A the skinny kernel takes (8 tiles of 16)
constexpr int KB = 2 * SK, X_STRIDE = KB + 8;         // k per block of the workgroup; +8 bf16 of padding

// The kernel for at most 16 rows: a thread keeps 8 pieces while the products run (more would cost the kernel its second
// workgroup per compute unit); 64 threads share a row where there are at most 8 rows, 32 otherwise.
constexpr int SLIM_PIECES = 8;
// Outputs of fewer than so many strips of 16 weight rows take strips of 8, twice the workgroups; with up to 8 rows of A, where a
// strip of 8 leaves no lane idle (FOLD = 1 below), of fewer than twice as many (measured at N = 4096 to 6144: 1 to 2 % of the
// decode step at 1 to 8 rows, and 7 % the other way at 12 and 16 rows); a product that adds onto rows and hands a norm on does
// so up to 3 rows only (N = 4096, K = 4096 and 14336 at 8 rows: 18.5 us with strips of 16 against 20.5, the step of the 8B shape
// 4.47 -> 4.3 ms; equal at 4 rows, 0.5 % the other way at 1 and 2).
constexpr int SLIM_NARROW_STRIPS = 256;
__host__ __device__ constexpr int slim_max_parts(int M) { return SLIM_PIECES * (M <= 8 ? 64 : 32); }
// The kernels for 17 to 128 rows: the kernel that adds the partial sums onto x writes one piece per 1024 columns.
constexpr int REDUCE_COLUMNS = 1024, REDUCE_MAX_PARTS = 8;


// The same for all M rows into `scales` (LDS, at least 32 floats or M), by a workgroup of 512 threads; the caller puts a barrier
// before the use.  With many pieces (the writer was a kernel for at most 32 rows with a piece per workgroup: at most
// TILES_MAX_PARTS for 17 to 32 rows, slim_max_parts for fewer) 16 or 32 threads share a row and ask for 16 pieces each at once.
constexpr int TILES_MAX_PARTS = 256;
__device__ __forceinline__ void row_scales_into(float* scales, const NormIn& n, int M) {
    const int tid = threadIdx.x;
    if (n.parts <= REDUCE_MAX_PARTS) {
        if (tid < M) scales[tid] = row_scale_of(n, tid);
        return;
    }
    const int sharing = M <= 16 ? 32 : 16, row = tid / sharing, at = tid % sharing;        // M <= 32 here
    float piece[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int p = at + sharing * i;
        piece[i] = (row < M && p < n.parts) ? n.squares[(size_t)row * n.parts + p] : 0.f;
    }
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) sum += piece[i];
    if (sharing == 32) sum += __shfl_xor(sum, 16, 64);
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (at == 0 && row < M) scales[row] = 1.0f / sqrtf(sum / (float)n.dim + n.eps);
}

template <int MT, int EPI, bool PARTIAL>
__global__ __launch_bounds__(512, MT == 2 ? 4 : 2) void gemm_bf16_skinny_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ C,
                                                              float* __restrict__ P, int M, int N, int K, long lda, long ldw, long ldc,
                                                              int k_per_split, NormIn norm_in) {
    __shared__ __attribute__((aligned(16))) bf16_t Xs[MT * 16 * X_STRIDE];
    __shared__ float other[4][MT][64][4];
    __shared__ float row_scale[MT * 16 < 32 ? 32 : MT * 16];
    const bool scaled_rows = !PARTIAL && norm_in.squares != nullptr;       // the rows of A lack their norm's rsqrt(mean square + eps)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int strip = wave & 3, half = wave >> 2;
    const int r = lane & 15, q = lane >> 4;
    const int n = blockIdx.x * 64 + strip * 16 + r;
    const int k_begin = blockIdx.y * k_per_split, k_end = min(K, k_begin + k_per_split);
    const bf16_t* wrow = W + (size_t)min(n, N - 1) * ldw + SK * half + 8 * q;

    floatx4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = floatx4{};

    // Every load of the loop is issued by every lane in every block (addresses beyond the range are clamped into it) and the
    // barriers wait for LDS only, so the compiler counts the loads in flight exactly: a block waits for its own activations and
    // weights and leaves the two blocks of weights and the block of activations behind them on their way (with a load that some
    // lanes or blocks skip it waits for all of them at the first use).  What a clamped load brings is finite and meets a zero or
    // is dropped: weights of k beyond the range are replaced by zeros where the range's last block is ragged, and results of rows
    // beyond M are never written.
    uint4 w_buf[3][4], x_reg[MT];
    const int w_last = K - 8 - (SK * half + 8 * q);           // the last 16 bytes of a weight row, from `wrow`
    auto fetch_w = [&](int k0, uint4 (&w)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) w[j] = load16(wrow + min(k0 + 32 * j, w_last));
    };
    const int x_row = tid / (KB / 8), x_k = (tid % (KB / 8)) * 8;             // of this thread's first 16 bytes of a block; its others lie 16 rows further each
    auto fetch_x = [&](int k0) {
#pragma unroll
        for (int c = 0; c < MT; ++c) x_reg[c] = load16(A + (size_t)min(x_row + 16 * c, M - 1) * lda + min(k0 + x_k, K - 8));
    };
    fetch_x(k_begin);
    fetch_w(k_begin, w_buf[0]);
    fetch_w(k_begin + KB, w_buf[1]);
    if (scaled_rows) row_scales_into(row_scale, norm_in, M);                   // (the loop's barriers lie before its use)
    // One block of 256 k: `w_use` holds its weights, `w_fill` takes those of the block after the next.  The activations of the
    // products' next 32 k are read from LDS while those of these 32 are multiplied.
    auto block = [&](int kk, const uint4 (&w_use)[4], uint4 (&w_fill)[4]) __attribute__((always_inline)) {
        barrier_lds();                                // everyone has finished reading the previous block
#pragma unroll
        for (int c = 0; c < MT; ++c) {
            const int e = tid + 512 * c;
            *reinterpret_cast<uint4*>(&Xs[(e / (KB / 8)) * X_STRIDE + (e % (KB / 8)) * 8]) = x_reg[c];
        }
        barrier_lds();
        fetch_x(kk + KB);
        fetch_w(kk + 2 * KB, w_fill);
        const bool ragged = kk + KB > k_end;          // the same for the whole workgroup
        const bf16_t* x_rows = &Xs[r * X_STRIDE + SK * half + 8 * q];
        bf16x8 a[2][MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) a[0][t] = as_bf16x8(*reinterpret_cast<const uint4*>(x_rows + t * 16 * X_STRIDE));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (j + 1 < 4) {
#pragma unroll
                for (int t = 0; t < MT; ++t) a[(j + 1) & 1][t] = as_bf16x8(*reinterpret_cast<const uint4*>(x_rows + t * 16 * X_STRIDE + 32 * (j + 1)));
            }
            uint4 w = w_use[j];
            if (ragged && kk + SK * half + 32 * j + 8 * q >= k_end) w = uint4{0, 0, 0, 0};
            const bf16x8 b = as_bf16x8(w);
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j & 1][t], b, acc[t], 0, 0, 0);
        }
    };
    int kk = k_begin;
    for (; kk + 2 * KB < k_end; kk += 3 * KB) {       // three blocks a trip (the last may be ragged): the buffers' roles come round
        block(kk, w_buf[0], w_buf[2]);
        block(kk + KB, w_buf[1], w_buf[0]);
        block(kk + 2 * KB, w_buf[2], w_buf[1]);
    }
    if (kk < k_end) {
        block(kk, w_buf[0], w_buf[2]);
        if (kk + KB < k_end) block(kk + KB, w_buf[1], w_buf[0]);
    }
    // the second half's sums join the first's
    if (half == 1) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) other[strip][t][lane][v] = acc[t][v];
    }
    __syncthreads();
    if (half == 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[t][v] += other[strip][t][lane][v];
    }
    // Element v of a lane's 16x16 result: row (activation row) 4*(lane/16) + v, column (weight row) lane%16.
    if constexpr (EPI == EPI_GATED_BF16 && !PARTIAL) {
        // strips 0 and 2 hold gates, strips 1 and 3 the ups of the same outputs: the ups cross over through LDS
        __syncthreads();
        if (half == 0 && (strip & 1)) {
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int v = 0; v < 4; ++v) other[strip][t][lane][v] = acc[t][v];
        }
        __syncthreads();
        if (half == 0 && !(strip & 1) && n < N) {
#pragma unroll
            for (int t = 0; t < MT; ++t)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int m = t * 16 + 4 * q + v;
                    const float rs = scaled_rows ? row_scale[m] : 1.0f;
                    if (m < M) ((bf16_t*)C)[(size_t)m * ldc + blockIdx.x * 32 + (strip >> 1) * 16 + r] = f32_to_bf16(silu_gate(acc[t][v] * rs, other[strip + 1][t][lane][v] * rs));
                }
        }
    } else if (half == 0 && n < N) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int m = t * 16 + 4 * q + v;
                if (m >= M) continue;
                if constexpr (PARTIAL) P[((size_t)blockIdx.y * M + m) * N + n] = acc[t][v];
                else write_out<EPI>(C, (size_t)m * ldc + n, scaled_rows ? acc[t][v] * row_scale[m] : acc[t][v]);
            }
    }
}

// Adds the k-split partial sums [splits][M][N] in ascending split order and writes the result.  A thread takes VEC neighbouring
// columns and asks for its values of up to eight splits at once: the kernel is one round trip to memory, not one per split.
// With `norm_in` the sums are multiplied by their row's rsqrt(mean square + eps).  With `norm_out` (adding onto 32-bit rows, four
// columns a thread, rows of a multiple of 1024 columns: a workgroup then lies in one row, and no workgroup is cut short) the rows'
// new values times g go out in bfloat16 beside them, and the workgroup's share of the row's sum of squares.
template <int EPI, int VEC>
__global__ __launch_bounds__(256) void skinny_reduce_kernel(const float* __restrict__ P, void* __restrict__ C, int M, int N, int splits, long ldc,
                                                            NormIn norm_in, NormOut norm_out) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC, slab = (size_t)M * N;
    if (i >= slab) return;
    const size_t row = i / N, col = i % N, o = row * ldc + col;      // (VEC divides N: the VEC columns lie in one row)
    // Everything the result needs besides the partial sums (the row's pieces of the norm before, the old values and the gains of
    // the norm behind) is asked for ahead of them: one round trip to memory for all of it, not one after the other.
    [[maybe_unused]] RowPieces pieces;
    if (norm_in.squares != nullptr) pieces = row_pieces(norm_in, (int)row);
    [[maybe_unused]] float4 old4 = {0.f, 0.f, 0.f, 0.f}, gain4 = {0.f, 0.f, 0.f, 0.f};
    if constexpr (VEC == 4 && EPI == EPI_ADD_F32) {
        old4 = *reinterpret_cast<const float4*>((const float*)C + o);
        if (norm_out.scaled != nullptr) gain4 = *reinterpret_cast<const float4*>(norm_out.g + col);
    }
    float s[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) s[v] = 0.f;
    for (int sp0 = 0; sp0 < splits; sp0 += 8) {
        float part[8][VEC];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const float* src = P + (size_t)min(sp0 + u, splits - 1) * slab + i;
            if constexpr (VEC == 4) {
                const float4 x = *reinterpret_cast<const float4*>(src);
                part[u][0] = x.x; part[u][1] = x.y; part[u][2] = x.z; part[u][3] = x.w;
            } else {
                part[u][0] = *src;
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (sp0 + u < splits) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) s[v] += part[u][v];
            }
    }
    if (norm_in.squares != nullptr) {
        const float rs = row_scale_from(norm_in, (int)row, pieces);
#pragma unroll
        for (int v = 0; v < VEC; ++v) s[v] *= rs;
    }
    if constexpr (VEC == 4) {                                        // (the host has checked that rows of C start at multiples of 16 bytes)
        if constexpr (EPI == EPI_STORE_BF16) {
            uint2 packed;
            packed.x = (unsigned)f32_to_bf16(s[0]) | ((unsigned)f32_to_bf16(s[1]) << 16);
            packed.y = (unsigned)f32_to_bf16(s[2]) | ((unsigned)f32_to_bf16(s[3]) << 16);
            *reinterpret_cast<uint2*>((bf16_t*)C + o) = packed;
        } else {
            float4* dst = reinterpret_cast<float4*>((float*)C + o);
            float4 x = old4;
            x.x += s[0]; x.y += s[1]; x.z += s[2]; x.w += s[3];
            *dst = x;
            if constexpr (EPI == EPI_ADD_F32) {
                if (norm_out.scaled != nullptr) {                    // (the same for every thread of the kernel)
                    __shared__ float wave_squares[4];
                    const float4 g = gain4;
                    uint2 packed;
                    packed.x = (unsigned)f32_to_bf16(g.x * x.x) | ((unsigned)f32_to_bf16(g.y * x.y) << 16);
                    packed.y = (unsigned)f32_to_bf16(g.z * x.z) | ((unsigned)f32_to_bf16(g.w * x.w) << 16);
                    *reinterpret_cast<uint2*>(norm_out.scaled + row * norm_out.ld + col) = packed;
                    float square = (x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w);
#pragma unroll
                    for (int off = 32; off > 0; off >>= 1) square += __shfl_xor(square, off, 64);
                    if ((threadIdx.x & 63) == 0) wave_squares[threadIdx.x >> 6] = square;
                    __syncthreads();
                    if (threadIdx.x == 0) {
                        const int per_row = N / REDUCE_COLUMNS;
                        norm_out.squares[row * per_row + blockIdx.x % per_row] = (wave_squares[0] + wave_squares[1]) + (wave_squares[2] + wave_squares[3]);
                    }
                }
            }
        }
    } else {
        write_out<EPI>(C, o, s[0]);
    }
}

// The same for the gated product: columns 32b .. 32b+15 of the partial sums are gates, 32b+16 .. 32b+31 the ups of
// outputs 16b .. 16b+15; the output [M, N/2] is silu(gate) * up in bfloat16.
__global__ void skinny_reduce_gated_kernel(const float* __restrict__ P, bf16_t* __restrict__ C, int M, int N, int splits, long ldc) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int half = N / 2;
    if (i >= (size_t)M * half) return;
    const size_t m = i / half;
    const int c = (int)(i % half), col = (c >> 4) * 32 + (c & 15);
    float gate = 0.f, up = 0.f;
    for (int sp = 0; sp < splits; ++sp) {
        gate += P[((size_t)sp * M + m) * N + col];
        up += P[((size_t)sp * M + m) * N + col + 16];
    }
    C[m * ldc + c] = f32_to_bf16(silu_gate(gate, up));
}

// The same for the q/k/v product of an attention layer, N = (n_heads + 2 n_kv) * hd columns: the sums of a row are its queries,
// keys and values, and instead of writing them out for a kernel that rotates them and puts them into the cache, this one does
// that itself: queries rotated into q_out, keys rotated and values as they are into the page table[slot][pos / page_size] at
// place pos % page_size (pairs (i, i + hd/2): a' = a cos - b sin, b' = a sin + b cos; the page's layout as the attention
// kernels read it: keys [kv_head][place][hd], then values [kv_head][hd][place]).  A thread has four neighbouring columns; the
// other half of its pairs is with the thread hd/8 lanes away, in the same wave (hd a power of two from 8 to 256, and rows of a
// multiple of 256 columns, so that a wave lies in one row and holds whole heads).
__global__ __launch_bounds__(256) void skinny_reduce_rope_store_kernel(const float* __restrict__ P, int M, int N, int splits, NormIn norm_in, RopeStore rs) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4, slab = (size_t)M * N;
    if (i >= slab) return;                                   // (whole waves: 256 divides N, so the exchange below has all its lanes)
    const size_t row = i / N;
    const int col = (int)(i % N);
    const int a_dim = rs.n_heads * rs.hd, kv_dim = rs.n_kv * rs.hd, half = rs.hd / 2;
    const int which = col < a_dim ? 0 : col < a_dim + kv_dim ? 1 : 2;                        // queries, keys, values
    const int c = which == 0 ? col : which == 1 ? col - a_dim : col - a_dim - kv_dim;        // the column among them
    const int h = c / rs.hd, kk = c % rs.hd;
    // Everything is asked for at once, by every lane: position and slot first (the page number, which needs them, then waits for
    // them alone), the row's pieces of the norm, the angles (a lane with values asks too and drops them), the first eight splits.
    const int p = rs.pos[row], slot = rs.slot[row];
    [[maybe_unused]] RowPieces pieces;
    if (norm_in.squares != nullptr) pieces = row_pieces(norm_in, (int)row);
    float4 cc = {1.f, 1.f, 1.f, 1.f}, ss = {0.f, 0.f, 0.f, 0.f};
    if (rs.cos_t != nullptr) {
        cc = *reinterpret_cast<const float4*>(rs.cos_t + row * half + kk % half);
        ss = *reinterpret_cast<const float4*>(rs.sin_t + row * half + kk % half);
    }
    float4 part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) part[u] = *reinterpret_cast<const float4*>(P + (size_t)min(u, splits - 1) * slab + i);
    const long page = rs.table[(size_t)slot * rs.table_stride + p / rs.page_size];
    float s[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < 8; ++u)
        if (u < splits) {
            s[0] += part[u].x; s[1] += part[u].y; s[2] += part[u].z; s[3] += part[u].w;
        }
    for (int sp0 = 8; sp0 < splits; sp0 += 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) part[u] = *reinterpret_cast<const float4*>(P + (size_t)min(sp0 + u, splits - 1) * slab + i);
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (sp0 + u < splits) {
                s[0] += part[u].x; s[1] += part[u].y; s[2] += part[u].z; s[3] += part[u].w;
            }
    }
    if (norm_in.squares != nullptr) {
        const float scale = row_scale_from(norm_in, (int)row, pieces);
#pragma unroll
        for (int v = 0; v < 4; ++v) s[v] *= scale;
    }
    float out[4] = {s[0], s[1], s[2], s[3]};
    if (rs.cos_t != nullptr) {                               // (every lane takes part in the exchange, whatever it holds)
        float other[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) other[v] = __shfl_xor(s[v], half / 4, 64);
        if (which != 2) {
            const float cs[4] = {cc.x, cc.y, cc.z, cc.w}, sn[4] = {ss.x, ss.y, ss.z, ss.w};
#pragma unroll
            for (int v = 0; v < 4; ++v) out[v] = kk < half ? s[v] * cs[v] - other[v] * sn[v] : other[v] * sn[v] + s[v] * cs[v];
        }
    }
    uint2 packed;
    packed.x = (unsigned)f32_to_bf16(out[0]) | ((unsigned)f32_to_bf16(out[1]) << 16);
    packed.y = (unsigned)f32_to_bf16(out[2]) | ((unsigned)f32_to_bf16(out[3]) << 16);
    if (which == 0) {
        *reinterpret_cast<uint2*>(rs.q_out + row * a_dim + c) = packed;
        return;
    }
    const int place = p % rs.page_size;
    bf16_t* keys = rs.cache + page * rs.page_stride;
    bf16_t* values = keys + (size_t)rs.n_kv * rs.page_size * rs.hd;
    if (which == 1) {
        *reinterpret_cast<uint2*>(keys + ((size_t)h * rs.page_size + place) * rs.hd + kk) = packed;
    } else {
#pragma unroll
        for (int v = 0; v < 4; ++v) values[((size_t)h * rs.hd + kk + v) * rs.page_size + place] = f32_to_bf16(out[v]);
    }
}

// ------------------------------------------------------------------------------------------- slim
// At most 16 rows of A.  Workgroup: 8 waves = STRIPS strips of ROWS weight rows x (8 / STRIPS)
// slices of k; slice s takes the 128-wide blocks of k numbered s, s + slices, ...  Both operands go
// from global memory straight into registers (the activations are few and stay in cache): for the
// j-th product of a block, lane (r = lane%16, q = lane/16) holds k0 + 32j + 8q .. +8 of weight row r
// and of activation row r, so the four lanes of a row read 64 contiguous bytes per load.  Loads run
// two blocks ahead of the products.  The slices' sums meet in LDS and are added in slice order.
// ROWS = 8 leaves half of each product idle and doubles the number of workgroups for narrow outputs.
// HAND: with the two halves of a norm handed from product to product (`NormIn`, `NormOut` above).
// FOLD (ROWS = 8): the product's rows 8..15, idle otherwise on the weights' side, take the same 8 weight rows at the next 32 of k, and
// the other operand 8 rows of A at both places likewise, so that a block is 256 wide, every lane loads weights, and a row's eight
// lanes read 128 contiguous bytes; of the 16 x 16 result the two 8 x 8 blocks on the diagonal are the two halves' sums (the other
// two mix the halves and are dropped).  FOLD = 1: at most 8 rows of A, one product per weight fragment; FOLD = 2: up to 16, in two
// groups of 8 rows that share the weight fragment.
template <int STRIPS, int ROWS, int EPI, bool HAND, int FOLD = 0>
__global__ __launch_bounds__(512, 4) void gemm_bf16_slim_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ C,
                                                            int M, int N, int K, long lda, long ldw, long ldc, NormIn norm_in, NormOut norm_out) {
    static_assert(FOLD == 0 || ROWS == 8, "folding k into the idle rows needs strips of 8 weight rows");
    constexpr int BLOCK = FOLD ? 2 * SK : SK, SPAN = BLOCK / 4;       // k of a block, and of one of its four products
    constexpr int XT = FOLD == 2 ? 2 : 1;                             // groups of rows of A
    constexpr int SLICES = 8 / STRIPS, STEP = SLICES * BLOCK, DEPTH = FOLD == 2 ? 2 : 3;
    __shared__ float red[8][XT][64][4];
    __shared__ float row_scale[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int strip = wave % STRIPS, slice = wave / STRIPS;
    const int r = FOLD ? lane & 7 : lane & 15, q = lane >> 4;
    const int k_lane = 8 * q + (FOLD ? 32 * ((lane >> 3) & 1) : 0);   // where in a product's span of k this lane reads
    const int n = (blockIdx.x * STRIPS + strip) * ROWS + (r < ROWS ? r : ROWS - 1);      // (lanes beyond a strip of 10 or 12 rows ask for its last row again)
    // Every lane issues every load of a block (a row beyond the operand is clamped into it and lands in results that are never
    // written; in a row's last, ragged block k is clamped too and the activations beyond K become zeros), and what a wave skips it
    // skips as a whole: the compiler then counts the loads in flight, and a block's products wait for that block alone.
    const bf16_t* wrow = W + (size_t)min(n, N - 1) * ldw + k_lane;
    const bf16_t* xrow[XT];
#pragma unroll
    for (int t = 0; t < XT; ++t) xrow[t] = A + (size_t)min(8 * t + r, M - 1) * lda + k_lane;
    const int k_last = K - 8 - k_lane;                        // the last 16 bytes of a row, from `wrow` and `xrow`

    floatx4 acc[XT];
#pragma unroll
    for (int t = 0; t < XT; ++t) acc[t] = floatx4{};
    uint4 w_buf[DEPTH][4], x_buf[DEPTH][XT][4];
    auto fetch = [&](int k0, uint4* w, uint4 (*x)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int at = min(k0 + SPAN * j, k_last);
            w[j] = load16(wrow + at);
#pragma unroll
            for (int t = 0; t < XT; ++t) x[t][j] = load16(xrow[t] + at);
        }
    };
    // What the epilogue adds onto (the thread's element of the 32-bit rows, and the next norm's gain for its column) is asked for
    // before anything else: it comes from the memory-side cache while the weights stream, not behind them as one more round trip.
    [[maybe_unused]] float old_value = 0.f, gain = 0.f;
    if constexpr (EPI == EPI_ADD_F32) {
        const int e_m = (tid & 255) >> 4, e_col = (blockIdx.x * STRIPS + (tid >> 8) % STRIPS) * ROWS + (tid & 15);
        old_value = ((const float*)C)[(size_t)min(e_m, M - 1) * ldc + min(e_col, N - 1)];
        if constexpr (HAND) {
            if (norm_out.scaled != nullptr) gain = norm_out.g[min(e_col, N - 1)];
        }
    }
    // The pieces of the rows' sums of squares, 32 or 64 threads a row: asked for ahead of the first weights (loads come back in
    // the order they were issued) and added up behind the requests for those, so that one register waits for the epilogue, not eight.
    float piece[HAND ? SLIM_PIECES : 1];
    [[maybe_unused]] float pieces_sum = 0.f;
    const int sharing = M <= 8 ? 64 : 32, piece_row = M <= 8 ? tid >> 6 : tid >> 5;
    if constexpr (HAND) {
        if (norm_in.squares != nullptr) {
            const float* row_pieces = norm_in.squares + (size_t)min(piece_row, M - 1) * norm_in.parts;
#pragma unroll
            for (int i = 0; i < SLIM_PIECES; ++i) piece[i] = row_pieces[min((tid & (sharing - 1)) + sharing * i, norm_in.parts - 1)];
        }
    }
    const int k_first = slice * BLOCK;
    const int n_blocks = k_first < K ? (K - k_first + STEP - 1) / STEP : 0;       // of this wave
#pragma unroll
    for (int d = 0; d < DEPTH - 1; ++d)
        if (d < n_blocks) fetch(k_first + d * STEP, w_buf[d], x_buf[d]);
    if constexpr (HAND) {
        if (norm_in.squares != nullptr) {
#pragma unroll
            for (int i = 0; i < SLIM_PIECES; ++i)
                if (piece_row < M && (tid & (sharing - 1)) + sharing * i < norm_in.parts) pieces_sum += piece[i];
        }
    }
    // Block b of the wave lies in buffer b % DEPTH; its products are behind the request for block b + DEPTH - 1.
    auto products = [&](int b, uint4* w, uint4 (*x)[4]) __attribute__((always_inline)) {
        const int kb = k_first + b * STEP;
        if (kb + BLOCK > K) {                                 // the row's end lies in this block
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (kb + SPAN * j + k_lane >= K) {
#pragma unroll
                    for (int t = 0; t < XT; ++t) x[t][j] = uint4{0, 0, 0, 0};
                }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < XT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(x[t][j]), as_bf16x8(w[j]), acc[t], 0, 0, 0);
    };
    int b = 0;
    for (; b + 2 * DEPTH - 1 <= n_blocks; b += DEPTH) {      // trips in which nothing is skipped: exact waits
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            fetch(k_first + (b + d + DEPTH - 1) * STEP, w_buf[(d + DEPTH - 1) % DEPTH], x_buf[(d + DEPTH - 1) % DEPTH]);
            products(b + d, w_buf[d], x_buf[d]);
        }
    }
    for (; b < n_blocks; b += DEPTH) {                        // the end of the wave's blocks
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (b + d + DEPTH - 1 < n_blocks) fetch(k_first + (b + d + DEPTH - 1) * STEP, w_buf[(d + DEPTH - 1) % DEPTH], x_buf[(d + DEPTH - 1) % DEPTH]);
            if (b + d < n_blocks) products(b + d, w_buf[d], x_buf[d]);
        }
    }
#pragma unroll
    for (int t = 0; t < XT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave][t][lane][v] = acc[t][v];
    if constexpr (HAND) {
        if (norm_in.squares != nullptr) {
            float sum = pieces_sum;
            if (sharing == 64) sum += __shfl_xor(sum, 32, 64);
#pragma unroll
            for (int off = 16; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
            if ((tid & (sharing - 1)) == 0 && piece_row < 16) row_scale[piece_row] = 1.0f / sqrtf(sum / (float)norm_in.dim + norm_in.eps);
        }
    }
    __syncthreads();
    // Element v of a lane's result: activation row 4*q + v, weight row r of the strip (folded: of the group's 8 rows, and the
    // second half of k at row + 8, weight row + 8).
    if (tid < 256 * (EPI == EPI_GATED_BF16 ? 1 : STRIPS)) {
        const int st = tid >> 8, e = tid & 255, m = e >> 4, c = e & 15;
        const int group = FOLD ? m >> 3 : 0, m_in = FOLD ? m & 7 : m;
        const int src_lane = c + 16 * (m_in >> 2), v = m_in & 3;
        float r = 1.0f;
        if constexpr (HAND) r = norm_in.squares != nullptr ? row_scale[m] : 1.0f;
        float square = 0.f;
        if (m < M && c < ROWS && group < XT) {
            if constexpr (EPI == EPI_GATED_BF16) {
                float gate = 0.f, up = 0.f;
#pragma unroll
                for (int s = 0; s < SLICES; ++s) {
                    gate += red[s * STRIPS + 0][0][src_lane][v];
                    up += red[s * STRIPS + 1][0][src_lane][v];
                }
                if constexpr (HAND) { gate *= r; up *= r; }
                ((bf16_t*)C)[(size_t)m * ldc + blockIdx.x * 16 + c] = f32_to_bf16(silu_gate(gate, up));
            } else {
                float sum = 0.f;
#pragma unroll
                for (int s = 0; s < SLICES; ++s) sum += red[s * STRIPS + st][group][src_lane][v];
                if constexpr (FOLD != 0) {                      // the other half of k: row + 8, column + 8 of the product
#pragma unroll
                    for (int s = 0; s < SLICES; ++s) sum += red[s * STRIPS + st][group][src_lane + 40][v];
                }
                if constexpr (HAND) sum *= r;
                const int col = (blockIdx.x * STRIPS + st) * ROWS + c;
                if (col < N) {
                    if constexpr (EPI == EPI_ADD_F32) {
                        const float x = old_value + sum;
                        ((float*)C)[(size_t)m * ldc + col] = x;
                        if constexpr (HAND) {
                            if (norm_out.scaled != nullptr) {
                                norm_out.scaled[(size_t)m * norm_out.ld + col] = f32_to_bf16(gain * x);
                                square = x * x;
                            }
                        }
                    } else {
                        write_out<EPI>(C, (size_t)m * ldc + col, sum);
                    }
                }
            }
        }
        if constexpr (HAND && EPI == EPI_ADD_F32) {
            if (norm_out.scaled != nullptr) {                   // the 16 threads of a row: its columns of this workgroup
#pragma unroll
                for (int off = 8; off > 0; off >>= 1) square += __shfl_xor(square, off, 64);
                if (c == 0 && m < M) norm_out.squares[(size_t)m * (gridDim.x * STRIPS) + blockIdx.x * STRIPS + st] = square;
            }
        }
    }
}

// The same for a few more rows of A (MT tiles of 16) and outputs too narrow to fill the chip with strips of 64 weight rows: a workgroup owns 16
// weight rows and all of k, its 8 waves take interleaved 128-wide blocks of k, and each wave multiplies its weights with MT tiles
// of 16 activation rows, all straight from global memory into registers (the waves share nothing: every wave reads another part
// of k; the activations come from L2, as many bytes again for every 16 rows as the strip has weights, which pays up to 32 rows).
// One launch does the product and its epilogue; the alternative, k shared out over workgroups with partial sums in memory and a
// second kernel to add them, costs that kernel's launch and as many bytes of partial sums as the output projection has weights.
template <int MT, int EPI>
__global__ __launch_bounds__(512, 4) void gemm_bf16_slim_tiles_kernel(const bf16_t* __restrict__ A, const bf16_t* __restrict__ W, void* __restrict__ C,
                                                                  int M, int N, int K, long lda, long ldw, long ldc, NormIn norm_in, NormOut norm_out,
                                                                  int strip_rows) {
    constexpr int SLICES = 8, STEP = SLICES * SK, DEPTH = 2;
    __shared__ float red[SLICES][MT][64][4];
    __shared__ float row_scale[MT * 16 < 32 ? 32 : MT * 16];
    static_assert(MT == 2, "the epilogue's sums of squares take every thread's one result to lie in one row of 16 threads");
    const int tid = threadIdx.x, lane = tid & 63, slice = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    // strip_rows (8, 12 or 16) of the product's 16 weight rows are the workgroup's own; lanes beyond them ask for its last row again
    // (the same cache line) and their results are dropped
    const int n = blockIdx.x * strip_rows + min(r, strip_rows - 1);
    const bf16_t* wrow = W + (size_t)min(n, N - 1) * ldw + 8 * q;         // (every lane issues every load of a block, as in the kernel above)
    const bf16_t* xrow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) xrow[t] = A + (size_t)min(t * 16 + r, M - 1) * lda + 8 * q;
    const int k_last = K - 8 - 8 * q;
    floatx4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = floatx4{};
    uint4 w_buf[DEPTH][4], x_buf[DEPTH][MT][4];
    auto fetch = [&](int k0, uint4* w, uint4 (*x)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int at = min(k0 + 32 * j, k_last);
            w[j] = load16(wrow + at);
#pragma unroll
            for (int t = 0; t < MT; ++t) x[t][j] = load16(xrow[t] + at);
        }
    };
    // (what the epilogue adds onto is asked for first, as in the kernel above: every thread has one result, e = tid below)
    [[maybe_unused]] float old_value = 0.f, gain = 0.f;
    if constexpr (EPI == EPI_ADD_F32) {
        const int e_row = 16 * (tid >> 8) + ((tid >> 4) & 15), e_col = blockIdx.x * strip_rows + (tid & 15);
        old_value = ((const float*)C)[(size_t)min(e_row, M - 1) * ldc + min(e_col, N - 1)];
        if (norm_out.scaled != nullptr) gain = norm_out.g[min(e_col, N - 1)];
    }
    const int k_first = slice * SK;
    const int n_blocks = k_first < K ? (K - k_first + STEP - 1) / STEP : 0;       // of this wave
    if (n_blocks > 0) fetch(k_first, w_buf[0], x_buf[0]);
    if (norm_in.squares != nullptr) row_scales_into(row_scale, norm_in, M);      // (the barrier behind the products lies before its use)
    auto products = [&](int b, uint4* w, uint4 (*x)[4]) __attribute__((always_inline)) {
        const int kb = k_first + b * STEP;
        if (kb + SK > K) {                                    // the row's end lies in this block: weights of k beyond it become zeros
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (kb + 32 * j + 8 * q >= K) w[j] = uint4{0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(x[t][j]), as_bf16x8(w[j]), acc[t], 0, 0, 0);
    };
    int b = 0;
    for (; b + 2 * DEPTH - 1 <= n_blocks; b += DEPTH) {      // trips in which nothing is skipped
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            fetch(k_first + (b + d + 1) * STEP, w_buf[(d + 1) % DEPTH], x_buf[(d + 1) % DEPTH]);
            products(b + d, w_buf[d], x_buf[d]);
        }
    }
    for (; b < n_blocks; b += DEPTH) {                        // the end of the wave's blocks
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (b + d + 1 < n_blocks) fetch(k_first + (b + d + 1) * STEP, w_buf[(d + 1) % DEPTH], x_buf[(d + 1) % DEPTH]);
            if (b + d < n_blocks) products(b + d, w_buf[d], x_buf[d]);
        }
    }
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[slice][t][lane][v] = acc[t][v];
    __syncthreads();
    // Element v of a lane's result for tile t: activation row 16*t + 4*q + v, weight row r of the strip.
    for (int e = tid; e < MT * 256; e += 512) {
        const int t = e >> 8, m = (e >> 4) & 15, c = e & 15;
        const int src_lane = c + 16 * (m >> 2), v = m & 3, row = 16 * t + m, col = c < strip_rows ? blockIdx.x * strip_rows + c : N;
        float sum = 0.f;
#pragma unroll
        for (int s = 0; s < SLICES; ++s) sum += red[s][t][src_lane][v];
        if (norm_in.squares != nullptr && row < M) sum *= row_scale[row];
        if constexpr (EPI == EPI_ADD_F32) {
            if (norm_out.scaled != nullptr) {                   // (every thread comes here once: MT * 256 results, 512 threads)
                float square = 0.f;
                if (row < M && col < N) {
                    const float x = old_value + sum;
                    ((float*)C)[(size_t)row * ldc + col] = x;
                    norm_out.scaled[(size_t)row * norm_out.ld + col] = f32_to_bf16(gain * x);
                    square = x * x;
                }
#pragma unroll
                for (int off = 8; off > 0; off >>= 1) square += __shfl_xor(square, off, 64);
                if (c == 0 && row < M) norm_out.squares[(size_t)row * gridDim.x + blockIdx.x] = square;
                continue;
            }
            if (row < M && col < N) ((float*)C)[(size_t)row * ldc + col] = old_value + sum;
            continue;
        }
        if (row < M && col < N) write_out<EPI>(C, (size_t)row * ldc + col, sum);
    }
}

int epilogue_of(int c_dtype, int accumulate) {
    if (c_dtype == GI_F32) return accumulate ? EPI_ADD_F32 : EPI_STORE_F32;
    if (c_dtype == GI_BF16 && !accumulate) return EPI_STORE_BF16;
    return -1;
}

}  // namespace

// Number of k-splits of the skinny kernel for a product with 17..64 rows, so that the caller can size
// the scratch (splits * M * N floats); 0: the output is wide enough to fill the chip without a split,
// no scratch is needed.  Workgroups for three quarters of the chip or more, each with at least one block of k (measured at 33 to
// 64 rows, product and reduce kernel together: 192 to 384 workgroups on 256 compute units, with two blocks of k each, take 11 us for N = 3072, K = 2048 and
// 16 us for N = 2048, K = 8192; twice the workgroups with one block each 12.5 and 17.5 us, half of them 13 and 22 us).
GI_API int gi_gemm_bf16_skinny_splits(int N, int K) {
    const int strips = (N + 63) / 64, most_of_the_chip = gi_compute_units() * 3 / 4;
    if (strips >= most_of_the_chip) return 0;
    int splits = 1;
    while (strips * splits < most_of_the_chip && K / (splits * 2) >= KB) splits *= 2;
    return splits;
}

// Splits of k for the LDS-ring kernel (more than 64 rows): with fewer tiles of 128 x 128 than three quarters of the compute units the tiles alone
// leave compute units idle and the weights stream too slowly; every share keeps at least 256 of k.
GI_API int gi_gemm_bf16_piped_splits(int M, int N, int K) {
    if (M <= SKINNY_MAX_ROWS || K % PK != 0 || N < 128) return 1;
    const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
    const int most_of_the_chip = gi_compute_units() * 3 / 4;
    int splits = 1;
    while (tiles * splits < most_of_the_chip && K % (splits * 2 * PK) == 0 && K / (splits * 2) >= 256) splits *= 2;
    return splits;
}

// Floats of scratch a product of these sizes needs (partial sums of k-splits), 0 if none.
GI_API long gi_gemm_bf16_scratch_floats(int M, int N, int K) {
    if (M <= SKINNY_MAX_ROWS) return (long)gi_gemm_bf16_skinny_splits(N, K) * M * N;
    const int splits = gi_gemm_bf16_piped_splits(M, N, K);
    return splits > 1 ? (long)splits * M * N : 0;
}

// The most pieces a reader of M rows takes: what a writer of as many rows makes.
static int consumer_max_parts(int M) { return M <= 16 ? slim_max_parts(M) : M <= 32 ? TILES_MAX_PARTS : REDUCE_MAX_PARTS; }

// Whether a product of more than 128 rows takes the ping-pong kernel: 256 x 256 tiles for three quarters of the compute units or
// more.  (Measured on whole prompts, gate/up being the one product wide enough: with 192 tiles on 256 units 640 and 768 rows of
// the Llama-3.2-1B shape take 2.94 and 3.51 ms against 3.27 and 3.81 with tiles of 128 x 128, the 3B shape 7.4 and 7.6 against 8.1
// and 8.3, 320 to 512 rows of the 8B shape, 224 tiles, 10.7 to 11.0 against 12.1 to 12.5; with 128 tiles, half of the units, 512
// rows take 2.82 ms against 2.73.  Long prompts whose narrower products reach that many tiles gain as much although this kernel
// hands no norm on and the norm's own kernel runs again: 4,096 rows of the 3B shape 28.3 against 31.0 ms, 3,072 of the 8B shape
// 47.4 against 52.8.)
static bool takes_pingpong(int M, int N) { return (long)((M + 255) / 256) * ((N + 255) / 256) >= gi_compute_units() * 3 / 4; }

static const NormIn NO_NORM_IN = {nullptr, 0, 0.f, 1};
static const NormOut NO_NORM_OUT = {nullptr, nullptr, 0, nullptr};

static int reduce_partials(const float* scratch, void* C, int epi, int M, int N, int splits, long ldc, hipStream_t stream, NormIn norm_in = NO_NORM_IN,
                           NormOut norm_out = NO_NORM_OUT) {
    if (epi == EPI_GATED_BF16) {
        GI_REQUIRE(norm_in.squares == nullptr, "gemm_bf16: a gated product whose k is shared out cannot finish a norm handed on");
        skinny_reduce_gated_kernel<<<(unsigned)(((size_t)M * (N / 2) + 255) / 256), 256, 0, stream>>>(scratch, (bf16_t*)C, M, N, splits, ldc);
    } else {
#define REDUCE(VEC_)                                                                                                                    \
    do {                                                                                                                                \
        const unsigned blocks = (unsigned)(((size_t)M * N / VEC_ + 255) / 256);                                                         \
        if (epi == EPI_STORE_F32) skinny_reduce_kernel<EPI_STORE_F32, VEC_><<<blocks, 256, 0, stream>>>(scratch, C, M, N, splits, ldc, norm_in, norm_out);  \
        else if (epi == EPI_ADD_F32) skinny_reduce_kernel<EPI_ADD_F32, VEC_><<<blocks, 256, 0, stream>>>(scratch, C, M, N, splits, ldc, norm_in, norm_out); \
        else skinny_reduce_kernel<EPI_STORE_BF16, VEC_><<<blocks, 256, 0, stream>>>(scratch, C, M, N, splits, ldc, norm_in, norm_out);                      \
    } while (0)
        const bool four = N % 4 == 0 && ldc % 4 == 0 && ((uintptr_t)scratch & 15) == 0 && ((uintptr_t)C & 15) == 0;
        GI_REQUIRE(norm_out.scaled == nullptr || (four && epi == EPI_ADD_F32 && N % REDUCE_COLUMNS == 0 && N / REDUCE_COLUMNS <= REDUCE_MAX_PARTS && norm_out.ld % 4 == 0 &&
                                                  ((uintptr_t)norm_out.scaled & 7) == 0 && ((uintptr_t)norm_out.g & 15) == 0),
                   "gemm_bf16: handing a norm on from %d rows needs rows of a multiple of %d columns, at most %d, and aligned operands", M, REDUCE_COLUMNS,
                   REDUCE_COLUMNS * REDUCE_MAX_PARTS);
        if (four) REDUCE(4); else REDUCE(1);
#undef REDUCE
    }
    GI_CHECK_LAUNCH("gemm_bf16 (reduce)");
    return 0;
}

// Up to 16 rows the slim kernel (no LDS staging, one launch) is the faster one, except for wide outputs with more
// than a few rows, where its per-workgroup reading of the activations costs more than the skinny kernel's staging
// (measured crossovers, whole decode steps: 12 rows for 256 strips of 64 columns at K = 2048, 8 to 9 rows for 256 strips at
// K = 3072, 3 rows for 448 strips at K = 4096, where the 8B shape's step lost 3 to 5 % at 6 to 10 rows with the crossover at 12;
// 5 rows for the 2004 strips of the vocabulary at K = 2048): the longer the rows and the more strips, the sooner, as
// 12 * (2048 / K) * (256 / strips), between 3 and 12.
static bool takes_slim(int M, int N, int K) {
    const int strips64 = (N + 63) / 64;
    const double fitted = 12.0 * (2048.0 / K) * (256.0 / strips64);
    const int wide_rows = strips64 >= 1024 ? 5 : fitted < 3 ? 3 : fitted > 12 ? 12 : (int)(fitted + 0.5);
    const bool wide_skinny = gi_gemm_bf16_skinny_splits(N, K) == 0 && M >= wide_rows;
    return M <= 16 && !wide_skinny;
}

// Workgroups of the slim kernel for an output of N columns that is not gated: the pieces a row's sum of squares comes in.
// (A product that adds onto rows may hand a norm on, with one piece of the rows' sums of squares per workgroup: it takes strips
// of 8 only where the reader takes that many pieces.  N = 3072 at 9 to 16 rows: 384 strips of 8 would be more than the 256 pieces
// a reader of so many rows takes, and the norm's own kernel would run twice a layer; 192 strips of 16 hand it on.)
static bool slim_wide_strips(int M, int N, int epi) {
    const bool doubled = M <= 8 && (epi != EPI_ADD_F32 || M <= 3);
    const bool few = (N + 15) / 16 <= (doubled ? 2 * SLIM_NARROW_STRIPS : SLIM_NARROW_STRIPS) - 1;
    return !(few && (epi != EPI_ADD_F32 || (N + 7) / 8 <= slim_max_parts(M)));
}
// Weight rows per workgroup of the slim kernel for an output that is not gated: 16 or 8 by the rules above, unless that many
// workgroups fill the compute units unevenly (384 strips of 8 or 192 of 16 on 256 units: a quarter of the chip waits for the
// rest) and strips of 12 or 10 rows fill them evenly (3,072 columns: 256 strips of 12) with no more pieces than a reader takes.
// A product's 16 weight rows beyond such a strip repeat its last row (the same cache line, no further traffic) and their results
// are dropped.  Measured on the decode step: the 1B shape (q/k/v of 3,072 columns) 1 to 2 % faster at 1 to 16 rows, the 3B shape
// (rows of 3,072: 11.7 against 12.9 us a product at 8 rows) 3 to 5 %.  640 strips of 8 (5,120 columns, five sixths even) are
// faster than 512 of 10 (11.9 against 12.9 us): the even strips are taken where the usual ones are less than four fifths even.
static int slim_strip_rows(int M, int N, int epi) {
    const int usual = slim_wide_strips(M, N, epi) ? 16 : 8, units = gi_compute_units();
    auto evenness = [&](int rows) {
        const int groups = (N + rows - 1) / rows;
        return (double)groups / ((groups + units - 1) / units * units);
    };
    if (evenness(usual) >= 0.8) return usual;
    for (int rows : {12, 10})
        if (evenness(rows) >= 0.95 && (epi != EPI_ADD_F32 || (N + rows - 1) / rows <= slim_max_parts(M))) return rows;
    return usual;
}
static int slim_parts(int M, int N) {
    const int rows = slim_strip_rows(M, N, EPI_ADD_F32);
    return (N + rows - 1) / rows;
}

static int launch_slim(const void* A, const void* W, void* C, int epi, int M, int N, int K, long lda, long ldw, long ldc, NormIn norm_in,
                       NormOut norm_out, hipStream_t stream) {
    const bool hand = norm_in.squares != nullptr || norm_out.scaled != nullptr;
#define SLIM(STRIPS_, ROWS_, EPI_)                                                                                                                     \
    do {                                                                                                                                               \
        if (hand) gemm_bf16_slim_kernel<STRIPS_, ROWS_, EPI_, true><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldw, ldc, norm_in, norm_out); \
        else gemm_bf16_slim_kernel<STRIPS_, ROWS_, EPI_, false><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldw, ldc, norm_in, norm_out);     \
    } while (0)
    if (epi == EPI_GATED_BF16) {
        dim3 grid(N / 32);
        SLIM(2, 16, EPI_GATED_BF16);
    } else if (slim_strip_rows(M, N, epi) == 16) {
        dim3 grid((N + 15) / 16);
        if (epi == EPI_STORE_F32) SLIM(1, 16, EPI_STORE_F32); else if (epi == EPI_ADD_F32) SLIM(1, 16, EPI_ADD_F32); else SLIM(1, 16, EPI_STORE_BF16);
    } else if (slim_strip_rows(M, N, epi) == 12) {     // (the last 4 of a product's 16 weight rows are the strip's last row again; their results are dropped)
        dim3 grid((N + 11) / 12);
        if (epi == EPI_STORE_F32) SLIM(1, 12, EPI_STORE_F32); else if (epi == EPI_ADD_F32) SLIM(1, 12, EPI_ADD_F32); else SLIM(1, 12, EPI_STORE_BF16);
    } else if (slim_strip_rows(M, N, epi) == 10) {
        dim3 grid((N + 9) / 10);
        if (epi == EPI_STORE_F32) SLIM(1, 10, EPI_STORE_F32); else if (epi == EPI_ADD_F32) SLIM(1, 10, EPI_ADD_F32); else SLIM(1, 10, EPI_STORE_BF16);
    } else {                                   // a narrow output: strips of 8 rows, twice the workgroups
        dim3 grid((N + 7) / 8);
#define SLIM_FOLD(EPI_, FOLD_)                                                                                                                         \
    do {                                                                                                                                               \
        if (hand) gemm_bf16_slim_kernel<1, 8, EPI_, true, FOLD_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldw, ldc, norm_in, norm_out); \
        else gemm_bf16_slim_kernel<1, 8, EPI_, false, FOLD_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldw, ldc, norm_in, norm_out);     \
    } while (0)
        // the idle halves of the products take a further 32 of k: for up to 8 rows of A on both sides, for more on the weights' side
        if (M <= 8) {
            if (epi == EPI_STORE_F32) SLIM_FOLD(EPI_STORE_F32, 1); else if (epi == EPI_ADD_F32) SLIM_FOLD(EPI_ADD_F32, 1); else SLIM_FOLD(EPI_STORE_BF16, 1);
        } else {
            if (epi == EPI_STORE_F32) SLIM_FOLD(EPI_STORE_F32, 2); else if (epi == EPI_ADD_F32) SLIM_FOLD(EPI_ADD_F32, 2); else SLIM_FOLD(EPI_STORE_BF16, 2);
        }
#undef SLIM_FOLD
    }
#undef SLIM
    GI_CHECK_LAUNCH("gemm_bf16 (slim)");
    return 0;
}

// 17 to 32 rows, a narrow output and a short k: one launch of the slim kernel with two tiles of activation rows.  Measured at
// N = 3072 and 2048, K = 2048 against the skinny kernel's partial sums and their second kernel: 9 against 13 us at 17 and 32 rows,
// 11 against 13 at 48, 13 against 13 at 64; at K = 8192 (every workgroup reads all the activations: 1 MB at 64 rows) 21 to 43 us
// against 16 to 19, so longer k and more rows stay with the skinny kernel.  Rows beyond 32 given to further workgroups of two tiles (a
// second grid dimension: 256 workgroups at 64 rows and N = 2048, each with 64 KB of weights and its own 128 KB of A) measured
// equal at 33 to 64 rows and 3 % slower in the whole step from 65 rows on: not kept.
static bool takes_slim_tiles(int M, int N, int K, int epi) {
    return !takes_slim(M, N, K) && M <= 32 && K <= 2048 && epi != EPI_GATED_BF16 && gi_gemm_bf16_skinny_splits(N, K) > 0;
}

// Weight rows per workgroup of that kernel: 16, or 12 or 8 where strips of 16 fill the compute units unevenly and those fill
// them evenly (2,048 columns: 256 strips of 8, not 128 of 16; 3,072: 256 of 12, not 192 of 16: the decode step of the 1B shape at 17 to 32
// rows 1 to 1.5 % faster), never more strips than a reader takes pieces.
static int tiles_strip_rows(int N) {
    const int units = gi_compute_units();
    auto evenness = [&](int rows) {
        const int groups = (N + rows - 1) / rows;
        return (double)groups / ((groups + units - 1) / units * units);
    };
    if (evenness(16) >= 0.8) return 16;
    for (int rows : {12, 8})
        if (evenness(rows) >= 0.95 && (N + rows - 1) / rows <= TILES_MAX_PARTS) return rows;
    return 16;
}

static int launch_slim_tiles(const void* A, const void* W, void* C, int epi, int M, int N, int K, long lda, long ldw, long ldc, NormIn norm_in,
                             NormOut norm_out, hipStream_t stream) {
    const int strip_rows = tiles_strip_rows(N);
    dim3 grid((N + strip_rows - 1) / strip_rows);
#define SLIM_TILES(MT_)                                                                                                                             \
    do {                                                                                                                                            \
        if (epi == EPI_STORE_F32) gemm_bf16_slim_tiles_kernel<MT_, EPI_STORE_F32><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldw, ldc, norm_in, norm_out, strip_rows); \
        else if (epi == EPI_ADD_F32) gemm_bf16_slim_tiles_kernel<MT_, EPI_ADD_F32><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldw, ldc, norm_in, norm_out, strip_rows); \
        else gemm_bf16_slim_tiles_kernel<MT_, EPI_STORE_BF16><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldw, ldc, norm_in, norm_out, strip_rows); \
    } while (0)
    SLIM_TILES(2);
#undef SLIM_TILES
    GI_CHECK_LAUNCH("gemm_bf16 (slim, tiles)");
    return 0;
}

// Up to 128 rows the weights are the traffic and every workgroup streams its share of them once (measured on the decode step of
// the Llama-3.2-1B shape: 72 rows took 2.69 ms through the tiles of 128 rows of the kernels for more rows, against 2.11 ms at 64 rows).
static int launch_skinny(const void* A, const void* W, void* C, int epi, int M, int N, int K, long lda, long ldw, long ldc, float* scratch,
                         long scratch_floats, NormIn norm_in, NormOut norm_out, hipStream_t stream, const RopeStore* rope = nullptr) {
    const int splits = gi_gemm_bf16_skinny_splits(N, K), mt = (M + 15) / 16;
#define SKINNY_MT(EPI_, PARTIAL_)                                                                                                   \
    do {                                                                                                                            \
        if (mt == 1) gemm_bf16_skinny_kernel<1, EPI_, PARTIAL_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, scratch, M, N, K, lda, ldw, ldc, k_per_split, norm_in); \
        else if (mt == 2) gemm_bf16_skinny_kernel<2, EPI_, PARTIAL_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, scratch, M, N, K, lda, ldw, ldc, k_per_split, norm_in); \
        else if (mt == 3) gemm_bf16_skinny_kernel<3, EPI_, PARTIAL_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, scratch, M, N, K, lda, ldw, ldc, k_per_split, norm_in); \
        else if (mt == 4) gemm_bf16_skinny_kernel<4, EPI_, PARTIAL_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, scratch, M, N, K, lda, ldw, ldc, k_per_split, norm_in); \
        else if (mt == 5) gemm_bf16_skinny_kernel<5, EPI_, PARTIAL_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, scratch, M, N, K, lda, ldw, ldc, k_per_split, norm_in); \
        else if (mt == 6) gemm_bf16_skinny_kernel<6, EPI_, PARTIAL_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, scratch, M, N, K, lda, ldw, ldc, k_per_split, norm_in); \
        else if (mt == 7) gemm_bf16_skinny_kernel<7, EPI_, PARTIAL_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, scratch, M, N, K, lda, ldw, ldc, k_per_split, norm_in); \
        else gemm_bf16_skinny_kernel<8, EPI_, PARTIAL_><<<grid, 512, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, scratch, M, N, K, lda, ldw, ldc, k_per_split, norm_in); \
    } while (0)
    GI_REQUIRE(norm_in.squares == nullptr || norm_in.parts <= consumer_max_parts(M), "gemm_bf16: %d pieces of a sum of squares, at most %d for %d rows",
               norm_in.parts, consumer_max_parts(M), M);
    if (splits == 0) {                             // a wide output: every workgroup sees all of k and finishes its columns
        GI_REQUIRE(norm_out.scaled == nullptr && rope == nullptr, "gemm_bf16: a product this wide does not hand a norm on, or its rows to the cache");
        const int k_per_split = K;
        dim3 grid((N + 63) / 64, 1);
        if (epi == EPI_GATED_BF16) SKINNY_MT(EPI_GATED_BF16, false); else if (epi == EPI_STORE_F32) SKINNY_MT(EPI_STORE_F32, false);
        else if (epi == EPI_ADD_F32) SKINNY_MT(EPI_ADD_F32, false); else SKINNY_MT(EPI_STORE_BF16, false);
        GI_CHECK_LAUNCH("gemm_bf16 (skinny)");
        return 0;
    }
    GI_REQUIRE(scratch != nullptr && scratch_floats >= (long)splits * M * N, "gemm_bf16: scratch of %ld floats needed, %ld given",
               (long)splits * M * N, scratch_floats);
    int k_per_split = (K + splits - 1) / splits;
    k_per_split = (k_per_split + KB - 1) / KB * KB;
    dim3 grid((N + 63) / 64, splits);
    SKINNY_MT(EPI_STORE_F32, true);
#undef SKINNY_MT
    GI_CHECK_LAUNCH("gemm_bf16 (skinny)");
    if (rope != nullptr) {                         // the sums go where an attention layer wants its queries, keys and values
        skinny_reduce_rope_store_kernel<<<(unsigned)(((size_t)M * N / 4 + 255) / 256), 256, 0, stream>>>(scratch, M, N, splits, norm_in, *rope);
        GI_CHECK_LAUNCH("gemm_bf16 (reduce, rotate, store)");
        return 0;
    }
    return reduce_partials(scratch, C, epi, M, N, splits, ldc, stream, norm_in, norm_out);
}

static const RopeStore NO_ROPE = {nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr, nullptr, 0, 0, 0, 0, 0};

// The pieces per row that a product of more than 128 rows writes when it hands a norm on, 0 if it cannot: one per tile of 128 columns
// from the epilogue of the kernel with tiles of 128 x 128, one per 1024 columns where k is shared out and a second kernel adds the
// shares; not from the ping-pong kernel.
static int large_norm_parts(int M, int N, int K) {
    if (K % PK != 0 || N < 128 || takes_pingpong(M, N)) return 0;
    if (gi_gemm_bf16_piped_splits(M, N, K) > 1) return N % REDUCE_COLUMNS == 0 && N / REDUCE_COLUMNS <= REDUCE_MAX_PARTS ? N / REDUCE_COLUMNS : 0;
    return N % 128 == 0 && N / 128 <= PIPED_MAX_PARTS ? N / 128 : 0;
}

// More than 128 rows, K a multiple of 64, 128 columns or more: the kernels that load their operands straight into LDS.
// `rope` != null: the sums are those of an attention layer's q/k/v product and go where it says (`epi` is then not looked at).
static int launch_large(const void* A, const void* W, void* C, int epi, int M, int N, int K, long lda, long ldw, long ldc, float* scratch,
                        long scratch_floats, NormIn norm_in, const RopeStore* rope, hipStream_t stream, NormOut norm_out = NO_NORM_OUT) {
#define PIPED(BM_, BN_, WM_, WN_, ST_, EPI_, OUT_, LDC_, SPLITS_, KPS_, SLAB_, NORM_, ROPE_)                                            \
    do {                                                                                                                                \
        constexpr int bytes = ST_ * (BM_ + BN_) * 128;                                                                                  \
        static bool raised = false;                                                                                                     \
        if (!raised) {                                                                                                                  \
            if (hipFuncSetAttribute((const void*)gemm_bf16_piped_kernel<BM_, BN_, WM_, WN_, ST_, EPI_>, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) \
                return gi_fail("gemm_bf16: cannot reserve %d bytes of LDS", bytes);                                                     \
            raised = true;                                                                                                              \
        }                                                                                                                               \
        dim3 grid((N + BN_ - 1) / BN_, (M + BM_ - 1) / BM_, SPLITS_);                                                                   \
        gemm_bf16_piped_kernel<BM_, BN_, WM_, WN_, ST_, EPI_><<<grid, 64 * WM_ * WN_, bytes, stream>>>((const bf16_t*)A, (const bf16_t*)W, OUT_, M, N, K, lda, \
                                                                                                        ldw, LDC_, KPS_, SLAB_, NORM_, ROPE_, norm_out); \
    } while (0)
#define PIPED_EPI(BM_, BN_, WM_, WN_, ST_)                                                                                              \
    do {                                                                                                                                \
        if (rope != nullptr) PIPED(BM_, BN_, WM_, WN_, ST_, EPI_QKV_ROPE, nullptr, 0L, 1, K, 0L, norm_in, *rope);                       \
        else if (epi == EPI_STORE_F32) PIPED(BM_, BN_, WM_, WN_, ST_, EPI_STORE_F32, C, ldc, 1, K, 0L, NO_NORM_IN, NO_ROPE);            \
        else if (epi == EPI_ADD_F32) PIPED(BM_, BN_, WM_, WN_, ST_, EPI_ADD_F32, C, ldc, 1, K, 0L, NO_NORM_IN, NO_ROPE);                \
        else if (epi == EPI_STORE_BF16) PIPED(BM_, BN_, WM_, WN_, ST_, EPI_STORE_BF16, C, ldc, 1, K, 0L, NO_NORM_IN, NO_ROPE);          \
        else PIPED(BM_, BN_, WM_, WN_, ST_, EPI_GATED_BF16, C, ldc, 1, K, 0L, NO_NORM_IN, NO_ROPE);                                     \
    } while (0)
    const int splits = gi_gemm_bf16_piped_splits(M, N, K);
    if (splits > 1) {                              // few tiles: k is shared out, the sums are finished by the reduce kernel
        GI_REQUIRE(scratch != nullptr && scratch_floats >= (long)splits * M * N, "gemm_bf16: scratch of %ld floats needed, %ld given",
                   (long)splits * M * N, scratch_floats);
        const int k_per_split = K / splits;
        PIPED(128, 128, 2, 2, 2, EPI_STORE_F32, scratch, (long)N, splits, k_per_split, (long)M * N, NO_NORM_IN, NO_ROPE);
        GI_CHECK_LAUNCH("gemm_bf16 (piped, split)");
        if (rope != nullptr) {
            skinny_reduce_rope_store_kernel<<<(unsigned)(((size_t)M * N / 4 + 255) / 256), 256, 0, stream>>>(scratch, M, N, splits, norm_in, *rope);
            GI_CHECK_LAUNCH("gemm_bf16 (reduce, rotate, store)");
            return 0;
        }
        return reduce_partials(scratch, C, epi, M, N, splits, ldc, stream, norm_in, norm_out);
    }
    // Measured at 2,048 rows (K = 2048 and 8192): where 256 x 256 tiles give three quarters of the compute units one or more, they halve
    // the traffic into LDS and run the two groups of waves out of step (the ping-pong kernel); otherwise 128 x 128, two
    // workgroups per unit with two stages each when there are enough tiles, else one workgroup of eight waves with four stages.
    const long tiles128 = (long)((M + 127) / 128) * ((N + 127) / 128);
    GI_REQUIRE(norm_out.scaled == nullptr || (!takes_pingpong(M, N) && large_norm_parts(M, N, K) > 0), "gemm_bf16: a product of M %d, N %d, K %d hands no norm on", M, N, K);
    GI_REQUIRE(norm_in.squares == nullptr || rope != nullptr || (epi == EPI_GATED_BF16 && takes_pingpong(M, N) && norm_in.parts <= PIPED_MAX_PARTS),
               "gemm_bf16: a product of M %d, N %d, K %d takes no norm handed on in %d pieces", M, N, K, norm_in.parts);
    if (takes_pingpong(M, N) && rope == nullptr) {     // 256 x 256 tiles for most of the compute units: the ping-pong kernel
#define PINGPONG(EPI_)                                                                                                                  \
    do {                                                                                                                                \
        constexpr int bytes = 2 * 512 * 128;                                                                                            \
        static bool raised = false;                                                                                                     \
        if (!raised) {                                                                                                                  \
            if (hipFuncSetAttribute((const void*)gemm_bf16_pingpong_kernel<256, EPI_>, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) \
                return gi_fail("gemm_bf16: cannot reserve %d bytes of LDS", bytes);                                                     \
            raised = true;                                                                                                              \
        }                                                                                                                               \
        dim3 grid((N + 255) / 256, (M + 255) / 256);                                                                                    \
        gemm_bf16_pingpong_kernel<256, EPI_><<<grid, 512, bytes, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldw, ldc, norm_in); \
    } while (0)
        GI_REQUIRE(lda < (1L << 22) && ldw < (1L << 22), "gemm_bf16: row strides %ld, %ld are too large for the tile-relative addressing", lda, ldw);
        if (epi == EPI_STORE_F32) PINGPONG(EPI_STORE_F32); else if (epi == EPI_ADD_F32) PINGPONG(EPI_ADD_F32);
        else if (epi == EPI_STORE_BF16) PINGPONG(EPI_STORE_BF16); else PINGPONG(EPI_GATED_BF16);
#undef PINGPONG
        GI_CHECK_LAUNCH("gemm_bf16 (pingpong)");
        return 0;
    }
    if (tiles128 > gi_compute_units()) PIPED_EPI(128, 128, 2, 2, 2);
    else PIPED_EPI(128, 128, 2, 4, 4);
#undef PIPED_EPI
#undef PIPED
    GI_CHECK_LAUNCH("gemm_bf16 (piped)");
    return 0;
}

// The pieces per row that a product of these sizes writes when it hands a norm on (gi_gemm_bf16_handing with `scaled_out`);
// 0 if it cannot: a shape whose kernel does not do it.  One piece per workgroup from the kernels that finish a product of up to
// 16 or 32 rows in one launch; up to 128 rows one per 1024 columns, from the kernel that adds the partial sums of the shares of k
// onto the rows.
GI_API int gi_gemm_bf16_norm_parts(int M, int N, int K) {
    if (takes_slim(M, N, K)) {
        const int parts = slim_parts(M, N);
        return parts <= slim_max_parts(M) ? parts : 0;
    }
    if (takes_slim_tiles(M, N, K, EPI_ADD_F32)) {
        const int parts = (N + tiles_strip_rows(N) - 1) / tiles_strip_rows(N);
        return parts <= TILES_MAX_PARTS ? parts : 0;
    }
    if (M > SKINNY_MAX_ROWS) return large_norm_parts(M, N, K);
    if (M <= 16 || gi_gemm_bf16_skinny_splits(N, K) == 0) return 0;
    return N % REDUCE_COLUMNS == 0 && N / REDUCE_COLUMNS <= REDUCE_MAX_PARTS ? N / REDUCE_COLUMNS : 0;
}

// Whether a product of these sizes can read rows whose norm was handed on (gi_gemm_bf16_handing with `squares_in`) by a product
// of as many rows.
GI_API int gi_gemm_bf16_takes_norm(int M, int N, int K, int gated) {
    if (takes_slim(M, N, K) || takes_slim_tiles(M, N, K, gated ? EPI_GATED_BF16 : EPI_STORE_F32)) return 1;
    if (M > SKINNY_MAX_ROWS)                      // the rows of prompts: the gated product on the ping-pong kernel scales in its epilogue
        return gated && K % PK == 0 && N >= 128 && takes_pingpong(M, N) ? 1 : 0;
    if (gi_gemm_bf16_skinny_splits(N, K) == 0) return 1;      // the weight-streaming kernel finishes its columns and scales them
    return M > 32 && !gated ? 1 : 0;                          // the kernel that adds the shares of k scales: with a few pieces only
}

// gi_gemm_bf16 for at most 128 rows, with an RMS norm handed from one product to the next instead of a kernel of its own.
// squares_in != null: the rows A are g * x of some rows x, in bfloat16, and squares_in [M, parts_in] holds the pieces of every
// row's sum of x^2; the results are multiplied by rsqrt(sum / K + eps).  scaled_out != null (needs accumulate onto 32-bit C):
// beside C += A W^T, scaled_out [M, ld_scaled] = bfloat16(g * C) and squares_out [M, gi_gemm_bf16_norm_parts(M, N, K)] = the
// pieces of the rows' sums of C^2, for the next product.  Where the two queries above say no, it fails.
GI_API int gi_gemm_bf16_handing(const void* A, const void* W, void* C, int c_dtype, int accumulate, int gated, int M, int N, int K, long lda,
                                long ldw, long ldc, float* scratch, long scratch_floats, const float* squares_in, int parts_in, float eps,
                                const float* g, void* scaled_out, long ld_scaled, float* squares_out, hipStream_t stream) {
    GI_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_bf16: M %d, N %d, K %d must be positive", M, N, K);
    GI_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_bf16: K %d and the row strides (%ld, %ld) must be multiples of 8", K, lda, ldw);
    GI_REQUIRE(((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_bf16: operands must be 16-byte aligned");
    GI_REQUIRE(lda >= K && ldw >= K && ldc >= (gated ? N / 2 : N), "gemm_bf16: leading dimensions too small");
    int epi = epilogue_of(c_dtype, accumulate);
    if (gated) {
        GI_REQUIRE(N % 32 == 0 && c_dtype == GI_BF16 && !accumulate, "gemm_bf16: the gated product needs N %% 32 == 0 and a bfloat16 output");
        epi = EPI_GATED_BF16;
    }
    GI_REQUIRE(epi >= 0, "gemm_bf16: output dtype %d with accumulate %d is not supported", c_dtype, accumulate);
    GI_REQUIRE(squares_in == nullptr || (parts_in > 0 && gi_gemm_bf16_takes_norm(M, N, K, gated)),
               "gemm_bf16: a product of these sizes (M %d, N %d, K %d%s) cannot finish a norm handed on", M, N, K, gated ? ", gated" : "");
    GI_REQUIRE(scaled_out == nullptr || (epi == EPI_ADD_F32 && g != nullptr && squares_out != nullptr && ld_scaled >= N && gi_gemm_bf16_norm_parts(M, N, K) > 0),
               "gemm_bf16: handing a norm on needs a product that adds onto 32-bit rows, of sizes that allow it (M %d, N %d, K %d), the norm's weights and "
               "room for the sums of squares", M, N, K);
    const NormIn norm_in = {squares_in, parts_in, eps, K};
    const NormOut norm_out = {g, (bf16_t*)scaled_out, ld_scaled, squares_out};
    if (takes_slim(M, N, K)) {
        GI_REQUIRE(squares_in == nullptr || parts_in <= slim_max_parts(M), "gemm_bf16: %d pieces of a sum of squares, at most %d", parts_in, slim_max_parts(M));
        return launch_slim(A, W, C, epi, M, N, K, lda, ldw, ldc, norm_in, norm_out, stream);
    }
    if (takes_slim_tiles(M, N, K, epi)) {
        GI_REQUIRE(squares_in == nullptr || parts_in <= consumer_max_parts(M), "gemm_bf16: %d pieces of a sum of squares, at most %d", parts_in, consumer_max_parts(M));
        return launch_slim_tiles(A, W, C, epi, M, N, K, lda, ldw, ldc, norm_in, norm_out, stream);
    }
    if (M > SKINNY_MAX_ROWS) {                   // the rows of prompts: a norm is handed on (to a q/k/v product that takes it), none is taken
        GI_REQUIRE(scaled_out == nullptr || (ldc % 4 == 0 && ld_scaled % 4 == 0 && ((uintptr_t)C & 15) == 0 && ((uintptr_t)scaled_out & 7) == 0 && ((uintptr_t)g & 15) == 0),
                   "gemm_bf16: handing a norm on from %d rows needs aligned operands", M);
        return launch_large(A, W, C, epi, M, N, K, lda, ldw, ldc, scratch, scratch_floats, norm_in, nullptr, stream, norm_out);
    }
    return launch_skinny(A, W, C, epi, M, N, K, lda, ldw, ldc, scratch, scratch_floats, norm_in, norm_out, stream);
}

// Whether gi_gemm_bf16_qkv_rope_store takes a q/k/v product of these sizes with heads of hd channels.  17 or 33 to 128 rows: the
// shapes whose k is shared out over workgroups, whose sums a second kernel adds up anyway.  More rows: the kernels with tiles of
// 128 x 128, whose epilogue lays the tile into LDS and sends it off rotated (whole heads must lie inside a tile), or, where they
// share k out, that second kernel again; not where the ping-pong kernel with its larger tiles is the faster product.
GI_API int gi_gemm_bf16_qkv_rope_store_takes(int M, int N, int K, int hd) {
    if (hd < 8 || hd > 256 || (hd & (hd - 1)) != 0) return 0;
    if (M <= SKINNY_MAX_ROWS)
        return !takes_slim(M, N, K) && !takes_slim_tiles(M, N, K, EPI_STORE_F32) && gi_gemm_bf16_skinny_splits(N, K) > 0 && N % 256 == 0 ? 1 : 0;
    if (K % PK != 0 || N < 128 || takes_pingpong(M, N)) return 0;
    return gi_gemm_bf16_piped_splits(M, N, K) > 1 ? N % 256 == 0 : hd <= 128;
}

// The most pieces of a row's sum of squares that gi_gemm_bf16_qkv_rope_store reads for a product of M rows.
GI_API int gi_gemm_bf16_qkv_rope_store_max_parts(int M, int N, int K) {
    return M <= SKINNY_MAX_ROWS || gi_gemm_bf16_piped_splits(M, N, K) > 1 ? REDUCE_MAX_PARTS : PIPED_MAX_PARTS;
}

// The q/k/v product of an attention layer, A [M, K] x W [N, K]^T with N = (n_heads + 2 n_kv) * hd, whose results do not come back:
// the queries go, rotated, to q_out [M, n_heads * hd] in bfloat16, the keys (rotated) and values into the pages of a bfloat16
// cache, as gi_rope_store would put them (cos_t, sin_t [M, hd/2] or both null; pos, slot [M]; table, cache, page_stride, page_size
// as there).  squares_in, parts_in, eps: a norm handed on, as for gi_gemm_bf16_handing (null: none).
GI_API int gi_gemm_bf16_qkv_rope_store(const void* A, const void* W, int M, int N, int K, long lda, long ldw, float* scratch, long scratch_floats,
                                       const float* squares_in, int parts_in, float eps, const float* cos_t, const float* sin_t, const int* pos,
                                       const int* slot, const int* table, int table_stride, void* q_out, void* cache, long page_stride, int page_size,
                                       int n_heads, int n_kv, int hd, hipStream_t stream) {
    GI_REQUIRE(M > 0 && N > 0 && K > 0 && n_heads > 0 && n_kv > 0 && hd > 0 && N == (n_heads + 2 * n_kv) * hd,
               "gemm_bf16 (q/k/v): M %d, N %d, K %d, %d heads, %d key/value heads of %d do not fit together", M, N, K, n_heads, n_kv, hd);
    GI_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K, "gemm_bf16: K %d and the row strides (%ld, %ld) must be multiples of 8", K, lda, ldw);
    GI_REQUIRE(((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0 && ((uintptr_t)scratch & 15) == 0, "gemm_bf16: operands must be 16-byte aligned");
    GI_REQUIRE(gi_gemm_bf16_qkv_rope_store_takes(M, N, K, hd), "gemm_bf16 (q/k/v): sizes M %d, N %d, K %d, heads of %d are not taken", M, N, K, hd);
    GI_REQUIRE((cos_t == nullptr) == (sin_t == nullptr) && ((uintptr_t)cos_t & 15) == 0 && ((uintptr_t)sin_t & 15) == 0,
               "gemm_bf16 (q/k/v): cos and sin must both be given or both be absent, 16-byte aligned");
    GI_REQUIRE(pos != nullptr && slot != nullptr && table != nullptr && q_out != nullptr && cache != nullptr && page_size > 0 &&
               page_stride >= 2L * n_kv * page_size * hd && ((uintptr_t)q_out & 7) == 0 && ((uintptr_t)cache & 7) == 0 && page_stride % 4 == 0,
               "gemm_bf16 (q/k/v): positions, slots, a table, q_out and a cache with a page stride of at least 2*n_kv*page_size*hd are needed");
    GI_REQUIRE(squares_in == nullptr || (parts_in > 0 && parts_in <= gi_gemm_bf16_qkv_rope_store_max_parts(M, N, K)),
               "gemm_bf16 (q/k/v): %d pieces of a sum of squares, at most %d", parts_in, gi_gemm_bf16_qkv_rope_store_max_parts(M, N, K));
    const RopeStore rope = {cos_t, sin_t, pos, slot, table, table_stride, (bf16_t*)q_out, (bf16_t*)cache, page_stride, page_size, n_heads, n_kv, hd};
    if (M > SKINNY_MAX_ROWS)
        return launch_large(A, W, nullptr, EPI_STORE_F32, M, N, K, lda, ldw, (long)N, scratch, scratch_floats, NormIn{squares_in, parts_in, eps, K}, &rope, stream);
    return launch_skinny(A, W, nullptr, EPI_STORE_F32, M, N, K, lda, ldw, (long)N, scratch, scratch_floats, NormIn{squares_in, parts_in, eps, K}, NO_NORM_OUT,
                         stream, &rope);
}

// `gated` != 0: W is [gate; up] interleaved in groups of 16 rows (N rows in all, a multiple of 32)
// and C is bfloat16 [M, N/2] = silu(gate) * up.
GI_API int gi_gemm_bf16(const void* A, const void* W, void* C, int c_dtype, int accumulate, int gated, int M, int N, int K, long lda,
                        long ldw, long ldc, float* scratch, long scratch_floats, hipStream_t stream) {
    GI_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_bf16: M %d, N %d, K %d must be positive", M, N, K);
    GI_REQUIRE(K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0, "gemm_bf16: K %d and the row strides (%ld, %ld) must be multiples of 8", K, lda, ldw);
    GI_REQUIRE(((uintptr_t)A & 15) == 0 && ((uintptr_t)W & 15) == 0, "gemm_bf16: operands must be 16-byte aligned");
    GI_REQUIRE(lda >= K && ldw >= K && ldc >= (gated ? N / 2 : N), "gemm_bf16: leading dimensions too small");
    int epi = epilogue_of(c_dtype, accumulate);
    if (gated) {
        GI_REQUIRE(N % 32 == 0 && c_dtype == GI_BF16 && !accumulate, "gemm_bf16: the gated product needs N %% 32 == 0 and a bfloat16 output");
        epi = EPI_GATED_BF16;
    }
    GI_REQUIRE(epi >= 0, "gemm_bf16: output dtype %d with accumulate %d is not supported", c_dtype, accumulate);

    if (takes_slim(M, N, K)) return launch_slim(A, W, C, epi, M, N, K, lda, ldw, ldc, NO_NORM_IN, NO_NORM_OUT, stream);

    if (takes_slim_tiles(M, N, K, epi)) return launch_slim_tiles(A, W, C, epi, M, N, K, lda, ldw, ldc, NO_NORM_IN, NO_NORM_OUT, stream);
    if (M <= SKINNY_MAX_ROWS) return launch_skinny(A, W, C, epi, M, N, K, lda, ldw, ldc, scratch, scratch_floats, NO_NORM_IN, NO_NORM_OUT, stream);

    GI_REQUIRE((M + 63) / 64 <= 65535, "gemm_bf16: M %d is too large", M);
    if (K % PK == 0 && N >= 128) return launch_large(A, W, C, epi, M, N, K, lda, ldw, ldc, scratch, scratch_floats, NO_NORM_IN, nullptr, stream);
#define TILED(BM_, EPI_) gemm_bf16_tiled_kernel<BM_, EPI_><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, C, M, N, K, lda, ldw, ldc)
    if ((long)((M + 127) / 128) * ((N + BN - 1) / BN) < 512) {   // few tiles: smaller ones fill more of the chip
        dim3 grid((N + BN - 1) / BN, (M + 63) / 64);
        if (epi == EPI_STORE_F32) TILED(64, EPI_STORE_F32); else if (epi == EPI_ADD_F32) TILED(64, EPI_ADD_F32);
        else if (epi == EPI_STORE_BF16) TILED(64, EPI_STORE_BF16); else TILED(64, EPI_GATED_BF16);
    } else {
        dim3 grid((N + BN - 1) / BN, (M + 127) / 128);
        if (epi == EPI_STORE_F32) TILED(128, EPI_STORE_F32); else if (epi == EPI_ADD_F32) TILED(128, EPI_ADD_F32);
        else if (epi == EPI_STORE_BF16) TILED(128, EPI_STORE_BF16); else TILED(128, EPI_GATED_BF16);
    }
#undef TILED
    GI_CHECK_LAUNCH("gemm_bf16 (tiled)");
    return 0;
}
