// C[m, n] (=|+=) sum_k A[m, k] * W[n, k] in true 32-bit arithmetic.
//
// Both operands are row-major with k contiguous (activations [M, K], weights [N, K] as checkpoints
// store them).  Every output element is one chain of fused multiply-adds over k = 0 .. K-1 in
// ascending order, whatever M is and wherever the row lies in the batch: a row computed alone
// has the same bits as the same row inside a large batch (the reference keeps the same rule,
// src/gpu/device_kernels.inc:97-100).  Operands may be stored as bfloat16; they are widened
// exactly.  This kernel is the 32-bit path of every matrix product, and the slow stand-in of the
// bfloat16 path for shapes the matrix-core kernels refuse.
#include "common.h"

namespace {

constexpr int BM = 64, BN = 64, BK = 16, PAD = 4;

template <typename TA, typename TW, typename TC, bool ACCUMULATE>
__global__ __launch_bounds__(256) void gemm_exact_kernel(const TA* __restrict__ A, const TW* __restrict__ W, TC* __restrict__ C, int M, int N,
                                                         int K, long lda, long ldw, long ldc) {
    __shared__ float As[BK][BM + PAD];
    __shared__ float Ws[BK][BN + PAD];
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int e = tid + 256 * r, row = e >> 4, kk = e & 15;
            const int m = m0 + row, n = n0 + row, k = k0 + kk;
            As[kk][row] = (m < M && k < K) ? load_f32(A, (size_t)m * lda + k) : 0.f;
            Ws[kk][row] = (n < N && k < K) ? load_f32(W, (size_t)n * ldw + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                a[i] = As[kk][ty * 4 + i];
                w[i] = Ws[kk][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            const size_t o = (size_t)m * ldc + n;
            if constexpr (ACCUMULATE) store_f32(C, o, load_f32(C, o) + acc[i][j]);
            else store_f32(C, o, acc[i][j]);
        }
    }
}

// The same product for at most FEW_ROWS rows of 32-bit activations (decoding): one lane per output column walks its
// weight row alone, so that a product with a handful of rows is spread over N lanes instead of N / 64 workgroups.
// Every output is the same chain of fused multiply-adds over ascending k as in the kernel above: the bits do not
// depend on which of the two kernels a row met.  A lane reads 16 bytes of its own row at a time (the rows of a
// wave's lanes are K elements apart, so a cache line a lane has touched serves its next loads); the activations
// are the same for all lanes.
constexpr int FEW_ROWS = 4;

template <typename TW> struct Sixteen;                      // 16 bytes of a weight row, widened
template <> struct Sixteen<float> {
    static constexpr int N = 4;
    static __device__ __forceinline__ void load(const float* p, float (&w)[4]) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
    }
};
template <> struct Sixteen<bf16_t> {
    static constexpr int N = 8;
    static __device__ __forceinline__ void load(const bf16_t* p, float (&w)[8]) {
        const uint4 v = *reinterpret_cast<const uint4*>(p);
        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            w[2 * i] = __uint_as_float(u[i] << 16);
            w[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
        }
    }
};

template <typename TW, bool ACCUMULATE, int MR>
__global__ __launch_bounds__(64) void gemm_exact_few_rows_kernel(const float* __restrict__ A, const TW* __restrict__ W, float* __restrict__ C, int M,
                                                                 int N, int K, long lda, long ldw, long ldc) {
    constexpr int PIECE = Sixteen<TW>::N, AHEAD = 32;        // elements per load; loads in flight per lane (512 bytes: four cache lines of its row)
    const int n = blockIdx.x * 64 + threadIdx.x;
    const TW* wrow = W + (size_t)min(n, N - 1) * ldw;
    float acc[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[m] = 0.f;
    const int k_whole = K - K % (PIECE * AHEAD);
    for (int k0 = 0; k0 < k_whole; k0 += PIECE * AHEAD) {
        float w[AHEAD][PIECE];
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) Sixteen<TW>::load(wrow + k0 + u * PIECE, w[u]);
#pragma unroll
        for (int u = 0; u < AHEAD; ++u)
#pragma unroll
            for (int j = 0; j < PIECE; ++j)
#pragma unroll
                for (int m = 0; m < MR; ++m)
                    if (m < M) acc[m] = fmaf(A[(size_t)m * lda + k0 + u * PIECE + j], w[u][j], acc[m]);
    }
    for (int k = k_whole; k < K; ++k) {
        const float w = load_f32(wrow, (size_t)k);
#pragma unroll
        for (int m = 0; m < MR; ++m)
            if (m < M) acc[m] = fmaf(A[(size_t)m * lda + k], w, acc[m]);
    }
    if (n >= N) return;
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        if (m >= M) break;
        const size_t o = (size_t)m * ldc + n;
        C[o] = ACCUMULATE ? C[o] + acc[m] : acc[m];
    }
}

template <typename TW>
int launch_few_rows(const void* A, const void* W, void* C, int accumulate, int M, int N, int K, long lda, long ldw, long ldc, hipStream_t stream) {
    const unsigned blocks = (unsigned)((N + 63) / 64);
#define FEW(ACC, MR) gemm_exact_few_rows_kernel<TW, ACC, MR><<<blocks, 64, 0, stream>>>((const float*)A, (const TW*)W, (float*)C, M, N, K, lda, ldw, ldc)
    if (M == 1) { if (accumulate) FEW(true, 1); else FEW(false, 1); }
    else if (M == 2) { if (accumulate) FEW(true, 2); else FEW(false, 2); }
    else { if (accumulate) FEW(true, FEW_ROWS); else FEW(false, FEW_ROWS); }
#undef FEW
    return 0;
}

template <typename TA, typename TW>
int launch(const void* A, const void* W, void* C, int c_dtype, int accumulate, int M, int N, int K, long lda, long ldw, long ldc,
           hipStream_t stream) {
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
#define GO(TC, ACC) gemm_exact_kernel<TA, TW, TC, ACC><<<grid, 256, 0, stream>>>((const TA*)A, (const TW*)W, (TC*)C, M, N, K, lda, ldw, ldc)
    if (c_dtype == GI_F32 && accumulate) GO(float, true);
    else if (c_dtype == GI_F32) GO(float, false);
    else if (c_dtype == GI_BF16 && !accumulate) GO(bf16_t, false);
    else return gi_fail("gemm_exact: output dtype %d with accumulate %d is not supported", c_dtype, accumulate);
#undef GO
    return 0;
}

}  // namespace

GI_API int gi_gemm_exact(const void* A, int a_dtype, const void* W, int w_dtype, void* C, int c_dtype, int accumulate, int M, int N, int K,
                         long lda, long ldw, long ldc, hipStream_t stream) {
    GI_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_exact: M %d, N %d, K %d must be positive", M, N, K);
    GI_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_exact: leading dimensions (%ld, %ld, %ld) too small for K %d, N %d", lda, ldw, ldc, K, N);
    GI_REQUIRE((M + BM - 1) / BM <= 65535, "gemm_exact: M %d is too large", M);
    int rc;
    // a few rows of 32-bit activations into a 32-bit result: a lane per output column (the loads need 16-byte pieces of the weight rows)
    const long w_piece = w_dtype == GI_F32 ? 4 : 8;
    if (M <= FEW_ROWS && a_dtype == GI_F32 && c_dtype == GI_F32 && (w_dtype == GI_F32 || w_dtype == GI_BF16) && ldw % w_piece == 0 &&
        ((uintptr_t)W & 15) == 0) {
        rc = w_dtype == GI_F32 ? launch_few_rows<float>(A, W, C, accumulate, M, N, K, lda, ldw, ldc, stream)
                               : launch_few_rows<bf16_t>(A, W, C, accumulate, M, N, K, lda, ldw, ldc, stream);
        GI_CHECK_LAUNCH("gemm_exact (few rows)");
        return rc;
    }
    if (a_dtype == GI_F32 && w_dtype == GI_F32) rc = launch<float, float>(A, W, C, c_dtype, accumulate, M, N, K, lda, ldw, ldc, stream);
    else if (a_dtype == GI_F32 && w_dtype == GI_BF16) rc = launch<float, bf16_t>(A, W, C, c_dtype, accumulate, M, N, K, lda, ldw, ldc, stream);
    else if (a_dtype == GI_BF16 && w_dtype == GI_BF16) rc = launch<bf16_t, bf16_t>(A, W, C, c_dtype, accumulate, M, N, K, lda, ldw, ldc, stream);
    else if (a_dtype == GI_BF16 && w_dtype == GI_F32) rc = launch<bf16_t, float>(A, W, C, c_dtype, accumulate, M, N, K, lda, ldw, ldc, stream);
    else return gi_fail("gemm_exact: unknown operand dtypes %d, %d", a_dtype, w_dtype);
    if (rc) return rc;
    GI_CHECK_LAUNCH("gemm_exact");
    return 0;
}
