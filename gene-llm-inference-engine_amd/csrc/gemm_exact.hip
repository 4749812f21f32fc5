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
    if (a_dtype == GI_F32 && w_dtype == GI_F32) rc = launch<float, float>(A, W, C, c_dtype, accumulate, M, N, K, lda, ldw, ldc, stream);
    else if (a_dtype == GI_F32 && w_dtype == GI_BF16) rc = launch<float, bf16_t>(A, W, C, c_dtype, accumulate, M, N, K, lda, ldw, ldc, stream);
    else if (a_dtype == GI_BF16 && w_dtype == GI_BF16) rc = launch<bf16_t, bf16_t>(A, W, C, c_dtype, accumulate, M, N, K, lda, ldw, ldc, stream);
    else if (a_dtype == GI_BF16 && w_dtype == GI_F32) rc = launch<bf16_t, float>(A, W, C, c_dtype, accumulate, M, N, K, lda, ldw, ldc, stream);
    else return gi_fail("gemm_exact: unknown operand dtypes %d, %d", a_dtype, w_dtype);
    if (rc) return rc;
    GI_CHECK_LAUNCH("gemm_exact");
    return 0;
}
