// C[M, N] = A[M, K] . W[N, K]^T with float32 accumulation on the vector ALUs, for any
// M, N, K and any alignment.  This is the matrix product of the float32 path (no
// reduced-precision matrix mode: plain fmaf) and the fallback for shapes that the bf16
// matrix-core kernels refuse.  W is row-major [out, in] as the reference keeps it
// (src/model.c:157-158); out[row] = sum_col W[row, col] x[col]
// (src/quant/f32_scalar.c:4-32, src/quant/bf16_scalar.c:4-21).
//
// Every output element is summed over k = 0 .. K-1 in that order with fmaf, whatever M
// and N are and whichever tile variant runs, so a row's result does not depend on how
// many other rows are in the batch.
#include "common.h"

#define GT_BN 64
#define GT_BK 16

template <typename TA, typename TW, typename TO, int BM>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                         TO* __restrict__ C, int M, int N, int K,
                                                         int lda, int ldw, int ldc) {
    constexpr int TM = BM / 16;
    __shared__ float As[GT_BK][BM + 1];
    __shared__ float Ws[GT_BK][GT_BN + 1];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * GT_BN;
    float acc[TM][4];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GT_BK) {
        for (int idx = tid; idx < BM * GT_BK; idx += 256) {
            const int r = idx / GT_BK, kk = idx - r * GT_BK;
            const int m = m0 + r, k = k0 + kk;
            As[kk][r] = (m < M && k < K) ? to_f32(A[(size_t)m * lda + k]) : 0.f;
        }
        for (int idx = tid; idx < GT_BN * GT_BK; idx += 256) {
            const int r = idx / GT_BK, kk = idx - r * GT_BK;
            const int n = n0 + r, k = k0 + kk;
            Ws[kk][r] = (n < N && k < K) ? to_f32(W[(size_t)n * ldw + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GT_BK; ++kk) {
            float a[TM], w[4];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = As[kk][ty * TM + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + ty * TM + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) C[(size_t)m * ldc + n] = from_f32<TO>(acc[i][j]);
        }
    }
}

template <typename TA, typename TW, typename TO>
static int launch(const void* A, const void* W, void* C, int M, int N, int K, int lda, int ldw, int ldc,
                  hipStream_t s) {
    const unsigned gx = (N + GT_BN - 1) / GT_BN;
    if (M <= 16) {
        hipLaunchKernelGGL((gemm_tiled_kernel<TA, TW, TO, 16>), dim3(gx, (M + 15) / 16), dim3(256), 0, s,
                           (const TA*)A, (const TW*)W, (TO*)C, M, N, K, lda, ldw, ldc);
    } else {
        hipLaunchKernelGGL((gemm_tiled_kernel<TA, TW, TO, 64>), dim3(gx, (M + 63) / 64), dim3(256), 0, s,
                           (const TA*)A, (const TW*)W, (TO*)C, M, N, K, lda, ldw, ldc);
    }
    return bn_launch_status();
}

// in_dtype: type of A and W; out_dtype: type of C (float32 output from bf16 inputs is allowed).
extern "C" int bn_gemm_tiled(int in_dtype, int out_dtype, const void* A, const void* W, void* C, int M,
                             int N, int K, int lda, int ldw, int ldc, hipStream_t s) {
    if (M <= 0 || N <= 0 || K <= 0 || lda < K || ldw < K || ldc < N) return BN_ERR_ARG;
    if ((M + 15) / 16 > 65535) return BN_ERR_ARG;
    if (in_dtype == BN_DT_F32 && out_dtype == BN_DT_F32)
        return launch<float, float, float>(A, W, C, M, N, K, lda, ldw, ldc, s);
    if (in_dtype == BN_DT_BF16 && out_dtype == BN_DT_BF16)
        return launch<bf16, bf16, bf16>(A, W, C, M, N, K, lda, ldw, ldc, s);
    if (in_dtype == BN_DT_BF16 && out_dtype == BN_DT_F32)
        return launch<bf16, bf16, float>(A, W, C, M, N, K, lda, ldw, ldc, s);
    return BN_ERR_DTYPE;
}
