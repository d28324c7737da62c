// Matrix products C[M, N] = A[M, K] . B[N, K]^T (weights are [out, in] row-major
// like the reference's Linear, src/layers/linear.cu:169-215, which calls
// cublasSgemm).  This file holds the true 32-bit product (plain FMA, no matrix
// cores, no reduced-precision mode) and 16-bit-in / 32-bit-accumulate variants
// of the same tiling; the sum over k runs in index order whatever M is, so a
// row's result does not depend on what else is in the batch.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

template <typename TA, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_simt_kernel(const TA* __restrict__ A, const TA* __restrict__ B,
                                                           TC* __restrict__ C, int M, int N, int K, int64_t lda,
                                                           int64_t ldb, int64_t ldc) {
    __shared__ float As[GT_BK][GT_BM + 4];
    __shared__ float Bs[GT_BK][GT_BN + 4];
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const int64_t m0 = (int64_t)blockIdx.y * GT_BM, n0 = (int64_t)blockIdx.x * GT_BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GT_BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = threadIdx.x + 256 * i;
            const int r = idx / GT_BK, c = idx % GT_BK;
            const bool kin = k0 + c < K;
            As[c][r] = (kin && m0 + r < M) ? to_f32<TA>(A[(m0 + r) * lda + k0 + c]) : 0.f;
            Bs[c][r] = (kin && n0 + r < N) ? to_f32<TA>(B[(n0 + r) * ldb + k0 + c]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GT_BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t n = n0 + tx * 4 + j;
            if (n < N) C[m * ldc + n] = from_f32<TC>(acc[i][j]);
        }
    }
}

// in_dtype: type of A and B; out_dtype: type of C
extern "C" int lle_gemm_nt_simt(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda,
                                int64_t ldb, int64_t ldc, int in_dtype, int out_dtype, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM);
    if (grid.y > 65535) return (int)hipErrorInvalidValue;
    if (in_dtype == LLE_F32 && out_dtype == LLE_F32)
        gemm_nt_simt_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)A, (const float*)B, (float*)C, M,
                                                                     N, K, lda, ldb, ldc);
    else if (in_dtype == LLE_BF16 && out_dtype == LLE_F32)
        gemm_nt_simt_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)B, (float*)C,
                                                                      M, N, K, lda, ldb, ldc);
    else if (in_dtype == LLE_BF16 && out_dtype == LLE_BF16)
        gemm_nt_simt_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)B,
                                                                       (bf16_t*)C, M, N, K, lda, ldb, ldc);
    else
        return (int)hipErrorInvalidValue;
    LLE_RETURN_LAUNCH_STATUS();
}
