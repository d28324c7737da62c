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

// ---------------------------------------------------------------------------------
// Skinny product for decoding: M <= 64 rows of activations against a weight
// matrix that is read exactly once.  bfloat16 in, 32-bit accumulate, bfloat16 or
// 32-bit out.  HBM-bound: the kernel is shaped to keep whole 128-byte lines of W
// in flight from all CUs.
//   workgroup = 16 rows of W (one matrix-core tile), 8 wavefronts split K:
//   wavefront w takes the 64-element k steps w, w + 8, ... (neighbouring
//   wavefronts read neighbouring 128-byte pieces of the same rows);
//   C^T tile = W tile [16 n x 64 k] . X^T [64 k x 16 m] by two
//   v_mfma_f32_16x16x32_bf16 per 16 rows of X; lane (c = lane / 16, r = lane % 16)
//   loads 32 contiguous bytes W[n0 + r][k0 + 16c .. + 15]; X comes from L2.
//   The 8 partial tiles are added in LDS in wavefront order, so the sum over k
//   has one fixed order for every M.
// ---------------------------------------------------------------------------------
typedef bf16_t gbf16x8 __attribute__((ext_vector_type(8)));
typedef float gf32x4 __attribute__((ext_vector_type(4)));

#define SK_WAVES 8
#define SK_KSTEP 64

template <int MT, typename TC>
__global__ __launch_bounds__(SK_WAVES* LLE_WAVE) void gemm_skinny_kernel(const bf16_t* __restrict__ X,
                                                                         const bf16_t* __restrict__ W,
                                                                         TC* __restrict__ C, int M, int N, int K) {
    __shared__ float s_acc[SK_WAVES][MT][16][17];
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int c = lane / 16, r16 = lane % 16;
    const int64_t n0 = (int64_t)blockIdx.x * 16;
    const int64_t wrow = min(n0 + r16, (int64_t)N - 1);
    const bf16_t* wp = W + wrow * K + 16 * c;
    const bf16_t* xp[MT];
    bool xok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = 16 * mt + r16;
        xok[mt] = m < M;
        xp[mt] = X + (int64_t)(xok[mt] ? m : 0) * K + 16 * c;
    }
    gf32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = gf32x4{0.f, 0.f, 0.f, 0.f};
    const gbf16x8 zero = {(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f,
                          (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};

    const int full_steps = K / SK_KSTEP;
    int ss = wave;
#pragma unroll 4
    for (; ss < full_steps; ss += SK_WAVES) {
        const int k0 = ss * SK_KSTEP;
        const gbf16x8 w0 = *(const gbf16x8*)(wp + k0);
        const gbf16x8 w1 = *(const gbf16x8*)(wp + k0 + 8);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            gbf16x8 x0 = zero, x1 = zero;
            if (xok[mt]) {
                x0 = *(const gbf16x8*)(xp[mt] + k0);
                x1 = *(const gbf16x8*)(xp[mt] + k0 + 8);
            }
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, x0, acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, x1, acc[mt], 0, 0, 0);
        }
    }
    // the tail of K (a multiple of 8): one more step, taken by the wavefront whose turn it is
    if (full_steps * SK_KSTEP < K && ss == full_steps) {
        const int k0 = full_steps * SK_KSTEP;
        const bool in0 = k0 + 16 * c + 8 <= K, in1 = k0 + 16 * c + 16 <= K;
        const gbf16x8 w0 = in0 ? *(const gbf16x8*)(wp + k0) : zero;
        const gbf16x8 w1 = in1 ? *(const gbf16x8*)(wp + k0 + 8) : zero;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const gbf16x8 x0 = (in0 && xok[mt]) ? *(const gbf16x8*)(xp[mt] + k0) : zero;
            const gbf16x8 x1 = (in1 && xok[mt]) ? *(const gbf16x8*)(xp[mt] + k0 + 8) : zero;
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, x0, acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, x1, acc[mt], 0, 0, 0);
        }
    }
    // lane holds C^T[n = 4c + i][m = r16]
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) s_acc[wave][mt][4 * c + i][r16] = acc[mt][i];
    __syncthreads();
    for (int idx = threadIdx.x; idx < MT * 256; idx += blockDim.x) {
        const int mt = idx / 256, m = (idx / 16) % 16, n = idx % 16;
        const int64_t row = 16 * mt + m, col = n0 + n;
        if (row >= M || col >= N) continue;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) sum += s_acc[w][mt][n][m];
        C[row * N + col] = from_f32<TC>(sum);
    }
}

template <typename TC>
static int launch_skinny(const bf16_t* X, const bf16_t* W, TC* C, int M, int N, int K, hipStream_t stream) {
    const int blocks = (N + 15) / 16;
    const int mt = (M + 15) / 16;
    switch (mt) {
        case 1: gemm_skinny_kernel<1, TC><<<blocks, SK_WAVES * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K); break;
        case 2: gemm_skinny_kernel<2, TC><<<blocks, SK_WAVES * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K); break;
        case 3: gemm_skinny_kernel<3, TC><<<blocks, SK_WAVES * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K); break;
        case 4: gemm_skinny_kernel<4, TC><<<blocks, SK_WAVES * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K); break;
        default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}

// X [M, K] and W [N, K] bfloat16, contiguous; 1 <= M <= 64; K a multiple of 8.
extern "C" int lle_gemm_skinny_bf16(const void* X, const void* W, void* C, int M, int N, int K, int out_dtype,
                                    hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K % 8 != 0 || K <= 0) return (int)hipErrorInvalidValue;
    if (out_dtype == LLE_F32) return launch_skinny<float>((const bf16_t*)X, (const bf16_t*)W, (float*)C, M, N, K, stream);
    if (out_dtype == LLE_BF16)
        return launch_skinny<bf16_t>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)C, M, N, K, stream);
    return (int)hipErrorInvalidValue;
}
