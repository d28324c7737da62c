// Matrix products C[M, N] = A[M, K] . B[N, K]^T (weights are [out, in] row-major
// like the reference's Linear, src/layers/linear.cu:169-215, which calls
// cublasSgemm).  This file holds the true 32-bit product (plain FMA, no matrix
// cores, no reduced-precision mode; the sum over k runs in index order whatever
// M is, so a row's result does not depend on what else is in the batch), the
// bfloat16 weight-streaming product of decoding, and its 32-bit twin (32-bit
// operands through the 32-bit matrix instruction: products and sums in float32).
#include "common.h"
#include <type_traits>

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

// The same product through the 32-bit matrix instruction (v_mfma_f32_16x16x4_f32: float32
// operands, products and sums; no reduced-precision mode), for many rows: 64 x 64 tiles, four
// wavefronts of 32 x 32 each, k in steps of 16 through LDS.  Lane (c, r) reads 16 bytes
// T[row r][4c .. 4c + 3] of a tile; its four values are the k slot c of four instructions, for
// both operands alike.  The sum over k runs in the same order for every tile, whatever M is.
// K must be a multiple of 4 (16-byte loads).
typedef float mf32x4 __attribute__((ext_vector_type(4)));
#define GM_LD (GT_BK + 4)  // row stride in LDS: 80 bytes, 16-byte reads of 16 rows fall into different banks
__global__ __launch_bounds__(256) void gemm_nt_mfma_f32_kernel(const float* __restrict__ A, const float* __restrict__ B,
                                                               float* __restrict__ C, int M, int N, int K,
                                                               int64_t lda, int64_t ldb, int64_t ldc) {
    __shared__ __attribute__((aligned(16))) float As[GT_BM * GM_LD];
    __shared__ __attribute__((aligned(16))) float Bs[GT_BN * GM_LD];
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int c = lane / 16, r16 = lane % 16;
    const int64_t m0 = (int64_t)blockIdx.y * GT_BM, n0 = (int64_t)blockIdx.x * GT_BN;
    const int wm = (wave / 2) * 32, wn = (wave % 2) * 32;  // this wavefront's corner in the tile
    // the copy into LDS: thread -> (row of the tile, 4 consecutive k)
    const int lr = threadIdx.x / 4, lk = (threadIdx.x % 4) * 4;
    const bool a_row = m0 + lr < M, b_row = n0 + lr < N;
    const float* ap = A + (m0 + lr) * lda + lk;
    const float* bp = B + (n0 + lr) * ldb + lk;
    const mf32x4 zero = {0.f, 0.f, 0.f, 0.f};
    mf32x4 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = zero;

    for (int k0 = 0; k0 < K; k0 += GT_BK) {
        const bool kin = k0 + lk < K;  // K is a multiple of 4: a piece is inside or outside as a whole
        const mf32x4 av = (a_row && kin) ? *(const mf32x4*)(ap + k0) : zero;
        const mf32x4 bv = (b_row && kin) ? *(const mf32x4*)(bp + k0) : zero;
        __syncthreads();  // the tiles of the step before are read
        *(mf32x4*)(As + lr * GM_LD + lk) = av;
        *(mf32x4*)(Bs + lr * GM_LD + lk) = bv;
        __syncthreads();
        mf32x4 a[2], b[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) a[i] = *(const mf32x4*)(As + (wm + 16 * i + r16) * GM_LD + 4 * c);
#pragma unroll
        for (int j = 0; j < 2; ++j) b[j] = *(const mf32x4*)(Bs + (wn + 16 * j + r16) * GM_LD + 4 * c);
        // C^T tile [n][m] = B tile . A tile^T: lane holds C^T[n = 4c + e][m = r16], as in the skinny kernels
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[j][e], a[i][e], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t m = m0 + wm + 16 * i + r16;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t n = n0 + wn + 16 * j + 4 * c + e;
                if (n < N) C[m * ldc + n] = acc[i][j][e];
            }
    }
}

// float32 in, float32 out; K a multiple of 4, rows 16-byte aligned (lda, ldb multiples of 4)
extern "C" int lle_gemm_nt_mfma_f32(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda,
                                    int64_t ldb, int64_t ldc, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0 || K % 4 != 0 || lda % 4 != 0 || ldb % 4 != 0) return (int)hipErrorInvalidValue;
    dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM);
    if (grid.y > 65535) return (int)hipErrorInvalidValue;
    gemm_nt_mfma_f32_kernel<<<grid, 256, 0, stream>>>((const float*)A, (const float*)B, (float*)C, M, N, K, lda, ldb,
                                                       ldc);
    LLE_RETURN_LAUNCH_STATUS();
}

// float32 in, float32 out (in_dtype and out_dtype must say so)
extern "C" int lle_gemm_nt_simt(const void* A, const void* B, void* C, int M, int N, int K, int64_t lda,
                                int64_t ldb, int64_t ldc, int in_dtype, int out_dtype, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (in_dtype != LLE_F32 || out_dtype != LLE_F32) return (int)hipErrorInvalidValue;
    dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM);
    if (grid.y > 65535) return (int)hipErrorInvalidValue;
    gemm_nt_simt_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)A, (const float*)B, (float*)C, M, N, K,
                                                                 lda, ldb, ldc);
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------
// Skinny product for decoding: M <= 64 rows of activations against a weight
// matrix that is read exactly once.  bfloat16 in, 32-bit accumulate, bfloat16 or
// 32-bit out.  HBM-bound: the kernel is shaped to keep whole 128-byte lines of W
// in flight from all CUs.
//   workgroup = 16 rows of W (one matrix-core tile), 16 wavefronts split K:
//   wavefront w takes the 64-element k steps w, w + 16, ... (neighbouring
//   wavefronts read neighbouring 128-byte pieces of the same rows);
//   C^T tile = W tile [16 n x 64 k] . X^T [64 k x 16 m] by two
//   v_mfma_f32_16x16x32_bf16 per 16 rows of X; lane (c = lane / 16, r = lane % 16)
//   loads 32 contiguous bytes W[n0 + r][k0 + 16c .. + 15]; X comes from L2.
//   The 16 partial tiles are added in LDS in wavefront order, so the sum over k
//   has one fixed order for every M.
// ---------------------------------------------------------------------------------
typedef bf16_t gbf16x8 __attribute__((ext_vector_type(8)));
typedef float gf32x4 __attribute__((ext_vector_type(4)));

#define SK_KSTEP 64

// GATED: W holds gate rows [0, N/2) and then up rows [N/2, N); a workgroup takes 16 gate rows
// and the 16 up rows that go with them (NT = 2) and writes silu(gate) * up, C is [M, N/2].
//
// The RMSNorm between two products can be folded into them (up to 32 rows).  With
//   norm(h)[m][k] = h[m][k] * w[k] * r[m],  r[m] = 1 / sqrt(mean_k h[m][k]^2 + eps)
// the factor r[m] commutes with the product that follows, so
//   RESID (the product before the norm): its result is the delta of the residual stream; the
//     epilogue forms h = hidden + delta in 32-bit, writes it back, writes xw = h * w as the
//     next product's input, and leaves the sum of h^2 over its 16 columns per row in
//     ss_part[16 MT][workgroups];
//   SCALED (the product after the norm): adds up the parts, and multiplies its rows by r[m].
struct NormFold {
    float* hidden;          // RESID: residual stream [M, N], read and written
    const void* weight;     // RESID: norm weight [N]
    int weight_dtype;
    bf16_t* xw;             // RESID: out, [M, N]
    float* ss_out;          // RESID: out, [16][workgroups]
    const float* ss_in;     // SCALED: [16][parts]
    int parts;              // SCALED
    float eps;              // SCALED
};

template <int MT, int NT, bool GATED, bool RESID, bool SCALED, typename TC, int SK_WAVES, int UNROLL>
// one tile of W and up to 16 rows of X: two workgroups of 16 wavefronts a CU (8 wavefronts a SIMD),
// which 64 registers allow; the gated form measured faster with the registers it asks for
__global__ __launch_bounds__(SK_WAVES* LLE_WAVE, (MT == 1 && !GATED) ? 8 : 4) void gemm_skinny_kernel(const bf16_t* __restrict__ X,
                                                                         const bf16_t* __restrict__ W,
                                                                         TC* __restrict__ C, int M, int N, int K,
                                                                         int tile_rows, NormFold fold) {
    static_assert(!(RESID || SCALED) || MT <= 2, "the norm is folded for up to 32 rows");
    // `tile_rows` (at most 16) rows of W per tile: fewer than 16 where that makes the number of tiles a
    // multiple of the number of CUs (see skinny_tile_rows); the lanes past them read the tile's last
    // row again, which costs no traffic, and write nothing.  Forms with several tiles of W per
    // workgroup (NT > 1, not gated) keep whole tiles.
    // NT tiles of 16 rows of W per workgroup share the X operands they are multiplied with
    __shared__ float s_acc[SK_WAVES][NT][MT][16][17];
    __shared__ float s_inv[16 * MT];
    // A launch is short: what stands between its start and its first load of W counts.  All
    // arguments are read in one go (read where they are first used, each group costs a round
    // trip of its own), and the small loads beside W (parts of the norm's sums, residual
    // stream, norm weight) are asked for without a condition around them, so that nothing
    // waits for them before the loads of W are on their way.
    asm volatile("" ::"s"(X), "s"(W), "s"(C), "s"(M), "s"(N), "s"(K), "s"(tile_rows), "s"(fold.hidden), "s"(fold.weight),
                 "s"(fold.weight_dtype), "s"(fold.xw), "s"(fold.ss_out), "s"(fold.ss_in), "s"(fold.parts),
                 "s"(fold.eps));
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    // SCALED: wavefront w adds up the parts of the rows w, w + 16.  With one tile of rows the
    // first parts are asked for now and added after the products.
    static_assert(!SCALED || SK_WAVES == 16, "one wavefront per row of a tile of the norm");
    constexpr int EARLY_PARTS = (GATED || MT > 1) ? 0 : 4;  // the gated form measured faster without them
    float early[EARLY_PARTS + 1];
    if (SCALED) {
#pragma unroll
        for (int i = 0; i < EARLY_PARTS; ++i)  // past the parts: the last one again, dropped below
            early[i] = fold.ss_in[(int64_t)wave * fold.parts + min(lane + LLE_WAVE * i, fold.parts - 1)];
    }
    const int c = lane / 16, r16 = lane % 16;
    const int64_t n0 = (int64_t)blockIdx.x * ((GATED || NT == 1) ? tile_rows : 16 * NT);
    // RESID: thread (m, n) of the first 256 owns element [m][n0 + n]; what it needs of the
    // residual stream and of the norm weight is asked for now and has arrived by the epilogue
    // (all threads ask, for places that are there; the bits of the weight are read as they lie
    // and interpreted in the epilogue)
    float resid_h[MT];
    uint32_t resid_w = 0;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) resid_h[mt] = 0.f;
    if (RESID) {
        const int64_t col = min(n0 + min((int)(threadIdx.x % 16), tile_rows - 1), (int64_t)N - 1);
        if (fold.weight_dtype == LLE_F32)
            resid_w = ((const uint32_t*)fold.weight)[col];
        else
            resid_w = ((const uint16_t*)fold.weight)[col];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            resid_h[mt] = fold.hidden[(int64_t)min(16 * mt + (int)(threadIdx.x / 16) % 16, M - 1) * N + col];
    }
    const bf16_t* wp[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int rt = min(r16, tile_rows - 1);  // the lane's row of the tile
        const int64_t wrow = GATED ? min(n0 + rt, (int64_t)N / 2 - 1) + nt * ((int64_t)N / 2)
                                   : min(n0 + (NT == 1 ? rt : 16 * nt + r16), (int64_t)N - 1);
        wp[nt] = W + wrow * K + 16 * c;
    }
    // rows of X beyond M are never written back, so their lanes may read any valid row
    const bf16_t* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xp[mt] = X + (int64_t)min(16 * mt + r16, M - 1) * K + 16 * c;
    gf32x4 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = gf32x4{0.f, 0.f, 0.f, 0.f};
    const gbf16x8 zero = {(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f,
                          (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};

    const int full_steps = K / SK_KSTEP;
    int ss = wave;
    // UNROLL steps at a time: all their loads are issued before the first product
    for (; ss + (UNROLL - 1) * SK_WAVES < full_steps; ss += UNROLL * SK_WAVES) {
        gbf16x8 w0[UNROLL][NT], w1[UNROLL][NT], x0[UNROLL][MT], x1[UNROLL][MT];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k0 = (ss + u * SK_WAVES) * SK_KSTEP;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                w0[u][nt] = *(const gbf16x8*)(wp[nt] + k0);
                w1[u][nt] = *(const gbf16x8*)(wp[nt] + k0 + 8);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                x0[u][mt] = *(const gbf16x8*)(xp[mt] + k0);
                x1[u][mt] = *(const gbf16x8*)(xp[mt] + k0 + 8);
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[u][nt], x0[u][mt], acc[nt][mt], 0, 0, 0);
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[u][nt], x1[u][mt], acc[nt][mt], 0, 0, 0);
                }
    }
    // what is left of K: single steps; the last one may be partial (K is a multiple of 8),
    // and there both operands are zeroed beyond K so that nothing outside the matrices is read
    const int all_steps = (K + SK_KSTEP - 1) / SK_KSTEP;
    for (; ss < all_steps; ss += SK_WAVES) {
        const int k0 = ss * SK_KSTEP;
        const bool in0 = k0 + 16 * c + 8 <= K, in1 = k0 + 16 * c + 16 <= K;
        gbf16x8 x0[MT], x1[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            x0[mt] = in0 ? *(const gbf16x8*)(xp[mt] + k0) : zero;
            x1[mt] = in1 ? *(const gbf16x8*)(xp[mt] + k0 + 8) : zero;
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const gbf16x8 w0 = in0 ? *(const gbf16x8*)(wp[nt] + k0) : zero;
            const gbf16x8 w1 = in1 ? *(const gbf16x8*)(wp[nt] + k0 + 8) : zero;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, x0[mt], acc[nt][mt], 0, 0, 0);
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, x1[mt], acc[nt][mt], 0, 0, 0);
            }
        }
    }
    if (SCALED) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = 16 * mt + wave;
            float part = 0.f;
#pragma unroll
            for (int i = 0; i < EARLY_PARTS; ++i) part += lane + LLE_WAVE * i < fold.parts ? early[i] : 0.f;
            // what is left: four loads at a time (one after the other would each pay the way from memory)
            const float* in = fold.ss_in + (int64_t)m * fold.parts;
            for (int b = lane + LLE_WAVE * EARLY_PARTS; b < fold.parts; b += 4 * LLE_WAVE) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = in[min(b + i * LLE_WAVE, fold.parts - 1)];
#pragma unroll
                for (int i = 0; i < 4; ++i) part += b + i * LLE_WAVE < fold.parts ? v[i] : 0.f;
            }
            part = wave_sum(part);
            if (lane == 0) s_inv[m] = 1.0f / sqrtf(part / (float)K + fold.eps);
        }
    }
    // lane holds C^T[n = 4c + i][m = r16]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) s_acc[wave][nt][mt][4 * c + i][r16] = acc[nt][mt][i];
    __syncthreads();
    if (GATED) {
        for (int idx = threadIdx.x; idx < MT * 256; idx += blockDim.x) {
            const int mt = idx / 256, m = (idx / 16) % 16, n = idx % 16;
            const int64_t row = 16 * mt + m, col = n0 + n;
            if (row >= M || col >= N / 2 || n >= tile_rows) continue;
            float g = 0.f, u = 0.f;
#pragma unroll
            for (int w = 0; w < SK_WAVES; ++w) {
                g += s_acc[w][0][mt][n][m];
                u += s_acc[w][NT - 1][mt][n][m];
            }
            if (SCALED) {
                g *= s_inv[16 * mt + m];
                u *= s_inv[16 * mt + m];
            }
            C[row * (N / 2) + col] = from_f32<TC>(g / (1.0f + expf(-g)) * u);
        }
        return;
    }
    if (RESID) {  // NT = 1
        if (threadIdx.x < 256) {
            const int n = threadIdx.x % 16;
            const int64_t col = n0 + n;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int m16 = threadIdx.x / 16, m = 16 * mt + m16;
                float sq = 0.f;
                if (m < M && col < N && n < tile_rows) {
                    float sum = 0.f;
#pragma unroll
                    for (int w = 0; w < SK_WAVES; ++w) sum += s_acc[w][0][mt][n][m16];
                    const float h = resid_h[mt] + sum;
                    fold.hidden[(int64_t)m * N + col] = h;
                    fold.xw[(int64_t)m * N + col] =
                        (bf16_t)(h * __uint_as_float(fold.weight_dtype == LLE_F32 ? resid_w : resid_w << 16));
                    sq = h * h;
                }
#pragma unroll
                for (int o = 1; o < 16; o <<= 1) sq += __shfl_xor(sq, o, LLE_WAVE);
                if (n == 0) fold.ss_out[(int64_t)m * gridDim.x + blockIdx.x] = sq;
            }
        }
        return;
    }
    for (int idx = threadIdx.x; idx < NT * MT * 256; idx += blockDim.x) {
        const int nt = idx / (MT * 256), mt = (idx / 256) % MT, m = (idx / 16) % 16, n = idx % 16;
        const int64_t row = 16 * mt + m, col = n0 + 16 * nt + n;
        if (row >= M || col >= N || (NT == 1 && n >= tile_rows)) continue;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) sum += s_acc[w][nt][mt][n][m];
        if (SCALED) sum *= s_inv[16 * mt + m];
        C[row * N + col] = from_f32<TC>(sum);
    }
}

// ---------------------------------------------------------------------------------
// 17 to 128 rows of X against a weight with few rows per CU (N about 16 rows a CU: o_proj,
// down_proj): the product in SLICES of K.  With one 16-row tile of W per workgroup every
// workgroup reads all of X (at 64 rows four times the bytes of its share of W, through L2), and
// taller tiles leave CUs without work: so a workgroup takes 64 rows of W and one of `slices`
// equal parts of K, a grid of (N / 64) x slices workgroups, and writes its 64 x M partial sums in
// float32: out[slice][m][n].  Whoever reads the result adds up the slices (the residual add that
// follows these products does), in slice order: the sum over k has one order whatever else runs.
// A workgroup walks its part of K in stages of 256 columns:
//   * the sixteen wavefronts are 4 tiles of W rows x the 4 64-element steps of a stage; a
//     wavefront's W operands (the only bytes from HBM) and its share of X[:, stage] are asked for
//     three stages ahead, into registers;
//   * X[:, stage] then goes to LDS (two buffers), its 16-byte pieces XOR-swizzled so that the
//     sixteen lanes that a 16-byte LDS read serves in a cycle hit sixteen different columns of
//     the banks, and every wavefront multiplies its W operands with every 16-row tile of it;
//   * at the end the four steps of a tile are added up in LDS.
// Measured on MI355X against the library: o_proj sizes (4096 x 4096) 11.7 against 15.0 us at
// 64 rows and 15.8 against 24.3 at 128, down_proj sizes (4096 x 12288) 29.5 against 38.7 us and
// 37.2 against 67.6; a CU takes in about 29 GB/s of W and X together whatever the depth of the
// loads on their way, and at 128 rows a workgroup reads twice as much X as W.
// ---------------------------------------------------------------------------------
#define MID_ROWS 64    // rows of W per workgroup
#define MID_STEPS 4    // 64-element steps of K per stage: 4 x MID_STEPS wavefronts a workgroup
#define MID_UNIT_STAGES 4  // a slice of K is a whole number of these many stages (the register sets divide it)
#define MID_STAGE (64 * MID_STEPS)  // columns of K per stage
// The XOR of a 16-byte piece index in row r of a 16-row tile of X.  Lanes (c, r) read the pieces
// 2 c and 2 c + 1 of a step; a cycle serves c0 with r / 4 in {0, 3} and c0 + 1 with r / 4 in
// {1, 2} (or the other way round), whose pieces differ in bit 1: r % 4 goes to bits 2-3 and
// r / 8 to bit 0, which makes the sixteen columns different.
#define MID_SWIZZLE(r) ((((r) & 3) << 2) | (((r) >> 3) & 1))
// BUFFERS: register sets, i.e. the stages on their way from memory plus the one that is multiplied
// (four up to 64 rows of X; two at 128 rows, where a stage of X is four loads a thread and the
// sixteen wavefronts of a workgroup have 128 registers a lane each; one to four measured the same).
template <int M_TILES, int BUFFERS>
__global__ __launch_bounds__(4 * MID_STEPS * LLE_WAVE) void gemm_mid_slices_kernel(const bf16_t* __restrict__ X,
                                                                                  const bf16_t* __restrict__ W,
                                                                                  float* __restrict__ out, int M, int N,
                                                                                  int K, int stages) {
    constexpr int WAVES = 4 * MID_STEPS;
    constexpr int XBUF = 16 * M_TILES * MID_STAGE;                      // elements of a stage of X
    constexpr int XL = XBUF / (WAVES * LLE_WAVE * 8);                   // 16-byte loads of X per thread and stage
    static_assert(XL * WAVES * LLE_WAVE * 8 == XBUF, "a stage of X is a whole number of loads for every thread");
    constexpr int PIECES = MID_STAGE / 8;                               // 16-byte pieces of a row of a stage
    extern __shared__ __attribute__((aligned(16))) unsigned char mid_lds[];
    bf16_t* xs = (bf16_t*)mid_lds;  // [2][16 M_TILES][MID_STAGE], swizzled
    float* red = (float*)mid_lds;   // afterwards: [wavefronts][M_TILES][16 n][17]
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int c = lane / 16, r16 = lane % 16;
    const int tile = wave % 4, step = wave / 4;
    const int64_t n0 = (int64_t)blockIdx.x * MID_ROWS;
    const int k_begin = blockIdx.y * stages * MID_STAGE;
    // W: lane (c, r) holds W[n0 + 16 tile + r][k + 16 c .. + 15] of the wavefront's step of a stage
    const bf16_t* wp = W + min(n0 + 16 * tile + r16, (int64_t)N - 1) * K + k_begin + step * SK_KSTEP + 16 * c;
    // X: thread t copies the pieces t, t + threads, ... of a stage (row = piece / PIECES), through
    // registers; piece p of row m goes to piece p ^ swizzle(m % 16) of the row in LDS
    const bf16_t* xsrc[XL];
    int xdst[XL];
#pragma unroll
    for (int i = 0; i < XL; ++i) {
        const int piece = threadIdx.x + WAVES * LLE_WAVE * i;
        const int m = piece / PIECES, p = piece % PIECES;
        xsrc[i] = X + (int64_t)min(m, M - 1) * K + k_begin + 8 * p;
        xdst[i] = m * MID_STAGE + 8 * (p ^ MID_SWIZZLE(m % 16));
    }
    gbf16x8 w0[BUFFERS], w1[BUFFERS], xr[BUFFERS][XL];
    auto issue = [&](int st, auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
        w0[buf] = *(const gbf16x8*)(wp + st * MID_STAGE);
        w1[buf] = *(const gbf16x8*)(wp + st * MID_STAGE + 8);
#pragma unroll
        for (int i = 0; i < XL; ++i) xr[buf][i] = *(const gbf16x8*)(xsrc[i] + st * MID_STAGE);
    };
    gf32x4 acc[M_TILES];
#pragma unroll
    for (int mt = 0; mt < M_TILES; ++mt) acc[mt] = gf32x4{0.f, 0.f, 0.f, 0.f};
    const int sw = MID_SWIZZLE(r16);
    const int piece0 = 8 * step + 2 * c;  // logical pieces 2 c and 2 c + 1 of the wavefront's step
    const int x_read0 = r16 * MID_STAGE + 8 * (piece0 ^ sw), x_read1 = r16 * MID_STAGE + 8 * ((piece0 + 1) ^ sw);
    // Stage st waits in register set st % BUFFERS (BUFFERS - 1 stages are on their way from
    // memory while one is multiplied) and is multiplied from LDS buffer st % 2.
    auto run_stage = [&](int st, auto buf_c) {
        constexpr int buf = decltype(buf_c)::value;
        bf16_t* xb = xs + (st % 2) * XBUF;
#pragma unroll
        for (int i = 0; i < XL; ++i) *(gbf16x8*)(xb + xdst[i]) = xr[buf][i];
        // the stores to LDS are waited for by hand and the barrier is the bare instruction: a
        // __syncthreads() would also wait for the loads that are meant to stay on their way
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();  // all of stage st is in LDS, and nobody reads stage st - 1 any more
        // (asked for under no condition, past the end the last stage again: where paths meet the
        // compiler would wait for every load that one of them may have issued)
        issue(min(st + BUFFERS - 1, stages - 1), std::integral_constant<int, (buf + BUFFERS - 1) % BUFFERS>{});
#pragma unroll
        for (int mt = 0; mt < M_TILES; ++mt) {
            const gbf16x8 x0 = *(const gbf16x8*)(xb + 16 * mt * MID_STAGE + x_read0);
            const gbf16x8 x1 = *(const gbf16x8*)(xb + 16 * mt * MID_STAGE + x_read1);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0[buf], x0, acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1[buf], x1, acc[mt], 0, 0, 0);
        }
    };
    static_assert(BUFFERS >= 2 && BUFFERS <= 4 && MID_UNIT_STAGES % BUFFERS == 0, "register sets for the stages on their way");
    // the number of stages is a multiple of MID_UNIT_STAGES, and so of BUFFERS (the caller sees to it)
#define MID_FOR_BUFFERS(F) F(0) F(1) F(2) F(3)
#define MID_ISSUE_FIRST(B) if constexpr (B < BUFFERS - 1) issue(min(B, stages - 1), std::integral_constant<int, B % BUFFERS>{});
    MID_FOR_BUFFERS(MID_ISSUE_FIRST)
    for (int st = 0; st < stages; st += BUFFERS) {
#define MID_RUN(B) if constexpr (B < BUFFERS) run_stage(st + B, std::integral_constant<int, B % BUFFERS>{});
        MID_FOR_BUFFERS(MID_RUN)
    }
#undef MID_RUN
#undef MID_ISSUE_FIRST
#undef MID_FOR_BUFFERS
    __syncthreads();  // X is no longer needed: its space takes the partial tiles
    // lane holds C^T[n = 4 c + i][m = r16] of tile `tile`, step `step`
#pragma unroll
    for (int mt = 0; mt < M_TILES; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((wave * M_TILES + mt) * 16 + 4 * c + i) * 17 + r16] = acc[mt][i];
    __syncthreads();
    float* dst = out + (int64_t)blockIdx.y * M * N;
    for (int idx = threadIdx.x; idx < 4 * M_TILES * 256; idx += blockDim.x) {
        const int n = idx % 16, t = (idx / 16) % 4, m = idx / 64;  // consecutive threads: consecutive columns
        const int64_t col = n0 + 16 * t + n;
        if (m >= M || col >= N) continue;
        const int mt = m / 16, m16 = m % 16;
        float sum = 0.f;
#pragma unroll
        for (int ph = 0; ph < MID_STEPS; ++ph) sum += red[(((4 * ph + t) * M_TILES + mt) * 16 + n) * 17 + m16];
        dst[(int64_t)m * N + col] = sum;
    }
}

// out [slices][M][N] float32; M <= 128, N a multiple of 64, K a multiple of slices x 4 stages of 256 columns
extern "C" int lle_gemm_mid_slices_unit(void) { return MID_STAGE * MID_UNIT_STAGES; }
extern "C" int lle_gemm_mid_slices_max_rows(void) { return 128; }

extern "C" int lle_gemm_mid_slices_bf16(const void* X, const void* W, void* out, int M, int N, int K, int slices,
                                        hipStream_t stream) {
    if (M <= 0 || M > 128 || N % MID_ROWS != 0 || slices <= 0 || slices > 65535 || K % (MID_STAGE * MID_UNIT_STAGES * slices) != 0)
        return (int)hipErrorInvalidValue;
    const dim3 grid(N / MID_ROWS, slices);
    const int stages = K / (MID_STAGE * slices);
#define LLE_MID_LAUNCH(T, B)                                                                                          \
    {                                                                                                                 \
        constexpr size_t tiles = (size_t)2 * 16 * T * MID_STAGE * sizeof(bf16_t);                           \
        constexpr size_t sums = (size_t)4 * MID_STEPS * T * 16 * 17 * sizeof(float);                                  \
        constexpr size_t lds = tiles > sums ? tiles : sums;                                                           \
        static bool ready = false; /* more than 64 KB of LDS has to be asked for once */                              \
        if (!ready) {                                                                                                 \
            if (hipFuncSetAttribute((const void*)gemm_mid_slices_kernel<T, B>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                    (int)lds) != hipSuccess)                                                          \
                return (int)hipGetLastError();                                                                        \
            ready = true;                                                                                             \
        }                                                                                                             \
        gemm_mid_slices_kernel<T, B><<<grid, 4 * MID_STEPS * LLE_WAVE, lds, stream>>>(                                    \
            (const bf16_t*)X, (const bf16_t*)W, (float*)out, M, N, K, stages);                                        \
    }
    if (M <= 32)
        LLE_MID_LAUNCH(2, 4)
    else if (M <= 64)
        LLE_MID_LAUNCH(4, 4)
    else if (M <= 96)
        LLE_MID_LAUNCH(6, 2)
    else
        LLE_MID_LAUNCH(8, 2)
#undef LLE_MID_LAUNCH
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------
// The product as a STREAM, for K = 64 * 16 * XS (XS steps per wavefront, all of X that a
// wavefront needs held in registers) and up to 16 rows of X; plain or gated, with or
// without the row factors of a folded norm.
// How fast a CU reads is bounded by the loads it can have on their way, so the chip is
// fastest when every CU has the same share of W.  There is one workgroup per CU, and it
// takes `share` rows of W (share = rows / CUs, rounded up) in tiles of 16, the last of
// which may be lower: tile t of all workgroups together is one block of consecutive rows
// (the memory channels see what they see of a plain sweep over W), of which workgroup b
// takes the b-th piece.  The lanes of a tile that is not full read its last row again,
// which costs no traffic.  A wavefront keeps two sets of W operands (two steps each where
// XS is even and small, one step otherwise): while one is multiplied the loads of the next are on
// their way, also across the end of a tile, where the partial tiles are added up in LDS
// and written out.  X is read once per workgroup instead of once per tile, and the sums of
// the folded norm are added up once.
// ---------------------------------------------------------------------------------
// MT = 2: up to 32 rows of X (two tiles of matrix-core columns), where all of X that a wavefront
// needs still fits its registers (XS <= 2: narrow models, the only ones whose norms are folded at
// more than 16 rows);
// the head of the 0.6B sizes (151936 x 1024) at 32 rows: 73.6 us, against 112.1 for the
// one-tile-per-workgroup kernel with four tiles a workgroup and 66.8 at 16 rows.
template <bool GATED, bool SCALED, int XS, typename TC, int MT = 1>
__global__ __launch_bounds__(16 * LLE_WAVE, 4) void gemm_skinny_stream_kernel(const bf16_t* __restrict__ X,
                                                                              const bf16_t* __restrict__ W,
                                                                              TC* __restrict__ C, int M, int N, int K,
                                                                              int share, NormFold fold) {
    constexpr int WAVES = 16;
    constexpr int NT = GATED ? 2 : 1;
    constexpr int SS = (XS % 2 == 0 && XS <= 6) ? 2 : 1;  // steps of a set (one where X takes most of the registers)
    constexpr int SPT = XS / SS;             // sets of a tile
    static_assert(MT == 1 || (MT == 2 && (XS <= 2 || (!GATED && XS <= 4))), "two tiles of X rows only while X fits the registers");
    __shared__ float s_acc[2][WAVES][NT][MT][16][17];  // tiles take the two halves in turn: one barrier a tile
    __shared__ float s_inv[16 * MT];
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int c = lane / 16, r16 = lane % 16;
    const int rows = GATED ? N / 2 : N;
    const int tiles = (share + 15) / 16;
    // rows [tile_begin(t), tile_end(t)) of this workgroup's tile t; none where W ends before them
    auto tile_begin = [&](int t) { return (int)gridDim.x * 16 * t + (int)blockIdx.x * min(16, share - 16 * t); };
    auto tile_end = [&](int t) { return min(rows, tile_begin(t) + min(16, share - 16 * t)); };

    // a set: SS 64-element steps of the tile (and of the up tile that goes with a gate tile)
    struct Set {
        gbf16x8 g0[SS], g1[SS], u0[SS], u1[SS];
    };
    // the load cursor: tile and step of the set that is asked for next
    int load_tile = 0, load_step = 0;
    const bf16_t* wp = nullptr;
    auto aim = [&]() {
        const int t = min(load_tile, tiles - 1);
        const int row = max(0, min(tile_begin(t) + r16, tile_end(t) - 1));  // a tile without rows reads rows that are there
        wp = W + (int64_t)row * K + 16 * c + wave * SK_KSTEP;
    };
    auto load = [&](Set& set) {
#pragma unroll
        for (int i = 0; i < SS; ++i) {
            const bf16_t* g = wp + (load_step + i) * (WAVES * SK_KSTEP);
            set.g0[i] = *(const gbf16x8*)g;
            set.g1[i] = *(const gbf16x8*)(g + 8);
            if (GATED) {
                const bf16_t* u = g + (int64_t)rows * K;
                set.u0[i] = *(const gbf16x8*)u;
                set.u1[i] = *(const gbf16x8*)(u + 8);
            }
        }
        load_step += SS;
        if (load_step == XS) {
            load_step = 0;
            ++load_tile;
            aim();
        }
    };
    Set sets[2];
    aim();
    load(sets[0]);
    // rows of X beyond M are never written back, so their lanes may read any valid row
    gbf16x8 x0[MT][XS], x1[MT][XS];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const bf16_t* xp = X + (int64_t)min(16 * mt + r16, M - 1) * K + 16 * c + wave * SK_KSTEP;
#pragma unroll
        for (int j = 0; j < XS; ++j) {
            x0[mt][j] = *(const gbf16x8*)(xp + j * (WAVES * SK_KSTEP));
            x1[mt][j] = *(const gbf16x8*)(xp + j * (WAVES * SK_KSTEP) + 8);
        }
    }
    if (SCALED) {
        // the row factors of the folded norm: wavefront w adds up the parts of row w (and of row
        // 16 + w), four loads at a time
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const float* in = fold.ss_in + (int64_t)(16 * mt + wave) * fold.parts;
            float part = 0.f;
            for (int p0 = lane; p0 < fold.parts; p0 += 4 * LLE_WAVE) {
                float v[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) v[i] = in[min(p0 + i * LLE_WAVE, fold.parts - 1)];
#pragma unroll
                for (int i = 0; i < 4; ++i) part += p0 + i * LLE_WAVE < fold.parts ? v[i] : 0.f;
            }
            part = wave_sum(part);
            if (lane == 0) s_inv[16 * mt + wave] = 1.0f / sqrtf(part / (float)K + fold.eps);
        }
    }
    gf32x4 acc_g[MT], acc_u[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc_g[mt] = acc_u[mt] = gf32x4{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const Set& set, int j) {
#pragma unroll
        for (int i = 0; i < SS; ++i)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                acc_g[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(set.g0[i], x0[mt][j + i], acc_g[mt], 0, 0, 0);
                acc_g[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(set.g1[i], x1[mt][j + i], acc_g[mt], 0, 0, 0);
                if (GATED) {
                    acc_u[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(set.u0[i], x0[mt][j + i], acc_u[mt], 0, 0, 0);
                    acc_u[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(set.u1[i], x1[mt][j + i], acc_u[mt], 0, 0, 0);
                }
            }
    };
    int half = 0;
    auto finish_tile = [&](int tile) {
        // lane holds C^T[n = 4c + i][m = 16 mt + r16]
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s_acc[half][wave][0][mt][4 * c + i][r16] = acc_g[mt][i];
                if (GATED) s_acc[half][wave][NT - 1][mt][4 * c + i][r16] = acc_u[mt][i];
            }
            acc_g[mt] = acc_u[mt] = gf32x4{0.f, 0.f, 0.f, 0.f};
        }
        __syncthreads();
        if (threadIdx.x < 256 * MT) {
            const int m = threadIdx.x / 16, n = threadIdx.x % 16;
            const int64_t col = (int64_t)tile_begin(tile) + n;
            if (m < M && col < tile_end(tile)) {
                float g = 0.f, u = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) {
                    g += s_acc[half][w][0][m / 16][n][m % 16];
                    if (GATED) u += s_acc[half][w][NT - 1][m / 16][n][m % 16];
                }
                if (SCALED) {
                    g *= s_inv[m];
                    u *= s_inv[m];
                }
                C[(int64_t)m * rows + col] = from_f32<TC>(GATED ? g / (1.0f + expf(-g)) * u : g);
            }
        }
        // The other half is written next; this one again only after the next tile's barrier,
        // which the threads that are still adding here have then passed.
        half ^= 1;
    };
    // One tile: its sets in turn, the one after each asked for before it is multiplied (also the
    // first of the next tile; the share's last tile asks for nothing beyond itself).  `first` is
    // the buffer that holds the tile's first set: the sets alternate between the two buffers
    // across tiles, so with an odd number of sets a tile every other tile starts in buffer 1.
    auto run_tile = [&](int tile, auto first_c, bool last) {
        constexpr int first = decltype(first_c)::value;
#pragma unroll
        for (int s = 0; s < SPT; ++s) {
            if (!(last && s == SPT - 1)) load(sets[(first + s + 1) % 2]);
            multiply(sets[(first + s) % 2], s * SS);
        }
        finish_tile(tile);
    };
    using Buf0 = std::integral_constant<int, 0>;
    using Buf1 = std::integral_constant<int, 1>;
    int tile = 0;
    if constexpr (SPT % 2 == 0) {
        for (; tile + 1 < tiles; ++tile) run_tile(tile, Buf0{}, false);
        run_tile(tile, Buf0{}, true);
    } else {
        for (; tile + 2 < tiles; tile += 2) {
            run_tile(tile, Buf0{}, false);
            run_tile(tile + 1, Buf1{}, false);
        }
        if (tile + 1 < tiles) {
            run_tile(tile, Buf0{}, false);
            run_tile(tile + 1, Buf1{}, true);
        } else {
            run_tile(tile, Buf0{}, true);
        }
    }
}

// CUs of the current device (asked once per device)
static int gemm_compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

// The streaming kernel takes the product when K is a number of whole rounds of its 16 wavefronts
// (1024 elements a round) that its registers hold, X has up to 16 rows, and W has more than one
// tile of rows for every CU.
template <bool GATED, bool SCALED, typename TC>
static bool launch_skinny_stream(const bf16_t* X, const bf16_t* W, TC* C, int M, int N, int K,
                                 const NormFold& fold, hipStream_t stream) {
    if (M > 32 || K % (SK_KSTEP * 16) != 0) return false;
    const int rows = GATED ? N / 2 : N;
    const int units = gemm_compute_units();
    const int share = (rows + units - 1) / units;
    if (share <= 16) return false;
    const int blocks = (rows + share - 1) / share;
    if (M > 16) {  // two tiles of X rows: while all of X that a wavefront needs fits its registers
        if (K == SK_KSTEP * 16) {
            gemm_skinny_stream_kernel<GATED, SCALED, 1, TC, 2><<<blocks, 16 * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K, share, fold);
            return true;
        }
        if (K == 2 * SK_KSTEP * 16) {
            gemm_skinny_stream_kernel<GATED, SCALED, 2, TC, 2><<<blocks, 16 * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K, share, fold);
            return true;
        }
        if constexpr (!GATED) {
            if (K == 3 * SK_KSTEP * 16) {
                gemm_skinny_stream_kernel<GATED, SCALED, 3, TC, 2><<<blocks, 16 * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K, share, fold);
                return true;
            }
            if (K == 4 * SK_KSTEP * 16) {
                gemm_skinny_stream_kernel<GATED, SCALED, 4, TC, 2><<<blocks, 16 * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K, share, fold);
                return true;
            }
        }
        return false;
    }
#define LLE_STREAM_CASE(XSV)                                                                                          \
    case XSV:                                                                                                         \
        gemm_skinny_stream_kernel<GATED, SCALED, XSV, TC><<<blocks, 16 * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K, share, \
                                                                                               fold);                \
        return true;
    switch (K / (SK_KSTEP * 16)) {
        LLE_STREAM_CASE(1)
        LLE_STREAM_CASE(2)
        LLE_STREAM_CASE(3)
        LLE_STREAM_CASE(4)
        LLE_STREAM_CASE(5)
        case 6:
        case 8:
            if constexpr (!GATED) {  // the gated form's two tiles leave no registers for this much of X
                if (K / (SK_KSTEP * 16) == 6) {
                    gemm_skinny_stream_kernel<GATED, SCALED, 6, TC><<<blocks, 16 * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K,
                                                                                                          share, fold);
                } else {
                    gemm_skinny_stream_kernel<GATED, SCALED, 8, TC><<<blocks, 16 * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K,
                                                                                                          share, fold);
                }
                return true;
            }
            return false;
    }
#undef LLE_STREAM_CASE
    return false;
}

// Rows of W per tile of the one-tile-per-workgroup kernel: as many as give every CU the same share.
// More 16-row tiles than CUs: as many rows as make the last round full (with 320 tiles of 16 rows on
// 256 CUs a quarter of the CUs reads twice what the others read and the launch lasts as long as two
// rounds, with 512 tiles of 10 rows every CU reads the same).  Fewer tiles than CUs (narrow models):
// lower tiles, down to 4 rows, so that every CU takes part: such a launch is short, and the share of
// W that a workgroup has to wait for is what is left to shorten (measured at 16 rows of X: 1024 x 3072
// 8.4 -> 7.3 us, 2048 x 6144 13.6 -> 12.1, 2560 x 9728 21.1 -> 18.9; tiles of 8 rows no better than of 4).
static int skinny_tile_rows(int rows) {
    const int units = gemm_compute_units();
    const int tiles16 = (rows + 15) / 16;
    if (tiles16 <= units) {
        const int per_unit = (rows + units - 1) / units;
        return per_unit < 4 ? 4 : (per_unit > 16 ? 16 : per_unit);
    }
    const int rounds = (tiles16 + units - 1) / units;
    const int per_tile = (int)(((int64_t)rows + (int64_t)rounds * units - 1) / ((int64_t)rounds * units));
    return per_tile < 1 ? 1 : (per_tile > 16 ? 16 : per_tile);
}

// tiles of lle_gemm_skinny_resid_bf16 for a weight of N rows: the second size of its ss_part
extern "C" int lle_gemm_skinny_resid_parts(int N) {
    if (N <= 0) return 0;
    const int tr = skinny_tile_rows(N);
    return (N + tr - 1) / tr;
}

template <typename TC, int NT, bool GATED>
static int launch_skinny(const bf16_t* X, const bf16_t* W, TC* C, int M, int N, int K, hipStream_t stream) {
    constexpr int WAVES = 16, UNROLL = 4 / NT;
    const int rows = GATED ? N / 2 : N;
    const int tile_rows = (GATED || NT == 1) ? skinny_tile_rows(rows) : 16;
    const int per_block = (GATED || NT == 1) ? tile_rows : 16 * NT;
    const int blocks = (rows + per_block - 1) / per_block;
    const int mt = (M + 15) / 16;
    const NormFold none = {};
    switch (mt) {
        case 1: gemm_skinny_kernel<1, NT, GATED, false, false, TC, WAVES, UNROLL><<<blocks, WAVES * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K, tile_rows, none); break;
        case 2: gemm_skinny_kernel<2, NT, GATED, false, false, TC, WAVES, UNROLL><<<blocks, WAVES * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K, tile_rows, none); break;
        case 3: gemm_skinny_kernel<3, NT, GATED, false, false, TC, WAVES, UNROLL><<<blocks, WAVES * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K, tile_rows, none); break;
        case 4: gemm_skinny_kernel<4, NT, GATED, false, false, TC, WAVES, UNROLL><<<blocks, WAVES * LLE_WAVE, 0, stream>>>(X, W, C, M, N, K, tile_rows, none); break;
        default: return (int)hipErrorInvalidValue;
    }
    return (int)hipGetLastError();
}

// X [M, K] and W [N, K] bfloat16, contiguous; 1 <= M <= 64; K a multiple of 8.
extern "C" int lle_gemm_skinny_bf16(const void* X, const void* W, void* C, int M, int N, int K, int out_dtype,
                                    hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K % 8 != 0 || K <= 0) return (int)hipErrorInvalidValue;
    const bf16_t* x = (const bf16_t*)X;
    const bf16_t* w = (const bf16_t*)W;
    // one tile of W rows per workgroup measured best up to 16 rows of X (two tiles share the X
    // operands but halve the number of workgroups; they only pay off from 16 rows on)
    if (out_dtype == LLE_F32) {
        if (launch_skinny_stream<false, false, float>(x, w, (float*)C, M, N, K, NormFold{}, stream)) LLE_RETURN_LAUNCH_STATUS();
        return launch_skinny<float, 1, false>(x, w, (float*)C, M, N, K, stream);
    }
    if (out_dtype == LLE_BF16) {
        if (launch_skinny_stream<false, false, bf16_t>(x, w, (bf16_t*)C, M, N, K, NormFold{}, stream)) LLE_RETURN_LAUNCH_STATUS();
        return launch_skinny<bf16_t, 1, false>(x, w, (bf16_t*)C, M, N, K, stream);
    }
    return (int)hipErrorInvalidValue;
}

// The gated feed-forward's first half in one launch: W [2I, K] holds the gate rows and then the
// up rows; C [M, I] = silu(X gate^T) * (X up^T), the activation in 32-bit.  1 <= M <= 32.
extern "C" int lle_gemm_skinny_gated_bf16(const void* X, const void* W, void* C, int M, int N2, int K,
                                          hipStream_t stream) {
    if (M <= 0 || N2 <= 0) return 0;
    if (M > 32 || K % 8 != 0 || K <= 0 || N2 % 2 != 0) return (int)hipErrorInvalidValue;
    if (launch_skinny_stream<true, false, bf16_t>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)C, M, N2, K, NormFold{}, stream))
        LLE_RETURN_LAUNCH_STATUS();
    return launch_skinny<bf16_t, 2, true>((const bf16_t*)X, (const bf16_t*)W, (bf16_t*)C, M, N2, K, stream);
}

// The product BEFORE a folded norm: delta = X W^T [M, N] is added into `hidden` (float32 [M, N],
// in place), xw = hidden * norm_weight goes to `xw` (bfloat16 [M, N]) and the sums of squares of
// the new hidden over each workgroup's columns to ss_part [16 or 32][lle_gemm_skinny_resid_parts(N)]
// (32 rows when M > 16).  1 <= M <= 32.
extern "C" int lle_gemm_skinny_resid_bf16(const void* X, const void* W, void* hidden, const void* norm_weight,
                                          int weight_dtype, void* xw, void* ss_part, int M, int N, int K,
                                          hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 32 || K % 8 != 0 || K <= 0) return (int)hipErrorInvalidValue;
    NormFold fold = {};
    fold.hidden = (float*)hidden;
    fold.weight = norm_weight;
    fold.weight_dtype = weight_dtype;
    fold.xw = (bf16_t*)xw;
    fold.ss_out = (float*)ss_part;
    const int tr = skinny_tile_rows(N), blocks = (N + tr - 1) / tr;
    if (M <= 16)
        gemm_skinny_kernel<1, 1, false, true, false, bf16_t, 16, 4><<<blocks, 16 * LLE_WAVE, 0, stream>>>(
            (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)nullptr, M, N, K, tr, fold);
    else
        gemm_skinny_kernel<2, 1, false, true, false, bf16_t, 16, 4><<<blocks, 16 * LLE_WAVE, 0, stream>>>(
            (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)nullptr, M, N, K, tr, fold);
    LLE_RETURN_LAUNCH_STATUS();
}

// The product AFTER a folded norm: X is the xw of lle_gemm_skinny_resid_bf16 and ss_part its
// (16 or 32) x `parts` sums; the rows of the result are scaled by 1 / sqrt(sum / K + eps).
// gated != 0: W is [2 I, K] and C [M, I] = silu(gate) * up as in lle_gemm_skinny_gated_bf16.
// C is bfloat16, or float32 for a product that is not gated (an output head).  1 <= M <= 32.
#ifndef SCALED_TILES_AT_32_ROWS
#define SCALED_TILES_AT_32_ROWS 4
#endif
template <typename TC>
static void launch_skinny_scaled(const bf16_t* x, const bf16_t* w, TC* c, int M, int N, int K, const NormFold& fold,
                                 hipStream_t stream) {
    if (launch_skinny_stream<false, true, TC>(x, w, c, M, N, K, fold, stream)) return;
    const int threads = 16 * LLE_WAVE;
    const int tr = skinny_tile_rows(N), blocks = (N + tr - 1) / tr;
    if (M <= 16) {
        gemm_skinny_kernel<1, 1, false, false, true, TC, 16, 4><<<blocks, threads, 0, stream>>>(x, w, c, M, N, K, tr, fold);
    } else if (N >= 16 * SCALED_TILES_AT_32_ROWS * gemm_compute_units()) {
        // 17 to 32 rows of X are twice the bytes of a tile of W: with one tile a workgroup a product
        // with many tiles (an output head) spends its time on X; several tiles share what they read of it
        // (the head of the 0.6B sizes, 151936 x 1024, at 32 rows: 137.6 us with one tile, 126.8 with two, 112.1 with four)
        constexpr int NT = SCALED_TILES_AT_32_ROWS;
        gemm_skinny_kernel<2, NT, false, false, true, TC, 16, 4 / NT>
            <<<(N + 16 * NT - 1) / (16 * NT), threads, 0, stream>>>(x, w, c, M, N, K, 16, fold);
    } else {
        gemm_skinny_kernel<2, 1, false, false, true, TC, 16, 4><<<blocks, threads, 0, stream>>>(x, w, c, M, N, K, tr, fold);
    }
}

extern "C" int lle_gemm_skinny_scaled_bf16(const void* X, const void* W, void* C, const void* ss_part, int parts,
                                           float eps, int M, int N, int K, int gated, int out_dtype,
                                           hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 32 || K % 8 != 0 || K <= 0 || parts <= 0 || (gated && N % 2 != 0)) return (int)hipErrorInvalidValue;
    if (out_dtype != LLE_BF16 && !(out_dtype == LLE_F32 && !gated)) return (int)hipErrorInvalidValue;
    NormFold fold = {};
    fold.ss_in = (const float*)ss_part;
    fold.parts = parts;
    fold.eps = eps;
    const bf16_t* x = (const bf16_t*)X;
    const bf16_t* w = (const bf16_t*)W;
    bf16_t* c = (bf16_t*)C;
    const int threads = 16 * LLE_WAVE;
    if (!gated) {
        if (out_dtype == LLE_F32)
            launch_skinny_scaled<float>(x, w, (float*)C, M, N, K, fold, stream);
        else
            launch_skinny_scaled<bf16_t>(x, w, c, M, N, K, fold, stream);
    } else if (launch_skinny_stream<true, true, bf16_t>(x, w, c, M, N, K, fold, stream)) {
    } else {
        const int rows = N / 2;
        const int tr = skinny_tile_rows(rows), blocks = (rows + tr - 1) / tr;
        if (M <= 16)
            gemm_skinny_kernel<1, 2, true, false, true, bf16_t, 16, 2><<<blocks, threads, 0, stream>>>(x, w, c, M, N, K, tr, fold);
        else
            gemm_skinny_kernel<2, 2, true, false, true, bf16_t, 16, 2><<<blocks, threads, 0, stream>>>(x, w, c, M, N, K, tr, fold);
    }
    LLE_RETURN_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------------
// The same for float32 operands: the true 32-bit path of decoding.  W is read once;
// v_mfma_f32_16x16x4_f32 multiplies and adds in float32 (no reduced-precision mode).
// Lane (c, r) loads 16 contiguous bytes W[n0 + r][k0 + 4c .. + 3]; its four values are the
// k slot c of four instructions, and the X operand is laid out the same way.
// ---------------------------------------------------------------------------------
#define SKF_KSTEP 16
template <int MT, int SK_WAVES, int UNROLL>
__global__ __launch_bounds__(SK_WAVES* LLE_WAVE) void gemm_skinny_f32_kernel(const float* __restrict__ X,
                                                                             const float* __restrict__ W,
                                                                             float* __restrict__ C, int M, int N, int K,
                                                                             int tile_rows) {
    // `tile_rows` (at most 16) rows of W per workgroup, as in the bfloat16 kernel (skinny_tile_rows):
    // the lanes past them read the tile's last row again and write nothing
    __shared__ float s_acc[SK_WAVES][MT][16][17];
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int c = lane / 16, r16 = lane % 16;
    const int64_t n0 = (int64_t)blockIdx.x * tile_rows;
    const float* wp = W + min(n0 + min(r16, tile_rows - 1), (int64_t)N - 1) * K + 4 * c;
    // rows of X beyond M are never written back, so their lanes may read any valid row
    const float* xp[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xp[mt] = X + (int64_t)min(16 * mt + r16, M - 1) * K + 4 * c;
    gf32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = gf32x4{0.f, 0.f, 0.f, 0.f};

    const int full_steps = K / SKF_KSTEP;
    int ss = wave;
    for (; ss + (UNROLL - 1) * SK_WAVES < full_steps; ss += UNROLL * SK_WAVES) {
        gf32x4 w[UNROLL], x[UNROLL][MT];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k0 = (ss + u * SK_WAVES) * SKF_KSTEP;
            w[u] = *(const gf32x4*)(wp + k0);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) x[u][mt] = *(const gf32x4*)(xp[mt] + k0);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u][j], x[u][mt][j], acc[mt], 0, 0, 0);
    }
    // what is left of K: single steps, the last one may be partial (K is a multiple of 4)
    const int all_steps = (K + SKF_KSTEP - 1) / SKF_KSTEP;
    const gf32x4 zero = {0.f, 0.f, 0.f, 0.f};
    for (; ss < all_steps; ss += SK_WAVES) {
        const int k0 = ss * SKF_KSTEP;
        const bool in = k0 + 4 * c + 4 <= K;
        const gf32x4 w = in ? *(const gf32x4*)(wp + k0) : zero;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const gf32x4 x = in ? *(const gf32x4*)(xp[mt] + k0) : zero;
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[j], x[j], acc[mt], 0, 0, 0);
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
        if (row >= M || col >= N || n >= tile_rows) continue;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w) sum += s_acc[w][mt][n][m];
        C[row * N + col] = sum;
    }
}

// X [M, K] and W [N, K] float32, contiguous; C [M, N] float32; 1 <= M <= 64; K a multiple of 4.
extern "C" int lle_gemm_skinny_f32(const void* X, const void* W, void* C, int M, int N, int K, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K % 4 != 0 || K <= 0) return (int)hipErrorInvalidValue;
    const int tr = skinny_tile_rows(N), blocks = (N + tr - 1) / tr;
    const float* x = (const float*)X;
    const float* w = (const float*)W;
    float* c = (float*)C;
    switch ((M + 15) / 16) {
        case 1: gemm_skinny_f32_kernel<1, 16, 4><<<blocks, 16 * LLE_WAVE, 0, stream>>>(x, w, c, M, N, K, tr); break;
        case 2: gemm_skinny_f32_kernel<2, 16, 4><<<blocks, 16 * LLE_WAVE, 0, stream>>>(x, w, c, M, N, K, tr); break;
        case 3: gemm_skinny_f32_kernel<3, 16, 2><<<blocks, 16 * LLE_WAVE, 0, stream>>>(x, w, c, M, N, K, tr); break;
        default: gemm_skinny_f32_kernel<4, 16, 2><<<blocks, 16 * LLE_WAVE, 0, stream>>>(x, w, c, M, N, K, tr); break;
    }
    LLE_RETURN_LAUNCH_STATUS();
}
