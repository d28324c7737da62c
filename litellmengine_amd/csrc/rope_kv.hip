// Per-head q/k RMSNorm + rotary position encoding + paged K/V write, one launch.
// In the reference these are five reshape copies, two RMSNorm launches, two
// rotary launches and one cudaMemcpy per token and tensor
// (src/model/qwen3.cpp:391-481, src/layers/rotary.cu:153-195,
// src/engine/paged_kv_cache.cpp:138-167).
//
// qkv [N, (nq + 2 nkv) d]: q heads, then k heads, then v heads of one token.
//   q head:  norm over d (weight [d]) -> rotate -> q_out [N, nq, d]
//   k head:  norm over d (weight [d]) -> rotate -> K page of the token's slot
//   v head:  copy                               -> V page of the token's slot
// Rotation pairs element i with i + rot/2 (half split) for i < rot/2; elements
// >= rot pass through.  angle = float(pos) * inv_freq[i], all in 32-bit; cosine and sine of
// every (token, i) are computed once per step by rope_table_kernel ([N][rot/2][2] floats) and
// shared by all heads and all layers.
// A cache page holds K as [nkv][page_size][d] and then V as [nkv][d][page_size]
// (V is kept transposed so that the matrix-core attention kernels find the keys
// of one value column next to each other); slot = page * page_size + offset;
// slot < 0 skips the write.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

template <typename T>
__global__ __launch_bounds__(64) void qk_norm_rope_write_kernel(
    const T* __restrict__ qkv, const int32_t* __restrict__ slots, const void* __restrict__ q_weight,
    const void* __restrict__ k_weight, int weight_dtype, const float* __restrict__ cos_sin, int rot, float eps,
    T* __restrict__ q_out, T* __restrict__ kv_layer, int nq, int nkv, int d, int page_size, int64_t page_stride,
    int write_kv) {
    const int64_t n = blockIdx.x;
    const int head = blockIdx.y;  // 0..nq-1 q, then nkv k, then nkv v
    const int lane = threadIdx.x;
    const int width = (nq + 2 * nkv) * d;
    const T* src = qkv + n * width + (int64_t)head * d;

    const bool is_q = head < nq;
    const bool is_k = !is_q && head < nq + nkv;
    T* dst;
    if (is_q) {
        dst = q_out + (n * nq + head) * d;
    } else {
        if (!write_kv) return;
        const int slot = slots[n];
        if (slot < 0) return;
        const int kvh = is_k ? head - nq : head - nq - nkv;
        const int64_t page = slot / page_size;
        const int off = slot - (int)page * page_size;
        T* page_base = kv_layer + page * page_stride;
        if (!is_k) {  // v: copy into the transposed page, element i of the head at [i][off]
            T* v = page_base + ((int64_t)nkv + kvh) * page_size * d + off;
            for (int i = lane; i < d; i += LLE_WAVE) v[(int64_t)i * page_size] = src[i];
            return;
        }
        dst = page_base + ((int64_t)kvh * page_size + off) * d;
    }

    const void* w = is_q ? q_weight : k_weight;
    float inv = 1.0f;
    if (w) {
        float ss = 0.f;
        for (int i = lane; i < d; i += LLE_WAVE) {
            const float v = to_f32<T>(src[i]);
            ss += v * v;
        }
        ss = wave_sum(ss);
        inv = 1.0f / sqrtf(ss / (float)d + eps);
    }
    const int half = rot / 2;
    const float2* cs = (const float2*)cos_sin + n * half;
    for (int i = lane; i < half; i += LLE_WAVE) {
        float x1 = to_f32<T>(src[i]) * inv;
        float x2 = to_f32<T>(src[i + half]) * inv;
        if (w) {
            x1 *= load_as_f32(w, i, weight_dtype);
            x2 *= load_as_f32(w, i + half, weight_dtype);
        }
        const float c = cs[i].x, s = cs[i].y;
        dst[i] = from_f32<T>(x1 * c - x2 * s);
        dst[i + half] = from_f32<T>(x2 * c + x1 * s);
    }
    for (int i = rot + lane; i < d; i += LLE_WAVE) {
        float x = to_f32<T>(src[i]) * inv;
        if (w) x *= load_as_f32(w, i, weight_dtype);
        dst[i] = from_f32<T>(x);
    }
}

// The same for bfloat16 heads of 16, 32, 64, 128 or 256 elements with a rotation over a
// multiple of 16 elements (or none): a lane holds 8 consecutive elements (16-byte loads and
// stores), d / 8 lanes hold a head, a wavefront holds 512 / d heads of one token.  The partner of
// element i in the rotation is i +- rot / 2, which lies rot / 16 lanes away.
typedef bf16_t rbf16x8 __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(256) void qk_norm_rope_write_vec_kernel(
    const bf16_t* __restrict__ qkv, const int32_t* __restrict__ slots, const void* __restrict__ q_weight,
    const void* __restrict__ k_weight, int weight_dtype, const float* __restrict__ cos_sin, int rot, float eps,
    bf16_t* __restrict__ q_out, bf16_t* __restrict__ kv_layer, int nq, int nkv, int d, int page_size,
    int64_t page_stride, int write_kv, int total_heads) {
    // write_kv: 0 = q only, 1 = K and V, 2 = K only (another kernel writes V)
    const int lph = d / 8;  // lanes per head
    const int lane = threadIdx.x % LLE_WAVE;
    const int heads_per_wave = LLE_WAVE / lph;
    const int64_t gw = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / LLE_WAVE;  // global wavefront
    const int64_t flat = gw * heads_per_wave + lane / lph;                           // (token, head)
    const int hl = lane % lph;                                                        // lane inside the head
    const int per_token = nq + 2 * nkv;
    const bool live = flat < (int64_t)total_heads;
    const int64_t n = live ? flat / per_token : 0;
    const int head = live ? (int)(flat - n * per_token) : 0;
    const bool is_q = head < nq;
    const bool is_k = !is_q && head < nq + nkv;
    const int e0 = 8 * hl;

    float x[8];
    {
        const rbf16x8 v = *(const rbf16x8*)(qkv + (n * per_token + head) * d + e0);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = (float)v[i];
    }
    if (is_q || is_k) {
        const void* w = is_q ? q_weight : k_weight;
        if (w) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
            for (int o = 1; o < lph; o <<= 1) ss += __shfl_xor(ss, o, LLE_WAVE);
            const float inv = 1.0f / sqrtf(ss / (float)d + eps);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = x[i] * inv * load_as_f32(w, e0 + i, weight_dtype);
        }
        if (rot > 0) {
            const int half = rot / 2;
            const int dl = half / 8;  // lanes between partners
            const bool low = e0 < half, in_rot = e0 < rot;
            float other[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                // lanes of the low half read from lane + dl, those of the high half from lane - dl
                const float up = __shfl_down(x[i], dl, LLE_WAVE), down = __shfl_up(x[i], dl, LLE_WAVE);
                other[i] = low ? up : down;
            }
            if (in_rot) {
                // 8 (cos, sin) pairs = four 16-byte loads
                const float4* tab = (const float4*)(cos_sin + (n * half + (low ? e0 : e0 - half)) * 2);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float4 t = tab[i];  // cos, sin of element 2i, then of 2i + 1
                    x[2 * i] = low ? x[2 * i] * t.x - other[2 * i] * t.y : x[2 * i] * t.x + other[2 * i] * t.y;
                    x[2 * i + 1] = low ? x[2 * i + 1] * t.z - other[2 * i + 1] * t.w
                                       : x[2 * i + 1] * t.z + other[2 * i + 1] * t.w;
                }
            }
        }
    }
    if (!live) return;
    rbf16x8 y;
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = (bf16_t)x[i];
    if (is_q) {
        *(rbf16x8*)(q_out + (n * nq + head) * d + e0) = y;
        return;
    }
    if (!write_kv) return;
    const int slot = slots[n];
    if (slot < 0) return;
    const int64_t page = slot / page_size;
    const int off = slot - (int)page * page_size;
    bf16_t* page_base = kv_layer + page * page_stride;
    if (is_k) {
        *(rbf16x8*)(page_base + ((int64_t)(head - nq) * page_size + off) * d + e0) = y;
    } else if (write_kv == 1) {
        bf16_t* v = page_base + ((int64_t)nkv + (head - nq - nkv)) * page_size * d + off;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[(int64_t)(e0 + i) * page_size] = y[i];
    }
}

// The V heads of many tokens into the transposed pages.  A workgroup takes 16 consecutive
// tokens of the batch and one kv head: the rows are read whole into LDS, and every thread
// writes one value element of 8 tokens, as one 16-byte store when those tokens sit in
// consecutive slots of one page starting at a multiple of 8 (prompt portions do), else one by one.
#define VW_TOKENS 16
__device__ __forceinline__ void v_write_transposed_block(const bf16_t* __restrict__ qkv,
                                                         const int32_t* __restrict__ slots,
                                                         bf16_t* __restrict__ kv_layer, int N, int nq, int nkv, int d,
                                                         int page_size, int64_t page_stride, int t0, int kvh,
                                                         bf16_t* tile /* [VW_TOKENS][d + 2] */, int* s_slot) {
    const int width = (nq + 2 * nkv) * d;
    const int row = d + 2;
    for (int idx = threadIdx.x; idx < VW_TOKENS * (d / 8); idx += blockDim.x) {
        const int t = idx / (d / 8), ch = idx % (d / 8);
        if (t0 + t < N) {
            const rbf16x8 v = *(const rbf16x8*)(qkv + (int64_t)(t0 + t) * width + (int64_t)(nq + nkv + kvh) * d + 8 * ch);
#pragma unroll
            for (int i = 0; i < 8; ++i) tile[t * row + 8 * ch + i] = v[i];
        }
    }
    if (threadIdx.x < VW_TOKENS) s_slot[threadIdx.x] = t0 + threadIdx.x < N ? slots[t0 + threadIdx.x] : -1;
    __syncthreads();
    for (int idx = threadIdx.x; idx < 2 * d; idx += blockDim.x) {
        const int g = idx / d, e = idx - g * d;  // tokens 8 g .. 8 g + 7, value element e
        const int first = s_slot[8 * g];
        bool run = first >= 0 && first % 8 == 0 && first % page_size + 8 <= page_size;
#pragma unroll
        for (int i = 1; i < 8; ++i) run = run && s_slot[8 * g + i] == first + i;
        if (run) {
            const int64_t page = first / page_size;
            const int off = first - (int)page * page_size;
            rbf16x8 y;
#pragma unroll
            for (int i = 0; i < 8; ++i) y[i] = tile[(8 * g + i) * row + e];
            *(rbf16x8*)(kv_layer + page * page_stride + ((int64_t)nkv + kvh) * page_size * d + (int64_t)e * page_size + off) = y;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int slot = s_slot[8 * g + i];
                if (slot < 0) continue;
                const int64_t page = slot / page_size;
                const int off = slot - (int)page * page_size;
                kv_layer[page * page_stride + ((int64_t)nkv + kvh) * page_size * d + (int64_t)e * page_size + off] =
                    tile[(8 * g + i) * row + e];
            }
        }
    }
}
__global__ __launch_bounds__(256) void v_write_transposed_kernel(const bf16_t* __restrict__ qkv,
                                                                  const int32_t* __restrict__ slots,
                                                                  bf16_t* __restrict__ kv_layer, int N, int nq, int nkv,
                                                                  int d, int page_size, int64_t page_stride) {
    extern __shared__ bf16_t tile[];  // [VW_TOKENS][d + 2]
    __shared__ int s_slot[VW_TOKENS];
    v_write_transposed_block(qkv, slots, kv_layer, N, nq, nkv, d, page_size, page_stride, blockIdx.x * VW_TOKENS,
                             blockIdx.y, tile, s_slot);
}

// The same for a rotation over the whole head (rot == d): a lane holds eight elements of the
// low half and their eight partners of the high half (16-byte loads and stores), so the rotation
// needs no exchange between lanes, and one (cos, sin) pair serves both partners.  `per_token`
// heads of a token are this kernel's: q and k, and v too unless the transposing workgroups take it.
__device__ __forceinline__ void load_weights8(const void* w, int e, int dtype, float (&out)[8]) {
    if (dtype == LLE_F32) {
        const float4 a = *(const float4*)((const float*)w + e), b = *(const float4*)((const float*)w + e + 4);
        out[0] = a.x, out[1] = a.y, out[2] = a.z, out[3] = a.w, out[4] = b.x, out[5] = b.y, out[6] = b.z, out[7] = b.w;
    } else {
        const rbf16x8 v = *(const rbf16x8*)((const bf16_t*)w + e);
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = (float)v[i];
    }
}
__global__ __launch_bounds__(256) void qk_norm_rope_write_pair_kernel(
    const bf16_t* __restrict__ qkv, const int32_t* __restrict__ slots, const void* __restrict__ q_weight,
    const void* __restrict__ k_weight, int weight_dtype, const float* __restrict__ cos_sin, float eps,
    bf16_t* __restrict__ q_out, bf16_t* __restrict__ kv_layer, int nq, int nkv, int d, int page_size,
    int64_t page_stride, int write_kv, int64_t total_heads, int per_token, int head_blocks, int N) {
    // write_kv == 2: the workgroups after the first `head_blocks` take the V heads of 16 tokens and
    // one kv head each into the transposed pages (the same launch: the two kinds of work overlap)
    if ((int)blockIdx.x >= head_blocks) {
        extern __shared__ bf16_t tile[];  // [VW_TOKENS][d + 2]
        __shared__ int s_slot[VW_TOKENS];
        const int vb = blockIdx.x - head_blocks;
        v_write_transposed_block(qkv, slots, kv_layer, N, nq, nkv, d, page_size, page_stride, (vb / nkv) * VW_TOKENS,
                                 vb % nkv, tile, s_slot);
        return;
    }
    const int lph = d / 16;  // lanes per head
    const int lane = threadIdx.x % LLE_WAVE;
    const int heads_per_wave = LLE_WAVE / lph;
    const int64_t gw = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / LLE_WAVE;
    const int64_t flat = gw * heads_per_wave + lane / lph;  // (token, head)
    const int hl = lane % lph;
    const bool live = flat < total_heads;
    const int64_t n = live ? flat / per_token : 0;
    const int head = live ? (int)(flat - n * per_token) : 0;
    const bool is_q = head < nq;
    const bool is_k = !is_q && head < nq + nkv;
    const int half = d / 2;
    const int e_lo = 8 * hl, e_hi = half + 8 * hl;

    float lo[8], hi[8];
    {
        const bf16_t* src = qkv + (n * (nq + 2 * nkv) + head) * d;
        const rbf16x8 a = *(const rbf16x8*)(src + e_lo), b = *(const rbf16x8*)(src + e_hi);
#pragma unroll
        for (int i = 0; i < 8; ++i) lo[i] = (float)a[i], hi[i] = (float)b[i];
    }
    if (is_q || is_k) {
        // the rotation table is asked for beside the row itself
        const float4* tab = (const float4*)(cos_sin + (n * half + e_lo) * 2);  // (cos, sin) of e_lo .. e_lo + 7
        const float4 t0 = tab[0], t1 = tab[1], t2 = tab[2], t3 = tab[3];
        const void* w = is_q ? q_weight : k_weight;
        if (w) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) ss += lo[i] * lo[i] + hi[i] * hi[i];
            for (int o = 1; o < lph; o <<= 1) ss += __shfl_xor(ss, o, LLE_WAVE);
            const float inv = 1.0f / sqrtf(ss / (float)d + eps);
            float wl[8], wh[8];
            load_weights8(w, e_lo, weight_dtype, wl);
            load_weights8(w, e_hi, weight_dtype, wh);
#pragma unroll
            for (int i = 0; i < 8; ++i) lo[i] = lo[i] * inv * wl[i], hi[i] = hi[i] * inv * wh[i];
        }
        const float cs[8] = {t0.x, t0.z, t1.x, t1.z, t2.x, t2.z, t3.x, t3.z};
        const float sn[8] = {t0.y, t0.w, t1.y, t1.w, t2.y, t2.w, t3.y, t3.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float a = lo[i], b = hi[i];
            lo[i] = a * cs[i] - b * sn[i];
            hi[i] = b * cs[i] + a * sn[i];
        }
    }
    if (!live) return;
    rbf16x8 ylo, yhi;
#pragma unroll
    for (int i = 0; i < 8; ++i) ylo[i] = (bf16_t)lo[i], yhi[i] = (bf16_t)hi[i];
    if (is_q) {
        bf16_t* dst = q_out + (n * nq + head) * d;
        *(rbf16x8*)(dst + e_lo) = ylo;
        *(rbf16x8*)(dst + e_hi) = yhi;
        return;
    }
    if (!write_kv) return;
    const int slot = slots[n];
    if (slot < 0) return;
    const int64_t page = slot / page_size;
    const int off = slot - (int)page * page_size;
    bf16_t* page_base = kv_layer + page * page_stride;
    if (is_k) {
        bf16_t* dst = page_base + ((int64_t)(head - nq) * page_size + off) * d;
        *(rbf16x8*)(dst + e_lo) = ylo;
        *(rbf16x8*)(dst + e_hi) = yhi;
    } else if (write_kv == 1) {
        bf16_t* v = page_base + ((int64_t)nkv + (head - nq - nkv)) * page_size * d + off;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            v[(int64_t)(e_lo + i) * page_size] = ylo[i];
            v[(int64_t)(e_hi + i) * page_size] = yhi[i];
        }
    }
}

// cos and sin of float(pos) * inv_freq[i] for every token of the step: out [N][half][2]
__global__ __launch_bounds__(256) void rope_table_kernel(const int32_t* __restrict__ positions,
                                                          const float* __restrict__ inv_freq,
                                                          float* __restrict__ out, int64_t total, int half) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int64_t n = idx / half;
    const int i = (int)(idx - n * half);
    float s, c;
    sincosf((float)positions[n] * inv_freq[i], &s, &c);
    ((float2*)out)[idx] = make_float2(c, s);
}

extern "C" int lle_rope_table(const void* positions, const void* inv_freq, void* out, int N, int half,
                              hipStream_t stream) {
    const int64_t total = (int64_t)N * half;
    if (total <= 0) return 0;
    rope_table_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>((const int32_t*)positions,
                                                                      (const float*)inv_freq, (float*)out, total, half);
    LLE_RETURN_LAUNCH_STATUS();
}

extern "C" int lle_qk_norm_rope_write(const void* qkv, const void* slots,
                                      const void* q_weight, const void* k_weight, int weight_dtype,
                                      const void* cos_sin, int rot, float eps, void* q_out, void* kv_layer,
                                      int N, int nq, int nkv, int d, int page_size, int64_t page_stride,
                                      int write_kv, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    const bool pow2 = d == 16 || d == 32 || d == 64 || d == 128 || d == 256;
    if (dtype == LLE_BF16 && pow2 && rot % 16 == 0 && (int64_t)N * (nq + 2 * nkv) < (1ll << 31)) {
        const int total_heads = N * (nq + 2 * nkv);
        const int heads_per_block = 4 * (LLE_WAVE / (d / 8));
        const int blocks = (total_heads + heads_per_block - 1) / heads_per_block;
        // many tokens: V goes through the transposing kernel (16-byte stores into the pages)
        const bool split_v = write_kv && N >= 64 && page_size % 8 == 0 && (N + VW_TOKENS - 1) / VW_TOKENS <= 0x7fffffff;
        const int64_t v_blocks = split_v ? (int64_t)((N + VW_TOKENS - 1) / VW_TOKENS) * nkv : 0;
        if (rot == d) {
            // the pair kernel: 16 elements a lane; with the transposing workgroups in the same launch
            // the V heads are theirs alone (without a cache write nobody needs them)
            const bool own_v = write_kv && !split_v;
            const int per_token = nq + nkv + (own_v ? nkv : 0);
            const int64_t pair_heads = (int64_t)N * per_token;
            const int pair_heads_per_block = 4 * (LLE_WAVE / (d / 16));
            const int64_t pair_blocks = (pair_heads + pair_heads_per_block - 1) / pair_heads_per_block;
            const bool one_launch = pair_blocks + v_blocks <= 0x7fffffff;
            qk_norm_rope_write_pair_kernel<<<(unsigned)(one_launch ? pair_blocks + v_blocks : pair_blocks), 256,
                                             split_v && one_launch ? VW_TOKENS * (d + 2) * sizeof(bf16_t) : 0, stream>>>(
                (const bf16_t*)qkv, (const int32_t*)slots, q_weight, k_weight, weight_dtype, (const float*)cos_sin, eps,
                (bf16_t*)q_out, (bf16_t*)kv_layer, nq, nkv, d, page_size, page_stride,
                write_kv ? (split_v ? 2 : 1) : 0, pair_heads, per_token, (int)pair_blocks, N);
            if (one_launch) LLE_RETURN_LAUNCH_STATUS();
        } else
            qk_norm_rope_write_vec_kernel<<<blocks, 256, 0, stream>>>(
                (const bf16_t*)qkv, (const int32_t*)slots, q_weight, k_weight, weight_dtype, (const float*)cos_sin, rot,
                eps, (bf16_t*)q_out, (bf16_t*)kv_layer, nq, nkv, d, page_size, page_stride,
                write_kv ? (split_v ? 2 : 1) : 0, total_heads);
        if (split_v)
            v_write_transposed_kernel<<<dim3((N + VW_TOKENS - 1) / VW_TOKENS, nkv), 256,
                                        VW_TOKENS * (d + 2) * sizeof(bf16_t), stream>>>(
                (const bf16_t*)qkv, (const int32_t*)slots, (bf16_t*)kv_layer, N, nq, nkv, d, page_size, page_stride);
        LLE_RETURN_LAUNCH_STATUS();
    }
    dim3 grid(N, nq + 2 * nkv);
    if (dtype == LLE_F32)
        qk_norm_rope_write_kernel<float><<<grid, 64, 0, stream>>>(
            (const float*)qkv, (const int32_t*)slots, q_weight, k_weight, weight_dtype, (const float*)cos_sin, rot, eps,
            (float*)q_out, (float*)kv_layer, nq, nkv, d, page_size, page_stride, write_kv);
    else
        qk_norm_rope_write_kernel<bf16_t><<<grid, 64, 0, stream>>>(
            (const bf16_t*)qkv, (const int32_t*)slots, q_weight, k_weight, weight_dtype, (const float*)cos_sin, rot, eps,
            (bf16_t*)q_out, (bf16_t*)kv_layer, nq, nkv, d, page_size, page_stride, write_kv);
    LLE_RETURN_LAUNCH_STATUS();
}
