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
// >= rot pass through.  angle = float(pos) * inv_freq[i], all in 32-bit.
// A cache page holds K as [nkv][page_size][d] and then V as [nkv][d][page_size]
// (V is kept transposed so that the matrix-core attention kernels find the keys
// of one value column next to each other); slot = page * page_size + offset;
// slot < 0 skips the write.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

template <typename T>
__global__ __launch_bounds__(64) void qk_norm_rope_write_kernel(
    const T* __restrict__ qkv, const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
    const void* __restrict__ q_weight, const void* __restrict__ k_weight, int weight_dtype,
    const float* __restrict__ inv_freq, int rot, float eps, T* __restrict__ q_out, T* __restrict__ kv_layer,
    int nq, int nkv, int d, int page_size, int64_t page_stride, int write_kv) {
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
    const float pos = (float)positions[n];
    for (int i = lane; i < half; i += LLE_WAVE) {
        float x1 = to_f32<T>(src[i]) * inv;
        float x2 = to_f32<T>(src[i + half]) * inv;
        if (w) {
            x1 *= load_as_f32(w, i, weight_dtype);
            x2 *= load_as_f32(w, i + half, weight_dtype);
        }
        const float ang = pos * inv_freq[i];
        float s, c;
        sincosf(ang, &s, &c);
        dst[i] = from_f32<T>(x1 * c - x2 * s);
        dst[i + half] = from_f32<T>(x2 * c + x1 * s);
    }
    for (int i = rot + lane; i < d; i += LLE_WAVE) {
        float x = to_f32<T>(src[i]) * inv;
        if (w) x *= load_as_f32(w, i, weight_dtype);
        dst[i] = from_f32<T>(x);
    }
}

extern "C" int lle_qk_norm_rope_write(const void* qkv, const void* positions, const void* slots,
                                      const void* q_weight, const void* k_weight, int weight_dtype,
                                      const void* inv_freq, int rot, float eps, void* q_out, void* kv_layer,
                                      int N, int nq, int nkv, int d, int page_size, int64_t page_stride,
                                      int write_kv, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    dim3 grid(N, nq + 2 * nkv);
    if (dtype == LLE_F32)
        qk_norm_rope_write_kernel<float><<<grid, 64, 0, stream>>>(
            (const float*)qkv, (const int32_t*)positions, (const int32_t*)slots, q_weight, k_weight, weight_dtype,
            (const float*)inv_freq, rot, eps, (float*)q_out, (float*)kv_layer, nq, nkv, d, page_size, page_stride,
            write_kv);
    else
        qk_norm_rope_write_kernel<bf16_t><<<grid, 64, 0, stream>>>(
            (const bf16_t*)qkv, (const int32_t*)positions, (const int32_t*)slots, q_weight, k_weight, weight_dtype,
            (const float*)inv_freq, rot, eps, (bf16_t*)q_out, (bf16_t*)kv_layer, nq, nkv, d, page_size, page_stride,
            write_kv);
    LLE_RETURN_LAUNCH_STATUS();
}
