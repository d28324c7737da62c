// Paged grouped-query attention over the cache, for any mix of prompt portions
// and single decoded tokens in one launch.
//
// The reference has three kernels, none of which covers a prompt portion after
// a past: flash_attention_kernel (prefill of one request over its own K/V,
// src/ops/attention.cu:320-426), flash_attention_kv_cache_kernel (:429-535) and
// flash_attention_paged_kv_cache_batch_kernel (:537-669, decode rows through a
// block table packed and uploaded per layer and step, :959-1020).  Here the K/V
// of the step's tokens are already in their pages, the block tables live on the
// device, and every query token attends through them:
//   query at cache position p (= kv_len - q_len + its index in the portion)
//   sees keys lo..p,  lo = max(0, p - window + 1) with a window, else 0
//   score_j = (q . k_j) * scale;  softmax over j streamed in 32-bit (m, l, acc)
//   kv head of q head h = h / (nq / nkv)                  (:577-668 for the maths)
// A cache page holds [2 (K, V)][nkv][page_size][d].
#include "common.h"

LLE_DEFINE_ERROR_STRING()

#define ATT_WAVES 4
#define ATT_MAX_R 4  // head_dim <= 256

// One workgroup per (query token, q head); each wavefront walks every fourth
// key, lanes split the head dimension.  Any head_dim <= 256, page size, window.
template <typename T>
__global__ __launch_bounds__(ATT_WAVES* LLE_WAVE) void paged_attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ kv_layer, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ kv_lens, const int32_t* __restrict__ token_seq, T* __restrict__ out, int nq,
    int nkv, int d, int page_size, int64_t page_stride, int max_pages, int window, float scale) {
    __shared__ float s_m[ATT_WAVES], s_l[ATT_WAVES];
    __shared__ float s_acc[ATT_WAVES][ATT_MAX_R * LLE_WAVE];

    const int64_t tok = blockIdx.x;
    const int h = blockIdx.y;
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int s = token_seq[tok];
    const int kv_len = kv_lens[s];
    const int q_start = cu_tokens[s];
    const int q_len = cu_tokens[s + 1] - q_start;
    const int pos = kv_len - q_len + (int)(tok - q_start);
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int kvh = h / (nq / nkv);
    const int32_t* table = block_tables + (int64_t)seq_slots[s] * max_pages;

    float qv[ATT_MAX_R], acc[ATT_MAX_R];
#pragma unroll
    for (int r = 0; r < ATT_MAX_R; ++r) {
        const int e = lane + LLE_WAVE * r;
        qv[r] = e < d ? to_f32<T>(q[(tok * nq + h) * d + e]) : 0.f;
        acc[r] = 0.f;
    }
    float m = -FLT_MAX, l = 0.f;
    const int64_t v_off = (int64_t)nkv * page_size * d;
    for (int j = lo + wave; j <= pos; j += ATT_WAVES) {
        const int lp = j / page_size;
        const int64_t page = table[lp];
        const T* kp = kv_layer + page * page_stride + ((int64_t)kvh * page_size + (j - lp * page_size)) * d;
        const T* vp = kp + v_off;
        float dot = 0.f;
#pragma unroll
        for (int r = 0; r < ATT_MAX_R; ++r) {
            const int e = lane + LLE_WAVE * r;
            if (e < d) dot += qv[r] * to_f32<T>(kp[e]);
        }
        const float score = wave_sum(dot) * scale;
        const float new_m = fmaxf(m, score);
        const float alpha = expf(m - new_m);
        const float beta = expf(score - new_m);
        l = l * alpha + beta;
#pragma unroll
        for (int r = 0; r < ATT_MAX_R; ++r) {
            const int e = lane + LLE_WAVE * r;
            if (e < d) acc[r] = acc[r] * alpha + beta * to_f32<T>(vp[e]);
        }
        m = new_m;
    }
    if (lane == 0) {
        s_m[wave] = m;
        s_l[wave] = l;
    }
#pragma unroll
    for (int r = 0; r < ATT_MAX_R; ++r) s_acc[wave][lane + LLE_WAVE * r] = acc[r];
    __syncthreads();
    float big = s_m[0];
    for (int w = 1; w < ATT_WAVES; ++w) big = fmaxf(big, s_m[w]);
    for (int e = threadIdx.x; e < d; e += blockDim.x) {
        float num = 0.f, den = 0.f;
        for (int w = 0; w < ATT_WAVES; ++w) {
            const float f = expf(s_m[w] - big);  // a wavefront without keys has l = 0, acc = 0
            num += s_acc[w][e] * f;
            den += s_l[w] * f;
        }
        out[(tok * nq + h) * d + e] = from_f32<T>(num / den);
    }
}

extern "C" int lle_paged_attention_generic(const void* q, const void* kv_layer, const void* block_tables,
                                           const void* seq_slots, const void* cu_tokens, const void* kv_lens,
                                           const void* token_seq, void* out, int N, int nq, int nkv, int d,
                                           int page_size, int64_t page_stride, int max_pages, int window,
                                           float scale, int dtype, hipStream_t stream) {
    if (N <= 0) return 0;
    if (d > ATT_MAX_R * LLE_WAVE) return (int)hipErrorInvalidValue;
    dim3 grid(N, nq);
    if (dtype == LLE_F32)
        paged_attention_generic_kernel<float><<<grid, ATT_WAVES * LLE_WAVE, 0, stream>>>(
            (const float*)q, (const float*)kv_layer, (const int32_t*)block_tables, (const int32_t*)seq_slots,
            (const int32_t*)cu_tokens, (const int32_t*)kv_lens, (const int32_t*)token_seq, (float*)out, nq, nkv, d,
            page_size, page_stride, max_pages, window, scale);
    else
        paged_attention_generic_kernel<bf16_t><<<grid, ATT_WAVES * LLE_WAVE, 0, stream>>>(
            (const bf16_t*)q, (const bf16_t*)kv_layer, (const int32_t*)block_tables, (const int32_t*)seq_slots,
            (const int32_t*)cu_tokens, (const int32_t*)kv_lens, (const int32_t*)token_seq, (bf16_t*)out, nq, nkv,
            d, page_size, page_stride, max_pages, window, scale);
    LLE_RETURN_LAUNCH_STATUS();
}
