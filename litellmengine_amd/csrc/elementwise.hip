// Embedding row gather, SiLU-and-mul and the bias of a projection.
// Counterparts in the reference: embedding_forward_kernel
// (src/layers/embedding.cu:91-118) and silu_and_mul_kernel
// (src/ops/silu_and_mul.cu:64-80); both are 32-bit only there.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

// out[n, :] = table[ids[n], :] as 32-bit (the residual stream is 32-bit in
// every mode).  The host has checked 0 <= id < V.
// An id below zero stands for "the token that the last step picked for this token's request": it
// is read from feedback[seq_slots[token_seq[n]]], where the picking kernel left it (a step that
// was launched before the host had read the step before it; the picking kernel only writes ids
// of the vocabulary).
template <typename T>
__global__ __launch_bounds__(256) void embedding_kernel(const int32_t* __restrict__ ids,
                                                         const T* __restrict__ table,
                                                         float* __restrict__ out, int H,
                                                         const int32_t* __restrict__ feedback,
                                                         const int32_t* __restrict__ token_seq,
                                                         const int32_t* __restrict__ seq_slots) {
    const int64_t n = blockIdx.x;
    int id = ids[n];
    if (id < 0) id = feedback ? feedback[seq_slots[token_seq[n]]] : 0;
    const T* row = table + (int64_t)id * H;
    float* o = out + n * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f32<T>(row[i]);
}

// `feedback`, `token_seq` [N] and `seq_slots`: all three or none
extern "C" int lle_embedding_feedback(const void* ids, const void* table, void* out, int N, int H, int dtype,
                                      const void* feedback, const void* token_seq, const void* seq_slots,
                                      hipStream_t stream) {
    if (N <= 0) return 0;
    if ((feedback != nullptr) != (token_seq != nullptr) || (feedback != nullptr) != (seq_slots != nullptr))
        return (int)hipErrorInvalidValue;
    if (dtype == LLE_F32)
        embedding_kernel<float><<<N, 256, 0, stream>>>((const int32_t*)ids, (const float*)table, (float*)out, H,
                                                        (const int32_t*)feedback, (const int32_t*)token_seq,
                                                        (const int32_t*)seq_slots);
    else
        embedding_kernel<bf16_t><<<N, 256, 0, stream>>>((const int32_t*)ids, (const bf16_t*)table, (float*)out, H,
                                                         (const int32_t*)feedback, (const int32_t*)token_seq,
                                                         (const int32_t*)seq_slots);
    LLE_RETURN_LAUNCH_STATUS();
}

extern "C" int lle_embedding(const void* ids, const void* table, void* out, int N, int H, int dtype,
                             hipStream_t stream) {
    return lle_embedding_feedback(ids, table, out, N, H, dtype, nullptr, nullptr, nullptr, stream);
}

// gate_up [N, 2I] (gate columns first) -> out [N, I] = gate / (1 + exp(-gate)) * up, in 32-bit
template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out,
                                                        int64_t total, int I) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t n = idx / I;
        const int i = (int)(idx - n * I);
        const float g = to_f32<T>(gate_up[n * 2 * I + i]);
        const float u = to_f32<T>(gate_up[n * 2 * I + I + i]);
        out[idx] = from_f32<T>(g / (1.0f + expf(-g)) * u);
    }
}

// the same for bfloat16 rows whose width is a multiple of 8: 16-byte loads and stores
typedef bf16_t ebf16x8 __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(256) void silu_mul_vec_kernel(const bf16_t* __restrict__ gate_up,
                                                            bf16_t* __restrict__ out, int64_t total8, int I8) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total8;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t n = idx / I8;
        const int i = (int)(idx - n * I8);
        const ebf16x8 g = *(const ebf16x8*)(gate_up + (n * 2 * I8 + i) * 8);
        const ebf16x8 u = *(const ebf16x8*)(gate_up + (n * 2 * I8 + I8 + i) * 8);
        ebf16x8 o;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float gf = (float)g[k];
            o[k] = (bf16_t)(gf / (1.0f + expf(-gf)) * (float)u[k]);
        }
        *(ebf16x8*)(out + idx * 8) = o;
    }
}

extern "C" int lle_silu_mul(const void* gate_up, void* out, int N, int I, int dtype, hipStream_t stream) {
    const int64_t total = (int64_t)N * I;
    if (total <= 0) return 0;
    if (dtype == LLE_BF16 && I % 8 == 0) {
        const int64_t total8 = total / 8;
        int64_t vblocks = (total8 + 255) / 256;
        if (vblocks > 16384) vblocks = 16384;
        silu_mul_vec_kernel<<<(int)vblocks, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, total8, I / 8);
        LLE_RETURN_LAUNCH_STATUS();
    }
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (dtype == LLE_F32)
        silu_mul_kernel<float><<<(int)blocks, 256, 0, stream>>>((const float*)gate_up, (float*)out, total, I);
    else
        silu_mul_kernel<bf16_t><<<(int)blocks, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, total, I);
    LLE_RETURN_LAUNCH_STATUS();
}

// x[m, :] += bias[:] in place, the sum in 32-bit (the reference's Linear has the same optional
// bias, src/layers/linear.cu:169-215; Qwen3 uses none).  `bias` holds TB, x holds T.
template <typename T, typename TB>
__global__ __launch_bounds__(256) void add_bias_kernel(T* __restrict__ x, const TB* __restrict__ bias, int64_t total,
                                                        int N) {
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x)
        x[idx] = from_f32<T>(to_f32<T>(x[idx]) + to_f32<TB>(bias[idx % N]));
}

extern "C" int lle_add_bias(void* x, const void* bias, int M, int N, int dtype, int bias_dtype, hipStream_t stream) {
    const int64_t total = (int64_t)M * N;
    if (total <= 0) return 0;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
#define LLE_BIAS_CASE(T, TB) add_bias_kernel<T, TB><<<(int)blocks, 256, 0, stream>>>((T*)x, (const TB*)bias, total, N)
    if (dtype == LLE_F32 && bias_dtype == LLE_F32) LLE_BIAS_CASE(float, float);
    else if (dtype == LLE_F32) LLE_BIAS_CASE(float, bf16_t);
    else if (bias_dtype == LLE_F32) LLE_BIAS_CASE(bf16_t, float);
    else LLE_BIAS_CASE(bf16_t, bf16_t);
#undef LLE_BIAS_CASE
    LLE_RETURN_LAUNCH_STATUS();
}
