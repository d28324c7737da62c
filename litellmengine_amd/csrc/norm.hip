// RMSNorm fused with the residual add (and, for the first norm of a model, with the embedding).
// Reference counterparts: rms_norm_forward_kernel (src/layers/rms_norm.cu:97-141)
// and add_fp32_kernel (src/ops/add.cu:16-27), two launches there.
//
//   h = hidden[row] (+ delta[row])          32-bit sum, the residual stream
//   out[r] = h * rsqrt(mean(h^2) + eps) * w
// With `rows == nullptr` row r is r and h is written back to `hidden`; with a
// row list (the output head: only the wanted rows) nothing is written back.
#include "common.h"

LLE_DEFINE_ERROR_STRING()

template <typename T>
__global__ __launch_bounds__(1024) void add_rmsnorm_kernel(float* __restrict__ hidden, const T* __restrict__ delta,
                                                            const int32_t* __restrict__ rows,
                                                            const void* __restrict__ weight, int weight_dtype,
                                                            T* __restrict__ out, int H, float eps) {
    __shared__ float red[16];
    const int64_t r = blockIdx.x;
    const int64_t row = rows ? (int64_t)rows[r] : r;
    float* h = hidden + row * H;
    const T* dl = delta ? delta + row * H : nullptr;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = h[i];
        if (dl) v += to_f32<T>(dl[i]);
        if (!rows && dl) h[i] = v;
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    T* o = out + r * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        float v = h[i];
        if (rows && dl) v += to_f32<T>(dl[i]);
        o[i] = from_f32<T>(v * inv * load_as_f32(weight, i, weight_dtype));
    }
}

// four consecutive elements of either type as 32-bit floats
template <typename T> struct Quad;
template <> struct Quad<float> {
    static __device__ __forceinline__ float4 load(const float* p) { return *(const float4*)p; }
    static __device__ __forceinline__ void store(float* p, float4 v) { *(float4*)p = v; }
};
template <> struct Quad<bf16_t> {
    typedef bf16_t vec __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ float4 load(const bf16_t* p) {
        const vec v = *(const vec*)p;
        return make_float4((float)v[0], (float)v[1], (float)v[2], (float)v[3]);
    }
    static __device__ __forceinline__ void store(bf16_t* p, float4 v) {
        *(vec*)p = vec{(bf16_t)v.x, (bf16_t)v.y, (bf16_t)v.z, (bf16_t)v.w};
    }
};

__device__ __forceinline__ float4 load_weight4(const void* w, int i, int dtype) {
    return dtype == LLE_F32 ? Quad<float>::load((const float*)w + i) : Quad<bf16_t>::load((const bf16_t*)w + i);
}

// The same sums in one pass for rows of up to 256 * 4 * NORM_CHUNKS elements (a multiple of 4):
// every thread keeps its part of the row in registers between the sum and the scaling.
#define NORM_CHUNKS 8
// `delta` may come as `slices` partial sums of type TD, `slice_stride` elements apart (a product
// over slices of K leaves them so): they are added in slice order.
template <typename T, typename TD = T, bool SLICED = false>
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(float* __restrict__ hidden, const TD* __restrict__ delta,
                                                              const int32_t* __restrict__ rows,
                                                              const void* __restrict__ weight, int weight_dtype,
                                                              T* __restrict__ out, int H, float eps, int slices = 1,
                                                              int64_t slice_stride = 0) {
    __shared__ float red[16];
    const int64_t r = blockIdx.x;
    const int64_t row = rows ? (int64_t)rows[r] : r;
    float* h = hidden + row * H;
    const TD* dl = delta ? delta + row * H : nullptr;
    float4 v[NORM_CHUNKS], wv[NORM_CHUNKS];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NORM_CHUNKS; ++k) {  // the weights do not wait for the sum
        const int i = (k * 256 + threadIdx.x) * 4;
        if (i < H) wv[k] = load_weight4(weight, i, weight_dtype);
    }
    if constexpr (SLICED) {
        // all of a row's loads of one kind are asked for together (a load that waits for the one before
        // it pays the memory's latency once more): the row and the first slice, then slice by slice
        float4 d[NORM_CHUNKS];
    #pragma unroll
        for (int k = 0; k < NORM_CHUNKS; ++k) {
            const int i = (k * 256 + threadIdx.x) * 4;
            if (i < H) {
                v[k] = *(const float4*)(h + i);
                if (dl) d[k] = Quad<TD>::load(dl + i);
            }
        }
        if (dl) {
    #pragma unroll 2
            for (int sl = 1; sl < slices; ++sl) {
                float4 e[NORM_CHUNKS];
    #pragma unroll
                for (int k = 0; k < NORM_CHUNKS; ++k) {
                    const int i = (k * 256 + threadIdx.x) * 4;
                    if (i < H) e[k] = Quad<TD>::load(dl + sl * slice_stride + i);
                }
    #pragma unroll
                for (int k = 0; k < NORM_CHUNKS; ++k) {
                    const int i = (k * 256 + threadIdx.x) * 4;
                    if (i < H) {
                        d[k].x += e[k].x;
                        d[k].y += e[k].y;
                        d[k].z += e[k].z;
                        d[k].w += e[k].w;
                    }
                }
            }
        }
    #pragma unroll
        for (int k = 0; k < NORM_CHUNKS; ++k) {
            const int i = (k * 256 + threadIdx.x) * 4;
            if (i < H) {
                float4 x = v[k];
                if (dl) {
                    x.x += d[k].x;
                    x.y += d[k].y;
                    x.z += d[k].z;
                    x.w += d[k].w;
                    if (!rows) *(float4*)(h + i) = x;
                }
                v[k] = x;
                ss += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < NORM_CHUNKS; ++k) {
            const int i = (k * 256 + threadIdx.x) * 4;
            if (i < H) {
                float4 x = *(const float4*)(h + i);
                if (dl) {
                    const float4 d = Quad<TD>::load(dl + i);
                    x.x += d.x;
                    x.y += d.y;
                    x.z += d.z;
                    x.w += d.w;
                    if (!rows) *(float4*)(h + i) = x;
                }
                v[k] = x;
                ss += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
            }
        }
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    T* o = out + r * H;
#pragma unroll
    for (int k = 0; k < NORM_CHUNKS; ++k) {
        const int i = (k * 256 + threadIdx.x) * 4;
        if (i < H) {
            const float4 w = wv[k];
            Quad<T>::store(o + i, make_float4(v[k].x * inv * w.x, v[k].y * inv * w.y, v[k].z * inv * w.z,
                                              v[k].w * inv * w.w));
        }
    }
}

// hidden += sums[0] + sums[1] + ... (float32 [slices][N][H], rows of hidden and of a slice alike), then
// the norm as lle_add_rmsnorm; H a multiple of 4 up to 256 * 4 * NORM_CHUNKS
// The first rows of the residual stream and their first norm in one launch: hidden[n] =
// table[id(n)] as 32-bit (the embedding, src/layers/embedding.cu:75-87), out[n] its RMSNorm.
// An id below zero stands for feedback[seq_slots[token_seq[n]]] (the token that the step before
// picked for the row's request and left on the device), as in the embedding kernel itself.
// VEC: rows of a multiple of 4 and at most 256 * 4 * NORM_CHUNKS elements, kept in registers.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void embedding_rmsnorm_kernel(const int32_t* __restrict__ ids,
                                                                const T* __restrict__ table,
                                                                float* __restrict__ hidden,
                                                                const void* __restrict__ weight, int weight_dtype,
                                                                T* __restrict__ out, int H, float eps,
                                                                const int32_t* __restrict__ feedback,
                                                                const int32_t* __restrict__ token_seq,
                                                                const int32_t* __restrict__ seq_slots) {
    __shared__ float red[16];
    const int64_t n = blockIdx.x;
    int id = ids[n];
    if (id < 0) id = feedback ? feedback[seq_slots[token_seq[n]]] : 0;
    const T* row = table + (int64_t)id * H;
    float* h = hidden + n * H;
    T* o = out + n * H;
    float ss = 0.f;
    if constexpr (VEC) {
        float4 v[NORM_CHUNKS], wv[NORM_CHUNKS];
#pragma unroll
        for (int k = 0; k < NORM_CHUNKS; ++k) {
            const int i = (k * 256 + threadIdx.x) * 4;
            if (i < H) {
                wv[k] = load_weight4(weight, i, weight_dtype);
                v[k] = Quad<T>::load(row + i);
            }
        }
#pragma unroll
        for (int k = 0; k < NORM_CHUNKS; ++k) {
            const int i = (k * 256 + threadIdx.x) * 4;
            if (i < H) {
                *(float4*)(h + i) = v[k];
                ss += v[k].x * v[k].x + v[k].y * v[k].y + v[k].z * v[k].z + v[k].w * v[k].w;
            }
        }
        ss = block_sum(ss, red);
        const float inv = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
        for (int k = 0; k < NORM_CHUNKS; ++k) {
            const int i = (k * 256 + threadIdx.x) * 4;
            if (i < H) {
                const float4 w = wv[k];
                Quad<T>::store(o + i, make_float4(v[k].x * inv * w.x, v[k].y * inv * w.y, v[k].z * inv * w.z,
                                                  v[k].w * inv * w.w));
            }
        }
    } else {
        for (int i = threadIdx.x; i < H; i += blockDim.x) {
            const float v = to_f32<T>(row[i]);
            h[i] = v;
            ss += v * v;
        }
        ss = block_sum(ss, red);
        const float inv = 1.0f / sqrtf(ss / (float)H + eps);
        // (each thread reads back the elements that it wrote itself)
        for (int i = threadIdx.x; i < H; i += blockDim.x)
            o[i] = from_f32<T>(h[i] * inv * load_as_f32(weight, i, weight_dtype));
    }
}

// ids int32 [N], table [V, H] and out [N, H] of `dtype`, hidden float32 [N, H]; `feedback`,
// `token_seq` [N] and `seq_slots`: all three or none.  The host has checked the ids.
extern "C" int lle_embedding_rmsnorm(const void* ids, const void* table, void* hidden, const void* weight,
                                     int weight_dtype, void* out, int N, int H, float eps, int dtype,
                                     const void* feedback, const void* token_seq, const void* seq_slots,
                                     hipStream_t stream) {
    if (N <= 0 || H <= 0) return 0;
    if ((feedback != nullptr) != (token_seq != nullptr) || (feedback != nullptr) != (seq_slots != nullptr))
        return (int)hipErrorInvalidValue;
    const bool vec = H % 4 == 0 && H <= 256 * 4 * NORM_CHUNKS;
#define LLE_EMBED_NORM(T, VEC)                                                                                  \
    embedding_rmsnorm_kernel<T, VEC><<<N, 256, 0, stream>>>(                                                    \
        (const int32_t*)ids, (const T*)table, (float*)hidden, weight, weight_dtype, (T*)out, H, eps,            \
        (const int32_t*)feedback, (const int32_t*)token_seq, (const int32_t*)seq_slots)
    if (dtype == LLE_F32) {
        if (vec) LLE_EMBED_NORM(float, true); else LLE_EMBED_NORM(float, false);
    } else if (dtype == LLE_BF16) {
        if (vec) LLE_EMBED_NORM(bf16_t, true); else LLE_EMBED_NORM(bf16_t, false);
    } else {
        return (int)hipErrorInvalidValue;
    }
#undef LLE_EMBED_NORM
    LLE_RETURN_LAUNCH_STATUS();
}

extern "C" int lle_add_rmsnorm_sums(void* hidden, const void* sums, int slices, int64_t slice_stride, const void* rows,
                                    const void* weight, int weight_dtype, void* out, int R, int H, float eps, int dtype,
                                    hipStream_t stream) {
    if (R <= 0) return 0;
    if (H % 4 != 0 || H > 256 * 4 * NORM_CHUNKS || slices < 1 || !sums) return (int)hipErrorInvalidValue;
    if (dtype == LLE_F32)
        add_rmsnorm_vec_kernel<float, float, true><<<R, 256, 0, stream>>>((float*)hidden, (const float*)sums,
                                                                     (const int32_t*)rows, weight, weight_dtype,
                                                                     (float*)out, H, eps, slices, slice_stride);
    else
        add_rmsnorm_vec_kernel<bf16_t, float, true><<<R, 256, 0, stream>>>((float*)hidden, (const float*)sums,
                                                                      (const int32_t*)rows, weight, weight_dtype,
                                                                      (bf16_t*)out, H, eps, slices, slice_stride);
    LLE_RETURN_LAUNCH_STATUS();
}

extern "C" int lle_add_rmsnorm(void* hidden, const void* delta, const void* rows, const void* weight,
                               int weight_dtype, void* out, int R, int H, float eps, int dtype,
                               hipStream_t stream) {
    if (R <= 0) return 0;
    if (H % 4 == 0 && H <= 256 * 4 * NORM_CHUNKS) {
        if (dtype == LLE_F32)
            add_rmsnorm_vec_kernel<float><<<R, 256, 0, stream>>>((float*)hidden, (const float*)delta,
                                                                  (const int32_t*)rows, weight, weight_dtype,
                                                                  (float*)out, H, eps);
        else
            add_rmsnorm_vec_kernel<bf16_t><<<R, 256, 0, stream>>>((float*)hidden, (const bf16_t*)delta,
                                                                   (const int32_t*)rows, weight, weight_dtype,
                                                                   (bf16_t*)out, H, eps);
        LLE_RETURN_LAUNCH_STATUS();
    }
    int threads = 256;
    if (H > 2048) threads = 512;
    if (H > 8192) threads = 1024;
    if (dtype == LLE_F32)
        add_rmsnorm_kernel<float><<<R, threads, 0, stream>>>((float*)hidden, (const float*)delta,
                                                              (const int32_t*)rows, weight, weight_dtype,
                                                              (float*)out, H, eps);
    else
        add_rmsnorm_kernel<bf16_t><<<R, threads, 0, stream>>>((float*)hidden, (const bf16_t*)delta,
                                                               (const int32_t*)rows, weight, weight_dtype,
                                                               (bf16_t*)out, H, eps);
    LLE_RETURN_LAUNCH_STATUS();
}

// plain RMSNorm of activation rows x [R, H] of type T (no residual): out = norm(x) * w
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const T* __restrict__ x, const void* __restrict__ weight,
                                                       int weight_dtype, T* __restrict__ out, int H, float eps) {
    __shared__ float red[16];
    const int64_t r = blockIdx.x;
    const T* xr = x + r * H;
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float v = to_f32<T>(xr[i]);
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
    T* o = out + r * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x)
        o[i] = from_f32<T>(to_f32<T>(xr[i]) * inv * load_as_f32(weight, i, weight_dtype));
}

extern "C" int lle_rmsnorm(const void* x, const void* weight, int weight_dtype, void* out, int R, int H, float eps,
                           int dtype, hipStream_t stream) {
    if (R <= 0) return 0;
    if (dtype == LLE_F32)
        rmsnorm_kernel<float><<<R, 256, 0, stream>>>((const float*)x, weight, weight_dtype, (float*)out, H, eps);
    else
        rmsnorm_kernel<bf16_t><<<R, 256, 0, stream>>>((const bf16_t*)x, weight, weight_dtype, (bf16_t*)out, H, eps);
    LLE_RETURN_LAUNCH_STATUS();
}
