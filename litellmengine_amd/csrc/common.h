// Shared device helpers for the gfx950 kernels: element types, conversions,
// wavefront (64 lanes) and workgroup reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <float.h>

typedef __bf16 bf16_t;

// dtype codes shared with the Python side (csrc/ops.py)
#define LLE_F32 0
#define LLE_BF16 1

#define LLE_WAVE 64

template <typename T> __device__ __forceinline__ float to_f32(T x);
template <> __device__ __forceinline__ float to_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t x) { return (float)x; }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return (bf16_t)x; }

// a value of either float type behind a void pointer (norm weights may be
// stored in 32-bit while activations are 16-bit)
__device__ __forceinline__ float load_as_f32(const void* p, int64_t i, int dtype) {
    return dtype == LLE_F32 ? ((const float*)p)[i] : (float)((const bf16_t*)p)[i];
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = LLE_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, LLE_WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = LLE_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, LLE_WAVE));
    return v;
}

// Sum over a workgroup of up to 1024 threads; `smem` holds >= 16 floats.
// Every thread gets the result; the order of the additions is fixed.
__device__ __forceinline__ float block_sum(float v, float* smem) {
    const int lane = threadIdx.x % LLE_WAVE, wave = threadIdx.x / LLE_WAVE;
    const int nwaves = (blockDim.x + LLE_WAVE - 1) / LLE_WAVE;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int w = 0; w < nwaves; ++w) total += smem[w];
    return total;
}

__device__ __forceinline__ float block_max(float v, float* smem) {
    const int lane = threadIdx.x % LLE_WAVE, wave = threadIdx.x / LLE_WAVE;
    const int nwaves = (blockDim.x + LLE_WAVE - 1) / LLE_WAVE;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    float total = smem[0];
    for (int w = 1; w < nwaves; ++w) total = fmaxf(total, smem[w]);
    return total;
}

// launch check shared by the extern "C" entry points: 0 or the hipError_t
#define LLE_RETURN_LAUNCH_STATUS() return (int)hipGetLastError()

extern "C" const char* lle_error_string(int code);
#define LLE_DEFINE_ERROR_STRING() \
    extern "C" const char* lle_error_string(int code) { return hipGetErrorString((hipError_t)code); }
