// Measured peaks of the machine the engine runs on, for the benchmark's rooflines: how fast
// a kernel that does nothing but read streams a buffer from HBM, and how fast the matrix
// cores multiply operands that never leave the registers.  (The reference measures no such
// thing; its benchmark reports tokens per second only, src/benchmark/generation_benchmark.cpp:531-578.)
#include "common.h"

LLE_DEFINE_ERROR_STRING()

typedef bf16_t pbf16x8 __attribute__((ext_vector_type(8)));
typedef float pf32x4 __attribute__((ext_vector_type(4)));

// Every thread reads 16-byte pieces `stride` apart, UNROLL of them on their way at a time, and
// folds them into one word; the word is stored only if it is a value that no real buffer
// gives, so the loads cannot be dropped and nothing is written.
#define READ_UNROLL 8
__global__ __launch_bounds__(1024) void read_stream_kernel(const uint4* __restrict__ data, int64_t pieces,
                                                           uint32_t* __restrict__ sink) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t fold = 0;
    for (; i + (READ_UNROLL - 1) * stride < pieces; i += READ_UNROLL * stride) {
        uint4 v[READ_UNROLL];
#pragma unroll
        for (int u = 0; u < READ_UNROLL; ++u) v[u] = data[i + u * stride];
#pragma unroll
        for (int u = 0; u < READ_UNROLL; ++u) fold ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < pieces; i += stride) {
        const uint4 v = data[i];
        fold ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    if (fold == 0x9e3779b9u && sink) sink[0] = fold;
}

// `data`: `bytes` (a multiple of 16) of device memory; `sink`: one word (written almost never)
extern "C" int lle_probe_read_stream(const void* data, int64_t bytes, int blocks, void* sink, hipStream_t stream) {
    if (bytes <= 0 || bytes % 16 != 0 || blocks <= 0) return (int)hipErrorInvalidValue;
    read_stream_kernel<<<blocks, 1024, 0, stream>>>((const uint4*)data, bytes / 16, (uint32_t*)sink);
    LLE_RETURN_LAUNCH_STATUS();
}

// Four independent chains of v_mfma_f32_16x16x32_bf16 per wavefront (an instruction can
// issue while the one before it is still in the pipeline), `iters` rounds of them.
// One instruction is 16 x 16 x 32 multiply-adds = 16384 flops.
__global__ __launch_bounds__(256) void mfma_bf16_kernel(int iters, float* __restrict__ sink) {
    pbf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = (bf16_t)(0.001f * (float)(threadIdx.x % 7 + i));
        b[i] = (bf16_t)(0.002f * (float)(threadIdx.x % 5 + i));
    }
    pf32x4 acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = pf32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[c], 0, 0, 0);
    }
    float total = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) total += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
    if (total == 12345.678f && sink) sink[0] = total;
}

// the same with v_mfma_f32_16x16x4_f32 (float32 operands): 16 x 16 x 4 multiply-adds = 2048 flops
__global__ __launch_bounds__(256) void mfma_f32_kernel(int iters, float* __restrict__ sink) {
    const float a = 0.001f * (float)(threadIdx.x % 7 + 1), b = 0.002f * (float)(threadIdx.x % 5 + 1);
    pf32x4 acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = pf32x4{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[c], 0, 0, 0);
    }
    float total = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) total += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
    if (total == 12345.678f && sink) sink[0] = total;
}

// blocks of 256 threads (4 wavefronts); every wavefront issues 16 * iters matrix instructions.
// dtype: LLE_BF16 or LLE_F32.
extern "C" int lle_probe_mfma(int dtype, int blocks, int iters, void* sink, hipStream_t stream) {
    if (blocks <= 0 || iters <= 0) return (int)hipErrorInvalidValue;
    if (dtype == LLE_BF16)
        mfma_bf16_kernel<<<blocks, 256, 0, stream>>>(iters, (float*)sink);
    else if (dtype == LLE_F32)
        mfma_f32_kernel<<<blocks, 256, 0, stream>>>(iters, (float*)sink);
    else
        return (int)hipErrorInvalidValue;
    LLE_RETURN_LAUNCH_STATUS();
}
