// Picking tokens from 32-bit logits rows: greedy (first maximum wins, as
// argmax_each_row_kernel, src/ops/argmax.cu:181-241) and temperature sampling
// (the reference parses --temperature and then only warns, src/main.cpp:175-178).
#include "common.h"
#include "sampling.h"
#include <mutex>

extern "C" const char* lle_error_string(int code) {
    if (code == LLE_ERROR_STATIC_SCRATCH_TOO_SMALL)
        return "lle_argmax_rows_static takes at most 256 rows (LLE_ARGMAX_STATIC_MAX_ROWS): its buffer has a fixed size";
    return hipGetErrorString((hipError_t)code);
}

#define SAMPLE_THREADS 1024

#define ARGMAX_THREADS 256

// (value, index) of the first maximum among the candidates of one workgroup; a NaN never
// wins a ">" comparison; ties go to the smaller index.  Valid in thread 0.
__device__ __forceinline__ void block_argmax(float& best, int& best_i, float* s_val, int* s_idx) {
    for (int o = LLE_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, LLE_WAVE);
        const int oi = __shfl_xor(best_i, o, LLE_WAVE);
        if (ov > best || (ov == best && oi < best_i)) {
            best = ov;
            best_i = oi;
        }
    }
    const int lane = threadIdx.x % LLE_WAVE, wave = threadIdx.x / LLE_WAVE;
    if (lane == 0) {
        s_val[wave] = best;
        s_idx[wave] = best_i;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int nwaves = (blockDim.x + LLE_WAVE - 1) / LLE_WAVE;
        for (int w = 1; w < nwaves; ++w)
            if (s_val[w] > best || (s_val[w] == best && s_idx[w] < best_i)) {
                best = s_val[w];
                best_i = s_idx[w];
            }
    }
}

// stage 1: grid (rows, chunks): the first maximum of one chunk of a row
__global__ __launch_bounds__(ARGMAX_THREADS) void argmax_chunks_kernel(const float* __restrict__ logits,
                                                                        float* __restrict__ part_val,
                                                                        int32_t* __restrict__ part_idx, int V) {
    __shared__ float s_val[ARGMAX_THREADS / LLE_WAVE];
    __shared__ int s_idx[ARGMAX_THREADS / LLE_WAVE];
    const float* row = logits + (int64_t)blockIdx.x * V;
    const int chunks = gridDim.y;
    const int per = (V + chunks - 1) / chunks;
    const int lo = min(V, (int)blockIdx.y * per), hi = min(V, lo + per);
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
        const float v = row[i];
        if (v > best || best_i == 0x7fffffff) {  // ascending: the first maximum of this thread
            best = v;
            best_i = i;
        }
    }
    block_argmax(best, best_i, s_val, s_idx);
    if (threadIdx.x == 0) {
        part_val[blockIdx.x * chunks + blockIdx.y] = best;
        part_idx[blockIdx.x * chunks + blockIdx.y] = best_i;
    }
}

// stage 2: grid rows, one wavefront: the first maximum among the chunks' winners
__global__ __launch_bounds__(LLE_WAVE) void argmax_final_kernel(const float* __restrict__ part_val,
                                                                const int32_t* __restrict__ part_idx,
                                                                int32_t* __restrict__ out, int chunks) {
    __shared__ float s_val[1];
    __shared__ int s_idx[1];
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int k = threadIdx.x; k < chunks; k += blockDim.x) {
        const float v = part_val[blockIdx.x * chunks + k];
        const int i = part_idx[blockIdx.x * chunks + k];
        if (i != 0x7fffffff && (v > best || best_i == 0x7fffffff || (v == best && i < best_i))) {
            best = v;
            best_i = i;
        }
    }
    block_argmax(best, best_i, s_val, s_idx);
    if (threadIdx.x == 0) out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;
}

// `part_val`, `part_idx`: workspaces of R * chunks elements
extern "C" int lle_argmax_rows(const void* logits, void* out, void* part_val, void* part_idx, int R, int V,
                               int chunks, hipStream_t stream) {
    if (R <= 0) return 0;
    if (chunks <= 0 || chunks > 65535) return (int)hipErrorInvalidValue;
    argmax_chunks_kernel<<<dim3(R, chunks), ARGMAX_THREADS, 0, stream>>>((const float*)logits, (float*)part_val,
                                                                          (int32_t*)part_idx, V);
    argmax_final_kernel<<<R, LLE_WAVE, 0, stream>>>((const float*)part_val, (const int32_t*)part_idx, (int32_t*)out,
                                                     chunks);
    LLE_RETURN_LAUNCH_STATUS();
}

// Chunks of a row: enough workgroups to stream a long row from all CUs.
static int argmax_chunks_for(int V) {
    const int c = V / 2048;
    return c < 1 ? 1 : (c > LLE_ARGMAX_STATIC_MAX_CHUNKS ? LLE_ARGMAX_STATIC_MAX_CHUNKS : c);
}

// The chunk winners of lle_argmax_rows_static: values (float) of up to MAX_ROWS * MAX_CHUNKS
// chunks, then their indices (int32).  In host code this name is only a handle for
// hipGetSymbolAddress; the address that kernels get is looked up once per device.
static __device__ __align__(256) unsigned char scratch[LLE_ARGMAX_STATIC_BYTES];

static int static_scratch_address(void** ptr) {
    static std::mutex lock;
    static void* address[64] = {nullptr};  // per device: every GPU holds its own copy of the array
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= 64) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> guard(lock);
    if (address[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return (int)hipErrorInvalidSymbol;
        address[dev] = p;
    }
    *ptr = address[dev];
    return 0;
}

// see sampling.h
extern "C" int lle_argmax_rows_static(const void* logits, void* out, int R, int V, hipStream_t stream) {
    if (R <= 0) return 0;
    if (V <= 0 || logits == nullptr || out == nullptr) return (int)hipErrorInvalidValue;
    if (R > LLE_ARGMAX_STATIC_MAX_ROWS) return LLE_ERROR_STATIC_SCRATCH_TOO_SMALL;
    void* base = nullptr;
    const int err = static_scratch_address(&base);
    if (err != 0) return err;
    const int chunks = argmax_chunks_for(V);
    float* part_val = (float*)base;
    int32_t* part_idx = (int32_t*)((unsigned char*)base + LLE_ARGMAX_STATIC_BYTES / 2);
    argmax_chunks_kernel<<<dim3(R, chunks), ARGMAX_THREADS, 0, stream>>>((const float*)logits, part_val, part_idx, V);
    argmax_final_kernel<<<R, LLE_WAVE, 0, stream>>>(part_val, part_idx, (int32_t*)out, chunks);
    LLE_RETURN_LAUNCH_STATUS();
}

// p_i = exp((x_i - max) / T); the pick is the first i whose running sum of p
// exceeds u * sum(p).  Thread t owns the contiguous ids [t c, (t + 1) c), so the
// running sum is taken in id order.  Rows with T <= 0 are picked greedily.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(const float* __restrict__ logits,
                                                                     const float* __restrict__ temperature,
                                                                     const float* __restrict__ uniform,
                                                                     int32_t* __restrict__ out, int V) {
    __shared__ float red[16];
    __shared__ float s_part[SAMPLE_THREADS];
    __shared__ int s_pick;
    const float* row = logits + (int64_t)blockIdx.x * V;
    const float T = temperature[blockIdx.x];
    const int t = threadIdx.x;
    const int chunk = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int lo = min(V, t * chunk), hi = min(V, lo + chunk);

    float mx = -INFINITY;
    int mx_i = V;
    for (int i = lo; i < hi; ++i)
        if (row[i] > mx) {
            mx = row[i];
            mx_i = i;
        }
    const float big = block_max(mx, red);
    if (T <= 0.f) {  // greedy: smallest index that reaches the maximum
        if (t == 0) s_pick = V;
        __syncthreads();
        if (mx == big && mx_i < V) atomicMin(&s_pick, mx_i);
        __syncthreads();
        if (t == 0) out[blockIdx.x] = s_pick < V ? s_pick : 0;
        return;
    }
    const float inv_t = 1.0f / T;
    float part = 0.f;
    for (int i = lo; i < hi; ++i) part += expf((row[i] - big) * inv_t);
    s_part[t] = part;
    __syncthreads();
    if (t == 0) {
        // sequential scan over 1024 partial sums: fixed order, once per row
        float run = 0.f;
        for (int k = 0; k < SAMPLE_THREADS; ++k) {
            const float p = s_part[k];
            s_part[k] = run;  // exclusive prefix
            run += p;
        }
        red[0] = run;
        s_pick = V;
    }
    __syncthreads();
    const float total = red[0];
    const float target = uniform[blockIdx.x] * total;
    const float before = s_part[t];
    if (lo < hi && target >= before && target < before + part) {
        float run = before;
        int pick = hi - 1;
        for (int i = lo; i < hi; ++i) {
            run += expf((row[i] - big) * inv_t);
            if (run > target) {
                pick = i;
                break;
            }
        }
        atomicMin(&s_pick, pick);
    }
    __syncthreads();
    if (t == 0) out[blockIdx.x] = s_pick < V ? s_pick : V - 1;
}

extern "C" int lle_sample_rows(const void* logits, const void* temperature, const void* uniform, void* out, int R,
                               int V, hipStream_t stream) {
    if (R <= 0) return 0;
    sample_rows_kernel<<<R, SAMPLE_THREADS, 0, stream>>>((const float*)logits, (const float*)temperature,
                                                          (const float*)uniform, (int32_t*)out, V);
    LLE_RETURN_LAUNCH_STATUS();
}
