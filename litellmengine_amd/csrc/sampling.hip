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
// With `scatter_dst` the pick of row r also goes to scatter_dst[scatter_index[r]] (the token that
// a request's slot decodes next, kept on the device for a step that is launched before the host
// has read this one's picks).
__global__ __launch_bounds__(LLE_WAVE) void argmax_final_kernel(const float* __restrict__ part_val,
                                                                const int32_t* __restrict__ part_idx,
                                                                int32_t* __restrict__ out, int chunks,
                                                                int32_t* __restrict__ scatter_dst = nullptr,
                                                                const int32_t* __restrict__ scatter_index = nullptr) {
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
    if (threadIdx.x == 0) {
        const int pick = best_i == 0x7fffffff ? 0 : best_i;
        out[blockIdx.x] = pick;
        if (scatter_dst) scatter_dst[scatter_index[blockIdx.x]] = pick;
    }
}

// `part_val`, `part_idx`: workspaces of R * chunks elements; `scatter_dst` (int32) and
// `scatter_index` (int32 [R], in range of scatter_dst) both or neither: see argmax_final_kernel
extern "C" int lle_argmax_rows_scatter(const void* logits, void* out, void* part_val, void* part_idx, int R, int V,
                                       int chunks, void* scatter_dst, const void* scatter_index, hipStream_t stream) {
    if (R <= 0) return 0;
    if (chunks <= 0 || chunks > 65535 || (scatter_dst == nullptr) != (scatter_index == nullptr))
        return (int)hipErrorInvalidValue;
    argmax_chunks_kernel<<<dim3(R, chunks), ARGMAX_THREADS, 0, stream>>>((const float*)logits, (float*)part_val,
                                                                          (int32_t*)part_idx, V);
    argmax_final_kernel<<<R, LLE_WAVE, 0, stream>>>((const float*)part_val, (const int32_t*)part_idx, (int32_t*)out,
                                                     chunks, (int32_t*)scatter_dst, (const int32_t*)scatter_index);
    LLE_RETURN_LAUNCH_STATUS();
}

extern "C" int lle_argmax_rows(const void* logits, void* out, void* part_val, void* part_idx, int R, int V,
                               int chunks, hipStream_t stream) {
    return lle_argmax_rows_scatter(logits, out, part_val, part_idx, R, V, chunks, nullptr, nullptr, stream);
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

// p_i = exp((x_i - max) / T); the pick is the first i whose running sum of p exceeds
// u * sum(p); if rounding leaves none, the last i with p_i > 0.  Rows with T <= 0 are picked
// greedily (first maximum).  One workgroup per row, every read of the row coalesced:
//   1. the first maximum (threads stride over the row);
//   2. the row is cut into segments of whole 1024-element lines (one line a segment up to
//      2 M ids); a wavefront sums a line with 16 loads of 64 neighbouring ids;
//   3. one wavefront scans the segment sums in id order and finds the segment that the
//      target falls into;
//   4. the workgroup scans that segment id by id (wavefront scans, joined in order).
// The running sum is taken in id order at every level, so the pick differs from an exact
// cumulative sum only where the target lies within rounding of a boundary.
#define SAMPLE_WAVES (SAMPLE_THREADS / LLE_WAVE)
#define SAMPLE_LINE 1024
#define SAMPLE_MAX_SEGMENTS 2048
#define SAMPLE_NONE 0x7fffffff

__device__ __forceinline__ float wave_inclusive_scan(float v, int lane) {
#pragma unroll
    for (int o = 1; o < LLE_WAVE; o <<= 1) {
        const float n = __shfl_up(v, o, LLE_WAVE);
        if (lane >= o) v += n;
    }
    return v;
}

// The weight of one id.  A logit that is no number (or an infinite one beside an infinite
// maximum) has none: it is never picked and moves no other id's share of the running sum.
__device__ __forceinline__ float sample_weight(float logit, float big, float inv_t) {
    const float e = expf((logit - big) * inv_t);
    return e == e ? e : 0.f;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_rows_kernel(const float* __restrict__ logits,
                                                                     const float* __restrict__ temperature,
                                                                     const float* __restrict__ uniform,
                                                                     int32_t* __restrict__ out, int V) {
    __shared__ float s_val[SAMPLE_WAVES];
    __shared__ int s_idx[SAMPLE_WAVES];
    __shared__ float s_seg[SAMPLE_MAX_SEGMENTS];
    __shared__ float s_wave[SAMPLE_WAVES];
    __shared__ float s_big, s_before, s_target;
    __shared__ int s_big_i, s_seg_pick, s_pick, s_last;
    const float* row = logits + (int64_t)blockIdx.x * V;
    const float T = temperature[blockIdx.x];
    const int t = threadIdx.x, lane = t % LLE_WAVE, wave = t / LLE_WAVE;

    float mx = -INFINITY;
    int mx_i = SAMPLE_NONE;
    for (int i = t; i < V; i += SAMPLE_THREADS) {  // ascending: the first maximum of this thread
        const float v = row[i];
        if (v > mx) {
            mx = v;
            mx_i = i;
        }
    }
    block_argmax(mx, mx_i, s_val, s_idx);
    if (t == 0) {
        s_big = mx;
        s_big_i = mx_i == SAMPLE_NONE ? 0 : mx_i;
        s_pick = SAMPLE_NONE;
        s_last = -1;
    }
    __syncthreads();
    const float big = s_big;
    if (T <= 0.f) {
        if (t == 0) out[blockIdx.x] = s_big_i;
        return;
    }
    const float inv_t = 1.0f / T;
    const int nlines = (V + SAMPLE_LINE - 1) / SAMPLE_LINE;
    const int per_seg = (nlines + SAMPLE_MAX_SEGMENTS - 1) / SAMPLE_MAX_SEGMENTS;  // lines a segment
    const int nseg = (nlines + per_seg - 1) / per_seg;
    for (int seg = wave; seg < nseg; seg += SAMPLE_WAVES) {
        float part = 0.f;
        for (int g = 0; g < per_seg; ++g) {
            const int64_t base = ((int64_t)seg * per_seg + g) * SAMPLE_LINE;
            if (base >= V) break;
            float v[SAMPLE_LINE / LLE_WAVE];
#pragma unroll
            for (int j = 0; j < SAMPLE_LINE / LLE_WAVE; ++j) {
                const int64_t i = base + lane + LLE_WAVE * j;
                v[j] = row[i < V ? i : V - 1];
            }
#pragma unroll
            for (int j = 0; j < SAMPLE_LINE / LLE_WAVE; ++j)
                part += base + lane + LLE_WAVE * j < V ? sample_weight(v[j], big, inv_t) : 0.f;
        }
        part = wave_sum(part);
        if (lane == 0) s_seg[seg] = part;
    }
    __syncthreads();
    if (wave == 0) {
        // lane l owns the segments [l * each, (l + 1) * each)
        const int each = (nseg + LLE_WAVE - 1) / LLE_WAVE;
        float own = 0.f;
        for (int k = 0; k < each; ++k) {
            const int seg = lane * each + k;
            own += seg < nseg ? s_seg[seg] : 0.f;
        }
        const float inclusive = wave_inclusive_scan(own, lane);
        const float total = __shfl(inclusive, LLE_WAVE - 1, LLE_WAVE);
        float before = __shfl_up(inclusive, 1, LLE_WAVE);
        if (lane == 0) before = 0.f;
        // a uniform number of exactly 1 (a double just below 1 rounds to it) would pick nothing
        const float target = fminf(uniform[blockIdx.x], 0x1.fffffep-1f) * total;
        int found = SAMPLE_NONE, last = -1;
        float found_before = 0.f, last_before = 0.f, run = before;
        for (int k = 0; k < each; ++k) {
            const int seg = lane * each + k;
            const float sum = seg < nseg ? s_seg[seg] : 0.f;
            if (sum > 0.f) {
                if (found == SAMPLE_NONE && run + sum > target) {
                    found = seg;
                    found_before = run;
                }
                last = seg;
                last_before = run;
            }
            run += sum;
        }
        // the first lane that found one holds the first such segment; without any, the last
        // segment that has weight at all
        const unsigned long long have = __builtin_amdgcn_ballot_w64(found != SAMPLE_NONE);
        const unsigned long long any = __builtin_amdgcn_ballot_w64(last >= 0);
        int src = 0;
        if (have)
            src = __builtin_ctzll(have);
        else if (any)
            src = 63 - __builtin_clzll(any);
        const int seg_pick = __shfl(have ? found : last, src, LLE_WAVE);
        const float seg_before = __shfl(have ? found_before : last_before, src, LLE_WAVE);
        if (lane == 0) {
            s_seg_pick = (have || any) ? seg_pick : -1;
            s_before = seg_before;
            s_target = target;
        }
    }
    __syncthreads();
    const int seg = s_seg_pick;
    if (seg < 0) {  // no id has weight (a row of NaN, or an infinite maximum): the greedy pick
        if (t == 0) out[blockIdx.x] = s_big_i;
        return;
    }
    const float target = s_target;
    float carry = s_before;
    for (int g = 0; g < per_seg; ++g) {
        const int64_t base = ((int64_t)seg * per_seg + g) * SAMPLE_LINE;
        if (base >= V) break;
        const int64_t i = base + t;
        const float p = i < V ? sample_weight(row[i], big, inv_t) : 0.f;
        const float inclusive = wave_inclusive_scan(p, lane);
        if (lane == LLE_WAVE - 1) s_wave[wave] = inclusive;
        __syncthreads();
        float ahead = 0.f, all = 0.f;
#pragma unroll
        for (int w = 0; w < SAMPLE_WAVES; ++w) {
            if (w < wave) ahead += s_wave[w];
            all += s_wave[w];
        }
        if (p > 0.f) {
            if (carry + ahead + inclusive > target) atomicMin(&s_pick, (int)i);
            atomicMax(&s_last, (int)i);
        }
        carry += all;
        __syncthreads();
    }
    if (t == 0) out[blockIdx.x] = s_pick != SAMPLE_NONE ? s_pick : (s_last >= 0 ? s_last : s_big_i);
}

extern "C" int lle_sample_rows(const void* logits, const void* temperature, const void* uniform, void* out, int R,
                               int V, hipStream_t stream) {
    if (R <= 0) return 0;
    sample_rows_kernel<<<R, SAMPLE_THREADS, 0, stream>>>((const float*)logits, (const float*)temperature,
                                                          (const float*)uniform, (int32_t*)out, V);
    LLE_RETURN_LAUNCH_STATUS();
}
