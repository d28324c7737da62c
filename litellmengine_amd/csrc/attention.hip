// Paged grouped-query attention over the cache, for any mix of prompt portions
// and single decoded tokens in one step.
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
// A cache page holds K as [nkv][page_size][d], then V as [nkv][d][page_size].
//
// Kernels:
//  * paged_attention_generic_kernel: any type, head size <= 256, page size,
//    window; one workgroup per (token, q head).  The 32-bit path and odd sizes.
//  * mfma_decode_kernel (+ mfma_combine_kernel): bfloat16, head size a multiple of
//    32, page size a multiple of 16.  One workgroup per (request, kv head, key
//    split); the q heads of the group (and up to 16 / group tokens) are the 16
//    columns of v_mfma_f32_16x16x32_bf16 tiles, so every K/V byte is read once
//    per group; the four wavefronts take every fourth 32-key step, their loads
//    two steps ahead; partial (m, l, acc) of the splits are merged by the combine
//    kernel.  In decode steps it can also do what comes before it: the q/k norm,
//    the rotation and the write of the new K and V (FusedQKV).
//  * mfma_prefill_kernel: same tile code, 32 rows (token, head) per wavefront,
//    all keys up to each row's own position; the four wavefronts of a workgroup
//    share the K/V tiles through LDS, two workgroups share a CU.
#include "common.h"
#include <type_traits>
#include <mutex>

LLE_DEFINE_ERROR_STRING()

#define ATT_WAVES 4
#define ATT_MAX_R 4  // head_dim <= 256
#define ATT_KEYS 4   // keys a wavefront works on at a time

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
    const int64_t v_base = ((int64_t)nkv + kvh) * page_size * d;
    // A wavefront takes ATT_KEYS consecutive keys at a time, so that the loads of several keys
    // are on their way together (one key after the other, each would wait for its own K row and
    // then for its own V row).  Which keys share a step depends on (lo, pos) only.
    // (keys j0 .. j0 + ATT_KEYS - 1 lie in one page, side by side, when the steps start at a
    // multiple of ATT_KEYS and pages hold a multiple of it; the last step of a row may reach
    // past `pos`, but not past its page)
    const bool keys_in_one_piece = lo % ATT_KEYS == 0 && page_size % ATT_KEYS == 0;
    for (int j0 = lo + wave * ATT_KEYS; j0 <= pos; j0 += ATT_WAVES * ATT_KEYS) {
        const T* vp[ATT_KEYS];
        float dot[ATT_KEYS];
#pragma unroll
        for (int i = 0; i < ATT_KEYS; ++i) {
            const int j = min(j0 + i, pos);  // past the row's last key: that key again, weighted 0 below
            const int lp = j / page_size;
            const int off = j - lp * page_size;
            // the same for the whole wavefront: a scalar load
            const T* page = kv_layer + (int64_t)table[__builtin_amdgcn_readfirstlane(lp)] * page_stride;
            const T* kp = page + ((int64_t)kvh * page_size + off) * d;
            vp[i] = page + v_base + off;  // element e of the value row at vp[e * page_size]
            dot[i] = 0.f;
#pragma unroll
            for (int r = 0; r < ATT_MAX_R; ++r) {
                const int e = lane + LLE_WAVE * r;
                if (e < d) dot[i] += qv[r] * to_f32<T>(kp[e]);
            }
        }
        float vals[ATT_KEYS][ATT_MAX_R];
        if (keys_in_one_piece) {
            // the ATT_KEYS values of an element lie side by side in the page: one load for all of them
            typedef T piece_t __attribute__((ext_vector_type(ATT_KEYS)));
#pragma unroll
            for (int r = 0; r < ATT_MAX_R; ++r) {
                const int e = lane + LLE_WAVE * r;
                if (e < d) {
                    const piece_t piece = *(const piece_t*)(vp[0] + (int64_t)e * page_size);
#pragma unroll
                    for (int i = 0; i < ATT_KEYS; ++i)  // what lies past `pos` was never written: not even times 0
                        vals[i][r] = j0 + i <= pos ? to_f32<T>(piece[i]) : 0.f;
                } else {
#pragma unroll
                    for (int i = 0; i < ATT_KEYS; ++i) vals[i][r] = 0.f;
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < ATT_KEYS; ++i)
#pragma unroll
                for (int r = 0; r < ATT_MAX_R; ++r) {
                    const int e = lane + LLE_WAVE * r;
                    vals[i][r] = e < d ? to_f32<T>(vp[i][(int64_t)e * page_size]) : 0.f;
                }
        }
        float score[ATT_KEYS];
        float new_m = m;
#pragma unroll
        for (int i = 0; i < ATT_KEYS; ++i) {
            score[i] = wave_sum(dot[i]) * scale;
            if (j0 + i <= pos) new_m = fmaxf(new_m, score[i]);
        }
        const float alpha = expf(m - new_m);
        float beta[ATT_KEYS];
        l *= alpha;
#pragma unroll
        for (int i = 0; i < ATT_KEYS; ++i) {
            beta[i] = j0 + i <= pos ? expf(score[i] - new_m) : 0.f;
            l += beta[i];
        }
#pragma unroll
        for (int r = 0; r < ATT_MAX_R; ++r) {
            float a = acc[r] * alpha;
#pragma unroll
            for (int i = 0; i < ATT_KEYS; ++i) a += beta[i] * vals[i][r];
            acc[r] = a;
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

// ---------------------------------------------------------------------------------
// matrix-core kernels (bfloat16)
// ---------------------------------------------------------------------------------
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define NEG_BIG (-1.0e30f)
#define LAZY_MAX 8.0f  // a row's reference maximum may lag its true one by this much (base 2)
#define KSTEP 32  // keys per step: two 16-key tiles; pages hold a multiple of 16 keys
#define KEY_OF_ROW(r, x) (8 * ((r) / 4) + 4 * (x) + (r) % 4)
// LDS tiles of the prompt kernel.  LDS has 64 banks of 4 bytes; a 16-byte read of a wavefront
// is served sixteen lanes a cycle, and the sixteen are not consecutive (measured: a cycle takes
// lanes 0-3, 12-15, 20-23, 24-27, the next 4-11, 16-19, 28-31, then the same of the upper 32).
// With lane = (c, r) = (lane / 16, lane % 16) a cycle holds c0 with r / 4 in {0, 3} and c0 + 1
// with r / 4 in {1, 2}, or the other way round, r % 4 taking all its values.  The tiles have no
// padding; a lane reads 16-byte piece (logical piece) ^ swizzle of its row instead, and the
// swizzle is such that a cycle's sixteen lanes hit the sixteen 16-byte columns of the banks:
//   Q4(q) for q = r / 4: 0, 2, 3, 1, so that c ^ Q4 differs between the four (c, r / 4) of a cycle;
//   V^T rows are 64 bytes (32 keys): element e uses Q4((e / 4) % 4); e % 4 picks the columns 4 (e % 4) ..
//   K rows are 64 DK bytes, key j = 8 (r / 4) + 4 x + r % 4 of the step: the low bits of j
//   choose among what the row's own offset leaves the same: none for odd DK (rows 64 bytes
//   apart mod 256), bit 1 for DK = 2, 6 (128 bytes), bits 1 and 0 for DK = 4, 8 (0 bytes).
#define Q4(q) ((((q) >> 1) & 1) | ((((q) ^ ((q) >> 1)) & 1) << 1))
#define K_SWIZZLE(j, DK) ((Q4(((j) >> 3) & 3) | ((((j) >> 1) & 1) << 2) | (((j) & 1) << 3)) & ((DK) % 4 == 0 ? 15 : (DK) % 2 == 0 ? 7 : 3))
#define V_SWIZZLE(e) Q4(((e) >> 2) & 3)

// What one lane knows about the query row it serves (row = lane % 16 of a 16-row tile).
struct RowInfo {
    const bf16_t* q;  // start of the row's head in q, or nullptr for a row that does not exist
    int pos;          // last key the row sees
    int lo;           // first key the row sees
};

// One wavefront runs `RT` tiles of 16 query rows over the 32-key steps
// step_begin, step_begin + step_stride, ... < step_end.  Products:
//   S^T = K Q^T   (A = K tile [16 keys x 32], B = Q^T [32 x 16 rows])
//   O^T += V^T P^T (A = V^T tile [16 d x 32 keys], B = P^T [32 keys x 16 rows])
// With v_mfma_f32_16x16x32_bf16 a lane (c = lane / 16, r = lane % 16) holds, of a
// result tile, column r and rows 4c..4c+3: for S^T that is query row r and four keys
// — exactly what the B operand of the second product wants, so P never leaves
// registers, and the softmax state of row r sits in the lanes r + 16c.
// Which key a row of a K tile stands for is free.  The two tiles of a step take the keys
//   row r of tile x  <->  key 8 (r / 4) + 4 x + r % 4   of the step        (KEY_OF_ROW)
// so that a lane's eight scores (rows 4c..4c+3 of both tiles) are the CONSECUTIVE keys
// 8c..8c+7: the V^T operand of the second product is then one 16-byte piece per lane
// (keys 8c..8c+7 of one value element), inside one page.
template <int DK, int RT>
struct RowState {
    bf16x8 qv[RT][DK];             // Q^T operands of the lane's row
    int open_lo[RT], open_hi[RT];  // steps with open_lo <= j0 and j0 + 31 <= open_hi need no mask
    f32x4 o[RT][2 * DK];           // O^T tiles: value elements 16 n + 4 c .. + 3 of row r16
    float m[RT], l[RT];            // running maximum (base 2) and this lane's share of the sum
};

// LOAD_Q = false: the caller has filled st.qv itself
template <int DK, int RT, bool LOAD_Q = true>
__device__ __forceinline__ void init_rows(RowState<DK, RT>& st, const RowInfo (&row)[RT]) {
    const int c = (threadIdx.x % LLE_WAVE) / 16;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        if (LOAD_Q) {
#pragma unroll
            for (int ks = 0; ks < DK; ++ks) {
                if (row[t].q) {
                    st.qv[t][ks] = *(const bf16x8*)(row[t].q + 32 * ks + 8 * c);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) st.qv[t][ks][i] = (bf16_t)0.0f;
                }
            }
        }
#pragma unroll
        for (int n = 0; n < 2 * DK; ++n) st.o[t][n] = f32x4{0.f, 0.f, 0.f, 0.f};
        st.m[t] = NEG_BIG;
        st.l[t] = 0.f;
        int lo_max = row[t].q ? row[t].lo : 0, pos_min = row[t].q ? row[t].pos : 0x7fffffff;
#pragma unroll
        for (int off = 1; off < LLE_WAVE; off <<= 1) {
            lo_max = max(lo_max, __shfl_xor(lo_max, off, LLE_WAVE));
            pos_min = min(pos_min, __shfl_xor(pos_min, off, LLE_WAVE));
        }
        // (the same in every lane: kept in scalar registers, so that the test is a scalar branch)
        st.open_lo[t] = __builtin_amdgcn_readfirstlane(lo_max);
        st.open_hi[t] = __builtin_amdgcn_readfirstlane(pos_min == 0x7fffffff ? -1 : pos_min);
    }
    // The rows of Q are waited for here, once.  Left pending, their first use lies inside the
    // key loop, where the wait for them also waits for the K/V loads just issued for a later
    // step: the loop would run at the latency of memory.
    if (LOAD_Q) {
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int ks = 0; ks < DK; ++ks) asm volatile("" : "+v"(st.qv[t][ks]));
    }
}

// The largest of eight scores, none of which is a NaN (masked scores are NEG_BIG, not infinite).
// Written with the instruction itself: from fmaxf the compiler first passes every operand that a
// select may have produced through an instruction of its own (x = max(x, x), which quiets a
// signalling NaN), 8 + 7 instructions for what takes 4.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float max_of_8(const float (&x)[8]) {
    const float a = max3(x[0], x[1], x[2]), b = max3(x[3], x[4], x[5]);
    return max3(max3(x[6], x[7], a), b, b);
}

// One 32-key step for RT tiles of 16 rows.  load_k(x, ks): for lane (c, r16) key
// KEY_OF_ROW(r16, x) of the step, elements 32 ks + 8 c .. + 7.  load_v(n): value element
// 16 n + r16, keys 8c..8c+7 of the step.  Each operand is fetched once and used by all row tiles.
template <int DK, int RT, typename LoadK, typename LoadV>
__device__ __forceinline__ void tile_step(RowState<DK, RT>& st, const RowInfo (&row)[RT], LoadK load_k,
                                          LoadV load_v, int j0, float scale_log2) {
    const int c = (threadIdx.x % LLE_WAVE) / 16;
    f32x4 s[RT][2];
#pragma unroll
    for (int t = 0; t < RT; ++t) s[t][0] = s[t][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
        for (int ks = 0; ks < DK; ++ks) {
            const bf16x8 k = load_k(x, ks);
#pragma unroll
            for (int t = 0; t < RT; ++t)
                s[t][x] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k, st.qv[t][ks], s[t][x], 0, 0, 0);
        }
    // the value operands are asked for before the softmax, whose arithmetic covers their way
    // from LDS; asked for one by one between the products, each would be waited for in turn
    bf16x8 vv[2 * DK];
#pragma unroll
    for (int n = 0; n < 2 * DK; ++n) vv[n] = load_v(n);
    __builtin_amdgcn_sched_barrier(0);
    // Scores relative to the row's reference m, in the base-2 domain: x = s * scale - m.  The
    // reference only has to be near the row's maximum, not equal to it: while no x exceeds
    // LAZY_MAX the weights are exp2(x) <= 2^LAZY_MAX and nothing else is touched.  Only when
    // some row of the wavefront goes beyond (the first keys of a row always do: m starts at
    // NEG_BIG) the maxima are agreed on between the four lanes of each row and m, l and the
    // accumulators are moved; that is rare after a row's first steps.
    float x[RT][8];
    bool raise = false;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[t][i] = fmaf(s[t][i / 4][i % 4], scale_log2, -st.m[t]);
        if (!(j0 >= st.open_lo[t] && j0 + KSTEP - 1 <= st.open_hi[t])) {  // same for the whole wavefront
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int j = j0 + 8 * c + i;  // score i of the lane: tile i / 4, row 4 c + i % 4
                if (j < row[t].lo || j > row[t].pos) x[t][i] = NEG_BIG;
            }
        }
        raise = raise || max_of_8(x[t]) > LAZY_MAX;
    }
    if (__builtin_amdgcn_ballot_w64(raise) != 0) {
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            // absolute scores again (x has lost them where m was still NEG_BIG)
            float sc[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) sc[i] = x[t][i] <= NEG_BIG ? NEG_BIG : s[t][i / 4][i % 4] * scale_log2;
            float tile_max = max_of_8(sc);
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, LLE_WAVE));
            tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, LLE_WAVE));
            const float new_m = fmaxf(st.m[t], tile_max);
            // while the row has seen no key new_m is NEG_BIG as its masked scores are, and
            // exp2(0) = 1 would count them: shift such rows so that they give 0
            const float base = new_m <= NEG_BIG ? 0.f : new_m;
            const float alpha = __builtin_amdgcn_exp2f(st.m[t] - base);
            st.m[t] = new_m;
            st.l[t] *= alpha;
#pragma unroll
            for (int n = 0; n < 2 * DK; ++n) st.o[t][n] *= alpha;
#pragma unroll
            for (int i = 0; i < 8; ++i) x[t][i] = sc[i] - base;
        }
    }
    bf16x8 pb[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        // two chains of additions instead of one: a dependent addition waits for the one before it
        float psum[2] = {0.f, 0.f};
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float p = __builtin_amdgcn_exp2f(x[t][i]);
            psum[i % 2] += p;
            pb[t][i] = (bf16_t)p;
        }
        st.l[t] += psum[0] + psum[1];
    }
#pragma unroll
    for (int n = 0; n < 2 * DK; ++n) {
#pragma unroll
        for (int t = 0; t < RT; ++t)
            st.o[t][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv[n], pb[t], st.o[t][n], 0, 0, 0);
    }
}

// the partial sums of a row sit in the four lanes r16 + 16 c
template <int DK, int RT>
__device__ __forceinline__ void finish_rows(RowState<DK, RT>& st) {
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        st.l[t] += __shfl_xor(st.l[t], 16, LLE_WAVE);
        st.l[t] += __shfl_xor(st.l[t], 32, LLE_WAVE);
    }
}

// The operands of one 32-key step as a wavefront loads them straight from the pages.
template <int DK>
struct StepOperands {
    bf16x8 k[2][DK];
    bf16x8 v[2 * DK];
};

// The steps step_begin, step_begin + step_stride, ... < step_end with the operands loaded by
// each wavefront straight from the pages, two steps ahead of their use: while one step is
// multiplied the loads of the next two are on their way.  Nothing in the loop stands under a
// condition (a load under a condition makes the compiler wait for every load where the paths
// meet again): the loop runs an even number of steps, loads past the end go to a page that is
// there, and the CALLER has limited the rows' `pos` to the last key of step_end - 1, so that a
// step past the end is masked out whole.
// `before_keys()` runs when the first table lookup is on its way and no operand is asked for yet:
// what the caller loads there travels beside the lookup, what it stores there is stored before
// this wavefront reads any key.  `after_first_loads()` runs once the first two steps are asked for.
template <int DK, int RT, bool LOAD_Q = true, typename BeforeKeys, typename AfterFirstLoads>
__device__ __forceinline__ void attend_rows(RowState<DK, RT>& st, const RowInfo (&row)[RT],
                                            const bf16_t* kv_layer, const int32_t* __restrict__ table,
                                            int kvh, int nkv, int P, int64_t page_stride, int step_begin,
                                            int step_end, int step_stride, int lo_min, int hi, float scale_log2,
                                            BeforeKeys before_keys, AfterFirstLoads after_first_loads) {
    constexpr int D = DK * 32;
    const int lane = threadIdx.x % LLE_WAVE;
    const int c = lane / 16, r16 = lane % 16;
    init_rows<DK, RT, LOAD_Q>(st, row);
    // the lane's keys of tile x lie in the 16-key half r16 / 8 of the step, its eight V keys in half c / 2
    const int k_half = r16 / 8, v_half = c / 2;
    const int64_t k_lane[2] = {(int64_t)kvh * P * D + (int64_t)(KEY_OF_ROW(r16, 0) % 16) * D + 8 * c,
                               (int64_t)kvh * P * D + (int64_t)(KEY_OF_ROW(r16, 1) % 16) * D + 8 * c};
    const int64_t v_lane = ((int64_t)nkv + kvh) * P * D + (int64_t)r16 * P + 8 * (c % 2);
    // Page and offset of a step's first key are carried from step to step instead of divided
    // out each time (the page size is no constant), and the table is read one load ahead.  A
    // half wholly outside [lo_min, hi] may lie in a page that is not there: the page index is
    // clamped to those of keys that are.
    const int page_lo = lo_min / P, page_hi = hi / P;
    const int adv_pages = (step_stride * KSTEP) / P, adv_off = (step_stride * KSTEP) % P;
    int look_page = (step_begin * KSTEP) / P, look_off = (step_begin * KSTEP) % P;
    int page_id[2], page_off[2];
    auto lookup = [&]() {
        const bool next_page = look_off + 16 == P;  // pages hold a multiple of 16 keys
        const int pg[2] = {look_page, next_page ? look_page + 1 : look_page};
        page_off[0] = look_off;
        page_off[1] = next_page ? 0 : look_off + 16;
#pragma unroll
        for (int x = 0; x < 2; ++x)  // the same for the whole wavefront: a scalar load, which no vector load waits for
            page_id[x] = table[__builtin_amdgcn_readfirstlane(min(max(pg[x], page_lo), page_hi))];
        look_page += adv_pages;
        look_off += adv_off;
        if (look_off >= P) {
            look_off -= P;
            ++look_page;
        }
    };
    auto load = [&](StepOperands<DK>& op) {
        const bf16_t* half0 = kv_layer + (int64_t)page_id[0] * page_stride;
        const bf16_t* half1 = kv_layer + (int64_t)page_id[1] * page_stride;
        const bf16_t* kpage = (k_half ? half1 : half0) + (int64_t)(k_half ? page_off[1] : page_off[0]) * D;
        const bf16_t* vp = (v_half ? half1 : half0) + v_lane + (v_half ? page_off[1] : page_off[0]);
#pragma unroll
        for (int x = 0; x < 2; ++x)
#pragma unroll
            for (int ks = 0; ks < DK; ++ks) op.k[x][ks] = *(const bf16x8*)(kpage + k_lane[x] + 32 * ks);
#pragma unroll
        for (int n = 0; n < 2 * DK; ++n) op.v[n] = *(const bf16x8*)(vp + (int64_t)16 * n * P);
        lookup();
    };
    auto multiply = [&](const StepOperands<DK>& op, int step) {
        tile_step<DK, RT>(
            st, row, [&](int x, int ks) { return op.k[x][ks]; }, [&](int n) { return op.v[n]; }, step * KSTEP,
            scale_log2);
    };
    StepOperands<DK> even, odd;
    lookup();
    before_keys();
    load(even);
    load(odd);
    after_first_loads();
    for (int step = step_begin; step < step_end; step += 2 * step_stride) {
        multiply(even, step);
        load(even);
        multiply(odd, step + step_stride);
        load(odd);
    }
    finish_rows<DK, RT>(st);
}

// row `r` of the (token, head-in-group) rows of one request and kv head
__device__ __forceinline__ RowInfo make_row(const bf16_t* q, int r, int nrows, int G, int q_start, int past, int nq,
                                            int kvh, int D, int window) {
    RowInfo info;
    if (r < nrows) {
        const int t = r / G, g = r - t * G;
        info.q = q + ((int64_t)(q_start + t) * nq + kvh * G + g) * D;
        info.pos = past + t;
        info.lo = window > 0 ? max(0, info.pos - window + 1) : 0;
    } else {
        info.q = nullptr;
        info.pos = -1;
        info.lo = 0;
    }
    return info;
}

// What the decode kernel needs to do the step before it as well: the RMSNorm of each q and k
// head, the rotation over the whole head, and the write of the new K and V into the pages.
// (Decode steps are short and every launch has a price; the prompt path keeps its own kernel.)
struct FusedQKV {
    const bf16_t* qkv;      // [N, (nq + 2 nkv) * D] as the projection left it
    const int32_t* slots;   // [N] place of each token in the pages (page * P + offset), < 0: not written
    const void* q_weight;   // [D] or nullptr: no norm
    const void* k_weight;
    int weight_dtype;
    const float* cos_sin;   // [N, D / 2, 2]
    float eps;
    int write_kv;
};

// Eight consecutive norm weights (float32 or bfloat16) as they lie in memory; what they mean is
// decided by weights8_as_f32 AFTER the loads have met again.  (Converted inside the branch that
// knows the type, every load would be waited for on the spot, one memory latency each.)
struct RawWeights8 {
    uint32_t bits[8];  // bfloat16: the first four words hold the eight values
};
__device__ __forceinline__ void load_raw_weights8(const void* w, int e, int dtype, RawWeights8& out) {
    if (dtype == LLE_F32) {
        const uint4 a = *(const uint4*)((const float*)w + e), b = *(const uint4*)((const float*)w + e + 4);
        out.bits[0] = a.x, out.bits[1] = a.y, out.bits[2] = a.z, out.bits[3] = a.w;
        out.bits[4] = b.x, out.bits[5] = b.y, out.bits[6] = b.z, out.bits[7] = b.w;
    } else {
        const uint4 a = *(const uint4*)((const bf16_t*)w + e);
        out.bits[0] = a.x, out.bits[1] = a.y, out.bits[2] = a.z, out.bits[3] = a.w;
        out.bits[4] = out.bits[5] = out.bits[6] = out.bits[7] = 0u;
    }
}
__device__ __forceinline__ float weights8_as_f32(const RawWeights8& raw, int i, bool is_f32) {
    const uint32_t word = raw.bits[i / 2];
    const uint32_t as_bf16 = (i % 2) ? (word & 0xffff0000u) : (word << 16);
    return __uint_as_float(is_f32 ? raw.bits[i] : as_bf16);
}
// one weight: the word it lies in (a bfloat16 value in the low half), read by weight_as_f32
__device__ __forceinline__ uint32_t load_raw_weight(const void* w, int e, int dtype) {
    if (dtype == LLE_F32) return ((const uint32_t*)w)[e];
    return ((const uint16_t*)w)[e];
}
__device__ __forceinline__ float weight_as_f32(uint32_t raw, bool is_f32) {
    return __uint_as_float(is_f32 ? raw : raw << 16);
}

// Q^T operands of the lane's row from the raw projection: norm over the head (its 4 * DK * 8
// elements sit in the four lanes r16 + 16 c), weight, rotation.  Element 32 ks + 8 c + i and its
// partner D / 2 further on are both in this lane (DK is even).  Rounded to bfloat16 as the
// separate kernel rounds q.  Everything is ASKED FOR in one go (load) and worked on later
// (finish): a load that followed the arithmetic on another would cost the memory's latency again.
template <int DK>
struct FusedQRow {
    static_assert(DK % 2 == 0, "rotation partners lie in one lane only for an even number of 32-element blocks");
    bf16x8 raw[DK];
    RawWeights8 w[DK];
    float4 tab[DK / 2][4];  // cos, sin of element 2 i, then of 2 i + 1

    // `src`: the head of a row that exists (lanes of rows that do not exist read another row's and drop it)
    __device__ __forceinline__ void load(const bf16_t* src, const FusedQKV& f, int64_t tok) {
        constexpr int D = DK * 32;
        const int c = (threadIdx.x % LLE_WAVE) / 16;
#pragma unroll
        for (int ks = 0; ks < DK; ++ks) raw[ks] = *(const bf16x8*)(src + 32 * ks + 8 * c);
#pragma unroll
        for (int ks = 0; ks < DK / 2; ++ks) {
            const float4* t = (const float4*)(f.cos_sin + (tok * (D / 2) + 32 * ks + 8 * c) * 2);
#pragma unroll
            for (int i = 0; i < 4; ++i) tab[ks][i] = t[i];
        }
        if (f.q_weight) {
#pragma unroll
            for (int ks = 0; ks < DK; ++ks) load_raw_weights8(f.q_weight, 32 * ks + 8 * c, f.weight_dtype, w[ks]);
        }
    }

    __device__ __forceinline__ void finish(bf16x8 (&qv)[DK], bool exists, const FusedQKV& f) const {
        constexpr int D = DK * 32;
        float x[DK][8];
#pragma unroll
        for (int ks = 0; ks < DK; ++ks)
#pragma unroll
            for (int i = 0; i < 8; ++i) x[ks][i] = exists ? (float)raw[ks][i] : 0.f;
        if (f.q_weight) {
            float ss = 0.f;
#pragma unroll
            for (int ks = 0; ks < DK; ++ks)
#pragma unroll
                for (int i = 0; i < 8; ++i) ss += x[ks][i] * x[ks][i];
            ss += __shfl_xor(ss, 16, LLE_WAVE);
            ss += __shfl_xor(ss, 32, LLE_WAVE);
            const float inv = 1.0f / sqrtf(ss / (float)D + f.eps);
            const bool is_f32 = f.weight_dtype == LLE_F32;
#pragma unroll
            for (int ks = 0; ks < DK; ++ks)
#pragma unroll
                for (int i = 0; i < 8; ++i) x[ks][i] = x[ks][i] * inv * weights8_as_f32(w[ks], i, is_f32);
        }
#pragma unroll
        for (int ks = 0; ks < DK / 2; ++ks) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float4 t = tab[ks][i];
                const float a0 = x[ks][2 * i], b0 = x[ks + DK / 2][2 * i];
                const float a1 = x[ks][2 * i + 1], b1 = x[ks + DK / 2][2 * i + 1];
                x[ks][2 * i] = a0 * t.x - b0 * t.y;
                x[ks + DK / 2][2 * i] = b0 * t.x + a0 * t.y;
                x[ks][2 * i + 1] = a1 * t.z - b1 * t.w;
                x[ks + DK / 2][2 * i + 1] = b1 * t.z + a1 * t.w;
            }
        }
#pragma unroll
        for (int ks = 0; ks < DK; ++ks)
#pragma unroll
            for (int i = 0; i < 8; ++i) qv[ks][i] = (bf16_t)x[ks][i];
    }
};

// One wavefront: K (norm, weight, rotation) and V of token `tok`, kv head `kvh`, into the pages.
// Lane l takes elements l, l + 64, ... < D / 2 and their partners D / 2 further on.  All loads
// are asked for before anything waits for one of them.
template <int DK>
__device__ __forceinline__ void fused_kv_write(const FusedQKV& f, int64_t tok, int kvh, int nq, int nkv,
                                               bf16_t* kv_layer, int P, int64_t page_stride) {
    constexpr int D = DK * 32, HALF = D / 2, PER = (HALF + LLE_WAVE - 1) / LLE_WAVE;
    const int lane = threadIdx.x % LLE_WAVE;
    const int slot = f.slots[tok];
    const bf16_t* ksrc = f.qkv + (tok * (nq + 2 * nkv) + nq + kvh) * D;
    const bf16_t* vsrc = ksrc + (int64_t)nkv * D;
    float lo[PER], hi[PER];
    uint32_t wlo[PER], whi[PER];
    bf16_t vlo[PER], vhi[PER];
    float2 tab[PER];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int e = min(lane + LLE_WAVE * j, HALF - 1);  // lanes past the half read its last element and drop it
        lo[j] = (float)ksrc[e];
        hi[j] = (float)ksrc[e + HALF];
        vlo[j] = vsrc[e];
        vhi[j] = vsrc[e + HALF];
        tab[j] = *(const float2*)(f.cos_sin + (tok * HALF + e) * 2);
        wlo[j] = whi[j] = 0x3f80u;  // 1 as bfloat16
    }
    const bool is_f32 = f.k_weight && f.weight_dtype == LLE_F32;
    if (f.k_weight) {
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int e = min(lane + LLE_WAVE * j, HALF - 1);
            wlo[j] = load_raw_weight(f.k_weight, e, f.weight_dtype);
            whi[j] = load_raw_weight(f.k_weight, e + HALF, f.weight_dtype);
        }
    }
    if (slot < 0) return;
    const int page = slot / P, off = slot - page * P;
    bf16_t* page_base = kv_layer + (int64_t)page * page_stride;
    bf16_t* kdst = page_base + ((int64_t)kvh * P + off) * D;
    bf16_t* vdst = page_base + ((int64_t)nkv + kvh) * P * D + off;  // element e at vdst[e * P]
    float inv = 1.f;
    if (f.k_weight) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < PER; ++j)
            if (lane + LLE_WAVE * j < HALF) ss += lo[j] * lo[j] + hi[j] * hi[j];
        ss = wave_sum(ss);
        inv = 1.0f / sqrtf(ss / (float)D + f.eps);
    }
#pragma unroll
    for (int j = 0; j < PER; ++j) {
        const int e = lane + LLE_WAVE * j;
        if (e < HALF) {
            const float a = lo[j] * inv * weight_as_f32(wlo[j], is_f32), b = hi[j] * inv * weight_as_f32(whi[j], is_f32);
            kdst[e] = (bf16_t)(a * tab[j].x - b * tab[j].y);
            kdst[e + HALF] = (bf16_t)(b * tab[j].x + a * tab[j].y);
            vdst[(int64_t)e * P] = vlo[j];
            vdst[(int64_t)(e + HALF) * P] = vhi[j];
        }
    }
}

// Requests whose rows (q_len * group) fit one 16-row tile: decoded tokens and very
// short portions.  grid = (requests, kv heads, splits).
#ifndef DEC_WAVES
#define DEC_WAVES 4
#endif
template <int DK, bool FUSED>
__global__ __launch_bounds__(DEC_WAVES* LLE_WAVE) void mfma_decode_kernel(
    const bf16_t* __restrict__ q, bf16_t* kv_layer, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ kv_lens, bf16_t* __restrict__ out, float* __restrict__ ws_o,
    float* __restrict__ ws_ml, int ws_stride, int nq, int nkv, int P, int64_t page_stride, int max_pages,
    int window, float scale_log2, FusedQKV fused) {
    constexpr int D = DK * 32;
    extern __shared__ float smem[];  // [waves][16][D] acc, then [waves][16] m, [waves][16] l
    float* s_o = smem;
    float* s_m = smem + DEC_WAVES * 16 * D;
    float* s_l = s_m + DEC_WAVES * 16;

    // A launch of this kernel is short, and what it waits for before its first key counts.  All
    // arguments are read here in one go, and so is all that is known of the request: read where
    // they are first used, each group would cost a round trip to memory of its own.
    // (The four tables that are read with scalar loads stay out of the statement: a pointer that
    // it has seen counts as written to, and loads through it would become vector loads.)
    asm volatile("" ::"s"(q), "s"(kv_layer), "s"(out), "s"(ws_o), "s"(ws_ml), "s"(ws_stride), "s"(nq), "s"(nkv), "s"(P),
                 "s"(page_stride), "s"(max_pages), "s"(window), "s"(scale_log2), "s"(fused.qkv), "s"(fused.slots),
                 "s"(fused.q_weight), "s"(fused.k_weight), "s"(fused.weight_dtype), "s"(fused.cos_sin),
                 "s"(fused.eps), "s"(fused.write_kv));
    const int s = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z, nsplit = gridDim.z;
    const int G = nq / nkv;
    const int q_start = cu_tokens[s], q_end = cu_tokens[s + 1], kv_len = kv_lens[s], seq_slot = seq_slots[s];
    asm volatile("" ::"s"(q_start), "s"(q_end), "s"(kv_len), "s"(seq_slot));
    const int q_len = q_end - q_start;
    const int nrows = q_len * G;
    if (nrows > 16 || nrows <= 0) return;  // the prefill kernel's, or nothing to do
    const int past = kv_len - q_len;
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int c = lane / 16, r16 = lane % 16;
    const int32_t* table = block_tables + (int64_t)seq_slot * max_pages;

    // FUSED: q is made here from the projection; the row's pointer only says that the row exists
    RowInfo row[1] = {make_row(FUSED ? fused.qkv : q, r16, nrows, G, q_start, past, nq, kvh, D, window)};
    const int lo_min = window > 0 ? max(0, past - window + 1) : 0;
    const int hi = kv_len - 1;
    const int first = lo_min / KSTEP, last = hi / KSTEP;
    const int per_split = (last - first + 1 + nsplit - 1) / nsplit;
    const int sb = first + split * per_split;
    const int se = min(last + 1, sb + per_split);
    // keys of later splits are not this workgroup's: attend_rows may run a step past `se`
    row[0].pos = min(row[0].pos, se * KSTEP - 1);
    // ... and asks for operands two steps ahead: past this split's last key those loads go to the
    // split's own last page (which the caches hold) instead of the next split's pages, which would
    // travel from memory twice, once for each of the two workgroups
    const int hi_loads = max(lo_min, min(hi, se * KSTEP - 1));

    RowState<DK, 1> st;
    if constexpr (FUSED) {
        // The raw q row, its rotation table and the norm weights are asked for while the table
        // lookup is on its way.  A new token's K and V go into the pages by the hand of the
        // wavefront that multiplies the token's step (step sb + wave, + DEC_WAVES, ...): it
        // stores them before it asks for any key, no other wavefront of this launch needs them
        // (one that runs a step past its share masks that step out whole), and so no barrier
        // stands between the write and the keys.
        FusedQRow<DK> qrow;
        const int rr = r16 < nrows ? r16 : 0;
        const int64_t tok = (int64_t)q_start + rr / G;
        attend_rows<DK, 1, false>(
            st, row, kv_layer, table, kvh, nkv, P, page_stride, sb + wave, se, DEC_WAVES, lo_min, hi_loads, scale_log2,
            [&]() {
                qrow.load(fused.qkv + (tok * (nq + 2 * nkv) + kvh * G + rr % G) * D, fused, tok);
                if (fused.write_kv) {
                    for (int t = 0; t < q_len; ++t) {
                        const int step_of = (past + t) / KSTEP;
                        if (step_of >= sb && step_of < se && (step_of - sb) % DEC_WAVES == wave)
                            fused_kv_write<DK>(fused, (int64_t)q_start + t, kvh, nq, nkv, kv_layer, P, page_stride);
                    }
                    // The keys are read through the same pointer (no `restrict` on it: the pages are
                    // written and read in this kernel), after this point in program order; the fence
                    // keeps the compiler from moving those loads above the stores.
                    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                    asm volatile("" ::: "memory");
                }
            },
            [&]() { qrow.finish(st.qv[0], r16 < nrows, fused); });
    } else {
        attend_rows<DK, 1, true>(
            st, row, kv_layer, table, kvh, nkv, P, page_stride, sb + wave, se, DEC_WAVES, lo_min, hi_loads, scale_log2,
            []() {}, []() {});
    }

    // merge the wavefronts (rows that do not exist are not worth the LDS traffic)
    if (r16 < nrows) {
#pragma unroll
        for (int n = 0; n < 2 * DK; ++n) *(f32x4*)(s_o + (wave * 16 + r16) * D + 16 * n + 4 * c) = st.o[0][n];
    }
    if (c == 0) {
        s_m[wave * 16 + r16] = st.m[0];
        s_l[wave * 16 + r16] = st.l[0];
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < nrows * D; idx += blockDim.x) {
        const int r = idx / D, e = idx - r * D;
        float big = s_m[r];
#pragma unroll
        for (int w = 1; w < DEC_WAVES; ++w) big = fmaxf(big, s_m[w * 16 + r]);
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) {
            const float f = exp2f(s_m[w * 16 + r] - big);
            num += s_o[(w * 16 + r) * D + e] * f;
            den += s_l[w * 16 + r] * f;
        }
        const int t = r / G, g = r - t * G;
        const int64_t head_row = (int64_t)(q_start + t) * nq + kvh * G + g;
        if (nsplit == 1) {
            out[head_row * D + e] = (bf16_t)(num / den);
        } else {
            ws_o[(head_row * ws_stride + split) * D + e] = num;
            if (e == 0) {
                ws_ml[(head_row * ws_stride + split) * 2] = big;
                ws_ml[(head_row * ws_stride + split) * 2 + 1] = den;
            }
        }
    }
}

// Merges the key splits.  grid = (tokens, q heads), one wavefront each; lane k holds (m, l) of
// split k (at most 64 splits).  A token of a request with at most 16 rows was split
// `nsplit_decode` ways by the decode kernel, any other `nsplit_prefill` ways by the prefill
// kernel; a token whose kernel did not split was written by that kernel itself.
__global__ __launch_bounds__(LLE_WAVE) void mfma_combine_kernel(const float* __restrict__ ws_o,
                                                                const float* __restrict__ ws_ml, int ws_stride,
                                                                const int32_t* __restrict__ cu_tokens,
                                                                const int32_t* __restrict__ token_seq,
                                                                bf16_t* __restrict__ out, int nq, int nkv, int D,
                                                                int nsplit_decode, int nsplit_prefill) {
    const int64_t tok = blockIdx.x;
    const int h = blockIdx.y;
    int nsplit = nsplit_decode;
    if (nsplit_decode != nsplit_prefill) {
        const int s = token_seq[tok];
        if ((cu_tokens[s + 1] - cu_tokens[s]) * (nq / nkv) > 16) nsplit = nsplit_prefill;
    }
    if (nsplit <= 1) return;
    const int lane = threadIdx.x;
    const int64_t head_row = tok * nq + h;
    // (m, l) of the lane's split and the first eight splits' partial sums of the lane's first two
    // elements are asked for together: the launch is as short as its chain of loads.
    const float* o = ws_o + head_row * ws_stride * D;
    const float2 ml = *(const float2*)(ws_ml + (head_row * ws_stride + min(lane, nsplit - 1)) * 2);
    const int e_first = min(2 * lane, D - 2);
    float2 first[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) first[j] = *(const float2*)(o + (int64_t)min(j, nsplit - 1) * D + e_first);
    const float m = lane < nsplit ? ml.x : NEG_BIG, l = lane < nsplit ? ml.y : 0.f;
    const float big = wave_max(m);
    const float f = exp2f(m - big);  // 0 for lanes without a split (l = 0 there anyway)
    const float den = wave_sum(l * f);
    // every lane needs every split's factor, also those of lanes that have no element below
    __shared__ float s_f[LLE_WAVE];
    s_f[lane] = f;
    __syncthreads();
    // A lane takes two neighbouring elements; the partial sums of eight splits are loaded
    // together (one load after the other would pay the memory's latency once per split).
    for (int e = 2 * lane; e < D; e += 2 * LLE_WAVE) {
        float2 num = {0.f, 0.f};
        for (int k0 = 0; k0 < nsplit; k0 += 8) {
            float2 part[8];
            if (k0 == 0 && e == e_first) {
#pragma unroll
                for (int j = 0; j < 8; ++j) part[j] = first[j];
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) part[j] = *(const float2*)(o + (int64_t)min(k0 + j, nsplit - 1) * D + e);
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const float fk = k0 + j < nsplit ? s_f[k0 + j] : 0.f;
                num.x += part[j].x * fk;
                num.y += part[j].y * fk;
            }
        }
        out[head_row * D + e] = (bf16_t)(num.x / den);
        out[head_row * D + e + 1] = (bf16_t)(num.y / den);
    }
}

// Requests with more than 16 rows.  grid = (kv heads, row blocks x key splits, requests); a
// workgroup takes a block of rows (token, head of the group) and walks the keys they see in steps
// of 32.  A short portion after a long past has few row blocks: its keys are then split over
// `nsplit` workgroups, which leave (m, l, acc) for the combine kernel.  The 32-key tiles of K and
// V^T are copied from the pages into LDS once per workgroup (all threads; two tiles are on their
// way while one is multiplied) and every wavefront reads its matrix-core operands from there:
// the rows of a workgroup share one pass over the keys.
//   LDS K tile:   [32 keys][D]    LDS V^T tile: [D][32 keys]
// both without padding, the 16-byte pieces of a row XOR-swizzled (K_SWIZZLE, V_SWIZZLE).
// Heads of 128 elements skip the registers: global_load_lds_dwordx4 writes the tiles into LDS
// directly (three buffers; see the DMA branch of the kernel).
// The shapes of a workgroup (PRE_WAVES wavefronts of PRE_RT tiles of 16 rows each):
//   4 x 1: 64 rows.  Twice the workgroups of half the height: for launches so small that these
//          all fit the chip at once.
//   4 x 2: 128 rows; every operand read from LDS serves both tiles of a wavefront.  Two
//          workgroups a CU in 256 registers a lane (heads up to 128; above, 4 x 1 only).
//   8 x 1: 128 rows, heads of 128 only.  Two workgroups a CU are four wavefronts a SIMD, in 128
//          registers each.  A wavefront issues about one instruction in eight cycles whatever
//          its kind, and a matrix instruction holds it for sixteen; the wavefronts of a SIMD run
//          side by side until they meet at an issue port, so four of them get more out of it
//          than two (measured: 118 against 128 us for 2048 rows over 4096 keys), although each
//          tile is then read from LDS by twice as many wavefronts.
#ifndef PRE_RT_MAX
#define PRE_RT_MAX 2
#endif
#define PRE_RT_OF(DK) ((DK) <= 4 ? PRE_RT_MAX : 1)
template <int DK, int PRE_RT, int PRE_WAVES = 4>
// (heads over 192 elements need more than the 256 registers a lane that two workgroups a CU leave)
__global__ __launch_bounds__(PRE_WAVES* LLE_WAVE, DK <= 6 ? 2 : 1) void mfma_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ kv_layer, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ kv_lens, bf16_t* __restrict__ out, float* __restrict__ ws_o,
    float* __restrict__ ws_ml, int ws_stride, int nsplit, int nq, int nkv, int P, int64_t page_stride, int max_pages,
    int window, float scale_log2, int complement_order) {
    constexpr int D = DK * 32;
    static_assert(PRE_RT <= PRE_RT_OF(DK), "the accumulators of two row tiles fit the registers up to heads of 128");
    constexpr int PRE_ROWS = PRE_WAVES * 16 * PRE_RT;
    constexpr bool DMA = DK == 4 && (PRE_WAVES == 4 || PRE_WAVES == 8);  // tiles straight into LDS (measured 4-5 % faster)
    static_assert(PRE_WAVES == 4 || (DK == 4 && PRE_RT == 1), "eight wavefronts: heads of 128, one row tile each");
    constexpr int TILE = 2 * KSTEP * D;  // elements of a tile: K [32 keys][D], then V^T [D][32 keys]
    __shared__ __attribute__((aligned(16))) bf16_t lds[(DMA ? 3 : 2) * TILE];

    // the kv head varies fastest: workgroups go to the eight dies in turn, each die has an L2 of
    // its own, and this way a die sees the K/V of few heads, which the row blocks of a head share
    const int s = blockIdx.z, kvh = blockIdx.x;
    const int G = nq / nkv;
    const int q_start = cu_tokens[s];
    const int q_len = cu_tokens[s + 1] - q_start;
    const int nrows = q_len * G;
    if (nrows <= 16) return;  // the decode kernel's
    // The last rows see the most keys: they are started first.  When the whole launch is
    // resident at once (two workgroups a CU) the order is: the heavy half of the row blocks,
    // heaviest first, then the light half, lightest first, so that the two workgroups that
    // come to share a CU (launch positions j and j + half) add up to about the same work.
    const int row_blocks = gridDim.y / nsplit;
    const int split = blockIdx.y / row_blocks;
    const int yb = blockIdx.y % row_blocks, heavy_blocks = (row_blocks + 1) / 2;
    const int block_row0 =
        (complement_order && yb >= heavy_blocks ? yb - heavy_blocks : row_blocks - 1 - yb) * PRE_ROWS;
    if (block_row0 >= nrows) return;
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int c = lane / 16, r16 = lane % 16;
    const int kv_len = kv_lens[s];
    const int past = kv_len - q_len;
    const int32_t* table = block_tables + (int64_t)seq_slots[s] * max_pages;

    // the workgroup's key range, and this wavefront's own
    const int block_last_row = min(nrows, block_row0 + PRE_ROWS) - 1;
    const int hi = past + block_last_row / G;
    const int block_first_pos = past + block_row0 / G;
    const int lo_min = window > 0 ? max(0, block_first_pos - window + 1) : 0;
    int first_step = lo_min / KSTEP, end_step = hi / KSTEP + 1;
    if (nsplit > 1) {  // this workgroup's share of the steps (it may be empty)
        const int per_split = (end_step - first_step + nsplit - 1) / nsplit;
        first_step = first_step + split * per_split;
        end_step = min(end_step, first_step + per_split);
    }

    const int row0 = block_row0 + wave * (16 * PRE_RT);
    RowInfo row[PRE_RT];
#pragma unroll
    for (int t = 0; t < PRE_RT; ++t) row[t] = make_row(q, row0 + 16 * t + r16, nrows, G, q_start, past, nq, kvh, D, window);
    int my_first = end_step, my_end = first_step;  // a wavefront without rows multiplies nothing
    if (row0 < nrows) {
        const int my_last_row = min(nrows, row0 + 16 * PRE_RT) - 1;
        const int my_lo = window > 0 ? max(0, past + row0 / G - window + 1) : 0;
        my_first = my_lo / KSTEP;
        my_end = min(end_step, (past + my_last_row / G) / KSTEP + 1);
    }
    // (the same in every lane of a wavefront: in scalar registers the tests on them are scalar branches)
    my_first = __builtin_amdgcn_readfirstlane(my_first);
    my_end = __builtin_amdgcn_readfirstlane(my_end);
    RowState<DK, PRE_RT> st;
    init_rows<DK, PRE_RT>(st, row);
    // what this lane reads from a tile in LDS: its two keys of a step and their swizzles
    const int kx[2] = {KEY_OF_ROW(r16, 0), KEY_OF_ROW(r16, 1)};
    const int ksw[2] = {K_SWIZZLE(kx[0], DK), K_SWIZZLE(kx[1], DK)};
    const int vsw = V_SWIZZLE(r16);

    const int64_t k_head = (int64_t)kvh * P * D;
    const int64_t v_head = ((int64_t)nkv + kvh) * P * D;
    // a tile holds 4 D 16-byte pieces of K and as many of V^T; this thread copies NP of each
    constexpr int PIECES = 4 * D;
    constexpr int NP = (PIECES + PRE_WAVES * LLE_WAVE - 1) / (PRE_WAVES * LLE_WAVE);
    // then the copies stand under no condition (see one_step on what a condition costs)
    constexpr bool EVERY_THREAD_COPIES = PIECES % (PRE_WAVES * LLE_WAVE) == 0;
    // two tiles are on their way from memory at any time (register sets 0 and 1); a tile is
    // written to LDS one step after its loads were issued and multiplied one step later still
    bf16x8 stage_k[2][NP], stage_v[2][NP];
    // The pages of the two 16-key halves of a step are looked up one fetch ahead, so that the
    // table's latency is not in the way of the loads that need it.  Fetches come in step order:
    // page and offset of the next half are carried along instead of divided out (the page size
    // is no constant).  A half wholly outside [lo_min, hi] may lie in a page that is not there:
    // the page index is clamped to those of keys that are.
    const int page_lo = lo_min / P, page_hi = hi / P;
    int look_page = __builtin_amdgcn_readfirstlane((first_step * KSTEP) / P);
    int look_off = __builtin_amdgcn_readfirstlane((first_step * KSTEP) % P);
    int page_id[2], page_off[2];
    auto lookup = [&]() {
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            page_id[x] = table[__builtin_amdgcn_readfirstlane(min(max(look_page, page_lo), page_hi))];
            page_off[x] = look_off;
            look_off += 16;  // pages hold a multiple of 16 keys
            if (look_off == P) {
                look_off = 0;
                ++look_page;
            }
        }
    };
    lookup();
    // Piece `piece` of a tile: the wavefront-sized run it lies in belongs to ONE 16-key half
    // (half = run / DK), so the half's page is the same for the whole wavefront and its address
    // stays in scalar registers; what differs between the threads is fixed for the kernel.
    //   K: the half's keys row by row, 16 bytes of a row per piece;
    //   V^T: the half's value elements one by one, each 16 keys = two pieces.
    int k_thread[NP], v_thread[NP];  // element offsets from the half's first key, in the page
    int k_lds[NP], v_lds[NP];        // element offsets in a tile in LDS
#pragma unroll
    for (int i = 0; i < NP; ++i) {
        const int q = (threadIdx.x + PRE_WAVES * LLE_WAVE * i) % (2 * D);  // piece within its half
        const int half = (threadIdx.x + PRE_WAVES * LLE_WAVE * i) / (2 * D);
        k_thread[i] = (q / (D / 8)) * D + (q % (D / 8)) * 8;
        v_thread[i] = (q / 2) * P + (q % 2) * 8;
        const int key = 16 * half + q / (D / 8);
        k_lds[i] = key * D + (((q % (D / 8)) ^ K_SWIZZLE(key, DK)) * 8);
        v_lds[i] = KSTEP * D + (q / 2) * KSTEP + (((2 * half + q % 2) ^ V_SWIZZLE(q / 2)) * 8);
    }
    auto fetch = [&](auto set_c) {
        constexpr int set = decltype(set_c)::value;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int piece = threadIdx.x + PRE_WAVES * LLE_WAVE * i;
            if (EVERY_THREAD_COPIES || piece < PIECES) {
                const int half = __builtin_amdgcn_readfirstlane(piece / (2 * D));
                const bf16_t* page = kv_layer + (int64_t)(half ? page_id[1] : page_id[0]) * page_stride;
                const int off = half ? page_off[1] : page_off[0];
                stage_k[set][i] = *(const bf16x8*)(page + k_head + (int64_t)off * D + k_thread[i]);
                stage_v[set][i] = *(const bf16x8*)(page + v_head + off + v_thread[i]);
            }
        }
        lookup();
    };
    auto stash = [&](int buf, auto set_c) {
        constexpr int set = decltype(set_c)::value;
        bf16_t* tile = lds + buf * TILE;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int piece = threadIdx.x + PRE_WAVES * LLE_WAVE * i;
            if (EVERY_THREAD_COPIES || piece < PIECES) {
                *(bf16x8*)(tile + k_lds[i]) = stage_k[set][i];
                *(bf16x8*)(tile + v_lds[i]) = stage_v[set][i];
            }
        }
    };
    // one step: tile `step` is in LDS buffer `buf`; tile step + 1 sits in register set `set`
    // (loads issued a step ago) and goes to the other buffer; tile step + 2 is requested now
    // into the other register set
    // Fetch and stash run in every step, also past the last tile (the lookup clamps to a page
    // that is there; what is stashed then is never read): a load under a condition makes the
    // compiler wait, where the paths meet again, for the loads that were issued last.
    auto one_step = [&](int step, int buf, auto set_c) {
        constexpr int set = decltype(set_c)::value;
        fetch(std::integral_constant<int, 1 - set>{});  // tile step + 2
        if (step >= my_first && step < my_end) {
            const bf16_t* kt = lds + buf * TILE;
            const bf16_t* vt = kt + KSTEP * D;
            tile_step<DK, PRE_RT>(
                st, row,
                [&](int x, int ks) { return *(const bf16x8*)(kt + kx[x] * D + (((4 * ks + c) ^ ksw[x]) * 8)); },
                [&](int n) { return *(const bf16x8*)(vt + (16 * n + r16) * KSTEP + ((c ^ vsw) * 8)); },
                step * KSTEP, scale_log2);
        }
        stash(buf ^ 1, set_c);
        __syncthreads();
    };

    if constexpr (DMA) {
        // Tiles go from the pages straight into LDS (no registers, no stores by the wavefronts):
        // a wavefront's load writes 1 KB of LDS in lane order (M0 holds where), so the swizzle is
        // in which piece each lane fetches: the logical piece that belongs at its place (physical
        // piece ^ swizzle).  The loads are written in assembly so that the waits are ours: the
        // compiler, seeing such a load, waits for ALL outstanding loads before every barrier.
        // vmcnt counts them in issue order, so "at most the 4 newest outstanding" means that
        // every tile requested before the last one has landed, whatever else was issued.
        // Three buffers: tile N is multiplied, N + 1 has landed or lands, N + 2 is requested.
        const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) void*)lds;
        const int tid = threadIdx.x;
        // A load's address is a base that is the same for the whole wavefront (scalar registers:
        // the page of one 16-key half) plus a byte offset per lane that never changes:
        //   K:   half i of the step, key q / 16 of it, physical piece q % 16        (q = thread + 256 i)
        //   V^T: half i of the step, element thread / 2, keys 8 (thread % 2) .. + 7 of the half
        // so V^T lies in LDS as [half][D][16 keys]: rows of 32 bytes, which the sixteen lanes that
        // a 16-byte read serves in a cycle (c0 and c0 + 1 of one half, eight different elements
        // mod 8 each) spread over the sixteen columns of the banks without a swizzle.
        constexpr int LOADS = 512 / (PRE_WAVES * LLE_WAVE);  // of K and of V^T, per thread and tile
        unsigned kd_lane[LOADS], vd_lane[LOADS];
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int q = tid + PRE_WAVES * LLE_WAVE * i;  // the half is q / 256: the same for a wavefront's load
            const int key = q / 16, pk = q % 16;
            kd_lane[i] = 2u * (unsigned)((key % 16) * D + ((pk ^ K_SWIZZLE(key, DK)) * 8));
            vd_lane[i] = 2u * (unsigned)(((q % 256) / 2) * P + (q % 2) * 8);
        }
        // With one load of K and one of V^T per wavefront and tile a wavefront needs the page of
        // its own half only, and follows that alone: half the scalar arithmetic a step.
        int own_page = 0, own_off = 0, own_id = 0;
        const int own_adv_pages = KSTEP / P, own_adv_off = KSTEP % P;
        auto own_lookup = [&]() { own_id = table[__builtin_amdgcn_readfirstlane(min(max(own_page, page_lo), page_hi))]; };
        if constexpr (LOADS == 1) {
            const int key0 = first_step * KSTEP + 16 * (wave / 4);
            own_page = __builtin_amdgcn_readfirstlane(key0 / P);
            own_off = __builtin_amdgcn_readfirstlane(key0 % P);
            own_lookup();
        }
        auto dma = [&](int buf) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) {
                const int first_piece = __builtin_amdgcn_readfirstlane(wave * LLE_WAVE + PRE_WAVES * LLE_WAVE * i);
                const int half = first_piece / 256;
                // (a page's offset as an unsigned 32 x 32 -> 64 bit product: two scalar instructions)
                const int id = LOADS == 1 ? own_id : (half ? page_id[1] : page_id[0]);
                const bf16_t* page = kv_layer + (uint64_t)(uint32_t)id * (uint64_t)(uint32_t)page_stride;
                const int off = LOADS == 1 ? own_off : (half ? page_off[1] : page_off[0]);
                const bf16_t* kb = page + k_head + (int64_t)off * D;
                const bf16_t* vb = page + v_head + off;
                const unsigned kdst = lds_base + 2 * (buf * TILE + first_piece * 8);
                const unsigned vdst = kdst + 2 * KSTEP * D;
                asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(kdst), "v"(kd_lane[i]), "s"(kb) : "memory", "m0");
                asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(vdst), "v"(vd_lane[i]), "s"(vb) : "memory", "m0");
            }
            if constexpr (LOADS == 1) {
                own_page += own_adv_pages;
                own_off += own_adv_off;
                if (own_off >= P) {
                    own_off -= P;
                    ++own_page;
                }
                own_lookup();
            } else {
                lookup();
            }
        };
        const int v_read = (c / 2) * (D * 16) + r16 * 16 + (c % 2) * 8;  // this lane's place in V^T for n = 0
        auto dma_step = [&](int step, int buf, int next_buf) {
            // the key operands are asked for first: the scalar arithmetic of the loads' addresses
            // then covers their way from LDS
            const bf16_t* kt = lds + buf * TILE;
            const bf16_t* vt = kt + KSTEP * D;
            bf16x8 kreg[2][DK];
#pragma unroll
            for (int x = 0; x < 2; ++x)
#pragma unroll
                for (int ks = 0; ks < DK; ++ks)
                    kreg[x][ks] = *(const bf16x8*)(kt + kx[x] * D + (((4 * ks + c) ^ ksw[x]) * 8));
            dma(next_buf);  // tile step + 2
            if (step >= my_first && step < my_end) {
                tile_step<DK, PRE_RT>(
                    st, row, [&](int x, int ks) { return kreg[x][ks]; },
                    [&](int n) { return *(const bf16x8*)(vt + v_read + n * 256); }, step * KSTEP, scale_log2);
            }
            // the loads just issued may stay in flight; the tile before them has landed
            if constexpr (LOADS == 2)
                asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
            else
                asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
            __builtin_amdgcn_s_barrier();
        };
        dma(0);  // tile first_step
        dma(1);  // tile first_step + 1
        if constexpr (LOADS == 2)
            asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else
            asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        for (int step = first_step; step < end_step; step += 3) {
            dma_step(step, 0, 2);
            dma_step(step + 1, 1, 0);
            dma_step(step + 2, 2, 1);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may land after the workgroup has gone
    } else {
        fetch(std::integral_constant<int, 0>{});  // tile first_step
        fetch(std::integral_constant<int, 1>{});  // tile first_step + 1
        stash(0, std::integral_constant<int, 0>{});
        __syncthreads();
        for (int step = first_step; step < end_step; step += 2) {
            one_step(step, 0, std::integral_constant<int, 1>{});
            one_step(step + 1, 1, std::integral_constant<int, 0>{});  // multiplies nothing past my_end
        }
    }
    finish_rows<DK, PRE_RT>(st);
#pragma unroll
    for (int t = 0; t < PRE_RT; ++t) {
        const int r = row0 + 16 * t + r16;
        if (r >= nrows) continue;
        const int tk = r / G, g = r - tk * G;
        const int64_t head_row = (int64_t)(q_start + tk) * nq + kvh * G + g;
        if (nsplit > 1) {
            float* po = ws_o + (head_row * ws_stride + split) * D;
#pragma unroll
            for (int n = 0; n < 2 * DK; ++n) *(f32x4*)(po + 16 * n + 4 * c) = st.o[t][n];
            if (c == 0) {
                ws_ml[(head_row * ws_stride + split) * 2] = st.m[t];
                ws_ml[(head_row * ws_stride + split) * 2 + 1] = st.l[t];
            }
            continue;
        }
        bf16_t* dst = out + head_row * D;
        const float inv = 1.0f / st.l[t];
#pragma unroll
        for (int n = 0; n < 2 * DK; ++n) {
            bf16x4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = (bf16_t)(st.o[t][n][i] * inv);
            *(bf16x4*)(dst + 16 * n + 4 * c) = v;
        }
    }
}

// ---------------------------------------------------------------------------------
// float32 on the matrix cores: v_mfma_f32_16x16x4_f32 multiplies and adds float32 (no
// reduced-precision mode), so this is still the true 32-bit path.  One kernel for every kind
// of request, head sizes in steps of 16 up to 256, pages that hold a multiple of 16 keys:
//   * a request with at most 16 rows (token, head of the group): one tile of rows, the four
//     wavefronts take every fourth 16-key step and are merged through LDS (decoding);
//   * any other: a workgroup takes 64 rows, each wavefront a tile of 16 of them and all keys
//     that its rows see.
// grid = (kv heads, row blocks x key splits, requests); with key splits the partial (m, l, acc)
// go to the workspaces and the combine kernel merges them.
// Operands (lane = (c, r), c = lane / 16, r = lane % 16): a lane loads 16 bytes, four
// consecutive elements, and its element e is the contraction slot c of instruction e:
//   S^T = K Q^T:    A = K[key r][16 q + 4 c + e],  B = Q[row r][16 q + 4 c + e]
//   O^T += V^T P^T: A = V^T[element 16 n + r][key 4 c + e],  B = P[key 4 c + e][row r]
// and the result tile S^T leaves lane (c, r) with keys 4 c .. 4 c + 3 of row r: exactly the B
// operand of the second product, so P never leaves its registers.
// ---------------------------------------------------------------------------------
#define F32_WAVES 4
#define F32_KEYS 16
template <int DQ>
__global__ __launch_bounds__(F32_WAVES* LLE_WAVE) void mfma_f32_attention_kernel(
    const float* __restrict__ q, const float* __restrict__ kv_layer, const int32_t* __restrict__ block_tables,
    const int32_t* __restrict__ seq_slots, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ kv_lens, float* __restrict__ out, float* __restrict__ ws_o,
    float* __restrict__ ws_ml, int nsplit, int nq, int nkv, int P, int64_t page_stride, int max_pages, int window,
    float scale_log2) {
    constexpr int D = 16 * DQ;
    extern __shared__ float smem[];  // [waves][16][D] acc, then [waves][16] m, [waves][16] l
    float* s_o = smem;
    float* s_m = smem + F32_WAVES * 16 * D;
    float* s_l = s_m + F32_WAVES * 16;
    const int s = blockIdx.z, kvh = blockIdx.x;
    const int G = nq / nkv;
    const int q_start = cu_tokens[s];
    const int q_len = cu_tokens[s + 1] - q_start;
    const int nrows = q_len * G;
    if (nrows <= 0) return;
    const int kv_len = kv_lens[s];
    const int past = kv_len - q_len;
    const int row_blocks = gridDim.y / nsplit;
    const int split = blockIdx.y / row_blocks, yb = blockIdx.y % row_blocks;
    const bool few = nrows <= 16;  // the same for the whole workgroup
    const int wave = threadIdx.x / LLE_WAVE, lane = threadIdx.x % LLE_WAVE;
    const int c = lane / 16, r16 = lane % 16;
    if (few ? yb != 0 : yb * (16 * F32_WAVES) >= nrows) return;
    const int row0 = few ? 0 : yb * (16 * F32_WAVES) + wave * 16;
    const bool wave_has_rows = row0 < nrows;
    const int32_t* table = block_tables + (int64_t)seq_slots[s] * max_pages;

    // the lane's row
    const int row = row0 + r16;
    const bool exists = row < nrows;
    const int tok = exists ? row / G : 0, g = exists ? row - tok * G : 0;
    const int64_t head_row = (int64_t)(q_start + tok) * nq + kvh * G + g;
    const int pos = exists ? past + tok : -1;
    const int lo = (exists && window > 0) ? max(0, pos - window + 1) : 0;
    f32x4 qf[DQ];
#pragma unroll
    for (int i = 0; i < DQ; ++i)
        qf[i] = exists ? *(const f32x4*)(q + head_row * D + 16 * i + 4 * c) : f32x4{0.f, 0.f, 0.f, 0.f};

    // the keys of this wavefront's tile, in steps of 16, and its share of them
    int step_begin = 0, step_end = 0, step_stride = 1;
    if (wave_has_rows) {
        const int last_row = min(nrows, row0 + 16) - 1;
        const int hi = past + last_row / G;
        const int lo_tile = window > 0 ? max(0, past + row0 / G - window + 1) : 0;
        const int first = lo_tile / F32_KEYS, end = hi / F32_KEYS + 1;
        const int per_split = (end - first + nsplit - 1) / nsplit;
        step_begin = first + split * per_split;
        step_end = min(end, step_begin + per_split);
        if (few) {
            step_begin += wave;
            step_stride = F32_WAVES;
        }
    }
    f32x4 o[DQ];
#pragma unroll
    for (int n = 0; n < DQ; ++n) o[n] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m = NEG_BIG, l = 0.f;
    const int64_t k_lane = ((int64_t)kvh * P + r16) * D + 4 * c;
    const int64_t v_lane = ((int64_t)nkv + kvh) * P * D + (int64_t)r16 * P + 4 * c;
    constexpr int NBUF = DQ <= 8 ? 2 : 1;
    f32x4 kf[NBUF][DQ], vf[NBUF][DQ];
    auto load = [&](int buf, int step) {
        const int j0 = step * F32_KEYS;
        const int lp = j0 / P, off = j0 - lp * P;  // 16 keys of a step lie in one page
        const float* page = kv_layer + (int64_t)table[__builtin_amdgcn_readfirstlane(lp)] * page_stride;
#pragma unroll
        for (int i = 0; i < DQ; ++i) kf[buf][i] = *(const f32x4*)(page + k_lane + (int64_t)off * D + 16 * i);
#pragma unroll
        for (int n = 0; n < DQ; ++n) vf[buf][n] = *(const f32x4*)(page + v_lane + (int64_t)16 * n * P + off);
    };
    auto multiply = [&](int buf, int step) {
        const int j0 = step * F32_KEYS;
        f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < DQ; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[buf][i][e], qf[i][e], sc, 0, 0, 0);
        float x[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int j = j0 + 4 * c + e;
            x[e] = (j < lo || j > pos) ? NEG_BIG : sc[e] * scale_log2;
        }
        float top = fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3]));
        top = fmaxf(top, __shfl_xor(top, 16, LLE_WAVE));
        top = fmaxf(top, __shfl_xor(top, 32, LLE_WAVE));
        const float new_m = fmaxf(m, top);
        // while the row has seen no key new_m is NEG_BIG as its masked scores are, and
        // exp2(0) = 1 would count them: shift such rows so that they give 0
        const float base = new_m <= NEG_BIG ? 0.f : new_m;
        const float alpha = exp2f(m - base);
        m = new_m;
        f32x4 p;
        float psum = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            p[e] = exp2f(x[e] - base);
            psum += p[e];
        }
        l = l * alpha + psum;
#pragma unroll
        for (int n = 0; n < DQ; ++n) {
            o[n] *= alpha;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[n] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[buf][n][e], p[e], o[n], 0, 0, 0);
        }
    };
    if constexpr (NBUF == 2) {
        // the operands of the next step are asked for before this one is multiplied
        if (step_begin < step_end) load(0, step_begin);
        int buf = 0;
        for (int step = step_begin; step < step_end; step += step_stride) {
            if (step + step_stride < step_end) {
                if (buf == 0) load(1, step + step_stride); else load(0, step + step_stride);
            }
            if (buf == 0) multiply(0, step); else multiply(1, step);
            buf ^= 1;
        }
    } else {  // heads over 128 elements: the registers hold one step's operands
        for (int step = step_begin; step < step_end; step += step_stride) {
            load(0, step);
            multiply(0, step);
        }
    }
    l += __shfl_xor(l, 16, LLE_WAVE);
    l += __shfl_xor(l, 32, LLE_WAVE);

    if (!few) {  // every wavefront writes the rows of its own tile
        if (!exists) return;
        if (nsplit > 1) {
            float* po = ws_o + (head_row * nsplit + split) * D;
#pragma unroll
            for (int n = 0; n < DQ; ++n) *(f32x4*)(po + 16 * n + 4 * c) = o[n];
            if (c == 0) {
                ws_ml[(head_row * nsplit + split) * 2] = m;
                ws_ml[(head_row * nsplit + split) * 2 + 1] = l;
            }
            return;
        }
        const float inv = 1.0f / l;
#pragma unroll
        for (int n = 0; n < DQ; ++n) *(f32x4*)(out + head_row * D + 16 * n + 4 * c) = o[n] * inv;
        return;
    }
    // few rows: the four wavefronts hold parts of the same rows
    if (exists) {
#pragma unroll
        for (int n = 0; n < DQ; ++n) *(f32x4*)(s_o + (wave * 16 + r16) * D + 16 * n + 4 * c) = o[n];
    }
    if (c == 0) {
        s_m[wave * 16 + r16] = m;
        s_l[wave * 16 + r16] = l;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < nrows * D; idx += blockDim.x) {
        const int r = idx / D, e = idx - r * D;
        float big = s_m[r];
#pragma unroll
        for (int w = 1; w < F32_WAVES; ++w) big = fmaxf(big, s_m[w * 16 + r]);
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < F32_WAVES; ++w) {
            const float f = exp2f(s_m[w * 16 + r] - big);  // a wavefront without keys has l = 0, acc = 0
            num += s_o[(w * 16 + r) * D + e] * f;
            den += s_l[w * 16 + r] * f;
        }
        const int t = r / G, gg = r - t * G;
        const int64_t hr = (int64_t)(q_start + t) * nq + kvh * G + gg;
        if (nsplit == 1) {
            out[hr * D + e] = num / den;
        } else {
            ws_o[(hr * nsplit + split) * D + e] = num;
            if (e == 0) {
                ws_ml[(hr * nsplit + split) * 2] = big;
                ws_ml[(hr * nsplit + split) * 2 + 1] = den;
            }
        }
    }
}

// merges the key splits of the kernel above: grid = (tokens, q heads), one wavefront each
__global__ __launch_bounds__(LLE_WAVE) void f32_combine_kernel(const float* __restrict__ ws_o,
                                                               const float* __restrict__ ws_ml, int nsplit,
                                                               float* __restrict__ out, int nq, int D) {
    const int64_t head_row = (int64_t)blockIdx.x * nq + blockIdx.y;
    const int lane = threadIdx.x;
    __shared__ float s_f[LLE_WAVE];
    const float2 ml = *(const float2*)(ws_ml + (head_row * nsplit + min(lane, nsplit - 1)) * 2);
    const float m = lane < nsplit ? ml.x : NEG_BIG, l = lane < nsplit ? ml.y : 0.f;
    const float big = wave_max(m);
    const float f = exp2f(m - big);
    const float den = wave_sum(l * f);
    s_f[lane] = f;
    __syncthreads();
    const float* o = ws_o + head_row * nsplit * D;
    for (int e = lane; e < D; e += LLE_WAVE) {
        float num = 0.f;
        for (int k = 0; k < nsplit; ++k) num += o[(int64_t)k * D + e] * s_f[k];
        out[head_row * D + e] = num / den;
    }
}

// float32, head_dim a multiple of 16 (<= 256), page size a multiple of 16.  `row_blocks`: the
// most 64-row blocks that a request of this batch has (1 when every request has at most 16
// rows); with nsplit > 1 the workspaces ws_o [N * nq * nsplit * d] and ws_ml [N * nq * nsplit * 2]
// floats are needed (nsplit <= 64).
extern "C" int lle_paged_attention_mfma_f32(const void* q, const void* kv_layer, const void* block_tables,
                                            const void* seq_slots, const void* cu_tokens, const void* kv_lens,
                                            void* out, void* ws_o, void* ws_ml, int N, int S, int nq, int nkv, int d,
                                            int page_size, int64_t page_stride, int max_pages, int window,
                                            float scale, int row_blocks, int nsplit, hipStream_t stream) {
    if (N <= 0) return 0;
    if (d % 16 != 0 || d > 256 || d <= 0 || page_size % 16 != 0 || nq % nkv != 0) return (int)hipErrorInvalidValue;
    if (S > 65535 || nkv <= 0 || row_blocks < 1 || nsplit < 1 || nsplit > 64 || (int64_t)row_blocks * nsplit > 65535)
        return (int)hipErrorInvalidValue;
    if (nsplit > 1 && (!ws_o || !ws_ml)) return (int)hipErrorInvalidValue;
    const float scale_log2 = scale * 1.44269504088896340736f;
    const dim3 grid(nkv, row_blocks * nsplit, S);
    const size_t smem = (size_t)(F32_WAVES * 16 * d + 2 * F32_WAVES * 16) * sizeof(float);
#define LLE_F32_CASE(DQV)                                                                                        \
    case DQV:                                                                                                    \
        if (smem > 64 * 1024) {                                                                                  \
            hipError_t e = hipFuncSetAttribute((const void*)mfma_f32_attention_kernel<DQV>,                       \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);           \
            if (e != hipSuccess) return (int)e;                                                                  \
        }                                                                                                        \
        mfma_f32_attention_kernel<DQV><<<grid, F32_WAVES * LLE_WAVE, smem, stream>>>(                             \
            (const float*)q, (const float*)kv_layer, (const int32_t*)block_tables, (const int32_t*)seq_slots,     \
            (const int32_t*)cu_tokens, (const int32_t*)kv_lens, (float*)out, (float*)ws_o, (float*)ws_ml, nsplit, \
            nq, nkv, page_size, page_stride, max_pages, window, scale_log2);                                      \
        break;
    switch (d / 16) {
        LLE_F32_CASE(1) LLE_F32_CASE(2) LLE_F32_CASE(3) LLE_F32_CASE(4) LLE_F32_CASE(5) LLE_F32_CASE(6)
        LLE_F32_CASE(7) LLE_F32_CASE(8) LLE_F32_CASE(9) LLE_F32_CASE(10) LLE_F32_CASE(11) LLE_F32_CASE(12)
        LLE_F32_CASE(13) LLE_F32_CASE(14) LLE_F32_CASE(15) LLE_F32_CASE(16)
    }
#undef LLE_F32_CASE
    if (nsplit > 1)
        f32_combine_kernel<<<dim3(N, nq), LLE_WAVE, 0, stream>>>((const float*)ws_o, (const float*)ws_ml, nsplit,
                                                                 (float*)out, nq, d);
    return (int)hipGetLastError();
}

// CUs of the current device (asked once per device)
static int compute_units() {
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

template <int DK, bool FUSED>
static int launch_decode(const bf16_t* q, bf16_t* kv_layer, const int32_t* block_tables, const int32_t* seq_slots,
                         const int32_t* cu_tokens, const int32_t* kv_lens, bf16_t* out, float* ws_o, float* ws_ml,
                         int ws_stride, int S, int nq, int nkv, int P, int64_t page_stride, int max_pages, int window,
                         float scale_log2, int nsplit, const FusedQKV& fused, hipStream_t stream) {
    constexpr int D = DK * 32;
    const size_t smem = (size_t)(DEC_WAVES * 16 * D + 2 * DEC_WAVES * 16) * sizeof(float);
    if (smem > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)mfma_decode_kernel<DK, FUSED>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return (int)e;
    }
    mfma_decode_kernel<DK, FUSED><<<dim3(S, nkv, nsplit), DEC_WAVES * LLE_WAVE, smem, stream>>>(
        q, kv_layer, block_tables, seq_slots, cu_tokens, kv_lens, out, ws_o, ws_ml, ws_stride, nq, nkv, P,
        page_stride, max_pages, window, scale_log2, fused);
    return 0;
}

// A second stream of this library's own (per device, made at first use, default priority) and the
// two events that fork it from and join it to the caller's stream: in a batch that holds prompt
// portions beside decoded tokens the two attention kernels work on different requests, one bound by
// memory and one by the matrix cores, and share the chip instead of taking turns.
struct SideLane {
    hipStream_t stream;
    hipEvent_t fork, join;
};
static SideLane* side_lane() {
    static SideLane lanes[64];
    static int state[64] = {0};  // 0: not made, 1: there, -1: could not be made
    static std::mutex lock;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    std::lock_guard<std::mutex> guard(lock);
    if (state[dev] == 0) {
        SideLane& l = lanes[dev];
        const bool ok = hipStreamCreateWithFlags(&l.stream, hipStreamNonBlocking) == hipSuccess &&
                        hipEventCreateWithFlags(&l.fork, hipEventDisableTiming) == hipSuccess &&
                        hipEventCreateWithFlags(&l.join, hipEventDisableTiming) == hipSuccess;
        state[dev] = ok ? 1 : -1;
    }
    return state[dev] == 1 ? &lanes[dev] : nullptr;
}

template <int DK>
static int launch_mfma(const bf16_t* q, bf16_t* kv_layer, const int32_t* block_tables,
                       const int32_t* seq_slots, const int32_t* cu_tokens, const int32_t* kv_lens,
                       const int32_t* token_seq, bf16_t* out, float* ws_o, float* ws_ml, int N, int S, int nq,
                       int nkv, int P, int64_t page_stride, int max_pages, int window, float scale_log2,
                       int run_decode, int nsplit_decode, int run_prefill, int nsplit_prefill, int max_q_len,
                       int prefill_form, const FusedQKV& fused, hipStream_t stream) {
    constexpr int D = DK * 32;
    const int G = nq / nkv;
    if (!run_decode) nsplit_decode = 1;
    if (!run_prefill) nsplit_prefill = 1;
    const int ws_stride = nsplit_decode > nsplit_prefill ? nsplit_decode : nsplit_prefill;
    if (fused.qkv && (run_prefill || !run_decode || DK % 2 != 0)) return (int)hipErrorInvalidValue;
    // both kinds in one batch: the decode kernel goes to the side stream, forked from and joined to `stream`
    SideLane* lane = (run_decode && run_prefill) ? side_lane() : nullptr;
    hipStream_t prefill_stream = stream;
    if (lane) {
        if (hipEventRecord(lane->fork, stream) != hipSuccess || hipStreamWaitEvent(lane->stream, lane->fork, 0) != hipSuccess)
            lane = nullptr;
    }
    if (lane) stream = lane->stream;  // for the decode kernel below
    if (run_decode) {
        int e;
        if constexpr (DK % 2 == 0) {
            e = fused.qkv ? launch_decode<DK, true>(q, kv_layer, block_tables, seq_slots, cu_tokens, kv_lens, out, ws_o,
                                                    ws_ml, ws_stride, S, nq, nkv, P, page_stride, max_pages, window,
                                                    scale_log2, nsplit_decode, fused, stream)
                          : launch_decode<DK, false>(q, kv_layer, block_tables, seq_slots, cu_tokens, kv_lens, out,
                                                     ws_o, ws_ml, ws_stride, S, nq, nkv, P, page_stride, max_pages,
                                                     window, scale_log2, nsplit_decode, fused, stream);
        } else {
            e = launch_decode<DK, false>(q, kv_layer, block_tables, seq_slots, cu_tokens, kv_lens, out, ws_o, ws_ml,
                                         ws_stride, S, nq, nkv, P, page_stride, max_pages, window, scale_log2,
                                         nsplit_decode, fused, stream);
        }
        if (e != 0) {
            if (lane) (void)hipStreamSynchronize(lane->stream);
            return e;
        }
    }
    // After the fork an error may not leave the side stream running behind the caller's back: the
    // caller frees `out` and the workspaces on its own stream, and the decode kernel still writes them.
    if (lane) {
        if (hipEventRecord(lane->join, lane->stream) != hipSuccess) {
            const int e = (int)hipGetLastError();
            (void)hipStreamSynchronize(lane->stream);
            return e;
        }
        stream = prefill_stream;
    }
    if (run_prefill) {
        const int rows = max_q_len * G;
        auto launch = [&](auto rt, auto waves) {
            constexpr int RT = decltype(rt)::value, WAVES = decltype(waves)::value;
            constexpr int PRE_ROWS = WAVES * 16 * RT;
            const int blocks = (rows + PRE_ROWS - 1) / PRE_ROWS;
            const int64_t workgroups = (int64_t)nkv * blocks * nsplit_prefill * S;
            mfma_prefill_kernel<DK, RT, WAVES><<<dim3(nkv, blocks * nsplit_prefill, S), WAVES * LLE_WAVE, 0, stream>>>(
                q, kv_layer, block_tables, seq_slots, cu_tokens, kv_lens, out, ws_o, ws_ml, ws_stride, nsplit_prefill,
                nq, nkv, P, page_stride, max_pages, window, scale_log2, workgroups <= 2 * compute_units() ? 1 : 0);
        };
        using Four = std::integral_constant<int, 4>;
        if (DK == 4 && prefill_form == 3) {
            if constexpr (DK == 4) launch(std::integral_constant<int, 1>{}, std::integral_constant<int, 8>{});
        } else if (PRE_RT_OF(DK) == 1 || prefill_form == 1) {
            launch(std::integral_constant<int, 1>{}, Four{});
        } else {
            launch(std::integral_constant<int, PRE_RT_OF(DK)>{}, Four{});
        }
    }
    if (lane && hipStreamWaitEvent(stream, lane->join, 0) != hipSuccess) {
        const int e = (int)hipGetLastError();
        (void)hipStreamSynchronize(lane->stream);
        return e;
    }
    if (ws_stride > 1)  // a batch of one kind needs no look at the tokens' requests
        mfma_combine_kernel<<<dim3(N, nq), LLE_WAVE, 0, stream>>>(
            ws_o, ws_ml, ws_stride, cu_tokens, token_seq, out, nq, nkv, D, run_decode ? nsplit_decode : nsplit_prefill,
            run_prefill ? nsplit_prefill : nsplit_decode);
    return (int)hipGetLastError();
}

// bfloat16, head_dim a multiple of 32 (<= 256), page size a multiple of 16.
// run_decode / run_prefill say which kinds of request the batch holds (requests
// with q_len * group <= 16 rows are the decode kernel's); with ns = max(nsplit_decode,
// nsplit_prefill) > 1 the workspaces ws_o [N * nq * ns * d] and ws_ml [N * nq * ns * 2]
// floats are needed (ns <= 64).
static int paged_attention_mfma(const void* q, void* kv_layer, const void* block_tables, const void* seq_slots,
                                const void* cu_tokens, const void* kv_lens, const void* token_seq, void* out,
                                void* ws_o, void* ws_ml, int N, int S, int nq, int nkv, int d, int page_size,
                                int64_t page_stride, int max_pages, int window, float scale, int run_decode,
                                int nsplit_decode, int run_prefill, int nsplit_prefill, int max_q_len,
                                int prefill_form, const FusedQKV& fused, hipStream_t stream) {
    if (N <= 0) return 0;
    if (d % 32 != 0 || d > 256 || page_size % 16 != 0 || nq % nkv != 0) return (int)hipErrorInvalidValue;
    if (S > 65535 || nkv > 65535 || page_stride < 0 || page_stride >= ((int64_t)1 << 32)) return (int)hipErrorInvalidValue;
    if (nsplit_decode < 1 || nsplit_decode > 64 || nsplit_prefill < 1 || nsplit_prefill > 64)
        return (int)hipErrorInvalidValue;
    const float scale_log2 = scale * 1.44269504088896340736f;
#define LLE_ATT_CASE(DKV)                                                                                          \
    case DKV:                                                                                                      \
        return launch_mfma<DKV>((const bf16_t*)q, (bf16_t*)kv_layer, (const int32_t*)block_tables,                  \
                                (const int32_t*)seq_slots, (const int32_t*)cu_tokens, (const int32_t*)kv_lens,      \
                                (const int32_t*)token_seq, (bf16_t*)out, (float*)ws_o, (float*)ws_ml, N, S, nq, nkv, \
                                page_size, page_stride, max_pages, window, scale_log2, run_decode, nsplit_decode,   \
                                run_prefill, nsplit_prefill, max_q_len, prefill_form, fused, stream);
    switch (d / 32) {
        LLE_ATT_CASE(1)
        LLE_ATT_CASE(2)
        LLE_ATT_CASE(3)
        LLE_ATT_CASE(4)
        LLE_ATT_CASE(5)
        LLE_ATT_CASE(6)
        LLE_ATT_CASE(7)
        LLE_ATT_CASE(8)
    }
#undef LLE_ATT_CASE
    return (int)hipErrorInvalidValue;
}

extern "C" int lle_paged_attention_mfma(const void* q, const void* kv_layer, const void* block_tables,
                                        const void* seq_slots, const void* cu_tokens, const void* kv_lens,
                                        const void* token_seq, void* out, void* ws_o, void* ws_ml, int N, int S,
                                        int nq, int nkv, int d, int page_size, int64_t page_stride, int max_pages,
                                        int window, float scale, int run_decode, int nsplit_decode, int run_prefill,
                                        int nsplit_prefill, int max_q_len, int prefill_form,
                                        hipStream_t stream) {
    const FusedQKV none = {};
    return paged_attention_mfma(q, (void*)kv_layer, block_tables, seq_slots, cu_tokens, kv_lens, token_seq, out, ws_o,
                                ws_ml, N, S, nq, nkv, d, page_size, page_stride, max_pages, window, scale, run_decode,
                                nsplit_decode, run_prefill, nsplit_prefill, max_q_len, prefill_form, none, stream);
}

// Decode steps only (every request has at most 16 / group tokens), head_dim a multiple of 64, a
// rotation over the whole head: the q/k norm, the rotation and the write of the new K and V
// (write_kv != 0; slots [N], < 0: not written) happen inside the attention launch.  qkv is
// [N, (nq + 2 nkv) * d] as the projection left it; q_weight / k_weight [d] or null; cos_sin
// [N, d / 2, 2] float32.
extern "C" int lle_qk_norm_rope_attention_decode(const void* qkv, const void* slots, const void* q_weight,
                                                 const void* k_weight, int weight_dtype, const void* cos_sin,
                                                 float eps, int write_kv, void* kv_layer, const void* block_tables,
                                                 const void* seq_slots, const void* cu_tokens, const void* kv_lens,
                                                 const void* token_seq, void* out, void* ws_o, void* ws_ml, int N,
                                                 int S, int nq, int nkv, int d, int page_size, int64_t page_stride,
                                                 int max_pages, int window, float scale, int nsplit_decode,
                                                 hipStream_t stream) {
    if (!qkv || !cos_sin || !slots || d % 64 != 0) return (int)hipErrorInvalidValue;
    if ((q_weight == nullptr) != (k_weight == nullptr)) return (int)hipErrorInvalidValue;
    FusedQKV fused;
    fused.qkv = (const bf16_t*)qkv;
    fused.slots = (const int32_t*)slots;
    fused.q_weight = q_weight;
    fused.k_weight = k_weight;
    fused.weight_dtype = weight_dtype;
    fused.cos_sin = (const float*)cos_sin;
    fused.eps = eps;
    fused.write_kv = write_kv;
    return paged_attention_mfma(nullptr, kv_layer, block_tables, seq_slots, cu_tokens, kv_lens, token_seq, out, ws_o,
                                ws_ml, N, S, nq, nkv, d, page_size, page_stride, max_pages, window, scale, 1,
                                nsplit_decode, 0, 1, 1, 0, fused, stream);
}
