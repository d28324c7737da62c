// Entry points of the sampling library (sampling.hip), as C callers see them.
// Every function returns 0 or an error code that lle_error_string() explains.
#pragma once
#include <hip/hip_runtime.h>

extern "C" {

// float32 logits [R, V] -> int32 out [R], first maximum wins.  `part_val` (float) and
// `part_idx` (int32) are workspaces of R * chunks elements that the caller brings.
int lle_argmax_rows(const void* logits, void* out, void* part_val, void* part_idx, int R, int V, int chunks,
                    hipStream_t stream);

// The same, and the pick of row r is also written to scatter_dst[scatter_index[r]] (both int32,
// both given or neither).
int lle_argmax_rows_scatter(const void* logits, void* out, void* part_val, void* part_idx, int R, int V, int chunks,
                            void* scatter_dst, const void* scatter_index, hipStream_t stream);

// float32 logits [R, V], temperature [R] (<= 0: greedy), uniform [R] in [0, 1) -> int32 out [R].
int lle_sample_rows(const void* logits, const void* temperature, const void* uniform, void* out, int R, int V,
                    hipStream_t stream);

// lle_argmax_rows for callers that cannot allocate: code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference
// (whose argmax, src/ops/argmax.cu:181-241, needs no workspace because it gives one
// workgroup a whole row).  The per-chunk winners go to a buffer that is part of the
// library's device image instead of a workspace argument: LLE_ARGMAX_STATIC_BYTES bytes on
// every GPU the library runs on, held until the process ends.  The function allocates
// nothing and calls no allocating routine; its first call on a device looks up the buffer's
// address there (hipGetSymbolAddress), later calls only launch.
//   * at most LLE_ARGMAX_STATIC_MAX_ROWS rows; more are refused with
//     LLE_ERROR_STATIC_SCRATCH_TOO_SMALL and nothing is launched;
//   * all calls on one GPU share that GPU's buffer: calls that overlap there (two streams,
//     two threads) race.  Calls on one stream are ordered and safe.  Nothing in the buffer
//     has to start at zero: every element that a call reads it has written before.
#define LLE_ARGMAX_STATIC_MAX_ROWS 256
#define LLE_ARGMAX_STATIC_MAX_CHUNKS 64
#define LLE_ARGMAX_STATIC_BYTES (LLE_ARGMAX_STATIC_MAX_ROWS * LLE_ARGMAX_STATIC_MAX_CHUNKS * 8)
#define LLE_ERROR_STATIC_SCRATCH_TOO_SMALL 100001
int lle_argmax_rows_static(const void* logits, void* out, int R, int V, hipStream_t stream);

const char* lle_error_string(int code);
}
