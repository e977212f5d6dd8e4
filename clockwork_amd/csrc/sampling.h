// C interface of the token-selection library (sampling.hip) for callers outside Python.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// Partial results per row that the arg-max kernels keep between their two stages.
int cw_argmax_chunks(int V);

// First index of the maximum of each of n float32 rows of V logits (rows row_stride floats apart)
// into out[n]. workspace: device memory of n * cw_argmax_chunks(V) * 8 bytes that the caller owns.
int cw_argmax(const float* logits, int64_t row_stride, int n, int V, int* out, void* workspace,
              int64_t workspace_bytes, hipStream_t stream);

// The same arg-max for callers that cannot allocate device memory: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference
// (whose arg-max is a library call that allocates its result). Inputs and outputs are the
// caller's; the partial results of the first stage go to a fixed array of
// CW_ARGMAX_STATIC_BYTES bytes inside the library instead of a workspace, of which every GPU the
// library runs on holds one copy until the process ends. The call allocates nothing and frees
// nothing (no hipMalloc, no hipFree, no allocating library routine).
//
//   * at most CW_ARGMAX_STATIC_MAX_ROWS rows a call: more returns CW_ERR_SIZE (-4) and launches
//     nothing;
//   * every call on a GPU uses that GPU's one array, which keeps the last call's contents: both
//     stages only read what the same call wrote, so nothing has to be cleared, but two calls that
//     overlap on one GPU (different streams, or two threads) race and must be ordered by the caller;
//   * the array's device address is looked up once per GPU, at the first call on that GPU or by
//     cw_argmax_static_init(), which a caller runs before a graph capture (the look-up itself is
//     not a stream operation). Both need that GPU to be the current device.
#define CW_ARGMAX_STATIC_MAX_ROWS 256
#define CW_ARGMAX_STATIC_BYTES (CW_ARGMAX_STATIC_MAX_ROWS * 64 * 8)
int cw_argmax_static_init(void);
int cw_argmax_static(const float* logits, int64_t row_stride, int n, int V, int* out, hipStream_t stream);

#ifdef __cplusplus
}
#endif
