// Entry points of the gfx950 kernel library that allocate nothing.
//
// They have no counterpart in the reference.  They are for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  Every other entry point of the library takes
// the scratch memory its kernels need from the caller (who allocates it); these keep it in a static array in device
// memory instead, one copy per GPU, held until the process ends.
#pragma once

#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Most (rows x runs of 4096 logits) one call may ask for: gi_argmax_no_alloc needs 8 bytes of scratch for each, so the
// static array is GI_NO_ALLOC_ARGMAX_MAX_PARTS * 8 bytes = 512 KiB per GPU.  128 rows of a 2,000,000-token vocabulary fit,
// or 2,048 rows of Llama's 128,256.
#define GI_NO_ALLOC_ARGMAX_MAX_PARTS 65536

// Set-up, once per device with that device current: finds the address of this GPU's copy of the static scratch array.
// gi_argmax_no_alloc does the same at its first call on a device; a caller that must not make its first call inside a
// graph capture calls this before.  Returns 0, or -1 with the text in gi_last_error().
__attribute__((visibility("default"))) int gi_no_alloc_prepare(void);

// out[r] = the lowest index of the largest of logits[r, 0 .. vocab) for r < n_rows; float32 logits with row stride
// `stride`, int32 out.  The result is gi_argmax's (the same kernels), without a scratch argument.
// Refuses n_rows * ceil(vocab / 4096) > GI_NO_ALLOC_ARGMAX_MAX_PARTS with a message.  Calls no hipMalloc, hipFree or
// other allocating routine.  All calls on one GPU share that GPU's scratch array: the kernels write every element of it
// that they later read, so nothing has to be cleared between calls, but two calls that overlap in time on one GPU (on
// different streams, or from different threads) race and give wrong tokens; calls on one stream are ordered and safe.
__attribute__((visibility("default"))) int gi_argmax_no_alloc(const float* logits, int* out, int n_rows, int vocab, long stride, hipStream_t stream);

#ifdef __cplusplus
}
#endif
