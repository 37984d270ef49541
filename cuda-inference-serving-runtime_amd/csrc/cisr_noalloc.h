// Entry points that allocate nothing.
//
// This declaration has no counterpart in the reference.  It is for callers that cannot
// allocate device memory: code that runs under HIP graph capture, tight serving loops, and
// harnesses that forbid hipMalloc.  Such a caller passes inputs and outputs only; what the
// kernels need beyond them lives in a fixed array in the library's device image (one copy on
// every GPU the library runs on, held until the process ends).
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Most rows of logits that cisr_argmax_noalloc takes in one call.  The array behind it is
// CISR_ARGMAX_NOALLOC_MAX_ROWS x 32 slices x 8 bytes = 256 KiB on each GPU.
#define CISR_ARGMAX_NOALLOC_MAX_ROWS 1024

// Resolves the device address of the fixed array on the current device (hipGetSymbolAddress) and keeps
// it.  Optional: cisr_argmax_noalloc does the same at its first call on a device.  A caller that records
// a graph calls this once per device beforehand.  Returns 0 or a HIP error code.
int cisr_noalloc_init(void);

// The limit above, for callers that read it at run time.
int cisr_argmax_noalloc_max_rows(void);

// out[r] = index of the largest of logits[r, 0..vocab-1] (the lowest index wins a tie): the same two
// kernels and the same results as cisr_argmax without `index`, with the slice winners kept in the fixed
// array instead of buffers that the caller brings.  logits float [rows, vocab], out int32 [rows], both
// on the current device.  Calls no hipMalloc, hipFree or allocating library routine.
// rows > CISR_ARGMAX_NOALLOC_MAX_ROWS, rows < 0, vocab <= 0 or a null pointer: nothing is launched, a
// line that names the limit goes to stderr and hipErrorInvalidValue is returned.
// Every call on a GPU uses that GPU's one array (nothing in it has to start at zero: the first kernel
// writes every entry that the second reads), so calls that overlap on one GPU, on different streams or
// from different threads, race; calls on one stream are ordered and safe.
int cisr_argmax_noalloc(const float* logits, int* out, int rows, int vocab, hipStream_t stream);

#ifdef __cplusplus
}
#endif
