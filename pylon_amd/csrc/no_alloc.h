// Entry points that allocate nothing.
//
// They have no counterpart in the reference engine.  They are for callers that cannot
// allocate device memory: code under HIP graph capture, tight serving loops, harnesses that
// forbid hipMalloc.  Where the ordinary entry point takes a scratch buffer from its caller,
// these use a fixed array in device memory that belongs to the library (each GPU the library
// runs on holds its own copy until the process ends) and refuse sizes beyond it.
#pragma once

#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Most rows pylon_argmax_static takes: its scratch array holds 64 partial results of 8
// bytes per row, 128 KiB in all.
#define PYLON_ARGMAX_STATIC_MAX_ROWS 256

// Resolves the address of the scratch array on the current device (once per device; later
// calls return at once).  pylon_argmax_static does this itself on its first call on a
// device; a caller that must not make even that runtime query later (under graph capture)
// calls this beforehand.  0, or 1 with the reason in pylon_last_error().
int pylon_argmax_static_init(void);

// As pylon_argmax (out[r] = index of the largest of logits[r, 0..vocab), the lowest among
// equals; with chosen and place also chosen[place[r]] = that index), but the partial
// results of its first launch live in the library's own array: no scratch argument, no
// allocation.  Refuses rows > PYLON_ARGMAX_STATIC_MAX_ROWS.  Every call on a GPU shares that
// GPU's array: calls that overlap on one GPU (different streams) race; calls on one stream
// do not.  Nothing in the array has to start at zero: each call overwrites what it reads.
int pylon_argmax_static(int* out, const float* logits, int rows, int vocab, long long row_stride,
                        int* chosen, const int* place, hipStream_t stream);

#ifdef __cplusplus
}
#endif
