// The one entry point of the kernel libraries that allocates nothing.
//
// It has no counterpart in the reference (axonn-ai/yalis lets torch allocate whatever a
// call needs).  It is for callers that cannot allocate device memory: code that runs while
// a HIP graph is being captured, tight serving loops, and harnesses that forbid hipMalloc.
//
// yk_argmax_static computes what yk_argmax computes (per row the index of the largest
// logit, the lowest index on ties; a row without any finite-or-infinite winner gives 0), with
// the same two kernels, but the per-slice partial results that yk_argmax keeps in a
// caller-supplied workspace live in a file-scope device array of the library instead
// (sampling.hip: yk_static_scratch, YK_ARGMAX_STATIC_MAX_ROWS rows x 32 slices x (float, int32)
// = 256 KiB; every GPU the library runs on holds its own copy until the process ends).
// The caller passes inputs and outputs only.
//
//  * Rows beyond YK_ARGMAX_STATIC_MAX_ROWS are refused (return -1, yk_last_error() says why);
//    nothing is launched then.
//  * No hipMalloc, hipFree or allocating library routine is called.  The array's device address
//    is looked up once per device with hipGetSymbolAddress: by yk_argmax_static_setup() (call it
//    on each device before a capture or a loop that must not do that lookup), else by the first
//    call of yk_argmax_static on that device.
//  * `stream` must be a stream of the device that is current at the call.
//  * Every call on one GPU uses that GPU's one array, which keeps the last call's contents.
//    Nothing in it has to start at zero: the first kernel writes every partial result that the
//    second reads.  Calls that overlap on one GPU (two streams, two threads) race on it: keep
//    them in stream order or serialise them.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define YK_ARGMAX_STATIC_MAX_ROWS 1024

extern "C" {
// Looks up this device's copy of the scratch array (idempotent).  0 on success, -1 on error.
int yk_argmax_static_setup(void);
// out[r] = argmax of logits[r, 0 .. vocab) for r < n_rows (float32, contiguous rows).
// 0 on success, -1 on error (bad sizes, more than YK_ARGMAX_STATIC_MAX_ROWS rows, a failed launch).
int yk_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, hipStream_t stream);
}
