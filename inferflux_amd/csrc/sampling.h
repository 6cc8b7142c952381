// Entry points of the sampling library that callers outside this package may link against.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

// Rows and slices the static scratch of ifx_argmax_static is sized for: 1,024 rows of 32 slices, a float and an int
// each = 256 KiB of device memory per GPU the library runs on, held until the process ends.
#define IFX_ARGMAX_STATIC_MAX_ROWS 1024

// Lowest index of the maximum of each row of float32 logits [R, V] into out [R] (int32), as ifx_argmax gives it, on
// `stream` (a hipStream_t).  This one has no counterpart in the reference.  It is for callers that cannot allocate: code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  ifx_argmax takes its two-stage
// scratch (the best of each of 32 slices of every row) from the caller as a workspace; this entry point keeps it
// in a file-scope device array instead, looked up once per device, and calls no allocator of any kind.
//
//  * R must be at most IFX_ARGMAX_STATIC_MAX_ROWS: more rows are refused (-1, text from ifx_last_error()), never
//    truncated.
//  * Every call on a GPU uses that GPU's one array, which keeps the last call's contents.  Nothing in it has to
//    start at zero: stage one writes every slot that stage two reads for the R rows of the call.
//  * Calls that overlap on one GPU (two streams, two threads) race on the array: serialise them.
//  * Inputs and outputs are the caller's: logits and out must be device memory of the current device.
int ifx_argmax_static(const float* logits, int R, int V, int* out, void* stream);

#ifdef __cplusplus
}
#endif
