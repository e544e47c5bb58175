// The one entry point of this library that neither takes a workspace nor allocates one.
//
// It has no counterpart in the reference. It is for callers that cannot allocate device
// memory: code that runs under HIP graph capture, tight serving loops, and harnesses that
// forbid hipMalloc. Every other launcher takes its workspace from the caller.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// The most rows a call may bring. The two-stage argmax keeps 64 (value, id) pairs a row between
// its stages: 1,024 rows x 64 pairs x 8 bytes = 512 KiB of device memory, which every GPU the
// library runs on holds from the library's load until the process ends.
#define LIYAB_ARGMAX_STATIC_MAX_ROWS 1024

extern "C" {

// Looks up, for the current device, the address of the library's own scratch array (a
// file-scope __device__ array in sampling.hip) and keeps it. Done once a device; later calls
// return at once. liyab_argmax_static calls it by itself at its first call on a device; a
// caller that will record that entry point into a graph calls it once before the capture.
// Returns 0, or a code with a message for liyab_last_error().
int liyab_argmax_static_init(void);

// out[r] = the first maximal element of logits[r] (ties go to the lowest id), r in [0, rows):
// what liyab_argmax computes, by the same two kernels, with the pairs between the stages in
// the library's own scratch array instead of a caller's workspace. logits: float32 [rows, ld],
// ld >= V. With scatter_index, row r's token also goes to scatter_out[scatter_index[r]].
// Calls no hipMalloc, hipFree or other allocating routine. rows beyond
// LIYAB_ARGMAX_STATIC_MAX_ROWS are refused. Nothing in the array has to start at zero: the first
// stage writes every pair the second reads. All calls on one GPU share that GPU's array: calls
// that overlap in time on one GPU (two streams, two threads) race; calls on one stream, or
// ordered by events, do not.
int liyab_argmax_static(int* out, const float* logits, int64_t ld, int rows, int V, const int* scatter_index,
                        int* scatter_out, hipStream_t stream);

}
