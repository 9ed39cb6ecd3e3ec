// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// ri_argmax_no_alloc is ri_argmax (sampling.hip) without the caller's scratch buffer: the slice
// maxima that the first kernel leaves for the second lie in a file-scope device array of
// RI_ARGMAX_NO_ALLOC_MAX_ROWS * 64 * 8 bytes (512 KiB; every GPU the library runs on holds its own
// copy until the process ends).  The caller still passes the logits and the output.  The call
// makes no hipMalloc, hipFree or allocating library call; rows beyond the maximum are refused
// with an error, as is a row count of more than 65535.  Nothing in the array has to start at
// zero: every word the second kernel reads is written by the first kernel of the same call.
// All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two
// host threads) race, and the caller must order them.
//
// ri_no_alloc_init looks the array's device address up for the current device
// (hipGetSymbolAddress, once a device); a caller that must not make even that call later, such
// as one under graph capture, calls it at set-up, with each device it uses current in turn.
// ri_argmax_no_alloc does the same at its first call on a device.
#pragma once
#include <hip/hip_runtime.h>

#define RI_ARGMAX_NO_ALLOC_MAX_ROWS 1024

extern "C" int ri_no_alloc_init();
extern "C" int ri_argmax_no_alloc_max_rows();
extern "C" int ri_argmax_no_alloc(const float* logits, int rows, int V, int ld, int* out, hipStream_t stream);
