// An entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory: code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
#pragma once

#include <stdint.h>

extern "C" {

// Lowest index of each row's maximum (logits float32 [n_rows, vocab], out int32 [n_rows]): what bc4g_argmax
// computes, without its workspace arguments.  The slices' bests go through an array of the library's own
// (512 KiB on every GPU the library runs on, held until the process ends); the call allocates nothing and
// calls no allocating routine.  At most bc4g_argmax_static_max_rows() = 1024 rows a call; more is refused
// with an error that says so (bc4g_last_error).  All calls on one GPU share the array, which keeps the last
// call's contents (nothing in it has to start at zero): calls that overlap on one GPU -- on different
// streams, or from different threads -- race.  The first call on a device asks the runtime for the array's
// address there; a caller that captures graphs makes one call outside a capture first.
// Returns 0 on success.
int bc4g_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, void* stream);
int bc4g_argmax_static_max_rows();

}  // extern "C"
