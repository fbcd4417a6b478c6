// The one entry point of the kernel library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory
// around a call: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
// Every other entry point that needs device memory beyond its inputs and outputs takes it from the
// caller as a workspace argument (which the caller had to allocate); this one keeps that memory in
// a file-scope __device__ array of a fixed, modest size instead.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// The (row, part) pairs the array holds: rows * ceil(vocab / 8192) of a call may not exceed this.
// 8 bytes a pair: 128 KB on every GPU the library runs on, held until the process ends.
#define ZI_ARGMAX_STATIC_MAX_PARTS 16384

// zi_argmax (the index of the highest value of each row, the lowest index among equals, and optionally
// the value) for rows long enough to be cut over several workgroups, with the parts' results kept in
// the library's own array instead of a workspace.  Same arguments as zi_argmax without the workspace;
// the device the tensors live on must be current.  Returns non-zero, with a message for
// zi_last_error(), when rows * ceil(vocab / 8192) exceeds ZI_ARGMAX_STATIC_MAX_PARTS.  It calls no
// hipMalloc, hipFree or allocating library routine.
//
// All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two
// threads) race on it; calls on one stream are ordered by the stream.  The array keeps the last call's
// contents; nothing in it has to start at zero, every part that is read has been written by the same
// call.
extern "C" int zi_argmax_static(int32_t* out_idx, float* out_val, const void* logits, int dt, int rows, int vocab,
                                int64_t ld, hipStream_t stream);

// ZI_ARGMAX_STATIC_MAX_PARTS, for callers that do not read this header.
extern "C" int zi_argmax_static_max_parts();
