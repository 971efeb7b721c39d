// Entry points for callers that cannot allocate device memory.
//
// tk_argmax_no_alloc has no counterpart in the reference.  It is for callers that
// cannot call hipMalloc: code under HIP graph capture, tight serving loops,
// harnesses that forbid allocation.  It computes what tk_argmax computes with
// the same kernels, but keeps the per-segment winners (the scratch that tk_argmax
// takes as `part_v`, `part_i`) in a fixed array inside the library instead of a
// buffer that the caller brings.
//
//   * The array holds TK_ARGMAX_NO_ALLOC_MAX_ROWS rows (256 KiB; every GPU the
//     library runs on holds it until the process ends).  More rows are refused
//     with status -3 and nothing is launched.
//   * It allocates nothing: no hipMalloc, hipFree or allocating library call.
//     The first call on a device looks the array's address up once
//     (hipGetSymbolAddress, with that device current) and keeps it per device.
//   * Every call on a GPU shares that GPU's array and the array keeps the last
//     call's contents.  Nothing in it has to start at zero: each launch writes
//     every entry it later reads.  Two calls that overlap on one GPU (two
//     streams, two threads) race on the array: order them on one stream.
//   * The device of `stream` must be the current device.
//
// Status: 0 ok; -1 bad sizes; -3 more than TK_ARGMAX_NO_ALLOC_MAX_ROWS rows;
// -4 the array's address could not be found; else a HIP error code of the launch.
#pragma once

#include <hip/hip_runtime.h>

#define TK_ARGMAX_NO_ALLOC_MAX_ROWS 1024

extern "C" __attribute__((visibility("default"))) int tk_argmax_no_alloc(
    const float* logits,  // [M, V] float32, rows `ld` floats apart
    int* out,             // [M] index of the first maximum of each row
    float* out_value,     // [M] the maxima, or nullptr
    int M, int V, long ld, hipStream_t stream);

extern "C" __attribute__((visibility("default"))) int tk_argmax_no_alloc_max_rows();
