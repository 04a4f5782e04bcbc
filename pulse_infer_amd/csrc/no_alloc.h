// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  Such a caller cannot bring the workspace
// that pulse_argmax asks for, so this variant keeps the chunk winners of its first stage in an array that lives in
// the library's own device image.
//
// pulse_argmax_static: out[r] = index of the largest logit of row r, the lowest index among equals, -1 if no entry
// of the row is a number: the result of pulse_argmax, from the same two kernels.
//
// * Limit: rows * pulse_argmax_chunks(vocab) <= PULSE_ARGMAX_STATIC_ENTRIES (65,536 pairs of a float and an int,
//   512 KiB, which every GPU the library runs on holds until the process ends).  At a vocabulary of 151,936
//   (75 chunks) that is 873 rows.  Larger inputs are refused with an error and nothing is launched.
// * The first call on a device looks up the array's address there (hipGetSymbolAddress, once per device, under a
//   lock); make that call outside a graph capture.  Later calls launch two kernels on `stream` and call no
//   allocating routine.
// * Every call on a GPU shares that GPU's array.  Calls on one stream follow each other and are safe; calls that
//   overlap on one GPU (two streams, two threads) race on the array and may return either call's winners.  Nothing
//   in the array has to start at zero: the first kernel writes every entry that the second one reads.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define PULSE_ARGMAX_STATIC_ENTRIES 65536

extern "C" int pulse_argmax_static(const float* logits, int rows, int vocab, int64_t row_stride, int* out,
                                   hipStream_t stream);
