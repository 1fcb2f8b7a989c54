// An entry point that allocates nothing.
//
// It has no counterpart in the reference. It is for callers that cannot allocate device memory:
// code that runs while a HIP graph is being captured, tight serving loops, harnesses that forbid
// hipMalloc. `distie_argmax` takes its two-stage scratch (the best value and index of every piece of
// every row) from the caller, who has to allocate it; `distie_argmax_static` computes the same result with
// the same kernels and keeps that scratch in a file-scope device array of fixed size, so the caller
// passes inputs and outputs only.
//
//   logits  float32 [rows, vocab] on the current device
//   out     int32 [rows]: index of the largest logit of each row, lowest index among equals
//   stream  the stream to launch on
//
// Returns 0 when launched, a hipError_t (> 0) when a HIP call failed, DISTIE_BAD_ARGUMENT (-1) for
// rows < 0 or vocab <= 0, and DISTIE_TOO_LARGE (-2) when rows exceeds DISTIE_ARGMAX_STATIC_MAX_ROWS or
// the pieces of all rows together exceed DISTIE_ARGMAX_STATIC_ENTRIES. `distie_argmax_static_limits`
// reports both numbers.
//
// The array (DISTIE_ARGMAX_STATIC_ENTRIES * 8 bytes = 8 KiB) exists once on every GPU the library runs
// on and stays until the process ends. Its address on a device is looked up once, by
// `distie_argmax_static_prepare` (with that device current) or by the first call of
// `distie_argmax_static` on the device. The lookup is no stream operation and must not happen while a
// stream captures: a caller that captures calls `distie_argmax_static_prepare` (or the entry point
// itself once, eagerly) on the device first; `distie_argmax_static` on a capturing stream of a device
// that was not prepared launches nothing and returns hipErrorStreamCaptureUnsupported. Every call on a GPU uses that GPU's one array, which keeps what the last call left: nothing
// in it has to start at zero, since a call writes every entry before it reads it; but two calls that
// overlap on one GPU (different streams, or threads) race on it. Calls that follow each other on one
// stream are safe.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define DISTIE_TOO_LARGE (-2)
#define DISTIE_ARGMAX_STATIC_ENTRIES 1024
#define DISTIE_ARGMAX_STATIC_MAX_ROWS 1024

extern "C" int distie_argmax_static(const float* logits, int32_t* out, int rows, int vocab, hipStream_t stream);
extern "C" int distie_argmax_static_prepare(void);      // 0, or a hipError_t
extern "C" void distie_argmax_static_limits(int* max_rows, int* max_entries);
