// The one entry point of this library that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot call
// hipMalloc: code that runs under HIP graph capture, tight serving loops that
// must never stall on the allocator, and harnesses that forbid allocation.
//
// cie_argmax_static is cie_argmax (csrc/sampling.hip: the first index of each
// row's largest float32 logit, in two stages) with the partial results of its
// first stage kept in a fixed array of device memory that the library itself
// holds, instead of in a workspace the caller brings.  The caller passes only
// the logits and the output.
//
//   logits  float32 [rows, ld], vocab <= ld numbers used of each row
//   out     int32 [rows]
//   chunk   numbers of a row that one workgroup of the first stage scans
//
// Limits: rows * ceil(vocab / chunk) <= CIE_ARGMAX_STATIC_MAX_ENTRIES (and the
// rows <= 65535 of cie_argmax).  Beyond that the call launches nothing and
// returns CIE_TOO_LARGE.  The array takes CIE_ARGMAX_STATIC_MAX_ENTRIES * 8
// bytes (128 KB) on every GPU the library runs on, from the library's load to
// the end of the process.
//
// Every call on a GPU uses that GPU's one array: calls that overlap on one GPU
// (two streams, two threads) race and give wrong tokens; calls on one stream,
// or ordered by events, do not.  Nothing in the array has to start at zero:
// each call's first stage writes every entry that its second stage reads, so
// what the call before left there is never seen.
//
// The array's address on a device is looked up once, at the first call with
// that device current (hipGetSymbolAddress; no allocation).  A failure of that
// lookup returns CIE_SETUP_FAILED.
#pragma once

#include "common.h"

#define CIE_ARGMAX_STATIC_MAX_ENTRIES 16384

CIE_API int cie_argmax_static(void* stream, const float* logits, int* out, int rows, int vocab, int ld, int chunk);
