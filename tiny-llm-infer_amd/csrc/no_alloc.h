// An entry point that allocates nothing.
//
// It has no counterpart in the reference.  It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  tli_sample needs a scratch buffer (the best score and token id of each of the
// pieces a row of logits is cut into) and takes it as an argument, which its caller has to
// allocate; tli_sample_no_alloc is the same operation with that buffer in a file-scope
// device array of the library.
//
//   int tli_sample_no_alloc(logits, rows, vocab, temperatures, seeds, top_p, out, stream)
//
// Arguments and result are those of tli_sample without `scratch`.  The caller still passes
// inputs and outputs.  It calls no hipMalloc, hipFree or allocating library routine; at its
// first call on a device it asks once for the address of that device's copy of the array.
// That first query must not fall inside a stream capture: before recording the entry point
// into a HIP graph, call tli_sample_no_alloc_prepare() (or the entry point itself, eagerly)
// once on that device, with that device current.
//
// Limit: rows <= TLI_SAMPLE_NO_ALLOC_MAX_ROWS (more is refused with an error, nothing
// launched).  The array takes 256 KiB on every GPU the library runs on until the process ends.
//
// Every call on a GPU uses that GPU's one array, which keeps the last call's contents; a
// call overwrites every entry it reads later, so nothing is cleared.  Two calls that overlap
// on one GPU (different streams, or different threads without an order between them) race
// for the array: give them an order.
#pragma once
#include <stdint.h>

#define TLI_SAMPLE_NO_ALLOC_MAX_ROWS 1024

extern "C" int tli_sample_no_alloc(const float* logits, int rows, int vocab, const float* temperatures,
                                   const uint32_t* seeds, const float* top_p, int* out, void* stream);
extern "C" int tli_sample_no_alloc_max_rows();
extern "C" int tli_sample_no_alloc_prepare();
