// C interface of libminiserve_hip.so for callers outside Python: the entry points
// that have no workspace arguments to size.  (The Python package declares every
// entry point's argument types itself, in ops/library.py.)
#pragma once

#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Message of the last entry point that returned non-zero on this thread.
const char* ms_last_error(void);

// Greedy tokens of float logits [rows, vocab] -> int32 out [rows]: the lowest index
// of the maximum, -1 for a row that holds a non-finite value.  chunk_max (float
// [rows, chunks]) and chunk_index (int32 [rows, chunks]) are partial results that the
// caller allocates; chunks is 1..64 and at most vocab.  Returns 0, or non-zero with
// a message in ms_last_error().
int ms_argmax_rows(const void* logits, void* chunk_max, void* chunk_index, void* out, int rows, int vocab,
                   int chunks, hipStream_t stream);

// The same choice for callers that cannot allocate: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc.  This entry point has no
// counterpart in the reference (its sampling runs in torch, which allocates as it
// goes).  It allocates nothing, neither with hipMalloc nor through any library: the
// partial results lie in a device array of the library itself (512 KiB on each GPU
// that the library runs on, held until the process ends), which takes at most 1024
// rows; more rows are refused with an error, as is anything else it cannot do.
// The caller passes logits and out as above and has the stream's device current.
// Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
// streams, two threads) race and give wrong tokens; calls on one stream do not.
// The array keeps the last call's contents; every entry that a call reads it has
// written before, so nothing is cleared.  The first call on a device asks the
// runtime for the array's address there (hipGetSymbolAddress) and must therefore
// not be made while a stream of that device is capturing; later calls may.
int ms_argmax_rows_static(const void* logits, void* out, int rows, int vocab, hipStream_t stream);

#ifdef __cplusplus
}
#endif
