// C interface of the sampling library (libtl_sampling.so).
//
// Every entry point returns 0 on success, else an error code whose text tl_last_error()
// gives; launches go to `stream` of the device that is current in the calling thread.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Chunks a row of `vocab` columns is scanned in (at most TL_SAMPLE_MAX_CHUNKS).
#define TL_SAMPLE_MAX_CHUNKS 128
int tl_sample_chunks(int vocab);

// One token per row of float32 logits [rows, vocab] (row stride ld): arg max where the row's
// temperature is 0 (or `temperature` is null), else a Gumbel-max draw keyed by keys[row].
// `scratch`: device memory of the caller, rows * tl_sample_chunks(vocab) * 8 bytes.
int tl_sample(const void* logits, int rows, int vocab, int ld, const void* temperature,
              const void* keys, void* out, void* scratch, hipStream_t stream);

// The same draw for callers that cannot allocate device memory: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference
// (whose sampling is a library arg max that allocates its result).  The candidates of the scan
// go through an array that the library itself holds in device memory, TL_SAMPLE_STATIC_MAX_ROWS *
// TL_SAMPLE_MAX_CHUNKS * 8 bytes (256 KiB) on every GPU the library is used on, until the
// process ends; the caller brings inputs and the output only.  More rows than
// TL_SAMPLE_STATIC_MAX_ROWS are refused.  It calls no hipMalloc, hipFree or allocating library
// routine.  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
// streams, two threads) race; calls on one stream are safe.  Nothing in the array has to start
// at zero: each call writes every candidate it reads.
#define TL_SAMPLE_STATIC_MAX_ROWS 256
int tl_sample_static(const void* logits, int rows, int vocab, int ld, const void* temperature,
                     const void* keys, void* out, hipStream_t stream);

#ifdef __cplusplus
}
#endif
