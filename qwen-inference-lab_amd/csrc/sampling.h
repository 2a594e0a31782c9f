// C interface of the next-token choice (sampling.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

// Bytes of scratch memory qil_sample needs for `rows` rows of `vocab` logits.
size_t qil_sample_workspace(int rows, int vocab);

// tokens[r], finite[r] from logits[r, :]: greedy where temperatures[r] == 0 (lowest index on ties), else a seeded
// Gumbel-max draw keyed by (seeds[r], counters[r]).  `workspace`: qil_sample_workspace(rows, vocab) bytes of device
// memory.  Returns 0, a HIP error code (> 0), or -1 for sizes it does not take.
int qil_sample(const float* logits, const float* temperatures, const int* seeds, const int* counters, int* tokens,
               int* finite, void* workspace, int rows, int vocab, hipStream_t stream);

// Most (row, 4096-logit chunk) cells of qil_sample_static: rows * ceil(vocab / 4096) may not exceed it.
#define QIL_SAMPLE_STATIC_CELLS 65536

// qil_sample without a workspace argument and without any allocation: the same two kernels, with their scratch
// memory in an array of QIL_SAMPLE_STATIC_CELLS * 12 bytes (768 KiB) that is part of the library's device image (every
// GPU the library runs on holds its own copy from load to process end).  This entry point has no counterpart in the
// reference; it is for callers that cannot allocate device memory: code inside a HIP graph capture, serving loops that
// must not touch the allocator, harnesses that forbid hipMalloc.  It calls no hipMalloc, hipFree or allocating
// library routine.  The first call on a device looks the array's address up (hipGetSymbolAddress) and keeps it;
// qil_sample_static_prepare() does only that, for callers that want it done before, say, a capture begins.
// Returns 0, a HIP error code (> 0), -1 for a size qil_sample refuses, or -2 if rows * ceil(vocab / 4096) exceeds
// QIL_SAMPLE_STATIC_CELLS.
// All calls on one GPU share that GPU's array: calls that may overlap there (different streams, different threads)
// race and must be ordered by the caller.  Nothing in the array has to start at zero, and nothing is cleared: the
// first kernel writes every cell that the second reads, so what an earlier, larger call left is never seen.
int qil_sample_static(const float* logits, const float* temperatures, const int* seeds, const int* counters,
                      int* tokens, int* finite, int rows, int vocab, hipStream_t stream);
int qil_sample_static_prepare(void);

#ifdef __cplusplus
}
#endif
