// C interface of the sampling library (sampling.hip).
#pragma once
#include <hip/hip_runtime.h>

extern "C" {

// Into how many chunks a vocabulary of V entries is cut; sa_sample's scratch arrays hold
// R * sa_sample_chunks(V) entries each.
int sa_sample_chunks(int V);

// One token per row of fp32 logits [R, V] into out[R]: argmax where temperature is null or 0,
// else argmax(logits / T - log q) with q from the row's key.  part_v (float) and part_i (int)
// are scratch arrays of R * sa_sample_chunks(V) entries that the caller allocates.
int sa_sample(const float* logits, const float* temperature, const unsigned long long* keys, int* out,
              float* part_v, int* part_i, int R, int V, hipStream_t stream);

// sa_sample for callers that cannot allocate device memory (code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
// The same kernels as sa_sample; the
// per-chunk partial results lie in an array that the library holds on every GPU it runs on
// (SA_SAMPLE_NOALLOC_ENTRIES entries of 8 bytes, 512 KiB, kept until the process ends) instead of
// in arrays the caller brings.  The call allocates nothing and frees nothing.
//   Limit: R * sa_sample_chunks(V) <= SA_SAMPLE_NOALLOC_ENTRIES, else SA_ERR_ARG (-1) and nothing runs.
//   Every entry the second kernel reads is written by the first one of the same call, so nothing
//   has to be cleared between calls.  All calls on one GPU share that GPU's array: calls that
//   overlap on one GPU (different streams, or threads) race; calls on one stream are ordered.
//   The first call on a device looks up the array's address there; hipError_t of that lookup is
//   returned as a positive code if it fails.
#define SA_SAMPLE_NOALLOC_ENTRIES 65536
int sa_sample_noalloc(const float* logits, const float* temperature, const unsigned long long* keys, int* out,
                      int R, int V, hipStream_t stream);

// The limit above, for callers that size their batches by it.
int sa_sample_noalloc_max_entries(void);

}  // extern "C"
