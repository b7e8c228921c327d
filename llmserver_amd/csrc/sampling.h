// Entry points of the sampling library (sampling.hip), for callers that load it without Python.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// Chunks a row of `vocab` logits is cut into (at most 64).
int lsa_sample_chunks(int vocab);

// One token per row of float32 `logits [n_rows, vocab]`: the first maximum where `temperature[row]` is 0, else the
// inverse of the cumulative distribution of softmax(logits / temperature) at `uniform[row]`.
// `workspace`: device memory of n_rows * lsa_sample_chunks(vocab) * 16 bytes that the caller brings.
int lsa_sample(const float* logits, const float* temperature, const float* uniform, int* out, void* workspace, int n_rows,
               int vocab, hipStream_t stream);

// The same result as lsa_sample, without a workspace argument and without allocating anything.
//
// This entry point has no counterpart in the reference.  It is for callers that cannot allocate device memory: code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The per-chunk statistics that
// lsa_sample keeps in the caller's workspace lie in a fixed array in the library's device image instead
// (LSA_SAMPLE_STATIC_MAX_ROWS * 64 chunks * 16 bytes = 1 MiB, held by every GPU the library runs on until the
// process ends).  Its address on the current device is looked up once per device, at the first call on that device;
// that first call should therefore come before a capture starts.
//
// Rows beyond LSA_SAMPLE_STATIC_MAX_ROWS are refused with LSA_SAMPLE_STATIC_TOO_MANY_ROWS and nothing is launched
// (lsa_sample_static_error gives the text for a code).  Every call on a GPU uses that GPU's one array: each call
// writes every entry it reads later, so nothing has to be cleared between calls, but two calls whose kernels
// overlap on one GPU (different streams, or graphs replayed concurrently) race on it.  Calls on one stream are safe.
#define LSA_SAMPLE_STATIC_MAX_ROWS 1024
#define LSA_SAMPLE_STATIC_TOO_MANY_ROWS (-2)
#define LSA_SAMPLE_STATIC_BAD_DEVICE (-3)
int lsa_sample_static(const float* logits, const float* temperature, const float* uniform, int* out, int n_rows, int vocab,
                      hipStream_t stream);
int lsa_sample_static_max_rows(void);
const char* lsa_sample_static_error(int code);

#ifdef __cplusplus
}
#endif
