// C entry points of sampling.hip: choosing next tokens from rows of float logits
// (greedy; temperature / top-k with the law of the reference's generate.py:40-57).
// All take device pointers and a stream and return a hipError_t as an int.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// One workgroup per row (small vocabularies).
int gfa_argmax(const float* logits, int* out, int n_rows, int V, size_t row_stride,
               hipStream_t stream);
int gfa_sample(const float* logits, size_t row_stride, int n_rows, int V, float temperature,
               int top_k, uint64_t seed, const uint32_t* seed_dev, const int* row_keys,
               const int* positions, int position_offset, int* out, float* probs_out,
               hipStream_t stream);

// A row spread over many workgroups (large vocabularies).  `workspace` holds
// gfa_sample_split_workspace(n_rows, V) bytes whose first n_rows * 4096 bytes are zero at
// the first call; the kernels leave them zero again.  temperature <= 0: greedy.
size_t gfa_sample_split_workspace(int n_rows, int V);
int gfa_sample_split(const float* logits, size_t row_stride, int n_rows, int V, float temperature,
                     int top_k, uint64_t seed, const uint32_t* seed_dev, const int* row_keys,
                     const int* positions, int position_offset, int* out, float* probs_out,
                     void* workspace, hipStream_t stream);

// The same as gfa_sample_split for callers that cannot allocate device memory: code under
// HIP graph capture, serving loops and harnesses that forbid hipMalloc.  It has no
// counterpart in the reference (whose sampler, generate.py:40-57, allocates through torch
// at every call).  It allocates nothing and calls no allocating routine: the workspace is
// a fixed array inside the library, GFA_SAMPLE_STATIC_BYTES per GPU, held from the
// library's load until the process ends, which bounds the input to
// GFA_SAMPLE_STATIC_MAX_ROWS rows of at most GFA_SAMPLE_STATIC_MAX_VOCAB logits; beyond
// that it returns hipErrorInvalidValue and gfa_sampling_last_error() says why.  The caller
// still passes inputs and outputs.  Every call on a GPU uses that GPU's one array, which
// keeps what the last call left: the part that must start at zero is cleared by a kernel
// at the start of every call, and calls that overlap on one GPU (two streams, two
// threads) race - run them one after another.
// The array's device address is looked up once per GPU, at the first call on it or by
// gfa_sampling_init(), which a caller that records graphs calls beforehand, with the GPU
// current, so that the look-up is not part of a recording.
#define GFA_SAMPLE_STATIC_MAX_ROWS 64
#define GFA_SAMPLE_STATIC_MAX_VOCAB 262144
#define GFA_SAMPLE_STATIC_BYTES (GFA_SAMPLE_STATIC_MAX_ROWS * (4 * 256 + 2 + 4 * (GFA_SAMPLE_STATIC_MAX_VOCAB / 4096)) * 4)
int gfa_sampling_init(void);
int gfa_sample_split_static(const float* logits, size_t row_stride, int n_rows, int V,
                            float temperature, int top_k, uint64_t seed,
                            const uint32_t* seed_dev, const int* row_keys, const int* positions,
                            int position_offset, int* out, float* probs_out, hipStream_t stream);
// Text of the last refusal of an entry point above on the calling thread ("" if none).
const char* gfa_sampling_last_error(void);

#ifdef __cplusplus
}
#endif
