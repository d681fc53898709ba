// Entry points that allocate nothing.
//
// For callers that cannot allocate device memory around a call: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// Status of a call whose partial results do not fit the static scratch array.
#define DLI_ERR_SCRATCH -3

// Size of the static scratch array in floats (8 MiB), held by each GPU that the library runs on
// until the process ends.
#define DLI_STATIC_SCRATCH_FLOATS (2 * 1024 * 1024)

extern "C" {

// Floats of scratch that dli_attention_decode_bf16_static needs for these sizes (0 for one split):
// requests * q_heads * splits * head_dim partial outputs, rounded up to 64, and two statistics
// per (request, head, split).
int64_t dli_attention_decode_static_floats(int requests, int q_heads, int head_dim, int splits);

// dli_attention_decode_bf16 (paged decode attention with the keys of each request cut into
// `splits` runs and a merge kernel) without the caller's partial-result buffers: they live in a
// file-scope device array of DLI_STATIC_SCRATCH_FLOATS floats. Calls no hipMalloc, hipFree or
// allocating library routine; inputs and `out` are the caller's. Same kernels, same results.
// Returns DLI_ERR_SCRATCH if dli_attention_decode_static_floats(...) exceeds the array,
// DLI_ERR_ARGUMENT for sizes that the kernels do not take, DLI_ERR_LAUNCH if the array's address
// on the current device cannot be found or a launch is refused.
// Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
// threads) race; calls on one stream are ordered. The array keeps the last call's contents and
// nothing in it has to start at zero.
int dli_attention_decode_bf16_static(const void* q, int64_t q_stride, const void* k_pages,
                                     const void* v_pages, void* out, int64_t out_stride,
                                     const int* kv_len, const int* block_tables, int table_stride,
                                     int requests, int q_heads, int kv_heads, int head_dim,
                                     int page_size, float scale, int window, int splits,
                                     hipStream_t stream);
}
