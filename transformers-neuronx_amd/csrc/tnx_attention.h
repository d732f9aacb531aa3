// Entry points of the attention library that a caller may reach through its C interface without the
// Python backend. All return 0, or non-zero with a message under tnx_last_error().
#pragma once
#include <hip/hip_runtime.h>

// The largest set of partial results the static array of `tnx_attention_decode_static` holds, in floats
// (4 MiB on every GPU the library runs on, until the process ends):
// requests x heads x splits x (head_size + 2) must not exceed it.
#define TNX_DECODE_SCRATCH_FLOATS (1 << 20)

extern "C" {

// Attention of single decoded tokens over the paged cache (bfloat16). The keys of a (request, head) are
// split over `num_splits` blocks; with more than one split the partial results (float32 weighted values,
// maximum and sum) pass through the caller's workspace: `part_o` of requests x heads x splits x head_size
// floats and `part_ml` of requests x heads x splits x 2. `page_pad`: elements between the end of one page
// and the start of the next (0: the pages lie one behind the other).
int tnx_attention_decode(const void* q, const void* k_pages, const void* v_pages, const int* run_start,
                         const int* cached_lens, const int* table, int table_width, int page_size, int num_pages,
                         const int* decode_runs, int num_decode, void* out, float* part_o, float* part_ml,
                         int num_heads, int num_kv, int head_size, int window, int num_splits, int waves,
                         const int* longest, int page_pad, hipStream_t stream);

// The same without a workspace argument, for callers that cannot allocate: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. The partial
// results go through an array that the library holds in device memory; the call allocates and frees
// nothing, on the host or the device. Sizes beyond TNX_DECODE_SCRATCH_FLOATS are refused with a message.
// The array's address is looked up at the first call on each device (that call is best made outside a
// capture). Every call on a GPU shares that GPU's array: calls that overlap on one GPU, on different
// streams or from different threads, race; calls on one stream are safe. Nothing in the array has to be
// cleared between calls: each call writes every partial result before its merge reads it. The pages lie one
// behind the other (no distance between them).
int tnx_attention_decode_static(const void* q, const void* k_pages, const void* v_pages, const int* run_start,
                                const int* cached_lens, const int* table, int table_width, int page_size,
                                int num_pages, const int* decode_runs, int num_decode, void* out, int num_heads,
                                int num_kv, int head_size, int window, int num_splits, int waves,
                                const int* longest, hipStream_t stream);
}
