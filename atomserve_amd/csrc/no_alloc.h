// An entry point for callers that cannot allocate device memory.
//
// It has no counterpart in the reference (aneesh-sathe/atomserve), whose kernels always
// receive scratch tensors that PyTorch allocated for the call.  It is for callers that
// cannot call hipMalloc (or an allocating library routine, torch's included) at the moment
// they need attention over the paged cache: code under HIP graph capture, tight serving
// loops, and harnesses that forbid allocation.
#pragma once
#include <hip/hip_runtime.h>

// Floats of the library's own scratch array: 8 MiB, held by every GPU the library runs on
// until the process ends.
#define AS_STATIC_SCRATCH_FLOATS (2u << 20)

// The entry point refuses a call whose partial results do not fit the scratch array.
#define AS_TOO_LARGE -4

extern "C" {

// as_attn_single_query with the partial results of a split context (part_m, part_l, part_acc)
// kept in the library's own scratch array instead of buffers the caller brings.  Same kernels,
// same arguments otherwise, same results.
//
//   needs  num_items * H * P * (D + 2) floats  <=  AS_STATIC_SCRATCH_FLOATS   (P > 1 only),
//   else returns AS_TOO_LARGE and launches nothing.
//
// Allocates nothing and frees nothing.  The array's device address is looked up once per
// device, at the first call on that device (hipGetSymbolAddress), which should therefore
// come before any graph capture.  All calls on one GPU share that GPU's array: calls that
// overlap on one GPU (two streams, two threads) race on it; calls on one stream do not.  The
// array keeps the last call's contents; the kernels write every element they later read, so
// nothing has to be cleared between calls.
int as_attn_single_query_static(const void* q, const void* k_pages, const void* v_pages, int dtype,
                                const int* items, int num_items, const int* positions, const int* tok_row,
                                const int* block_tables, int table_width, void* out, int H, int KV, int D,
                                int bs, float scale, int window, int part_size, int P, hipStream_t stream);
}
