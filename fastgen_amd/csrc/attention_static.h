// Decode attention for callers that cannot allocate.
//
// fg_attn_decode_static has no counterpart in the reference (facebookresearch/fastgen calls a
// library's attention, which brings its own work space).  It is for callers that cannot call
// hipMalloc: code under HIP graph capture, tight serving loops, harnesses that forbid allocation.
// It runs what fg_attn_plan + fg_attn_split run (plan, split and combine kernels, the same ones),
// but the plan and the chunks' partial results (max, sum, O), for which the other entry points take
// buffers from the caller, live in one file-scope device array of FG_ATTN_STATIC_BYTES per GPU and
// per loaded library (one library a head size).  It allocates nothing and frees nothing.
//
// Every call on a GPU uses that GPU's one array, which keeps what the last call left: nothing in it
// has to start at zero (the plan kernel writes every chunk record, in use or not, and a partial
// result is read only where this call's split kernel wrote it), and two calls that overlap on one
// GPU (two streams, two threads) race on it: order them.
#pragma once

#include <hip/hip_runtime.h>

#define FG_ATTN_STATIC_BYTES (16u << 20)  // 16 MiB
#define FG_ERR_SCRATCH 3  // the call needs more scratch than the static array holds, or the array has no address

extern "C" {
// The largest max_chunks that fits the array for n_kv kv heads at this library's head size.
int fg_attn_decode_static_max_chunks(int n_kv);

// items: int32 [n_items][4] on the device (sequence, first flat token, tokens, first position),
// 16-byte aligned; every item has at most 16 rows (tokens x query heads per kv head).  max_chunks as
// for fg_attn_plan (>= 2 * n_items), at most fg_attn_decode_static_max_chunks(n_kv): beyond it the
// call does nothing and returns FG_ERR_SCRATCH.  Same results as fg_attn_plan + fg_attn_split with
// these arguments.
int fg_attn_decode_static(const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
                          const void* v_pages, const int* block_table, int bt_stride, const int* items,
                          int n_items, int max_chunks, int min_tiles, int max_rows, int n_heads, int n_kv, int hd,
                          int page_size, float scale, int window, hipStream_t stream);

// What went wrong in this thread's last fg_attn_decode_static call that did not return 0 ("" if nothing).
const char* fg_attn_decode_static_error();
}
