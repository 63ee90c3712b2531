// C interface of attention_mfma.hip (one shared object per head size, -DHEAD_DIM=<d>).
// Every function returns 0 on success; otherwise mi_last_error() holds the message.  All pointers are device
// pointers unless said otherwise; work is queued on `stream`.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

int mi_attn_head_dim();
int mi_attn_macro_tile_keys();
int mi_attn_decode_waves();
int mi_attn_prefill_tokens_per_block(int nq, int nkv);

int mi_attn_prefill(const void* q, int64_t q_row_stride, void* out, int64_t out_row_stride, const void* k_pages,
                    const void* v_pages, const int* block_table, int table_width, const int* work, int num_work,
                    const int* cu_q, const int* kv_len, int nq, int nkv, int page_size, float scale, int window,
                    int variant, hipStream_t stream);

// Split-key attention of entries first_entry .. first_entry + num_entries - 1, one new token each.  The caller
// brings the scratch for the splits' partial results: part_o float [num_entries * nq * num_splits * D] and part_ml
// float [num_entries * nq * num_splits * 2].  stream_keys != 0: the keys and values are read with nontemporal loads;
// wide != 0: workgroups of twice the waves (for launches of two workgroups or more a compute unit, with half the splits).
int mi_attn_decode(const void* q, int64_t q_row_stride, void* out, int64_t out_row_stride, const void* k_pages,
                   const void* v_pages, const int* block_table, int table_width, const int* cu_q, const int* kv_len,
                   int first_entry, int num_entries, int num_splits, float* part_o, float* part_ml, int nq, int nkv,
                   int page_size, float scale, int window, int stream_keys, int wide, hipStream_t stream);

int mi_attn_decode_front(const void* qkv, int64_t qkv_row_stride, void* out, int64_t out_row_stride, void* k_pages,
                         void* v_pages, const int* block_table, int table_width, const int* cu_q, const int* kv_len,
                         int first_entry, int num_entries, int num_splits, float* part_o, float* part_ml, int nq,
                         int nkv, int page_size, float scale, int window, int stream_keys, int wide, const float* q_weight,
                         const float* k_weight, float eps, const float* cos_sin, int rotary_dim, int max_pos,
                         const int* positions, const int* slots, hipStream_t stream);

// mi_attn_decode for callers that cannot allocate device memory and have no workspace to pass: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference
// (tom-jerr/MiniInfer's attention backends allocate their split workspaces through torch).  Same kernels, same
// arguments (stream_keys = 0, wide = 0) and result as mi_attn_decode, but the partial results of the key splits live in a file-scope device
// array of MI_ATTN_STATIC_SCRATCH_FLOATS floats that each GPU holds, once per loaded shared object, until the
// process ends.  The function allocates nothing and calls no allocating routine.  It refuses a launch whose
// partials (num_entries * nq * num_splits * (D + 2) floats) do not fit.  Nothing in the array has to start at zero:
// every partial a merge reads was written by the launch before it.  All calls on one GPU share that GPU's array,
// so two calls that may overlap there (different streams, or graphs replayed side by side) race; calls on one
// stream are ordered and safe.  mi_attn_static_scratch_floats() returns the array's size.
#define MI_ATTN_STATIC_SCRATCH_FLOATS (1 << 20)
int mi_attn_static_scratch_floats();
int mi_attn_decode_static(const void* q, int64_t q_row_stride, void* out, int64_t out_row_stride,
                          const void* k_pages, const void* v_pages, const int* block_table, int table_width,
                          const int* cu_q, const int* kv_len, int first_entry, int num_entries, int num_splits,
                          int nq, int nkv, int page_size, float scale, int window, hipStream_t stream);

const char* mi_last_error();

}  // extern "C"
