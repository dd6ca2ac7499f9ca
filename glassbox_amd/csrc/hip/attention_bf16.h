// C entry points of the bfloat16 paged-attention library (attention_bf16.hip).
//
// Every function returns 0, or 1 after leaving a message for gb_last_error().  Pointers are device
// pointers unless said otherwise; `stream` is the HIP stream the kernels are launched on.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

extern "C" {

const char* gb_last_error();

int gb_attention_supported_head_size(int hd);

// Decoding: rows 0 .. n_decode-1 of q and out are requests with one token each, at positions[s], with block
// table tables[s * table_stride ...].  The context is cut into chunks of `chunk` keys (a multiple of 256);
// with more than one chunk (splits = ceil(max_context / chunk) > 1) the chunks' partial results pass through
// ws_acc (n_decode * nh * splits * hd floats) and ws_ml (n_decode * nh * splits * 2 floats), which the
// caller provides.
int gb_attention_decode_bf16(const void* q, int q_stride, void* out, int out_stride, void* ws_acc, void* ws_ml,
                             const int32_t* positions, const int32_t* tables, int table_stride, const void* k_pages,
                             const void* v_pages, int n_decode, int nh, int nkv, int hd, int page_size, float scale,
                             int window, int chunk, int max_context, hipStream_t stream);

// The same decoding for callers that cannot allocate device memory and have no workspace to pass: code under
// HIP graph capture, tight serving loops, harnesses that forbid allocation.  It has no counterpart in the
// reference (a CPU engine whose attention needs no partial results, crates/glassbox-core/src/model.rs:285-317).
//
// The chunks' partial results live in an array that the library itself holds on every GPU it runs on, of
// GB_DECODE_STATIC_FLOATS floats (4 MiB, until the process ends); its address on the current device is looked
// up at the first call on that device (make that call outside a graph capture).  The call allocates nothing,
// on the device or through any library.  It refuses, with a message, sizes whose partial results do not fit:
//     n_decode * nh * ceil(max_context / chunk) * (hd + 2)  <=  GB_DECODE_STATIC_FLOATS
// (one chunk needs nothing).  Inputs, outputs, kernels and results are those of gb_attention_decode_bf16.
//
// Every call on a GPU uses that GPU's one array: calls whose kernels may overlap on one GPU (two streams, two
// threads) race; calls on one stream are ordered and safe.  The array keeps the last call's contents; the
// kernels write every cell they read, so nothing needs clearing between calls.
#define GB_DECODE_STATIC_FLOATS (1 << 20)
int gb_attention_decode_bf16_static(const void* q, int q_stride, void* out, int out_stride, const int32_t* positions,
                                    const int32_t* tables, int table_stride, const void* k_pages, const void* v_pages,
                                    int n_decode, int nh, int nkv, int hd, int page_size, float scale, int window,
                                    int chunk, int max_context, hipStream_t stream);

int gb_attention_prefill_parts(int max_q_len, int max_context, int nh, int n_seqs, int hd);

int gb_attention_prefill_bf16(const void* q, int q_stride, void* out, int out_stride, const int32_t* q_start,
                              const int32_t* q_len, const int32_t* pos0, int seq_base, int n_seqs, int max_q_len,
                              int max_context, const int32_t* tables, int table_stride, const void* k_pages,
                              const void* v_pages, int nh, int nkv, int hd, int page_size, float scale, int window,
                              int first_row, int n_rows, float* part_ws, long long part_floats, hipStream_t stream);

}  // extern "C"
