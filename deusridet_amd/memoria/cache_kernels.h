// cache_kernels.h -- gather pages into a flat buffer and scatter them back.
// Same two entry points as the reference (src/memoria/cache_kernels.h:44-74),
// HIP vocabulary types.  Flat layout: [num_layers][2][num_tokens][num_kv_heads]
// [head_dim], K then V per layer.  A hole in the block table (entry < 0) is
// zero-filled by extract and skipped by inject (cache_kernels.cu:64-68, 120).
// Offsets are 64-bit (the reference computes them in 32-bit int,
// cache_kernels.cu:43-47, 75-84, and overflows past 2^31 elements).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

namespace deusridet {

void invoke_extract_kv_from_pages(__half* dst, const __half* kv_pool, const int* block_table, int start_token,
                                  int num_tokens, int num_layers, int num_kv_heads, int head_dim, int block_size,
                                  int max_phys_blocks, hipStream_t stream);

void invoke_inject_kv_to_pages(__half* kv_pool, const __half* src, const int* block_table, int start_token,
                               int num_tokens, int num_layers, int num_kv_heads, int head_dim, int block_size,
                               int max_phys_blocks, hipStream_t stream);

// Same for any storage type (DRK_* from drk_kv.h); an INT8 pool's fp16 scales go
// to / come from `scales` [num_layers][2][num_tokens][num_kv_heads] when it is
// not null.  Not in the reference (its cache is fp16 only).
void invoke_extract_kv_from_pages_typed(void* dst, void* dst_scales, const void* kv_pool, const int* block_table,
                                        int start_token, int num_tokens, int num_layers, int num_kv_heads,
                                        int head_dim, int block_size, int max_phys_blocks, int kv_dtype,
                                        hipStream_t stream);
void invoke_inject_kv_to_pages_typed(void* kv_pool, const void* src, const void* src_scales, const int* block_table,
                                     int start_token, int num_tokens, int num_layers, int num_kv_heads,
                                     int head_dim, int block_size, int max_phys_blocks, int kv_dtype,
                                     hipStream_t stream);

} // namespace deusridet
