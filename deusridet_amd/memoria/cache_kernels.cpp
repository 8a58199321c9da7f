// cache_kernels.cpp -- see cache_kernels.h.  Thin forwarders to the C ABI; like
// the reference's launchers they return nothing, a failure is logged.
#include "cache_kernels.h"
#include "../communis/log.h"
#include "drk_kv.h"

namespace deusridet {

static drk_kv_layout flat_layout(int num_layers, int num_kv_heads, int head_dim, int block_size, int max_phys_blocks,
                                 int kv_dtype)
{
    // the layer stride depends on max_phys_blocks only, so num_layers here is just
    // the number of layers the call touches; query heads play no part
    return drk_kv_layout{num_layers, num_kv_heads, num_kv_heads, head_dim, block_size, max_phys_blocks, kv_dtype, 0};
}

void invoke_extract_kv_from_pages_typed(void* dst, void* dst_scales, const void* kv_pool, const int* block_table,
                                        int start_token, int num_tokens, int num_layers, int num_kv_heads,
                                        int head_dim, int block_size, int max_phys_blocks, int kv_dtype,
                                        hipStream_t stream)
{
    if (num_layers <= 0 || num_tokens <= 0) return;
    drk_kv_layout g = flat_layout(num_layers, num_kv_heads, head_dim, block_size, max_phys_blocks, kv_dtype);
    if (drk_kv_extract(&g, dst, dst_scales, kv_pool, block_table, start_token, num_tokens, num_layers, stream) != DRK_OK)
        LOG_ERROR("Memoria", "extract_kv_from_pages: %s", drk_last_error());
}

void invoke_inject_kv_to_pages_typed(void* kv_pool, const void* src, const void* src_scales, const int* block_table,
                                     int start_token, int num_tokens, int num_layers, int num_kv_heads,
                                     int head_dim, int block_size, int max_phys_blocks, int kv_dtype,
                                     hipStream_t stream)
{
    if (num_layers <= 0 || num_tokens <= 0) return;
    drk_kv_layout g = flat_layout(num_layers, num_kv_heads, head_dim, block_size, max_phys_blocks, kv_dtype);
    if (drk_kv_inject(&g, kv_pool, src, src_scales, block_table, start_token, num_tokens, num_layers, stream) != DRK_OK)
        LOG_ERROR("Memoria", "inject_kv_to_pages: %s", drk_last_error());
}

void invoke_extract_kv_from_pages(__half* dst, const __half* kv_pool, const int* block_table, int start_token,
                                  int num_tokens, int num_layers, int num_kv_heads, int head_dim, int block_size,
                                  int max_phys_blocks, hipStream_t stream)
{
    invoke_extract_kv_from_pages_typed(dst, nullptr, kv_pool, block_table, start_token, num_tokens, num_layers,
                                       num_kv_heads, head_dim, block_size, max_phys_blocks, DRK_F16, stream);
}

void invoke_inject_kv_to_pages(__half* kv_pool, const __half* src, const int* block_table, int start_token,
                               int num_tokens, int num_layers, int num_kv_heads, int head_dim, int block_size,
                               int max_phys_blocks, hipStream_t stream)
{
    invoke_inject_kv_to_pages_typed(kv_pool, src, nullptr, block_table, start_token, num_tokens, num_layers,
                                    num_kv_heads, head_dim, block_size, max_phys_blocks, DRK_F16, stream);
}

} // namespace deusridet
