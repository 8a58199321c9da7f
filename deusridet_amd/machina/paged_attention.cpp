// paged_attention.cpp -- see paged_attention.h.  Forwarders to the C ABI.
#include "paged_attention.h"
#include "../communis/log.h"
#include "drk_kv.h"

#include <mutex>

namespace deusridet {

namespace {
std::mutex g_ws_mu;
void* g_ws = nullptr;
size_t g_ws_bytes = 0;

// grow-only; returns the workspace or null
void* workspace(size_t need)
{
    std::lock_guard<std::mutex> lock(g_ws_mu);
    if (need <= g_ws_bytes) return g_ws;
    if (g_ws) {
        drk_stream_synchronize(nullptr);
        drk_dev_free(g_ws);
        g_ws = nullptr;
        g_ws_bytes = 0;
    }
    size_t bytes = (need + (1u << 20) - 1) & ~(size_t)((1u << 20) - 1);
    if (drk_dev_malloc(&g_ws, bytes) != DRK_OK) {
        LOG_ERROR("Machina", "paged attention workspace of %zu bytes: %s", bytes, drk_last_error());
        g_ws = nullptr;
        return nullptr;
    }
    g_ws_bytes = bytes;
    return g_ws;
}
} // namespace

bool paged_attention_reserve_workspace(int max_branches, int max_seq_len, int max_prefill_rows, int block_size)
{
    drk_kv_layout g = ModelConfig::layout(1, block_size);
    const int B = max_branches > 0 ? max_branches : 1;
    size_t need = drk_decode_workspace_bytes(&g, B, max_seq_len);
    // the shared-prefix and the scored variants keep more partials than the plain call
    size_t s = drk_decode_shared_workspace_bytes(&g, B, max_seq_len, max_seq_len);
    if (s > need) need = s;
    s = drk_decode_mass_workspace_bytes(&g, B, max_seq_len);
    if (s > need) need = s;
    if (max_prefill_rows > 0) {
        // the last chunk of the longest context needs the most (0 for the MFMA prefill kernel)
        const int rows = max_prefill_rows < max_seq_len ? max_prefill_rows : max_seq_len;
        size_t p = drk_prefill_workspace_bytes(&g, max_seq_len - rows, rows);
        if (p > need) need = p;
        // ... and a short chunk behind a long context runs with the context split over the chip, which
        // keeps partial results: room for any chunk length up to max_prefill_rows
        for (int m = 64; m <= 256; m *= 2) {
            const int r = m < rows ? m : rows;
            p = drk_prefill_workspace_bytes(&g, max_seq_len - r, r);
            if (p > need) need = p;
        }
    }
    return need == 0 || workspace(need) != nullptr;
}

void paged_attention_release_workspace()
{
    std::lock_guard<std::mutex> lock(g_ws_mu);
    if (g_ws) drk_dev_free(g_ws);
    g_ws = nullptr;
    g_ws_bytes = 0;
}

void paged_kv_cache_write(const __half* src_k, const __half* src_v, __half* kv_pool, const int* d_block_table,
                          int fa_layer_idx, const int* d_pos, int max_phys_blocks, int block_size, hipStream_t stream)
{
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_kv_append_token(&g, kv_pool, d_block_table, fa_layer_idx, d_pos, src_k, src_v, ModelConfig::IO_DTYPE,
                            stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_kv_cache_write: %s", drk_last_error());
}

void paged_kv_cache_write_batch(const __half* src_k, const __half* src_v, __half* kv_pool, const int* d_block_table,
                                int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                                hipStream_t stream)
{
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_kv_append_batch(&g, kv_pool, d_block_table, fa_layer_idx, 1, pos_start, M, src_k, src_v,
                            ModelConfig::IO_DTYPE, stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_kv_cache_write_batch: %s", drk_last_error());
}

void paged_kv_cache_write_branches(const __half* src_k, const __half* src_v, __half* kv_pool, const int* d_tables,
                                   int table_stride, const int* d_pos, int B, int fa_layer_idx,
                                   int max_phys_blocks, int block_size, hipStream_t stream)
{
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_kv_append_branches(&g, kv_pool, d_tables, table_stride, d_pos, B, fa_layer_idx, 1, src_k, src_v,
                               ModelConfig::IO_DTYPE, stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_kv_cache_write_branches: %s", drk_last_error());
}

void paged_gqa_decode_attention(const __half* Q, __half* kv_pool, const int* d_block_table, __half* out,
                                int fa_layer_idx, int seq_len, int max_phys_blocks, int block_size, float scale,
                                hipStream_t stream)
{
    if (seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    size_t need = drk_decode_workspace_bytes(&g, 1, seq_len);
    void* ws = workspace(need);
    if (!ws) return;
    if (drk_paged_decode_attention(&g, Q, kv_pool, d_block_table, out, fa_layer_idx, seq_len, scale,
                                   ModelConfig::IO_DTYPE, ws, g_ws_bytes, stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention: %s", drk_last_error());
}

void paged_gqa_decode_attention_branches(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                         const int* d_seq_lens, int B, int max_seq_len, __half* out,
                                         int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                         hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    size_t need = drk_decode_workspace_bytes(&g, B, max_seq_len);
    void* ws = workspace(need);
    if (!ws) return;
    if (drk_paged_decode_attention_branches(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, out,
                                            fa_layer_idx, scale, ModelConfig::IO_DTYPE, 0, ws, g_ws_bytes,
                                            stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_branches: %s", drk_last_error());
}

void paged_gqa_decode_attention_shared(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                       const int* d_seq_lens, int B, int max_seq_len, int shared_tokens,
                                       __half* out, int fa_layer_idx, int max_phys_blocks, int block_size,
                                       float scale, hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    size_t need = drk_decode_shared_workspace_bytes(&g, B, max_seq_len, shared_tokens);
    void* ws = workspace(need);
    if (!ws) return;
    if (drk_paged_decode_attention_shared(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len,
                                          shared_tokens, out, fa_layer_idx, scale, ModelConfig::IO_DTYPE, ws,
                                          g_ws_bytes, stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_shared: %s", drk_last_error());
}

void paged_prefill_attention(const __half* Q, __half* kv_pool, const int* d_block_table, __half* out,
                             int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                             float scale, hipStream_t stream)
{
    if (M <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    size_t need = drk_prefill_workspace_bytes(&g, pos_start, M);
    void* ws = workspace(need);
    if (!ws && need) return;            // need == 0 (the MFMA kernel on a long chunk) and nothing reserved yet: no workspace
    if (drk_paged_prefill_attention(&g, Q, kv_pool, d_block_table, out, fa_layer_idx, pos_start, M, scale,
                                    ModelConfig::IO_DTYPE, ws, ws ? g_ws_bytes : 0, stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_prefill_attention: %s", drk_last_error());
}

namespace {
void fused_write(const char* who, const __half* qg, const __half* k, const __half* v, const __half* q_norm,
                 const __half* k_norm, __half* q_out, __half* kv_pool, const int* d_tables, int table_stride,
                 const int* d_pos, int pos_start, int T, int fa_layer_idx, int max_phys_blocks, int block_size,
                 const float* d_rope_table, int table_positions, hipStream_t stream)
{
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_qk_norm_rope_append(&g, kv_pool, d_tables, table_stride, d_pos, pos_start, T, fa_layer_idx, qg, k, v, q_norm,
                                k_norm, ModelConfig::RMS_EPS, ModelConfig::ROTARY_DIM, ModelConfig::ROPE_THETA,
                                d_rope_table, table_positions, q_out, ModelConfig::IO_DTYPE, stream) != DRK_OK)
        LOG_ERROR("Machina", "%s: %s", who, drk_last_error());
}
} // namespace

void paged_qk_norm_rope_write(const __half* qg, const __half* k, const __half* v, const __half* q_norm,
                              const __half* k_norm, __half* q_out, __half* kv_pool, const int* d_block_table,
                              int fa_layer_idx, const int* d_pos, int max_phys_blocks, int block_size,
                              const float* d_rope_table, int table_positions, hipStream_t stream)
{
    fused_write("paged_qk_norm_rope_write", qg, k, v, q_norm, k_norm, q_out, kv_pool, d_block_table, 0, d_pos, 0, 1,
                fa_layer_idx, max_phys_blocks, block_size, d_rope_table, table_positions, stream);
}

void paged_qk_norm_rope_write_batch(const __half* qg, const __half* k, const __half* v, const __half* q_norm,
                                    const __half* k_norm, __half* q_out, __half* kv_pool, const int* d_block_table,
                                    int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                                    const float* d_rope_table, int table_positions, hipStream_t stream)
{
    fused_write("paged_qk_norm_rope_write_batch", qg, k, v, q_norm, k_norm, q_out, kv_pool, d_block_table, 0, nullptr,
                pos_start, M, fa_layer_idx, max_phys_blocks, block_size, d_rope_table, table_positions, stream);
}

void paged_qk_norm_rope_write_branches(const __half* qg, const __half* k, const __half* v, const __half* q_norm,
                                       const __half* k_norm, __half* q_out, __half* kv_pool, const int* d_tables,
                                       int table_stride, const int* d_pos, int B, int fa_layer_idx,
                                       int max_phys_blocks, int block_size, const float* d_rope_table,
                                       int table_positions, hipStream_t stream)
{
    fused_write("paged_qk_norm_rope_write_branches", qg, k, v, q_norm, k_norm, q_out, kv_pool, d_tables, table_stride,
                d_pos, 0, B, fa_layer_idx, max_phys_blocks, block_size, d_rope_table, table_positions, stream);
}

void paged_gqa_decode_attention_gated_branches(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                               const int* d_seq_lens, int B, int max_seq_len, const __half* gate,
                                               int gate_stride, __half* out, int fa_layer_idx, int max_phys_blocks,
                                               int block_size, float scale, hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    size_t need = drk_decode_workspace_bytes(&g, B, max_seq_len);
    void* ws = workspace(need);
    if (!ws) return;
    if (drk_paged_decode_attention_gated(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, out,
                                         fa_layer_idx, scale, ModelConfig::IO_DTYPE, gate, (size_t)gate_stride, ws,
                                         g_ws_bytes, stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_gated_branches: %s", drk_last_error());
}

void paged_gqa_decode_attention_branches_scored(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                                const int* d_seq_lens, int B, int max_seq_len, __half* out,
                                                int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                                float* d_block_mass, bool accumulate, hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    size_t need = drk_decode_mass_workspace_bytes(&g, B, max_seq_len);
    if (need == 0) {
        LOG_ERROR("Machina", "paged_gqa_decode_attention_branches_scored: geometry not supported by the scored kernel");
        return;
    }
    void* ws = workspace(need);
    if (!ws) return;
    if (drk_paged_decode_attention_mass(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, out,
                                        fa_layer_idx, scale, ModelConfig::IO_DTYPE, d_block_mass, table_stride,
                                        accumulate ? 1 : 0, ws, g_ws_bytes, stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_branches_scored: %s", drk_last_error());
}

void paged_prefill_attention_gated(const __half* Q, __half* kv_pool, const int* d_block_table, const __half* gate,
                                   int gate_stride, __half* out, int fa_layer_idx, int pos_start, int M,
                                   int max_phys_blocks, int block_size, float scale, hipStream_t stream)
{
    if (M <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    size_t need = drk_prefill_workspace_bytes(&g, pos_start, M);
    void* ws = workspace(need);
    if (!ws && need) return;
    if (drk_paged_prefill_attention_gated(&g, Q, kv_pool, d_block_table, out, fa_layer_idx, pos_start, M, scale,
                                          ModelConfig::IO_DTYPE, gate, (size_t)gate_stride, ws, ws ? g_ws_bytes : 0,
                                          stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_prefill_attention_gated: %s", drk_last_error());
}

} // namespace deusridet
