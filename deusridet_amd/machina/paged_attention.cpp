// paged_attention.cpp -- see paged_attention.h.  Forwarders to the C ABI.
#include "paged_attention.h"
#include "../communis/log.h"
#include "drk_kv.h"

#include <cmath>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

namespace deusridet {

// ---- AttentionWorkspace ------------------------------------------------------------------

AttentionWorkspace::~AttentionWorkspace() { release(); }

bool AttentionWorkspace::reserve(size_t bytes)
{
    if (bytes <= bytes_) return true;
    if (ptr_) {
        LOG_ERROR("Machina", "attention workspace holds %zu bytes, %zu wanted: it is reserved once and never moved", bytes_, bytes);
        return false;
    }
    size_t rounded = (bytes + (1u << 20) - 1) & ~(size_t)((1u << 20) - 1);
    if (drk_dev_malloc(&ptr_, rounded) != DRK_OK) {
        LOG_ERROR("Machina", "paged attention workspace of %zu bytes: %s", rounded, drk_last_error());
        ptr_ = nullptr;
        return false;
    }
    bytes_ = rounded;
    return true;
}

// shared ranges nested deeper than this fall to the private tails (CacheManager::common_prefix_groups emits
// parents first, so the callers simply stop there)
static constexpr int kMaxForkTreeDepth = 4;

size_t paged_attention_workspace_bytes(int max_branches, int max_seq_len, int max_prefill_rows, int block_size)
{
    drk_kv_layout g = ModelConfig::layout(1, block_size);
    const int B = max_branches > 0 ? max_branches : 1;
    size_t need = drk_decode_workspace_bytes(&g, B, max_seq_len);
    // the shared-prefix and the scored variants keep more partials than the plain call
    size_t s = drk_decode_shared_workspace_bytes(&g, B, max_seq_len, max_seq_len);
    if (s > need) need = s;
    s = drk_decode_mass_workspace_bytes(&g, B, max_seq_len);
    if (s > need) need = s;
    s = drk_decode_grouped_workspace_bytes_max(&g, B, max_seq_len, kMaxForkTreeDepth);
    if (s > need) need = s;
    if (max_prefill_rows > 0) {
        // a short chunk behind a long context runs with the context split over the chip and keeps
        // partial results; other geometries run row by row through the decode kernel
        s = drk_prefill_workspace_bytes_max(&g, max_seq_len, max_prefill_rows);
        if (s > need) need = s;
    }
    return need;
}

bool AttentionWorkspace::reserve_for(int max_branches, int max_seq_len, int max_prefill_rows, int block_size)
{
    return reserve(paged_attention_workspace_bytes(max_branches, max_seq_len, max_prefill_rows, block_size));
}

void AttentionWorkspace::release()
{
    if (ptr_) drk_dev_free(ptr_);
    ptr_ = nullptr;
    bytes_ = 0;
}

// ---- one workspace per stream for the calls that take none ---------------------------------

namespace {
std::mutex g_ws_mu;
std::map<hipStream_t, std::unique_ptr<AttentionWorkspace>> g_ws;     // current buffer of each stream
std::vector<std::unique_ptr<AttentionWorkspace>> g_ws_retired;       // outgrown buffers: kept, never freed while in use

// The stream's workspace with at least `need` bytes, or null.  Growing means a new allocation;
// the outgrown buffer stays alive (launches already enqueued on the stream, or a graph captured
// from it, keep the memory they were given).  Nothing is allocated while the stream is captured.
AttentionWorkspace* stream_workspace(hipStream_t stream, size_t need, const char* who)
{
    std::lock_guard<std::mutex> lock(g_ws_mu);
    std::unique_ptr<AttentionWorkspace>& cur = g_ws[stream];
    if (cur && need <= cur->bytes()) return cur.get();
    if (!cur && need == 0) return nullptr;
    int capturing = 0;
    if (drk_stream_is_capturing(stream, &capturing) != DRK_OK || capturing) {
        LOG_ERROR("Machina", "%s: needs %zu bytes of workspace while its stream is being captured (%zu reserved): "
                  "call paged_attention_reserve_workspace for this stream first", who, need, cur ? cur->bytes() : (size_t)0);
        return nullptr;
    }
    const size_t want = cur && 2 * cur->bytes() > need ? 2 * cur->bytes() : need;
    std::unique_ptr<AttentionWorkspace> fresh(new AttentionWorkspace());
    if (!fresh->reserve(want) && !(want > need && fresh->reserve(need))) return nullptr;
    if (cur) g_ws_retired.push_back(std::move(cur));
    cur = std::move(fresh);
    return cur.get();
}
} // namespace

bool paged_attention_reserve_workspace(int max_branches, int max_seq_len, int max_prefill_rows, int block_size,
                                       hipStream_t stream)
{
    const size_t need = paged_attention_workspace_bytes(max_branches, max_seq_len, max_prefill_rows, block_size);
    return need == 0 || stream_workspace(stream, need, "paged_attention_reserve_workspace") != nullptr;
}

void paged_attention_release_workspace()
{
    std::lock_guard<std::mutex> lock(g_ws_mu);
    if (g_ws.empty() && g_ws_retired.empty()) return;
    drk_device_synchronize();
    g_ws.clear();
    g_ws_retired.clear();
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

void paged_gqa_decode_attention(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_block_table,
                                __half* out, int fa_layer_idx, int seq_len, int max_phys_blocks, int block_size,
                                float scale, hipStream_t stream)
{
    if (seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_decode_attention(&g, Q, kv_pool, d_block_table, out, fa_layer_idx, seq_len, scale,
                                   ModelConfig::IO_DTYPE, ws.ptr(), ws.bytes(), stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention: %s", drk_last_error());
}

void paged_gqa_decode_attention(const __half* Q, __half* kv_pool, const int* d_block_table, __half* out,
                                int fa_layer_idx, int seq_len, int max_phys_blocks, int block_size, float scale,
                                hipStream_t stream)
{
    if (seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    AttentionWorkspace* ws = stream_workspace(stream, drk_decode_workspace_bytes(&g, 1, seq_len), "paged_gqa_decode_attention");
    if (ws) paged_gqa_decode_attention(*ws, Q, kv_pool, d_block_table, out, fa_layer_idx, seq_len, max_phys_blocks, block_size, scale, stream);
}

void paged_gqa_decode_attention_branches(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_tables,
                                         int table_stride, const int* d_seq_lens, int B, int max_seq_len, __half* out,
                                         int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                         hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_decode_attention_branches(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, out,
                                            fa_layer_idx, scale, ModelConfig::IO_DTYPE, 0, ws.ptr(), ws.bytes(),
                                            stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_branches: %s", drk_last_error());
}

void paged_gqa_decode_attention_branches(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                         const int* d_seq_lens, int B, int max_seq_len, __half* out,
                                         int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                         hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    AttentionWorkspace* ws = stream_workspace(stream, drk_decode_workspace_bytes(&g, B, max_seq_len), "paged_gqa_decode_attention_branches");
    if (ws) paged_gqa_decode_attention_branches(*ws, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, out,
                                                fa_layer_idx, max_phys_blocks, block_size, scale, stream);
}

void paged_gqa_decode_attention_shared(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_tables,
                                       int table_stride, const int* d_seq_lens, int B, int max_seq_len,
                                       int shared_tokens, __half* out, int fa_layer_idx, int max_phys_blocks,
                                       int block_size, float scale, hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_decode_attention_shared(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len,
                                          shared_tokens, out, fa_layer_idx, scale, ModelConfig::IO_DTYPE, ws.ptr(),
                                          ws.bytes(), stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_shared: %s", drk_last_error());
}

size_t paged_decode_plan_bytes(int B, int max_seq_len, int max_phys_blocks, int block_size, int n_groups)
{
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    return drk_decode_plan_bytes(&g, B, max_seq_len, n_groups);
}

bool paged_decode_plan_build(void* d_plan, size_t plan_bytes, const int* d_tables, int table_stride, const int* d_seq_lens,
                             int B, int max_seq_len, const drk_prefix_group* groups, int n_groups, int max_phys_blocks,
                             int block_size, hipStream_t stream)
{
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_decode_plan_build(&g, d_tables, table_stride, d_seq_lens, B, max_seq_len, groups, n_groups, d_plan, plan_bytes,
                              stream) != DRK_OK) {
        LOG_ERROR("Machina", "paged_decode_plan_build: %s", drk_last_error());
        return false;
    }
    return true;
}

void paged_gqa_decode_attention_planned(AttentionWorkspace& ws, const void* d_plan, const __half* Q, __half* kv_pool,
                                        const int* d_tables, int table_stride, const int* d_seq_lens, int B, int max_seq_len,
                                        const drk_prefix_group* groups, int n_groups, const __half* gate, int gate_stride,
                                        __half* out, int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                        hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_decode_attention_planned(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, groups, n_groups,
                                           d_plan, out, fa_layer_idx, scale, ModelConfig::IO_DTYPE, gate, (size_t)gate_stride,
                                           ws.ptr(), ws.bytes(), stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_planned: %s", drk_last_error());
}

bool paged_gqa_decode_grouped_supported(int block_size)
{
    return ModelConfig::HEAD_DIM == 128 && block_size % 16 == 0 && ModelConfig::NUM_KV_HEADS > 0 &&
           ModelConfig::NUM_ATTN_HEADS / ModelConfig::NUM_KV_HEADS <= 16;
}

void paged_gqa_decode_attention_grouped(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_tables,
                                        int table_stride, const int* d_seq_lens, int B, int max_seq_len,
                                        const drk_prefix_group* groups, int n_groups, const __half* gate,
                                        int gate_stride, __half* out, int fa_layer_idx, int max_phys_blocks,
                                        int block_size, float scale, hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_decode_attention_grouped(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, groups,
                                           n_groups, out, fa_layer_idx, scale, ModelConfig::IO_DTYPE, gate,
                                           (size_t)gate_stride, ws.ptr(), ws.bytes(), stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_grouped: %s", drk_last_error());
}

void paged_gqa_decode_attention_shared(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                       const int* d_seq_lens, int B, int max_seq_len, int shared_tokens,
                                       __half* out, int fa_layer_idx, int max_phys_blocks, int block_size,
                                       float scale, hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    AttentionWorkspace* ws = stream_workspace(stream, drk_decode_shared_workspace_bytes(&g, B, max_seq_len, shared_tokens),
                                              "paged_gqa_decode_attention_shared");
    if (ws) paged_gqa_decode_attention_shared(*ws, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, shared_tokens,
                                              out, fa_layer_idx, max_phys_blocks, block_size, scale, stream);
}

void paged_gqa_decode_attention_grouped(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                        const int* d_seq_lens, int B, int max_seq_len, const drk_prefix_group* groups,
                                        int n_groups, __half* out, int fa_layer_idx, int max_phys_blocks, int block_size,
                                        float scale, hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    AttentionWorkspace* ws = stream_workspace(stream, drk_decode_grouped_workspace_bytes(&g, B, max_seq_len, groups, n_groups),
                                              "paged_gqa_decode_attention_grouped");
    if (ws) paged_gqa_decode_attention_grouped(*ws, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, groups,
                                               n_groups, nullptr, 0, out, fa_layer_idx, max_phys_blocks, block_size, scale, stream);
}

void paged_prefill_attention(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_block_table,
                             __half* out, int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                             float scale, hipStream_t stream)
{
    if (M <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_prefill_attention(&g, Q, kv_pool, d_block_table, out, fa_layer_idx, pos_start, M, scale,
                                    ModelConfig::IO_DTYPE, ws.ptr(), ws.bytes(), stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_prefill_attention: %s", drk_last_error());
}

namespace {
AttentionWorkspace g_no_workspace;      // stays empty: the MFMA prefill kernel on a long chunk needs none

AttentionWorkspace& prefill_workspace(hipStream_t stream, int pos_start, int M, int max_phys_blocks, int block_size, const char* who)
{
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    AttentionWorkspace* ws = stream_workspace(stream, drk_prefill_workspace_bytes(&g, pos_start, M), who);
    return ws ? *ws : g_no_workspace;
}
} // namespace

void paged_prefill_attention(const __half* Q, __half* kv_pool, const int* d_block_table, __half* out,
                             int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                             float scale, hipStream_t stream)
{
    if (M <= 0) return;
    paged_prefill_attention(prefill_workspace(stream, pos_start, M, max_phys_blocks, block_size, "paged_prefill_attention"), Q,
                            kv_pool, d_block_table, out, fa_layer_idx, pos_start, M, max_phys_blocks, block_size, scale, stream);
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

void paged_gqa_decode_attention_gated_branches(AttentionWorkspace& ws, const __half* Q, __half* kv_pool,
                                               const int* d_tables, int table_stride, const int* d_seq_lens, int B,
                                               int max_seq_len, const __half* gate, int gate_stride, __half* out,
                                               int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                               hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_decode_attention_gated(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, out,
                                         fa_layer_idx, scale, ModelConfig::IO_DTYPE, gate, (size_t)gate_stride, ws.ptr(),
                                         ws.bytes(), stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_gated_branches: %s", drk_last_error());
}

void paged_gqa_decode_attention_gated_branches(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                               const int* d_seq_lens, int B, int max_seq_len, const __half* gate,
                                               int gate_stride, __half* out, int fa_layer_idx, int max_phys_blocks,
                                               int block_size, float scale, hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    AttentionWorkspace* ws = stream_workspace(stream, drk_decode_workspace_bytes(&g, B, max_seq_len), "paged_gqa_decode_attention_gated_branches");
    if (ws) paged_gqa_decode_attention_gated_branches(*ws, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, gate,
                                                      gate_stride, out, fa_layer_idx, max_phys_blocks, block_size, scale, stream);
}

void paged_gqa_decode_attention_branches_scored(AttentionWorkspace& ws, const __half* Q, __half* kv_pool,
                                                const int* d_tables, int table_stride, const int* d_seq_lens, int B,
                                                int max_seq_len, __half* out, int fa_layer_idx, int max_phys_blocks,
                                                int block_size, float scale, float* d_block_mass, bool accumulate,
                                                hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_decode_attention_mass(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, out,
                                        fa_layer_idx, scale, ModelConfig::IO_DTYPE, d_block_mass, table_stride,
                                        accumulate ? 1 : 0, ws.ptr(), ws.bytes(), stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_branches_scored: %s", drk_last_error());
}

void paged_gqa_decode_attention_branches_scored(AttentionWorkspace& ws, const void* d_plan, const __half* Q, __half* kv_pool,
                                                const int* d_tables, int table_stride, const int* d_seq_lens, int B,
                                                int max_seq_len, const __half* gate, int gate_stride, __half* out,
                                                int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                                float* d_block_mass, bool accumulate, hipStream_t stream)
{
    if (B <= 0 || max_seq_len <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_decode_attention_mass_gated(&g, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, d_plan, out,
                                              fa_layer_idx, scale, ModelConfig::IO_DTYPE, gate, (size_t)gate_stride,
                                              d_block_mass, table_stride, accumulate ? 1 : 0, ws.ptr(), ws.bytes(),
                                              stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_gqa_decode_attention_branches_scored: %s", drk_last_error());
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
    AttentionWorkspace* ws = stream_workspace(stream, need, "paged_gqa_decode_attention_branches_scored");
    if (ws) paged_gqa_decode_attention_branches_scored(*ws, Q, kv_pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, out,
                                                       fa_layer_idx, max_phys_blocks, block_size, scale, d_block_mass, accumulate, stream);
}

void paged_prefill_attention_mass(const __half* Q, const __half* kv_pool, const int* d_block_table, int fa_layer_idx,
                                  int pos_start, int M, int max_phys_blocks, int block_size, float scale,
                                  float* d_block_mass, int mass_len, bool accumulate, hipStream_t stream)
{
    if (M <= 0 && accumulate) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_prefill_attention_mass(&g, Q, kv_pool, d_block_table, fa_layer_idx, pos_start, M, scale,
                                         ModelConfig::IO_DTYPE, d_block_mass, mass_len, accumulate ? 1 : 0, stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_prefill_attention_mass: %s", drk_last_error());
}

void paged_prefill_attention_mass(const __half* Q, const __half* kv_pool, const int* d_block_table, int fa_layer_idx,
                                  int pos_start, int M, int max_phys_blocks, int block_size, float scale,
                                  const float* d_row_lse, float* d_block_mass, int mass_len, bool accumulate,
                                  hipStream_t stream)
{
    if (M <= 0 && accumulate) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_prefill_attention_mass_lse(&g, Q, kv_pool, d_block_table, fa_layer_idx, pos_start, M, scale,
                                             ModelConfig::IO_DTYPE, d_row_lse, d_block_mass, mass_len, accumulate ? 1 : 0,
                                             stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_prefill_attention_mass: %s", drk_last_error());
}

void paged_prefill_attention_gated(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_block_table,
                                   const __half* gate, int gate_stride, __half* out, float* d_row_lse, int fa_layer_idx,
                                   int pos_start, int M, int max_phys_blocks, int block_size, float scale, hipStream_t stream)
{
    if (M <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_prefill_attention_lse(&g, Q, kv_pool, d_block_table, out, fa_layer_idx, pos_start, M, scale,
                                        ModelConfig::IO_DTYPE, gate, (size_t)gate_stride, d_row_lse, ws.ptr(), ws.bytes(),
                                        stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_prefill_attention_gated: %s", drk_last_error());
}

void paged_prefill_attention_gated(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_block_table,
                                   const __half* gate, int gate_stride, __half* out, int fa_layer_idx, int pos_start,
                                   int M, int max_phys_blocks, int block_size, float scale, hipStream_t stream)
{
    if (M <= 0) return;
    drk_kv_layout g = ModelConfig::layout(max_phys_blocks, block_size);
    if (drk_paged_prefill_attention_gated(&g, Q, kv_pool, d_block_table, out, fa_layer_idx, pos_start, M, scale,
                                          ModelConfig::IO_DTYPE, gate, (size_t)gate_stride, ws.ptr(), ws.bytes(),
                                          stream) != DRK_OK)
        LOG_ERROR("Machina", "paged_prefill_attention_gated: %s", drk_last_error());
}

void paged_prefill_attention_gated(const __half* Q, __half* kv_pool, const int* d_block_table, const __half* gate,
                                   int gate_stride, __half* out, int fa_layer_idx, int pos_start, int M,
                                   int max_phys_blocks, int block_size, float scale, hipStream_t stream)
{
    if (M <= 0) return;
    paged_prefill_attention_gated(prefill_workspace(stream, pos_start, M, max_phys_blocks, block_size, "paged_prefill_attention_gated"),
                                  Q, kv_pool, d_block_table, gate, gate_stride, out, fa_layer_idx, pos_start, M, max_phys_blocks,
                                  block_size, scale, stream);
}

// ---- the reference's two layer wrappers ---------------------------------------------------

namespace {
LinearForwardFn g_linear_forward = nullptr;
const float* g_rope_table = nullptr;
int g_rope_positions = 0;
}

void set_linear_forward(LinearForwardFn fn) { g_linear_forward = fn; }

void set_rope_table(const float* d_rope_table, int table_positions)
{
    g_rope_table = table_positions > 0 ? d_rope_table : nullptr;
    g_rope_positions = g_rope_table ? table_positions : 0;
}

// paged_attention.cu:314-376
void full_attention_forward_paged(const __half* x, const FullAttentionWeights& attn, __half* kv_pool,
                                  const int* d_block_table, int fa_layer_idx, int pos, int seq_len,
                                  int max_phys_blocks, int block_size, InferenceState& state, hipStream_t stream)
{
    using MC = ModelConfig;
    (void)pos;                                            // the kernels read the position from state.d_pos, as the reference's do
    if (!g_linear_forward) {
        LOG_ERROR("Machina", "full_attention_forward_paged: no projection registered (set_linear_forward)");
        return;
    }
    const int hd = MC::HEAD_DIM;
    // 1, 2: Q|gate, K and V projections (paged_attention.cu:326, 340-345)
    g_linear_forward(x, attn.fp16_q, state.q_buf, 1, stream);
    __half* k_buf = state.dn_z;
    __half* v_buf = state.dn_z + MC::NUM_KV_HEADS * hd;
    g_linear_forward(x, attn.fp16_k, k_buf, 1, stream);
    g_linear_forward(x, attn.fp16_v, v_buf, 1, stream);
    // 1b-5: split, per-head RMSNorm, partial RoPE, page write (paged_attention.cu:331-360), one launch
    __half* q_ptr = state.dn_qkv;
    paged_qk_norm_rope_write(state.q_buf, k_buf, v_buf, attn.q_norm, attn.k_norm, q_ptr, kv_pool, d_block_table,
                             fa_layer_idx, state.d_pos, max_phys_blocks, block_size, g_rope_table, g_rope_positions, stream);
    // 6: attention (paged_attention.cu:362-366)
    const float scale = 1.0f / std::sqrt((float)hd);
    paged_gqa_decode_attention(q_ptr, kv_pool, d_block_table, state.attn_out, fa_layer_idx, seq_len, max_phys_blocks,
                               block_size, scale, stream);
    // 7: gate, read where the projection left it (paged_attention.cu:368-370)
    if (drk_sigmoid_gate(state.attn_out, state.q_buf + hd, state.attn_out, (size_t)MC::NUM_ATTN_HEADS, hd, 2 * (size_t)hd,
                         MC::IO_DTYPE, stream) != DRK_OK)
        LOG_ERROR("Machina", "full_attention_forward_paged: gate: %s", drk_last_error());
    // 8: O projection (paged_attention.cu:372-374)
    g_linear_forward(state.attn_out, attn.fp16_o, state.norm_out, 1, stream);
}

// paged_attention.cu:563-638
void full_attention_forward_paged_prefill(const __half* x, const FullAttentionWeights& attn, __half* kv_pool,
                                          const int* d_block_table, int fa_layer_idx, int pos_start, int M,
                                          int seq_len, int max_phys_blocks, int block_size, InferenceState& state,
                                          hipStream_t stream)
{
    using MC = ModelConfig;
    (void)seq_len;                                        // = pos_start + M; the reference does not read it either
    if (M <= 0) return;
    if (!g_linear_forward) {
        LOG_ERROR("Machina", "full_attention_forward_paged_prefill: no projection registered (set_linear_forward)");
        return;
    }
    const int hd = MC::HEAD_DIM;
    // 1-3: projections (paged_attention.cu:576-582)
    g_linear_forward(x, attn.fp16_q, state.q_buf, M, stream);
    g_linear_forward(x, attn.fp16_k, state.kv_buf, M, stream);
    g_linear_forward(x, attn.fp16_v, state.dn_z, M, stream);
    // 4-7: split, norms, RoPE, page write (paged_attention.cu:587-619), one launch
    __half* q_sep = state.dn_qkv;
    paged_qk_norm_rope_write_batch(state.q_buf, state.kv_buf, state.dn_z, attn.q_norm, attn.k_norm, q_sep, kv_pool,
                                   d_block_table, fa_layer_idx, pos_start, M, max_phys_blocks, block_size, g_rope_table,
                                   g_rope_positions, stream);
    // 8, 9: causal attention with the gate in its epilogue (paged_attention.cu:621-634)
    paged_prefill_attention_gated(q_sep, kv_pool, d_block_table, state.q_buf + hd, 2 * hd, state.attn_out, fa_layer_idx,
                                  pos_start, M, max_phys_blocks, block_size, 1.0f / std::sqrt((float)hd), stream);
    // 10: O projection (paged_attention.cu:636-637)
    g_linear_forward(state.attn_out, attn.fp16_o, state.norm_out, M, stream);
}

} // namespace deusridet
