// host_capi.cpp -- the C shim declared in include/drk_host.h: one-line forwarders
// to the C++ host classes.
#include <mutex>
#include "drk_host.h"

#include "../machina/paged_attention.h"
#include "../machina/layer.h"
#include "../memoria/kv_swapper.h"
#include "../conscientia/kv_stream.h"
#include "../memoria/cache_kernels.h"
#include "../memoria/cache_manager.h"

#include <algorithm>

using namespace deusridet;

#define CM(p) (static_cast<CacheManager *>(p))
#define SC(p) (static_cast<ImportanceScorer *>(p))
#define SW(p) (static_cast<KVSwapper *>(p))
#define KS(p) (static_cast<KvStream *>(p))
#define H(p) (reinterpret_cast<__half *>(p))
#define CH(p) (reinterpret_cast<const __half *>(p))
#define ST(p) (static_cast<hipStream_t>(p))

extern "C" {

int drkh_set_attention_geometry(int num_fa_layers, int num_attn_heads, int num_kv_heads, int head_dim, int kv_dtype,
                                int io_dtype)
{
    return ModelConfig::set_attention_geometry(num_fa_layers, num_attn_heads, num_kv_heads, head_dim, kv_dtype,
                                               io_dtype) ? 1 : 0;
}

void *drkh_scorer_create(void) { return new ImportanceScorer(); }
void drkh_scorer_destroy(void *s) { delete SC(s); }
int drkh_scorer_init(void *s, int max_blocks, float decay) { return SC(s)->init(max_blocks, decay) ? 1 : 0; }
int drkh_scorer_init_detached(void *s, int max_blocks, float decay) { return SC(s)->init_detached(max_blocks, decay) ? 1 : 0; }
void drkh_scorer_update(void *s, const float *d, int n) { SC(s)->update(d, n); }
int drkh_scorer_least_important(void *s, const int *ids, int n) { return SC(s)->least_important(ids, n); }
float drkh_scorer_score(void *s, int b) { return SC(s)->score(b); }
void drkh_scorer_sync_to_host(void *s) { SC(s)->sync_to_host(); }
void drkh_scorer_load_host_scores(void *s, const float *scores, int n) { SC(s)->load_host_scores(scores, n); }

void *drkh_cm_create(void) { return new CacheManager(); }
void drkh_cm_destroy(void *cm) { delete CM(cm); }
int drkh_cm_init(void *cm, size_t budget, int block_size, void *scorer, int max_branches)
{
    return CM(cm)->init(budget, "", block_size, nullptr, SC(scorer), max_branches) ? 1 : 0;
}
int drkh_cm_init_ssd(void *cm, size_t budget, const char *cache_dir, int block_size, void *swapper, void *scorer,
                     int max_branches)
{
    return CM(cm)->init(budget, cache_dir ? cache_dir : "", block_size, SW(swapper), SC(scorer), max_branches) ? 1 : 0;
}
int drkh_cm_ssd_blocks_used(void *cm) { return CM(cm)->ssd_blocks_used(); }
void drkh_cm_prefetch_block(void *cm, int branch, int logical_idx) { CM(cm)->prefetch_block(branch, logical_idx); }
void *drkh_swapper_create(void) { return new KVSwapper(); }
void drkh_swapper_destroy(void *sw) { delete SW(sw); }
int drkh_swapper_init(void *sw, void *cm, const char *ssd_dir, int staging_blocks)
{
    return SW(sw)->init(CM(cm)->block_pool(), ssd_dir ? ssd_dir : "", staging_blocks) ? 1 : 0;
}
void drkh_swapper_shutdown(void *sw) { SW(sw)->shutdown(); }
void drkh_swapper_drain(void *sw) { SW(sw)->drain(); }
int drkh_swapper_pending(void *sw) { return SW(sw)->pending(); }
void drkh_swapper_prefetch(void *sw, int logical_block_idx, const char *path) { SW(sw)->prefetch(logical_block_idx, path ? path : ""); }
int drkh_swapper_is_prefetched(void *sw, int logical_block_idx) { return SW(sw)->is_prefetched(logical_block_idx) ? 1 : 0; }
size_t drkh_swapper_block_bytes(void *sw) { return SW(sw)->block_bytes(); }
int drkh_swapper_swap(void *sw, int direction, int logical_block_idx, int physical_block_id, const char *path)
{
    bool success = false;
    SwapRequest req;
    req.direction = direction == 0 ? SwapDirection::GPU_TO_SSD : SwapDirection::SSD_TO_GPU;
    req.logical_block_idx = logical_block_idx;
    req.physical_block_id = physical_block_id;
    req.ssd_path = path ? path : "";
    req.callback = [&success](bool ok) { success = ok; };
    SW(sw)->submit(std::move(req));
    SW(sw)->drain();
    return success ? 1 : 0;
}
int drkh_swapper_swap_many(void *sw, int n, const int32_t *direction, const int32_t *logical_block_idx,
                           const int32_t *physical_block_id, const char *const *path, int32_t *completion_order,
                           int32_t *ok)
{
    std::mutex mu;
    int done = 0;
    for (int i = 0; i < n; i++) {
        SwapRequest req;
        req.direction = direction[i] == 0 ? SwapDirection::GPU_TO_SSD : SwapDirection::SSD_TO_GPU;
        req.logical_block_idx = logical_block_idx[i];
        req.physical_block_id = physical_block_id[i];
        req.ssd_path = path[i] ? path[i] : "";
        req.callback = [&, i](bool success) {
            std::lock_guard<std::mutex> lock(mu);
            if (completion_order) completion_order[done] = i;
            if (ok) ok[i] = success ? 1 : 0;
            done++;
        };
        SW(sw)->submit(std::move(req));
    }
    SW(sw)->drain();
    std::lock_guard<std::mutex> lock(mu);
    return done;
}
void drkh_swapper_remove_writer_stream(void *sw, void *stream) { SW(sw)->remove_writer_stream(ST(stream)); }
int drkh_cm_init_detached(void *cm, int max_blocks, int block_size, void *scorer, int max_branches)
{
    return CM(cm)->init_detached(max_blocks, block_size, SC(scorer), max_branches) ? 1 : 0;
}
int drkh_cm_ensure_blocks_for(void *cm, int branch, int pos) { return CM(cm)->ensure_blocks_for(branch, pos) ? 1 : 0; }
int drkh_cm_ensure_blocks_for_range(void *cm, int branch, int pos_start, int M)
{
    return CM(cm)->ensure_blocks_for_range(branch, pos_start, M) ? 1 : 0;
}
void drkh_cm_sync_block_table(void *cm, void *stream) { CM(cm)->sync_block_table(ST(stream)); }
void drkh_cm_forget_stream(void *cm, void *stream) { CM(cm)->forget_stream(ST(stream)); }
const int32_t *drkh_cm_d_block_table(void *cm, int branch) { return CM(cm)->d_block_table(branch); }
const int32_t *drkh_cm_h_block_table(void *cm, int branch) { return CM(cm)->h_block_table(branch); }
int drkh_cm_table_stride(void *cm) { return CM(cm)->table_stride(); }
int drkh_cm_seq_len(void *cm, int branch) { return CM(cm)->seq_len(branch); }
void drkh_cm_set_seq_len(void *cm, int branch, int len) { CM(cm)->set_seq_len(branch, len); }
int drkh_cm_num_logical_blocks(void *cm, int branch) { return CM(cm)->num_logical_blocks(branch); }
int drkh_cm_fork_branch(void *cm, int parent, int pos) { return CM(cm)->fork_branch(parent, pos); }
void drkh_cm_release_branch(void *cm, int branch) { CM(cm)->release_branch(branch); }
void drkh_cm_touch_block(void *cm, int branch, int logical) { CM(cm)->touch_block(branch, logical); }
int drkh_cm_common_prefix_tokens(void *cm, const int32_t *branches, int n) { return CM(cm)->common_prefix_tokens(branches, n); }
int drkh_cm_common_prefix_groups(void *cm, const int32_t *branches, int n, int max_group_branches, int min_tokens, int32_t *out, int max_groups)
{
    return CM(cm)->common_prefix_groups(branches, n, max_group_branches, min_tokens, (drk_prefix_group *)out, max_groups);
}
int drkh_cm_block_location(void *cm, int branch, int logical) { return (int)CM(cm)->block_location(branch, logical); }
int drkh_cm_evict_blocks(void *cm, int n) { return CM(cm)->evict_blocks(n); }
int drkh_cm_ensure_free_blocks(void *cm, int n_free) { return CM(cm)->ensure_free_blocks(n_free) ? 1 : 0; }
int drkh_cm_gpu_blocks_used(void *cm) { return CM(cm)->gpu_blocks_used(); }
int drkh_cm_free_blocks(void *cm) { return CM(cm)->free_blocks(); }

int drkh_cm_lru_snapshot(void *cm, int32_t *bo, int32_t *lo, int cap)
{
    auto v = CM(cm)->lru_snapshot();
    int n = std::min<int>(cap, (int)v.size());
    for (int i = 0; i < n; i++) { bo[i] = v[i].first; lo[i] = v[i].second; }
    return (int)v.size();
}
int drkh_cm_take_pending_copies(void *cm, int32_t *so, int32_t *dn, int cap)
{
    auto v = CM(cm)->take_pending_copies();
    int n = std::min<int>(cap, (int)v.size());
    for (int i = 0; i < n; i++) { so[i] = v[i].first; dn[i] = v[i].second; }
    return (int)v.size();
}

int drkh_pool_alloc_block(void *cm) { return CM(cm)->block_pool().alloc_block(); }
void drkh_pool_free_block(void *cm, int id) { CM(cm)->block_pool().free_block(id); }
int drkh_pool_free_count(void *cm) { return CM(cm)->block_pool().free_count(); }
int drkh_pool_max_blocks(void *cm) { return CM(cm)->block_pool().max_blocks(); }
int drkh_pool_block_size(void *cm) { return CM(cm)->block_pool().block_size(); }
int drkh_pool_refcount(void *cm, int id) { return CM(cm)->block_pool().refcount(id); }
void *drkh_pool_ptr(void *cm) { return CM(cm)->block_pool().pool_raw(); }
size_t drkh_pool_k_offset(void *cm, int layer, int block) { return CM(cm)->block_pool().k_offset(layer, block); }
size_t drkh_pool_v_offset(void *cm, int layer, int block) { return CM(cm)->block_pool().v_offset(layer, block); }
size_t drkh_pool_total_bytes(void *cm) { return CM(cm)->block_pool().total_bytes(); }
int drkh_pool_free_stack(void *cm, int32_t *out, int cap)
{
    auto v = CM(cm)->block_pool().free_stack_snapshot();
    int n = std::min<int>(cap, (int)v.size());
    for (int i = 0; i < n; i++) out[i] = v[i];
    return (int)v.size();
}

void drkh_paged_kv_cache_write(const void *src_k, const void *src_v, void *kv_pool, const int32_t *d_block_table,
                               int fa_layer_idx, const int32_t *d_pos, int max_phys_blocks, int block_size,
                               void *stream)
{
    paged_kv_cache_write(CH(src_k), CH(src_v), H(kv_pool), d_block_table, fa_layer_idx, d_pos, max_phys_blocks,
                         block_size, ST(stream));
}
void drkh_paged_kv_cache_write_batch(const void *src_k, const void *src_v, void *kv_pool,
                                     const int32_t *d_block_table, int fa_layer_idx, int pos_start, int M,
                                     int max_phys_blocks, int block_size, void *stream)
{
    paged_kv_cache_write_batch(CH(src_k), CH(src_v), H(kv_pool), d_block_table, fa_layer_idx, pos_start, M,
                               max_phys_blocks, block_size, ST(stream));
}
void drkh_paged_kv_cache_write_branches(const void *src_k, const void *src_v, void *kv_pool,
                                        const int32_t *d_tables, int table_stride, const int32_t *d_pos, int B,
                                        int fa_layer_idx, int max_phys_blocks, int block_size, void *stream)
{
    paged_kv_cache_write_branches(CH(src_k), CH(src_v), H(kv_pool), d_tables, table_stride, d_pos, B, fa_layer_idx,
                                  max_phys_blocks, block_size, ST(stream));
}
void drkh_paged_gqa_decode_attention(const void *Q, void *kv_pool, const int32_t *d_block_table, void *out,
                                     int fa_layer_idx, int seq_len, int max_phys_blocks, int block_size,
                                     float scale, void *stream)
{
    paged_gqa_decode_attention(CH(Q), H(kv_pool), d_block_table, H(out), fa_layer_idx, seq_len, max_phys_blocks,
                               block_size, scale, ST(stream));
}
void drkh_paged_gqa_decode_attention_branches(const void *Q, void *kv_pool, const int32_t *d_tables,
                                              int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len,
                                              void *out, int fa_layer_idx, int max_phys_blocks, int block_size,
                                              float scale, void *stream)
{
    paged_gqa_decode_attention_branches(CH(Q), H(kv_pool), d_tables, table_stride, d_seq_lens, B, max_seq_len,
                                        H(out), fa_layer_idx, max_phys_blocks, block_size, scale, ST(stream));
}
void drkh_paged_gqa_decode_attention_shared(const void *Q, void *kv_pool, const int32_t *d_tables, int table_stride,
                                            const int32_t *d_seq_lens, int B, int max_seq_len, int shared_tokens,
                                            void *out, int fa_layer_idx, int max_phys_blocks, int block_size,
                                            float scale, void *stream)
{
    paged_gqa_decode_attention_shared(CH(Q), H(kv_pool), d_tables, table_stride, d_seq_lens, B, max_seq_len,
                                      shared_tokens, H(out), fa_layer_idx, max_phys_blocks, block_size, scale,
                                      ST(stream));
}
int drkh_paged_gqa_decode_grouped_supported(int block_size) { return paged_gqa_decode_grouped_supported(block_size) ? 1 : 0; }
void drkh_paged_gqa_decode_attention_grouped(const void *Q, void *kv_pool, const int32_t *d_tables, int table_stride,
                                             const int32_t *d_seq_lens, int B, int max_seq_len,
                                             const int32_t *groups, int n_groups, void *out, int fa_layer_idx,
                                             int max_phys_blocks, int block_size, float scale, void *stream)
{
    paged_gqa_decode_attention_grouped(CH(Q), H(kv_pool), d_tables, table_stride, d_seq_lens, B, max_seq_len,
                                       reinterpret_cast<const drk_prefix_group *>(groups),
                                       n_groups, H(out), fa_layer_idx, max_phys_blocks, block_size, scale, ST(stream));
}
void drkh_paged_prefill_attention(const void *Q, void *kv_pool, const int32_t *d_block_table, void *out,
                                  int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                                  float scale, void *stream)
{
    paged_prefill_attention(CH(Q), H(kv_pool), d_block_table, H(out), fa_layer_idx, pos_start, M, max_phys_blocks,
                            block_size, scale, ST(stream));
}
int drkh_set_rope(int rotary_dim, float theta, float rms_eps) { return ModelConfig::set_rope(rotary_dim, theta, rms_eps) ? 1 : 0; }
void drkh_sigmoid_gate(const void *x, const void *gate, void *out, int n, void *stream)
{
    sigmoid_gate(CH(x), CH(gate), H(out), n, (hipStream_t)stream);
}
void drkh_apply_rope(void *q, void *k, int num_heads, int num_kv_heads, int head_dim, int rotary_dim,
                     const int32_t *d_pos, float theta, void *stream)
{
    apply_rope(H(q), H(k), num_heads, num_kv_heads, head_dim, rotary_dim, d_pos, theta, (hipStream_t)stream);
}
void drkh_head_norm(const void *x, const void *weight, void *out, int num_heads, int head_dim, float eps,
                    void *stream)
{
    head_norm(CH(x), CH(weight), H(out), num_heads, head_dim, eps, (hipStream_t)stream);
}
void drkh_paged_qk_norm_rope_write_batch(const void *qg, const void *k, const void *v, const void *q_norm,
                                         const void *k_norm, void *q_out, void *kv_pool,
                                         const int32_t *d_block_table, int fa_layer_idx, int pos_start, int M,
                                         int max_phys_blocks, int block_size, const float *d_rope_table,
                                         int table_positions, void *stream)
{
    paged_qk_norm_rope_write_batch(CH(qg), CH(k), CH(v), CH(q_norm), CH(k_norm), H(q_out), H(kv_pool), d_block_table,
                                   fa_layer_idx, pos_start, M, max_phys_blocks, block_size, d_rope_table,
                                   table_positions, (hipStream_t)stream);
}
void drkh_paged_qk_norm_rope_write_branches(const void *qg, const void *k, const void *v, const void *q_norm,
                                            const void *k_norm, void *q_out, void *kv_pool, const int32_t *d_tables,
                                            int table_stride, const int32_t *d_pos, int B, int fa_layer_idx,
                                            int max_phys_blocks, int block_size, const float *d_rope_table,
                                            int table_positions, void *stream)
{
    paged_qk_norm_rope_write_branches(CH(qg), CH(k), CH(v), CH(q_norm), CH(k_norm), H(q_out), H(kv_pool), d_tables,
                                      table_stride, d_pos, B, fa_layer_idx, max_phys_blocks, block_size, d_rope_table,
                                      table_positions, (hipStream_t)stream);
}
void drkh_paged_gqa_decode_attention_gated_branches(const void *Q, void *kv_pool, const int32_t *d_tables,
                                                    int table_stride, const int32_t *d_seq_lens, int B,
                                                    int max_seq_len, const void *gate, int gate_stride, void *out,
                                                    int fa_layer_idx, int max_phys_blocks, int block_size,
                                                    float scale, void *stream)
{
    paged_gqa_decode_attention_gated_branches(CH(Q), H(kv_pool), d_tables, table_stride, d_seq_lens, B, max_seq_len,
                                              CH(gate), gate_stride, H(out), fa_layer_idx, max_phys_blocks,
                                              block_size, scale, (hipStream_t)stream);
}
void drkh_paged_prefill_attention_gated(const void *Q, void *kv_pool, const int32_t *d_block_table, const void *gate,
                                        int gate_stride, void *out, int fa_layer_idx, int pos_start, int M,
                                        int max_phys_blocks, int block_size, float scale, void *stream)
{
    paged_prefill_attention_gated(CH(Q), H(kv_pool), d_block_table, CH(gate), gate_stride, H(out), fa_layer_idx,
                                  pos_start, M, max_phys_blocks, block_size, scale, (hipStream_t)stream);
}
static KvLayerIO make_io(const void *qg, const void *k, const void *v, const void *q_norm, const void *k_norm,
                         void *q_scratch, void *attn_out)
{
    return KvLayerIO{CH(qg), CH(k), CH(v), CH(q_norm), CH(k_norm), H(q_scratch), H(attn_out)};
}
void *drkh_kvs_create(void) { return new KvStream(); }
void drkh_kvs_destroy(void *ks) { delete KS(ks); }
int drkh_kvs_init(void *ks, void *cm, int max_context_len, void *scorer, const float *d_rope_table, int table_positions,
                  int max_prefill_rows)
{
    return KS(ks)->init(*CM(cm), max_context_len, SC(scorer), d_rope_table, table_positions, max_prefill_rows) ? 1 : 0;
}
int drkh_kvs_begin_prefill(void *ks, int M, void *stream) { return KS(ks)->begin_prefill(M, (hipStream_t)stream) ? 1 : 0; }
void drkh_kvs_prefill_layer(void *ks, int fa_layer_idx, const void *qg, const void *k, const void *v, const void *q_norm,
                            const void *k_norm, void *q_scratch, void *attn_out, int M, void *stream)
{
    KS(ks)->prefill_layer(fa_layer_idx, make_io(qg, k, v, q_norm, k_norm, q_scratch, attn_out), M, (hipStream_t)stream);
}
void drkh_kvs_end_prefill(void *ks, int M, void *stream) { KS(ks)->end_prefill(M, (hipStream_t)stream); }
int drkh_kvs_current_pos(void *ks) { return KS(ks)->current_pos(); }
int drkh_kvs_open_branches(void *ks, int n) { return KS(ks)->open_branches(n); }
int drkh_kvs_set_branch_count(void *ks, int n) { return KS(ks)->set_branch_count(n); }
void drkh_kvs_close_branches(void *ks) { KS(ks)->close_branches(); }
int drkh_kvs_num_branches(void *ks) { return KS(ks)->num_branches(); }
int drkh_kvs_branch_id(void *ks, int i) { return KS(ks)->branch_id(i); }
int drkh_kvs_branch_pos(void *ks, int i) { return KS(ks)->branch_pos(i); }
int drkh_kvs_shared_tokens(void *ks) { return KS(ks)->shared_tokens(); }
void drkh_kvs_set_shared_prefix_policy(void *ks, int min_branches, int min_tokens) { KS(ks)->set_shared_prefix_policy(min_branches, min_tokens); }
int drkh_kvs_begin_decode_step(void *ks, void *stream) { return KS(ks)->begin_decode_step((hipStream_t)stream) ? 1 : 0; }
void drkh_kvs_decode_layer(void *ks, int fa_layer_idx, const void *qg, const void *k, const void *v, const void *q_norm,
                           const void *k_norm, void *q_scratch, void *attn_out, void *stream)
{
    KS(ks)->decode_layer(fa_layer_idx, make_io(qg, k, v, q_norm, k_norm, q_scratch, attn_out), (hipStream_t)stream);
}
void drkh_kvs_end_decode_step(void *ks, void *stream) { KS(ks)->end_decode_step((hipStream_t)stream); }
int drkh_kvs_capture_decode_step(void *ks, void (*layers)(void *stream, void *user), void *user, void *stream)
{
    return KS(ks)->capture_decode_step([&](hipStream_t s) { layers((void *)s, user); }, (hipStream_t)stream) ? 1 : 0;
}
int drkh_kvs_replay_decode_step(void *ks, void *stream) { return KS(ks)->replay_decode_step((hipStream_t)stream) ? 1 : 0; }
void *drkh_scorer_d_new_scores(void *s) { return SC(s)->d_new_scores(); }
void drkh_scorer_apply_new_scores(void *s, void *stream) { SC(s)->apply_new_scores((hipStream_t)stream); }
void drkh_scorer_apply_new_scores_range(void *sc, int first, int count, void *stream) { SC(sc)->apply_new_scores(first, count, ST(stream)); }
void drkh_paged_gqa_decode_attention_branches_scored(const void *Q, void *kv_pool, const int32_t *d_tables,
                                                     int table_stride, const int32_t *d_seq_lens, int B,
                                                     int max_seq_len, void *out, int fa_layer_idx,
                                                     int max_phys_blocks, int block_size, float scale,
                                                     float *d_block_mass, int accumulate, void *stream)
{
    paged_gqa_decode_attention_branches_scored(CH(Q), H(kv_pool), d_tables, table_stride, d_seq_lens, B, max_seq_len,
                                               H(out), fa_layer_idx, max_phys_blocks, block_size, scale, d_block_mass,
                                               accumulate != 0, (hipStream_t)stream);
}
int drkh_paged_attention_reserve_workspace(int max_branches, int max_seq_len, int max_prefill_rows, int block_size,
                                           void *stream)
{
    return paged_attention_reserve_workspace(max_branches, max_seq_len, max_prefill_rows, block_size, ST(stream)) ? 1 : 0;
}
size_t drkh_paged_attention_workspace_bytes(int max_branches, int max_seq_len, int max_prefill_rows, int block_size)
{
    return paged_attention_workspace_bytes(max_branches, max_seq_len, max_prefill_rows, block_size);
}

// The two layer wrappers with the projections served from buffers: the GEMMs are the model's
// code, so the shim registers a stand-in that copies M rows of a precomputed projection
// (Linear::weight points at it) into place, and passes the gated attention output through
// as the "O projection" (weight NULL).
static void projection_from_buffer(const __half *x, const Linear &w, __half *y, int M, hipStream_t stream)
{
    const void *src = w.weight ? (const void *)w.weight : (const void *)x;
    drk_memcpy_d2d_async(y, src, (size_t)M * w.out_features * sizeof(__half), stream);
}

static void wrapper_operands(FullAttentionWeights &attn, InferenceState &st, const void *qg_proj, const void *k_proj,
                             const void *v_proj, const void *q_norm, const void *k_norm, void *const *state_bufs,
                             int32_t *d_pos)
{
    const int qd = ModelConfig::NUM_ATTN_HEADS * ModelConfig::HEAD_DIM, kd = ModelConfig::NUM_KV_HEADS * ModelConfig::HEAD_DIM;
    attn.fp16_q.weight = H(const_cast<void *>(qg_proj)); attn.fp16_q.out_features = 2 * qd;
    attn.fp16_k.weight = H(const_cast<void *>(k_proj));  attn.fp16_k.out_features = kd;
    attn.fp16_v.weight = H(const_cast<void *>(v_proj));  attn.fp16_v.out_features = kd;
    attn.fp16_o.weight = nullptr;                        attn.fp16_o.out_features = qd;
    attn.q_norm = H(const_cast<void *>(q_norm));
    attn.k_norm = H(const_cast<void *>(k_norm));
    st.q_buf = H(state_bufs[0]); st.kv_buf = H(state_bufs[1]); st.dn_z = H(state_bufs[2]); st.dn_qkv = H(state_bufs[3]);
    st.attn_out = H(state_bufs[4]); st.norm_out = H(state_bufs[5]);
    st.d_pos = d_pos;
    set_linear_forward(projection_from_buffer);
}

void drkh_set_rope_table(const float *d_rope_table, int table_positions) { set_rope_table(d_rope_table, table_positions); }

void drkh_full_attention_forward_paged(const void *qg_proj, const void *k_proj, const void *v_proj, const void *q_norm,
                                       const void *k_norm, void *kv_pool, const int32_t *d_block_table, int fa_layer_idx,
                                       int pos, int seq_len, int max_phys_blocks, int block_size, void *const *state_bufs,
                                       int32_t *d_pos, void *stream)
{
    FullAttentionWeights attn;
    InferenceState st;
    wrapper_operands(attn, st, qg_proj, k_proj, v_proj, q_norm, k_norm, state_bufs, d_pos);
    full_attention_forward_paged(nullptr, attn, H(kv_pool), d_block_table, fa_layer_idx, pos, seq_len, max_phys_blocks,
                                 block_size, st, ST(stream));
}

void drkh_full_attention_forward_paged_prefill(const void *qg_proj, const void *k_proj, const void *v_proj,
                                               const void *q_norm, const void *k_norm, void *kv_pool,
                                               const int32_t *d_block_table, int fa_layer_idx, int pos_start, int M,
                                               int seq_len, int max_phys_blocks, int block_size, void *const *state_bufs,
                                               void *stream)
{
    FullAttentionWeights attn;
    InferenceState st;
    wrapper_operands(attn, st, qg_proj, k_proj, v_proj, q_norm, k_norm, state_bufs, nullptr);
    full_attention_forward_paged_prefill(nullptr, attn, H(kv_pool), d_block_table, fa_layer_idx, pos_start, M, seq_len,
                                         max_phys_blocks, block_size, st, ST(stream));
}
void drkh_paged_attention_release_workspace(void) { paged_attention_release_workspace(); }
void drkh_invoke_extract_kv_from_pages(void *dst, const void *kv_pool, const int32_t *block_table, int start_token,
                                       int num_tokens, int num_layers, int num_kv_heads, int head_dim,
                                       int block_size, int max_phys_blocks, void *stream)
{
    invoke_extract_kv_from_pages_typed(dst, nullptr, kv_pool, block_table, start_token, num_tokens, num_layers,
                                       num_kv_heads, head_dim, block_size, max_phys_blocks, ModelConfig::KV_DTYPE,
                                       ST(stream));
}
void drkh_invoke_inject_kv_to_pages(void *kv_pool, const void *src, const int32_t *block_table, int start_token,
                                    int num_tokens, int num_layers, int num_kv_heads, int head_dim, int block_size,
                                    int max_phys_blocks, void *stream)
{
    invoke_inject_kv_to_pages_typed(kv_pool, src, nullptr, block_table, start_token, num_tokens, num_layers,
                                    num_kv_heads, head_dim, block_size, max_phys_blocks, ModelConfig::KV_DTYPE,
                                    ST(stream));
}

} // extern "C"
