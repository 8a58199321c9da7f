/*
 * drk_host.h -- C shim over the C++ host classes (deusridet::CacheManager,
 * BlockPool, ImportanceScorer, ModelConfig and the paged_attention.h
 * functions), exported by libdeusridet_memoria.so for language bindings: the
 * Python tests and the benchmark drive the host classes through it.  C++ callers
 * include the class headers directly.  Every function forwards to the method of
 * the same name; see the headers under deusridet_amd/memoria and machina/paged_attention.h for
 * the semantics and the reference citations.
 */
#ifndef DRK_HOST_H
#define DRK_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ModelConfig::set_attention_geometry (src/machina/model.h:39-42, 73) */
int drkh_set_attention_geometry(int num_fa_layers, int num_attn_heads, int num_kv_heads, int head_dim,
                                int kv_dtype, int io_dtype);

/* ImportanceScorer (src/memoria/importance_scorer.h:25-67) */
void *drkh_scorer_create(void);
void  drkh_scorer_destroy(void *s);
int   drkh_scorer_init(void *s, int max_blocks, float decay);
int   drkh_scorer_init_detached(void *s, int max_blocks, float decay);
void  drkh_scorer_update(void *s, const float *d_block_scores, int num_blocks);
int   drkh_scorer_least_important(void *s, const int *ids, int n);
float drkh_scorer_score(void *s, int logical_block);
void  drkh_scorer_sync_to_host(void *s);
void  drkh_scorer_load_host_scores(void *s, const float *scores, int n);

/* CacheManager (src/memoria/cache_manager.h:52-169) and its BlockPool
 * (src/memoria/block_pool.h:58-123) */
void *drkh_cm_create(void);
void  drkh_cm_destroy(void *cm);
int   drkh_cm_init(void *cm, size_t kv_budget_bytes, int block_size, void *scorer, int max_branches);
/* with the overflow tier: cache_dir and a KVSwapper (src/memoria/cache_manager.h:60-64); the swapper is
 * initialised afterwards on the manager's pool with drkh_swapper_init */
int   drkh_cm_init_ssd(void *cm, size_t kv_budget_bytes, const char *cache_dir, int block_size, void *swapper,
                       void *scorer, int max_branches);
int   drkh_cm_ssd_blocks_used(void *cm);
void  drkh_cm_prefetch_block(void *cm, int branch, int logical_idx);
/* src/memoria/kv_swapper.h:50-114 */
void *drkh_swapper_create(void);
void  drkh_swapper_destroy(void *sw);
int   drkh_swapper_init(void *sw, void *cm, const char *ssd_dir, int staging_blocks);
void  drkh_swapper_shutdown(void *sw);
void  drkh_swapper_drain(void *sw);
int   drkh_swapper_pending(void *sw);
void  drkh_swapper_prefetch(void *sw, int logical_block_idx, const char *path);
int   drkh_swapper_is_prefetched(void *sw, int logical_block_idx);
size_t drkh_swapper_block_bytes(void *sw);
/* one synchronous request through the queue: direction 0 = GPU -> file, 1 = file -> GPU; returns success */
int   drkh_swapper_swap(void *sw, int direction, int logical_block_idx, int physical_block_id, const char *path);
/* n requests submitted one after the other, then drain(): completion_order[k] = index of the k-th request whose
 * callback ran, ok[i] = its result (either may be NULL); returns the number of callbacks.  physical_block_id < 0 with
 * direction 1 is a prefetch (file -> host cache). */
int   drkh_swapper_swap_many(void *sw, int n, const int32_t *direction, const int32_t *logical_block_idx,
                             const int32_t *physical_block_id, const char *const *path, int32_t *completion_order,
                             int32_t *ok);
void  drkh_swapper_remove_writer_stream(void *sw, void *stream);     /* KVSwapper::remove_writer_stream */
int   drkh_cm_init_detached(void *cm, int max_blocks, int block_size, void *scorer, int max_branches);
int   drkh_cm_ensure_blocks_for(void *cm, int branch, int pos);
int   drkh_cm_ensure_blocks_for_range(void *cm, int branch, int pos_start, int M);
void  drkh_cm_sync_block_table(void *cm, void *stream);
void  drkh_cm_forget_stream(void *cm, void *stream);      /* CacheManager::forget_stream: before the stream is destroyed */
const int32_t *drkh_cm_d_block_table(void *cm, int branch);
const int32_t *drkh_cm_h_block_table(void *cm, int branch);
int   drkh_cm_table_stride(void *cm);
int   drkh_cm_seq_len(void *cm, int branch);
void  drkh_cm_set_seq_len(void *cm, int branch, int len);
int   drkh_cm_num_logical_blocks(void *cm, int branch);
int   drkh_cm_fork_branch(void *cm, int parent, int pos);
void  drkh_cm_release_branch(void *cm, int branch);
void  drkh_cm_touch_block(void *cm, int branch, int logical);
int   drkh_cm_common_prefix_tokens(void *cm, const int32_t *branches, int n);
/* CacheManager::common_prefix_groups: out holds max_groups drk_prefix_group (4 x int32 each); returns the count */
int   drkh_cm_common_prefix_groups(void *cm, const int32_t *branches, int n, int max_group_branches, int min_tokens,
                                   int32_t *out, int max_groups);
int   drkh_cm_block_location(void *cm, int branch, int logical);
int   drkh_cm_evict_blocks(void *cm, int n);
int   drkh_cm_ensure_free_blocks(void *cm, int n_free);
int   drkh_cm_gpu_blocks_used(void *cm);
int   drkh_cm_free_blocks(void *cm);
int   drkh_cm_lru_snapshot(void *cm, int32_t *branch_out, int32_t *logical_out, int cap);
int   drkh_cm_take_pending_copies(void *cm, int32_t *src_out, int32_t *dst_out, int cap);
/* BlockPool through the manager */
int    drkh_pool_alloc_block(void *cm);
void   drkh_pool_free_block(void *cm, int id);
int    drkh_pool_free_count(void *cm);
int    drkh_pool_max_blocks(void *cm);
int    drkh_pool_block_size(void *cm);
int    drkh_pool_refcount(void *cm, int id);
void  *drkh_pool_ptr(void *cm);
size_t drkh_pool_k_offset(void *cm, int layer, int block);
size_t drkh_pool_v_offset(void *cm, int layer, int block);
size_t drkh_pool_total_bytes(void *cm);
int    drkh_pool_free_stack(void *cm, int32_t *out, int cap);

/* src/machina/paged_attention.h:27-73 and src/memoria/cache_kernels.h:44-74 */
void drkh_paged_kv_cache_write(const void *src_k, const void *src_v, void *kv_pool, const int32_t *d_block_table,
                               int fa_layer_idx, const int32_t *d_pos, int max_phys_blocks, int block_size,
                               void *stream);
void drkh_paged_kv_cache_write_batch(const void *src_k, const void *src_v, void *kv_pool,
                                     const int32_t *d_block_table, int fa_layer_idx, int pos_start, int M,
                                     int max_phys_blocks, int block_size, void *stream);
void drkh_paged_kv_cache_write_branches(const void *src_k, const void *src_v, void *kv_pool,
                                        const int32_t *d_tables, int table_stride, const int32_t *d_pos, int B,
                                        int fa_layer_idx, int max_phys_blocks, int block_size, void *stream);
void drkh_paged_gqa_decode_attention(const void *Q, void *kv_pool, const int32_t *d_block_table, void *out,
                                     int fa_layer_idx, int seq_len, int max_phys_blocks, int block_size,
                                     float scale, void *stream);
void drkh_paged_gqa_decode_attention_branches(const void *Q, void *kv_pool, const int32_t *d_tables,
                                              int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len,
                                              void *out, int fa_layer_idx, int max_phys_blocks, int block_size,
                                              float scale, void *stream);
void drkh_paged_gqa_decode_attention_shared(const void *Q, void *kv_pool, const int32_t *d_tables, int table_stride,
                                            const int32_t *d_seq_lens, int B, int max_seq_len, int shared_tokens,
                                            void *out, int fa_layer_idx, int max_phys_blocks, int block_size,
                                            float scale, void *stream);
/* branches that share pages as a fork tree (groups: n_groups x 4 int32 as drkh_cm_common_prefix_groups wrote them;
 * no reference counterpart) */
int  drkh_paged_gqa_decode_grouped_supported(int block_size);
void drkh_paged_gqa_decode_attention_grouped(const void *Q, void *kv_pool, const int32_t *d_tables, int table_stride,
                                             const int32_t *d_seq_lens, int B, int max_seq_len,
                                             const int32_t *groups, int n_groups, void *out, int fa_layer_idx,
                                             int max_phys_blocks, int block_size, float scale, void *stream);
void drkh_paged_prefill_attention(const void *Q, void *kv_pool, const int32_t *d_block_table, void *out,
                                  int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                                  float scale, void *stream);
/* src/machina/layer.h:77-79, 124-140 and the fused forms in machina/paged_attention.h */
int  drkh_set_rope(int rotary_dim, float theta, float rms_eps);
void drkh_sigmoid_gate(const void *x, const void *gate, void *out, int n, void *stream);
void drkh_apply_rope(void *q, void *k, int num_heads, int num_kv_heads, int head_dim, int rotary_dim,
                     const int32_t *d_pos, float theta, void *stream);
void drkh_head_norm(const void *x, const void *weight, void *out, int num_heads, int head_dim, float eps,
                    void *stream);
void drkh_paged_qk_norm_rope_write_batch(const void *qg, const void *k, const void *v, const void *q_norm,
                                         const void *k_norm, void *q_out, void *kv_pool,
                                         const int32_t *d_block_table, int fa_layer_idx, int pos_start, int M,
                                         int max_phys_blocks, int block_size, const float *d_rope_table,
                                         int table_positions, void *stream);
void drkh_paged_qk_norm_rope_write_branches(const void *qg, const void *k, const void *v, const void *q_norm,
                                            const void *k_norm, void *q_out, void *kv_pool, const int32_t *d_tables,
                                            int table_stride, const int32_t *d_pos, int B, int fa_layer_idx,
                                            int max_phys_blocks, int block_size, const float *d_rope_table,
                                            int table_positions, void *stream);
void drkh_paged_gqa_decode_attention_gated_branches(const void *Q, void *kv_pool, const int32_t *d_tables,
                                                    int table_stride, const int32_t *d_seq_lens, int B,
                                                    int max_seq_len, const void *gate, int gate_stride, void *out,
                                                    int fa_layer_idx, int max_phys_blocks, int block_size,
                                                    float scale, void *stream);
void drkh_paged_prefill_attention_gated(const void *Q, void *kv_pool, const int32_t *d_block_table, const void *gate,
                                        int gate_stride, void *out, int fa_layer_idx, int pos_start, int M,
                                        int max_phys_blocks, int block_size, float scale, void *stream);
/* conscientia/kv_stream.h: the KV side of ConscientiStream (src/conscientia/stream.cpp:145-401) */
void *drkh_kvs_create(void);
void  drkh_kvs_destroy(void *ks);
int   drkh_kvs_init(void *ks, void *cm, int max_context_len, void *scorer, const float *d_rope_table, int table_positions,
                    int max_prefill_rows);
int   drkh_kvs_begin_prefill(void *ks, int M, void *stream);
void  drkh_kvs_prefill_layer(void *ks, int fa_layer_idx, const void *qg, const void *k, const void *v, const void *q_norm,
                             const void *k_norm, void *q_scratch, void *attn_out, int M, void *stream);
void  drkh_kvs_end_prefill(void *ks, int M, void *stream);
int   drkh_kvs_current_pos(void *ks);
int   drkh_kvs_open_branches(void *ks, int n);
int   drkh_kvs_set_branch_count(void *ks, int n);
void  drkh_kvs_close_branches(void *ks);
int   drkh_kvs_num_branches(void *ks);
int   drkh_kvs_branch_id(void *ks, int i);
int   drkh_kvs_branch_pos(void *ks, int i);
int   drkh_kvs_shared_tokens(void *ks);
void  drkh_kvs_set_shared_prefix_policy(void *ks, int min_branches, int min_tokens);
int   drkh_kvs_begin_decode_step(void *ks, void *stream);
void  drkh_kvs_decode_layer(void *ks, int fa_layer_idx, const void *qg, const void *k, const void *v, const void *q_norm,
                            const void *k_norm, void *q_scratch, void *attn_out, void *stream);
void  drkh_kvs_end_decode_step(void *ks, void *stream);
/* layers(stream, user) enqueues one step's work (drkh_kvs_decode_layer per full-attention layer) */
int   drkh_kvs_capture_decode_step(void *ks, void (*layers)(void *stream, void *user), void *user, void *stream);
int   drkh_kvs_replay_decode_step(void *ks, void *stream);
void *drkh_scorer_d_new_scores(void *s);
void drkh_scorer_apply_new_scores(void *s, void *stream);
void  drkh_scorer_apply_new_scores_range(void *sc, int first, int count, void *stream);   /* cells [first, first + count): folded and their new scores cleared */
void drkh_paged_gqa_decode_attention_branches_scored(const void *Q, void *kv_pool, const int32_t *d_tables,
                                                     int table_stride, const int32_t *d_seq_lens, int B,
                                                     int max_seq_len, void *out, int fa_layer_idx,
                                                     int max_phys_blocks, int block_size, float scale,
                                                     float *d_block_mass, int accumulate, void *stream);
/* the workspace of `stream` (the calls above keep one per stream) */
int  drkh_paged_attention_reserve_workspace(int max_branches, int max_seq_len, int max_prefill_rows, int block_size,
                                            void *stream);
size_t drkh_paged_attention_workspace_bytes(int max_branches, int max_seq_len, int max_prefill_rows, int block_size);
/* full_attention_forward_paged / _paged_prefill (src/machina/paged_attention.h:75-106) with the four
 * projections served from buffers instead of GEMMs (which are the model's code): qg_proj [M, QH, 2 D],
 * k_proj, v_proj [M, KVH, D] are what the Q|gate, K and V projections would produce; the gated attention
 * output passes through the "O projection" unchanged.  state_bufs = {q_buf, kv_buf, dn_z, dn_qkv,
 * attn_out, norm_out} (InferenceState, src/machina/model.h:232-293). */
void drkh_set_rope_table(const float *d_rope_table, int table_positions);
void drkh_full_attention_forward_paged(const void *qg_proj, const void *k_proj, const void *v_proj, const void *q_norm,
                                       const void *k_norm, void *kv_pool, const int32_t *d_block_table, int fa_layer_idx,
                                       int pos, int seq_len, int max_phys_blocks, int block_size, void *const *state_bufs,
                                       int32_t *d_pos, void *stream);
void drkh_full_attention_forward_paged_prefill(const void *qg_proj, const void *k_proj, const void *v_proj,
                                               const void *q_norm, const void *k_norm, void *kv_pool,
                                               const int32_t *d_block_table, int fa_layer_idx, int pos_start, int M,
                                               int seq_len, int max_phys_blocks, int block_size, void *const *state_bufs,
                                               void *stream);
void drkh_paged_attention_release_workspace(void);
void drkh_invoke_extract_kv_from_pages(void *dst, const void *kv_pool, const int32_t *block_table, int start_token,
                                       int num_tokens, int num_layers, int num_kv_heads, int head_dim,
                                       int block_size, int max_phys_blocks, void *stream);
void drkh_invoke_inject_kv_to_pages(void *kv_pool, const void *src, const int32_t *block_table, int start_token,
                                    int num_tokens, int num_layers, int num_kv_heads, int head_dim, int block_size,
                                    int max_phys_blocks, void *stream);

#ifdef __cplusplus
}
#endif
#endif
