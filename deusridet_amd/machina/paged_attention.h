// paged_attention.h -- paged KV-cache write and paged GQA attention.  The first
// three functions have the reference's names, parameter order and meaning
// (src/machina/paged_attention.h:27-73) with HIP vocabulary types; head counts
// and head_dim come from ModelConfig's runtime statics exactly as in the
// reference's launchers (paged_attention.cu:110-114, 276-281).  Element types:
// ModelConfig::KV_DTYPE for the pool, ModelConfig::IO_DTYPE for Q / out / sources
// (both fp16 by default, as in the reference); the `__half*` in the signatures
// is then just "16-bit element".
//
// Launchers return void, are asynchronous on `stream`, and log a failure
// (the reference's launchers check nothing).  Order of use is write-then-attend:
// the token written at `pos` is visible to its own query, seq_len = pos + 1
// (paged_attention.cu:359-368, stream.cpp:319-334).
//
// The two full-layer wrappers of the reference (full_attention_forward_paged*,
// paged_attention.h:75-106) are at the end of this header: every step but the four
// projections is this library's; the projections go through a function the model code
// registers (set_linear_forward).
//
// Split-K partials.  The attention calls keep partial results in device memory.  The calls
// with the reference's signatures take that memory from a workspace this library keeps PER
// STREAM, so that a prefill on one stream and a decode on another never share partials.
// Such a workspace grows on demand -- by a new allocation; the old buffer is kept until
// paged_attention_release_workspace(), so work already enqueued, or a captured graph, never
// loses the memory it was launched with -- and never while its stream is being captured.
// Overloads that take an AttentionWorkspace use the caller's buffer instead and never
// allocate: a decode call that does not fit logs an error and launches nothing, a short
// prefill chunk that does not fit runs unsplit.
#pragma once

#include "model.h"
#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

namespace deusridet {

// Device memory for split-K partials, owned by the caller: reserved once, never moved.
class AttentionWorkspace {
public:
    AttentionWorkspace() = default;
    ~AttentionWorkspace();
    AttentionWorkspace(const AttentionWorkspace&) = delete;
    AttentionWorkspace& operator=(const AttentionWorkspace&) = delete;

    // Allocates `bytes` (16-byte aligned).  True when the workspace already holds at least
    // that much; false -- and nothing changes -- when it holds less (it is never reallocated:
    // launches already enqueued, or a captured graph, may be using it) or the allocation fails.
    bool reserve(size_t bytes);
    // Enough for every attention call of up to max_branches branches (and the shared-prefix and
    // scored variants), contexts up to max_seq_len and prefill chunks of up to max_prefill_rows.
    bool reserve_for(int max_branches, int max_seq_len, int max_prefill_rows, int block_size);
    // Frees the buffer; the caller makes sure nothing on the device still uses it.
    void release();
    void*  ptr() const { return ptr_; }
    size_t bytes() const { return bytes_; }

private:
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
};

// The size AttentionWorkspace::reserve_for allocates.
size_t paged_attention_workspace_bytes(int max_branches, int max_seq_len, int max_prefill_rows, int block_size);

// ---- the reference's entry points --------------------------------------------
void paged_kv_cache_write(const __half* src_k, const __half* src_v, __half* kv_pool, const int* d_block_table,
                          int fa_layer_idx, const int* d_pos, int max_phys_blocks, int block_size,
                          hipStream_t stream = 0);

void paged_kv_cache_write_batch(const __half* src_k, const __half* src_v, __half* kv_pool, const int* d_block_table,
                                int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                                hipStream_t stream = 0);

void paged_gqa_decode_attention(const __half* Q, __half* kv_pool, const int* d_block_table, __half* out,
                                int fa_layer_idx, int seq_len, int max_phys_blocks, int block_size, float scale,
                                hipStream_t stream = 0);

// The attention step of the reference's prefill wrapper (static kernel launched at
// paged_attention.cu:621-630): Q/out [M, NUM_ATTN_HEADS, HEAD_DIM], row t sees
// tokens 0 .. pos_start + t.
void paged_prefill_attention(const __half* Q, __half* kv_pool, const int* d_block_table, __half* out,
                             int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                             float scale, hipStream_t stream = 0);

// ---- several decode branches in one launch (not in the reference) ------------
// d_tables [B, table_stride] (CacheManager::d_block_tables()), d_pos / d_seq_lens
// [B] on the device, src [B, NUM_KV_HEADS, HEAD_DIM], Q/out [B, NUM_ATTN_HEADS,
// HEAD_DIM]; max_seq_len bounds every d_seq_lens[b].
void paged_kv_cache_write_branches(const __half* src_k, const __half* src_v, __half* kv_pool, const int* d_tables,
                                   int table_stride, const int* d_pos, int B, int fa_layer_idx,
                                   int max_phys_blocks, int block_size, hipStream_t stream = 0);

void paged_gqa_decode_attention_branches(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                         const int* d_seq_lens, int B, int max_seq_len, __half* out,
                                         int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                         hipStream_t stream = 0);

// Same, for branches whose first shared_tokens tokens live in the same physical
// pages (CacheManager::common_prefix_tokens): those pages are read from HBM once
// for all branches.
void paged_gqa_decode_attention_shared(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                       const int* d_seq_lens, int B, int max_seq_len, int shared_tokens,
                                       __half* out, int fa_layer_idx, int max_phys_blocks, int block_size,
                                       float scale, hipStream_t stream = 0);

// Same, for branches that share pages as a fork tree (CacheManager::common_prefix_groups): every shared range and
// every private tail is read once, in one launch.  head_dim 128 only (the call logs and leaves out untouched
// otherwise: check paged_gqa_decode_grouped_supported()).
bool paged_gqa_decode_grouped_supported(int block_size);
void paged_gqa_decode_attention_grouped(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                        const int* d_seq_lens, int B, int max_seq_len, const drk_prefix_group* groups,
                                        int n_groups, __half* out, int fa_layer_idx, int max_phys_blocks, int block_size,
                                        float scale, hipStream_t stream = 0);

// ---- fused layer steps (not in the reference as single functions) ---------------
// Steps 1b-5 of full_attention_forward_paged (paged_attention.cu:331-360) in one launch:
// qg is the interleaved Q|gate projection [T, NUM_ATTN_HEADS, 2*HEAD_DIM], k / v the K and
// V projections [T, NUM_KV_HEADS, HEAD_DIM]; q_out [T, NUM_ATTN_HEADS, HEAD_DIM] receives
// rope(norm(q)); rope(norm(k)) and v go into the pages.  RMS_EPS, ROTARY_DIM and ROPE_THETA
// come from ModelConfig.  d_rope_table (float [table_positions][ROTARY_DIM/2][2], see
// drk_rope_table_fill) may be null.  The gate halves stay in qg: pass qg + HEAD_DIM with
// stride 2*HEAD_DIM to the gated attention calls below.
void paged_qk_norm_rope_write(const __half* qg, const __half* k, const __half* v, const __half* q_norm,
                              const __half* k_norm, __half* q_out, __half* kv_pool, const int* d_block_table,
                              int fa_layer_idx, const int* d_pos, int max_phys_blocks, int block_size,
                              const float* d_rope_table = nullptr, int table_positions = 0, hipStream_t stream = 0);
void paged_qk_norm_rope_write_batch(const __half* qg, const __half* k, const __half* v, const __half* q_norm,
                                    const __half* k_norm, __half* q_out, __half* kv_pool, const int* d_block_table,
                                    int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                                    const float* d_rope_table = nullptr, int table_positions = 0,
                                    hipStream_t stream = 0);
void paged_qk_norm_rope_write_branches(const __half* qg, const __half* k, const __half* v, const __half* q_norm,
                                       const __half* k_norm, __half* q_out, __half* kv_pool, const int* d_tables,
                                       int table_stride, const int* d_pos, int B, int fa_layer_idx,
                                       int max_phys_blocks, int block_size, const float* d_rope_table = nullptr,
                                       int table_positions = 0, hipStream_t stream = 0);

// Attention with the sigmoid gate (paged_attention.cu:368-370, 633-634) folded into the
// epilogue; gate rows are gate_stride elements apart.
void paged_gqa_decode_attention_gated_branches(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                               const int* d_seq_lens, int B, int max_seq_len, const __half* gate,
                                               int gate_stride, __half* out, int fa_layer_idx, int max_phys_blocks,
                                               int block_size, float scale, hipStream_t stream = 0);
void paged_prefill_attention_gated(const __half* Q, __half* kv_pool, const int* d_block_table, const __half* gate,
                                   int gate_stride, __half* out, int fa_layer_idx, int pos_start, int M,
                                   int max_phys_blocks, int block_size, float scale, hipStream_t stream = 0);

// Decode attention that also reports the attention mass each block received (sum of the
// softmax probabilities of its tokens over all query heads) into d_block_mass
// [B, table_stride] -- ImportanceScorer::d_new_scores() for a CacheManager's tables.
// accumulate = false on the first full-attention layer of a step, true on the others.
void paged_gqa_decode_attention_branches_scored(const __half* Q, __half* kv_pool, const int* d_tables, int table_stride,
                                                const int* d_seq_lens, int B, int max_seq_len, __half* out,
                                                int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                                float* d_block_mass, bool accumulate, hipStream_t stream = 0);

// The attention mass a prefill chunk gives to each block of the context (sum of the softmax
// probabilities of the block's tokens over the chunk's rows and all query heads) into
// d_block_mass [mass_len] -- the stream's row of ImportanceScorer::d_new_scores().  A pass of its
// own after the chunk's attention: Q (normed, with RoPE) and the pool only, no workspace.
// accumulate = false on the first full-attention layer of a frame, true on the others.
void paged_prefill_attention_mass(const __half* Q, const __half* kv_pool, const int* d_block_table, int fa_layer_idx,
                                  int pos_start, int M, int max_phys_blocks, int block_size, float scale,
                                  float* d_block_mass, int mass_len, bool accumulate, hipStream_t stream = 0);
// The same measurement without the second walk over the keys: the gated attention call below leaves every row's
// log-sum-exp in d_row_lse [M * num_q_heads], this pass reads it.  The pass may run on another stream behind an
// event recorded after the attention call: it reads Q, the pages and d_row_lse only.
void paged_prefill_attention_mass(const __half* Q, const __half* kv_pool, const int* d_block_table, int fa_layer_idx,
                                  int pos_start, int M, int max_phys_blocks, int block_size, float scale,
                                  const float* d_row_lse, float* d_block_mass, int mass_len, bool accumulate,
                                  hipStream_t stream = 0);

// ---- the same attention calls on a workspace of the caller's ---------------------
void paged_gqa_decode_attention(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_block_table,
                                __half* out, int fa_layer_idx, int seq_len, int max_phys_blocks, int block_size,
                                float scale, hipStream_t stream = 0);
void paged_prefill_attention(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_block_table,
                             __half* out, int fa_layer_idx, int pos_start, int M, int max_phys_blocks, int block_size,
                             float scale, hipStream_t stream = 0);
void paged_gqa_decode_attention_branches(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_tables,
                                         int table_stride, const int* d_seq_lens, int B, int max_seq_len, __half* out,
                                         int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                         hipStream_t stream = 0);
void paged_gqa_decode_attention_shared(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_tables,
                                       int table_stride, const int* d_seq_lens, int B, int max_seq_len,
                                       int shared_tokens, __half* out, int fa_layer_idx, int max_phys_blocks,
                                       int block_size, float scale, hipStream_t stream = 0);
// The fork-tree call; gate may be null, otherwise as in the gated call below.
void paged_gqa_decode_attention_grouped(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_tables,
                                        int table_stride, const int* d_seq_lens, int B, int max_seq_len,
                                        const drk_prefix_group* groups, int n_groups, const __half* gate,
                                        int gate_stride, __half* out, int fa_layer_idx, int max_phys_blocks,
                                        int block_size, float scale, hipStream_t stream = 0);
// The layers of one decode step read the same tables and lengths: the decode kernels' unit descriptors can be built
// once per step (paged_decode_plan_build, one small launch) and read by every layer's attention call
// (paged_gqa_decode_attention_planned: the grouped call, or with n_groups = 0 the gated one; gate may be null).
// The plan must come from the same tables, lengths, B, max_seq_len and groups.  paged_decode_plan_bytes is 0 where
// the kernels take no plan (more than 64 branches, head dims other than 128 / 256).
size_t paged_decode_plan_bytes(int B, int max_seq_len, int max_phys_blocks, int block_size, int n_groups);
bool paged_decode_plan_build(void* d_plan, size_t plan_bytes, const int* d_tables, int table_stride, const int* d_seq_lens,
                             int B, int max_seq_len, const drk_prefix_group* groups, int n_groups, int max_phys_blocks,
                             int block_size, hipStream_t stream = 0);
void paged_gqa_decode_attention_planned(AttentionWorkspace& ws, const void* d_plan, const __half* Q, __half* kv_pool,
                                        const int* d_tables, int table_stride, const int* d_seq_lens, int B, int max_seq_len,
                                        const drk_prefix_group* groups, int n_groups, const __half* gate, int gate_stride,
                                        __half* out, int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                        hipStream_t stream = 0);
void paged_gqa_decode_attention_gated_branches(AttentionWorkspace& ws, const __half* Q, __half* kv_pool,
                                               const int* d_tables, int table_stride, const int* d_seq_lens, int B,
                                               int max_seq_len, const __half* gate, int gate_stride, __half* out,
                                               int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                               hipStream_t stream = 0);
void paged_prefill_attention_gated(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_block_table,
                                   const __half* gate, int gate_stride, __half* out, int fa_layer_idx, int pos_start,
                                   int M, int max_phys_blocks, int block_size, float scale, hipStream_t stream = 0);
void paged_prefill_attention_gated(AttentionWorkspace& ws, const __half* Q, __half* kv_pool, const int* d_block_table,
                                   const __half* gate, int gate_stride, __half* out, float* d_row_lse, int fa_layer_idx,
                                   int pos_start, int M, int max_phys_blocks, int block_size, float scale,
                                   hipStream_t stream = 0);
void paged_gqa_decode_attention_branches_scored(AttentionWorkspace& ws, const __half* Q, __half* kv_pool,
                                                const int* d_tables, int table_stride, const int* d_seq_lens, int B,
                                                int max_seq_len, __half* out, int fa_layer_idx, int max_phys_blocks,
                                                int block_size, float scale, float* d_block_mass, bool accumulate,
                                                hipStream_t stream = 0);
// The same with the step's plan (or null: every launch builds its descriptors) and the gate (or null) applied in
// the merge: what a layer of a decode step with a scorer attached needs in one call.
void paged_gqa_decode_attention_branches_scored(AttentionWorkspace& ws, const void* d_plan, const __half* Q, __half* kv_pool,
                                                const int* d_tables, int table_stride, const int* d_seq_lens, int B,
                                                int max_seq_len, const __half* gate, int gate_stride, __half* out,
                                                int fa_layer_idx, int max_phys_blocks, int block_size, float scale,
                                                float* d_block_mass, bool accumulate, hipStream_t stream = 0);

// ---- the per-stream workspaces behind the calls that take none ---------------------
// Reserve the workspace of `stream` up front for the largest shapes, so that the steady
// state is free of allocations (a device allocation is an implicit synchronisation, and is
// not allowed while a stream is being captured).  false on allocation failure.
bool paged_attention_reserve_workspace(int max_branches, int max_seq_len, int max_prefill_rows, int block_size,
                                       hipStream_t stream = 0);
// Waits for the device, then frees every per-stream workspace, retired buffers included.
void paged_attention_release_workspace();

// ---- the reference's two layer wrappers -----------------------------------------------
// The projections of the wrappers below (fp16_gemv / linear_forward in the reference,
// paged_attention.cu:326, 340-343, 373, 576-582, 637) are the model's code: y [M, out_features]
// = x [M, in_features] W^T.  Registered once; without it the wrappers log an error and return.
using LinearForwardFn = void (*)(const __half* x, const Linear& w, __half* y, int M, hipStream_t stream);
void set_linear_forward(LinearForwardFn fn);
// Optional cos/sin table for the wrappers' RoPE step (float [table_positions][ROTARY_DIM/2][2], see
// drk_rope_table_fill); without one, and for positions beyond it, the kernel evaluates
// pos * theta^(-2 pair / rotary_dim) and its cos / sin itself, as the reference's kernels do.
void set_rope_table(const float* d_rope_table, int table_positions);

// full_attention_forward_paged, paged_attention.h:75-86 / paged_attention.cu:314-376: one
// token at position `pos` (also in *state.d_pos), seq_len = pos + 1.  Q|gate, K and V
// projections (K, V into state.dn_z), then ONE launch for split + per-head RMSNorm + partial
// RoPE + page write (rope(norm(q)) lands in state.dn_qkv), attention into state.attn_out,
// sigmoid gate read in place from state.q_buf, O projection into state.norm_out.
void full_attention_forward_paged(const __half* x, const FullAttentionWeights& attn, __half* kv_pool,
                                  const int* d_block_table, int fa_layer_idx, int pos, int seq_len,
                                  int max_phys_blocks, int block_size, InferenceState& state, hipStream_t stream = 0);

// full_attention_forward_paged_prefill, paged_attention.h:92-104 / paged_attention.cu:563-638:
// M tokens at pos_start .. pos_start + M - 1; K into state.kv_buf, V into state.dn_z; two
// launches (fused split/norm/RoPE/write, MFMA prefill attention with the gate in its epilogue)
// between the projections.
void full_attention_forward_paged_prefill(const __half* x, const FullAttentionWeights& attn, __half* kv_pool,
                                          const int* d_block_table, int fa_layer_idx, int pos_start, int M,
                                          int seq_len, int max_phys_blocks, int block_size, InferenceState& state,
                                          hipStream_t stream = 0);

} // namespace deusridet
