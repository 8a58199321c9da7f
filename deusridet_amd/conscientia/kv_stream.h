// kv_stream.h -- the KV-cache side of the reference's ConscientiStream
// (src/conscientia/stream.cpp:145-401): who allocates blocks when, when the block table goes
// to the device, which position each token is written at, and when positions move on.
//
//   perception  (prefill_tokens, stream.cpp:145-238): ensure_blocks_for_range(current_pos, M),
//               sync_block_table, every layer with (pos_start = current_pos, M), then
//               current_pos += M and set_seq_len(current_pos);
//   decode      (stream.cpp:297-372): per token ensure_blocks_for(pos), sync_block_table,
//               position to the device, every layer with seq_len = pos + 1, pos++.
//
// What is new here is what the reference describes but does not have
// (docs/en/architecture/03-cogitatio.md:3-5, 18-22; scheduler.h:53-56: 1 / 2 / 4 decode
// branches by wakefulness state): decode runs on several branches forked copy-on-write from
// the perception stream, all of them in ONE launch per layer, and a whole decode step (all
// layers plus the caller's own kernels between them) can be captured once and replayed:
// positions and lengths live on the device and the captured step advances them itself; the
// host only makes sure blocks exist and uploads changed table entries before each replay.
//
// The model code (projections, MLP, ...) stays with the caller: per full-attention layer it
// hands over the raw projections and gets the gated attention output back.
#pragma once

#include "../machina/paged_attention.h"
#include "../memoria/cache_manager.h"
#include <functional>
#include <vector>

namespace deusridet {

struct KvLayerIO {               // one full-attention layer, T tokens (prefill chunk) or T branches (decode)
    const __half* qg;            // [T, NUM_ATTN_HEADS, 2*HEAD_DIM]  interleaved Q | gate projection
    const __half* k;             // [T, NUM_KV_HEADS, HEAD_DIM]      K projection (raw)
    const __half* v;             // [T, NUM_KV_HEADS, HEAD_DIM]
    const __half* q_norm;        // [HEAD_DIM]
    const __half* k_norm;        // [HEAD_DIM]
    __half* q_scratch;           // [T, NUM_ATTN_HEADS, HEAD_DIM]    rope(norm(q)) lands here
    __half* attn_out;            // [T, NUM_ATTN_HEADS, HEAD_DIM]    attention * sigmoid(gate)
};

class KvStream {
public:
    KvStream() = default;
    ~KvStream();
    KvStream(const KvStream&) = delete;
    KvStream& operator=(const KvStream&) = delete;

    // cm must be initialised with max_branches >= 1 + the decode branches ever open at once.
    // scorer (optional): decode attention reports the attention mass per block into it; it must
    // cover cm.max_branches() * cm.table_stride() cells (init fails otherwise).
    // d_rope_table (optional): see drk_rope_table_fill.
    // max_prefill_rows: the longest chunk begin_prefill will be given.
    // Two workspaces for split-K partials are reserved here, one for perception and one for
    // decode, sized for max_context_len, every branch and max_prefill_rows: perception and decode
    // may run on different streams at the same time, and nothing allocates after init -- a
    // captured step keeps the addresses it was recorded with.
    bool init(CacheManager& cm, int max_context_len, ImportanceScorer* scorer = nullptr,
              const float* d_rope_table = nullptr, int table_positions = 0, int max_prefill_rows = 2048);
    void destroy();

    // ---- perception: the persistent stream, branch 0 -------------------------------------
    // May run between the decode steps of open branches (time division): the branches keep the
    // pages they forked from, the stream copies a block it still shares before it writes into it.
    bool begin_prefill(int M, hipStream_t stream);
    void prefill_layer(int fa_layer_idx, const KvLayerIO& io, int M, hipStream_t stream);
    // With a scorer attached every layer's attention call also leaves its rows' log-sum-exps, and a pass over Q and
    // K on the scorer's stream (behind an event) turns them into the attention mass every block received; the next
    // layer's first launch waits for that pass, which reads q_scratch.  end_prefill folds the frame's masses into the
    // scores of the stream's own row (and clears them) on the scorer's stream, behind the passes, and makes the
    // layers' stream wait for the last pass; `stream` only keeps the reference's call shape.
    void end_prefill(int M, hipStream_t stream = nullptr);
    int  current_pos() const { return current_pos_; }

    // ---- decode branches ---------------------------------------------------------------------
    // Fork n branches from the stream at current_pos (copy-on-write: they share every block of
    // the prefix).  Returns how many were opened (fewer when the manager runs out of ids).
    int  open_branches(int n);
    // Change the number of open branches (the scheduler's 1 / 2 / 4 by wakefulness state,
    // scheduler.h:53-56): the youngest are closed, new ones fork at the stream's current position.
    // Returns the number open afterwards.  A captured step is dropped.
    int  set_branch_count(int n);
    void close_branches();
    int  num_branches() const { return (int)branches_.size(); }
    int  branch_id(int i) const { return branches_[i]; }
    int  branch_pos(int i) const { return pos_[i]; }
    // The prefix (whole blocks) all open branches share.  With at least min_branches open and
    // at least min_tokens shared, decode streams that prefix once for all branches instead of
    // once per branch.  Defaults: 4 branches, 4096 tokens.
    int  shared_tokens() const { return shared_tokens_; }
    // the open branches' fork tree as decode reads it: shared ranges, parents first (empty: nothing shared)
    const std::vector<drk_prefix_group>& shared_groups() const { return groups_; }
    void set_shared_prefix_policy(int min_branches, int min_tokens) { shared_min_branches_ = min_branches; shared_min_tokens_ = min_tokens; }

    // One decode step = begin, decode_layer for every full-attention layer, end.
    // begin: blocks for the token each branch is about to write, table sync (this also issues the
    // copy-on-write copies), positions to the device when they are not there yet.
    bool begin_decode_step(hipStream_t stream);
    void decode_layer(int fa_layer_idx, const KvLayerIO& io, hipStream_t stream);
    // end: positions and lengths + 1 on the device (in the stream) and on the host.
    void end_decode_step(hipStream_t stream);

    // Capture one step (layers(stream) must enqueue everything between begin and end, calling
    // decode_layer for each full-attention layer) and replay it: replay_decode_step() does the
    // host part of begin, launches the graph, does the host part of end.
    bool capture_decode_step(const std::function<void(hipStream_t)>& layers, hipStream_t stream);
    bool replay_decode_step(hipStream_t stream);
    bool has_graph() const { return graph_ != nullptr; }

    const int* d_pos() const { return d_pos_; }          // [num_branches] position each branch writes next
    const int* d_seq_lens() const { return d_len_; }     // = d_pos + 1 during a step

private:
    CacheManager* cm_ = nullptr;
    ImportanceScorer* scorer_ = nullptr;
    const float* d_rope_table_ = nullptr;
    int table_positions_ = 0;
    int max_context_len_ = 0;
    int current_pos_ = 0;
    std::vector<int> branches_;      // CacheManager branch ids of the open decode branches
    std::vector<int> pos_;           // host copy of the positions
    int* d_pos_ = nullptr;
    int* d_len_ = nullptr;
    bool positions_on_device_ = false;
    int shared_tokens_ = 0;          // prefix the open branches share (whole blocks)
    std::vector<drk_prefix_group> groups_;   // their fork tree: the ranges some of them share (CacheManager::common_prefix_groups)
    int shared_min_branches_ = 4;
    int shared_min_tokens_ = 4096;
    void* graph_ = nullptr;
    AttentionWorkspace ws_prefill_, ws_decode_;
    int max_prefill_rows_ = 0;
    int first_layer_of_step_ = -1;   // the layer whose scored call overwrites instead of accumulating
    int first_layer_of_frame_ = -1;  // the same for the mass pass of a perception frame
    void* d_plan_ = nullptr;               // the decode kernels' unit descriptors of the step under way
    size_t plan_bytes_ = 0;
    bool plan_built_ = false;
    bool step_plan(const int* tables, int stride, int B, int max_len, const drk_prefix_group* groups, int n_groups,
                   hipStream_t stream);
    hipStream_t frame_stream_ = nullptr;   // stream of the frame's layers
    hipStream_t mass_stream_ = nullptr;    // stream of the frame's mass passes (the scorer's)
    float* d_row_lse_ = nullptr;           // [2][max_prefill_rows][num_q_heads]: the rows' log-sum-exps, by turns
    float* d_frame_mass_ = nullptr;        // [table_stride]: the masses of the frame under way (same allocation)
    unsigned lse_turn_ = 0;
    void* ev_attn_ = nullptr;              // a layer's attention call has been issued (recorded on the caller's stream)
    void* ev_mass_ = nullptr;              // its mass pass has been issued (recorded on the scorer's stream)
    bool mass_pending_ = false;

    bool host_begin(hipStream_t stream);
    void host_end();
    void clear_mass_rows(int first_branch, int count);
    void find_shared_groups();
};

} // namespace deusridet
