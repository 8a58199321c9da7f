// kv_stream.cpp -- see kv_stream.h.
#include "kv_stream.h"
#include "../communis/log.h"
#include "drk_kv.h"

#include <cmath>

namespace deusridet {

KvStream::~KvStream() { destroy(); }

bool KvStream::init(CacheManager& cm, int max_context_len, ImportanceScorer* scorer, const float* d_rope_table,
                    int table_positions, int max_prefill_rows)
{
    destroy();
    // the scored attention call writes one row of table_stride() masses per branch into the scorer's
    // buffer, indexed like the block tables
    if (scorer && scorer->d_new_scores() &&
        (long long)scorer->max_blocks() < (long long)cm.max_branches() * cm.table_stride()) {
        LOG_ERROR("Conscientia", "KvStream: the scorer holds %d blocks, %d branches x %d table entries need %lld",
                  scorer->max_blocks(), cm.max_branches(), cm.table_stride(), (long long)cm.max_branches() * cm.table_stride());
        return false;
    }
    max_prefill_rows_ = max_prefill_rows;
    cm_ = &cm;
    scorer_ = scorer;
    d_rope_table_ = d_rope_table;
    table_positions_ = table_positions;
    max_context_len_ = max_context_len;
    current_pos_ = cm.seq_len(0);
    void* p = nullptr;
    size_t bytes = (size_t)cm.max_branches() * sizeof(int);
    if (drk_dev_malloc(&p, bytes) != DRK_OK) {
        LOG_ERROR("Conscientia", "KvStream: position buffer: %s", drk_last_error());
        return false;
    }
    d_pos_ = static_cast<int*>(p);
    if (drk_dev_malloc(&p, bytes) != DRK_OK) {
        LOG_ERROR("Conscientia", "KvStream: length buffer: %s", drk_last_error());
        destroy();
        return false;
    }
    d_len_ = static_cast<int*>(p);
    if (scorer && scorer->d_new_scores()) {
        // perception frames: two sets of row log-sum-exps (the attention call of one layer may run while the mass
        // pass of the layer before still reads its set) and the two events that order the passes
        // and the frame's masses, one per table entry of the stream's row (zero between frames)
        const size_t lse_floats = 2 * (size_t)max_prefill_rows * ModelConfig::NUM_ATTN_HEADS;
        const size_t mass_floats = (size_t)cm.table_stride();
        p = nullptr;
        if (drk_dev_malloc(&p, (lse_floats + mass_floats) * sizeof(float)) != DRK_OK || drk_event_create(&ev_attn_) != DRK_OK ||
            drk_event_create(&ev_mass_) != DRK_OK ||
            drk_dev_memset_async(static_cast<float*>(p) + lse_floats, 0, mass_floats * sizeof(float), nullptr) != DRK_OK ||
            drk_stream_synchronize(nullptr) != DRK_OK) {
            LOG_ERROR("Conscientia", "KvStream: buffers of the mass pass: %s", drk_last_error());
            d_row_lse_ = static_cast<float*>(p);
            destroy();
            return false;
        }
        d_row_lse_ = static_cast<float*>(p);
        d_frame_mass_ = d_row_lse_ + lse_floats;
    }
    // every attention call below finds its split-K workspace ready: nothing allocates later
    const int bs = cm.block_pool().block_size();
    // the decode kernels' unit descriptors, built once per step for all layers (where the kernels take a plan)
    plan_bytes_ = paged_decode_plan_bytes(cm.max_branches(), max_context_len, cm.block_pool().max_blocks(), bs, DRK_MAX_PREFIX_GROUPS);
    if (plan_bytes_) {
        p = nullptr;
        if (drk_dev_malloc(&p, plan_bytes_) != DRK_OK) {
            LOG_ERROR("Conscientia", "KvStream: plan buffer: %s", drk_last_error());
            destroy();
            return false;
        }
        d_plan_ = p;
    }
    if (!ws_decode_.reserve_for(cm.max_branches(), max_context_len, 0, bs) ||
        !ws_prefill_.reserve_for(1, max_context_len, max_prefill_rows, bs)) {
        destroy();
        return false;
    }
    return true;
}

void KvStream::destroy()
{
    if (graph_) {
        drk_graph_destroy(graph_);
        graph_ = nullptr;
    }
    scorer_ = nullptr;                            // borrowed, and possibly gone already: its rows are not cleared here
    if (cm_) close_branches();
    if (d_pos_) drk_dev_free(d_pos_);
    if (d_len_) drk_dev_free(d_len_);
    if (d_plan_) {
        drk_device_synchronize();                 // a launch may still be reading it
        drk_dev_free(d_plan_);
        d_plan_ = nullptr;
    }
    plan_bytes_ = 0;
    if (d_row_lse_ || ev_attn_ || ev_mass_) {
        drk_device_synchronize();                 // a mass pass may still be reading
        if (d_row_lse_) drk_dev_free(d_row_lse_);
        if (ev_attn_) drk_event_destroy(ev_attn_);
        if (ev_mass_) drk_event_destroy(ev_mass_);
        d_row_lse_ = d_frame_mass_ = nullptr;
        ev_attn_ = ev_mass_ = nullptr;
        mass_pending_ = false;
    }
    if (ws_decode_.ptr() || ws_prefill_.ptr()) {
        drk_device_synchronize();                 // launches that use the partials may still be running
        ws_decode_.release();
        ws_prefill_.release();
    }
    d_pos_ = d_len_ = nullptr;
    cm_ = nullptr;
    scorer_ = nullptr;
    positions_on_device_ = false;
}

// ---- perception (stream.cpp:145-238) -----------------------------------------------------------

bool KvStream::begin_prefill(int M, hipStream_t stream)
{
    if (!cm_ || M <= 0) return M == 0;
    // Decode branches may be open (time division: perception goes on while they think).  They
    // keep the pages they forked from; the stream's first write into a block it still shares
    // with them makes a private copy, as a branch's would.
    if (M > max_prefill_rows_) {
        LOG_ERROR("Conscientia", "KvStream: chunk of %d tokens exceeds max_prefill_rows %d", M, max_prefill_rows_);
        return false;
    }
    if (current_pos_ + M > max_context_len_) {
        LOG_ERROR("Conscientia", "KvStream: context of %d tokens exceeds max_context_len %d", current_pos_ + M, max_context_len_);
        return false;
    }
    if (!cm_->ensure_blocks_for_range(0, current_pos_, M)) {              // stream.cpp:151-155
        LOG_ERROR("Conscientia", "Block allocation failed for pos=%d M=%d", current_pos_, M);
        return false;
    }
    cm_->sync_block_table(stream);                                        // stream.cpp:156
    first_layer_of_frame_ = -1;
    return true;
}

void KvStream::prefill_layer(int fa_layer_idx, const KvLayerIO& io, int M, hipStream_t stream)
{
    const BlockPool& pool = cm_->block_pool();
    const int hd = ModelConfig::HEAD_DIM;
    const float scale = 1.0f / std::sqrt((float)hd);
    const bool scored = scorer_ && scorer_->d_new_scores() && d_row_lse_;
    // the mass pass of the layer before reads q_scratch on the scorer's stream: this layer's first launch rewrites it
    if (scored && mass_pending_ && drk_stream_wait_event(stream, ev_mass_) != DRK_OK)
        LOG_ERROR("Conscientia", "KvStream: waiting for the mass pass: %s", drk_last_error());
    // steps 4-9 of full_attention_forward_paged_prefill (paged_attention.cu:589-634) in two launches
    paged_qk_norm_rope_write_batch(io.qg, io.k, io.v, io.q_norm, io.k_norm, io.q_scratch, pool.pool_ptr(),
                                   cm_->d_block_table(0), fa_layer_idx, current_pos_, M, pool.max_blocks(),
                                   pool.block_size(), d_rope_table_, table_positions_, stream);
    if (!scored) {
        paged_prefill_attention_gated(ws_prefill_, io.q_scratch, pool.pool_ptr(), cm_->d_block_table(0), io.qg + hd, 2 * hd, io.attn_out,
                                      fa_layer_idx, current_pos_, M, pool.max_blocks(), pool.block_size(), scale, stream);
        return;
    }
    // What the frame's rows looked at, block by block, into a buffer of the stream's own
    // ("after each Prefill frame, record cumulative attention weight received by each KV block",
    // docs/en/architecture/02-memoria.md:40-44).  The attention call leaves every row's log-sum-exp; the mass pass
    // -- Q and K once more, no V -- runs on the scorer's stream behind an event, beside whatever the caller puts on
    // `stream` next (the layer's output projection and MLP).
    float* lse = d_row_lse_ + (size_t)(lse_turn_ & 1) * max_prefill_rows_ * ModelConfig::NUM_ATTN_HEADS;
    lse_turn_++;
    paged_prefill_attention_gated(ws_prefill_, io.q_scratch, pool.pool_ptr(), cm_->d_block_table(0), io.qg + hd, 2 * hd, io.attn_out,
                                  lse, fa_layer_idx, current_pos_, M, pool.max_blocks(), pool.block_size(), scale, stream);
    const bool first = first_layer_of_frame_ < 0;
    if (first) first_layer_of_frame_ = fa_layer_idx;
    frame_stream_ = stream;
    hipStream_t ms = scorer_->stream();
    if (drk_event_record(ev_attn_, stream) != DRK_OK || drk_stream_wait_event(ms, ev_attn_) != DRK_OK) {
        LOG_ERROR("Conscientia", "KvStream: ordering the mass pass: %s", drk_last_error());
        ms = stream;                                    // in line, then
    }
    paged_prefill_attention_mass(io.q_scratch, pool.pool_ptr(), cm_->d_block_table(0), fa_layer_idx, current_pos_, M,
                                 pool.max_blocks(), pool.block_size(), scale, lse, d_frame_mass_, cm_->table_stride(), !first, ms);
    mass_stream_ = ms;
    mass_pending_ = drk_event_record(ev_mass_, ms) == DRK_OK;
}

void KvStream::end_prefill(int M, hipStream_t stream)
{
    if (scorer_ && first_layer_of_frame_ >= 0) {
        // Fold the frame's masses into the scores of the stream's own row, and clear them in the same pass.  Only
        // that row: the rows of open decode branches still hold their last step's masses, which that step has
        // folded in already.  The fold goes behind the mass passes, on the stream they ran on, whatever the caller
        // passes (or leaves out) here; the caller's stream waits for the last pass, which still reads q_scratch.
        (void)stream;
        scorer_->fold_masses(0, cm_->table_stride(), d_frame_mass_, mass_stream_);
        if (mass_pending_ && mass_stream_ != frame_stream_ && drk_stream_wait_event(frame_stream_, ev_mass_) != DRK_OK)
            LOG_ERROR("Conscientia", "KvStream: waiting for the mass pass: %s", drk_last_error());
        mass_pending_ = false;
        first_layer_of_frame_ = -1;
    }
    current_pos_ += M;                                                    // stream.cpp:238-239
    cm_->set_seq_len(0, current_pos_);
}

// ---- decode branches ------------------------------------------------------------------------------

int KvStream::open_branches(int n)
{
    if (!cm_ || !branches_.empty()) return 0;
    return set_branch_count(n);
}

int KvStream::set_branch_count(int n)
{
    if (!cm_ || n < 0) return (int)branches_.size();
    if (n == (int)branches_.size()) return n;
    while ((int)branches_.size() > n) {                       // close the youngest
        clear_mass_rows(branches_.back(), 1);
        cm_->release_branch(branches_.back());
        branches_.pop_back();
        pos_.pop_back();
    }
    while ((int)branches_.size() < n) {                       // fork more, at the stream's position of now
        int id = cm_->fork_branch(0, current_pos_);
        if (id < 0) break;
        // launches address the branches' table rows as one [B, stride] array: ids must be consecutive
        if (!branches_.empty() && id != branches_.back() + 1) {
            cm_->release_branch(id);
            break;
        }
        branches_.push_back(id);
        pos_.push_back(current_pos_);
    }
    positions_on_device_ = false;
    shared_tokens_ = branches_.empty() ? 0 : cm_->common_prefix_tokens(branches_.data(), (int)branches_.size());
    find_shared_groups();
    if (graph_) {                        // a captured step is tied to the branch set it was recorded for
        drk_graph_destroy(graph_);
        graph_ = nullptr;
    }
    return (int)branches_.size();
}

// Branches forked at different moments form a tree: all of them share the context up to the oldest fork, the
// younger ones what the stream took in since.  (Forks never change a shared page -- a write takes a private copy
// -- so the tree found here holds until the branch set changes.)
void KvStream::find_shared_groups()
{
    groups_.clear();
    const int B = (int)branches_.size();
    if (B < 2 || !paged_gqa_decode_grouped_supported(cm_->block_pool().block_size()) || ModelConfig::KV_DTYPE > DRK_BF16) return;
    const int per_group = 64 / (ModelConfig::NUM_ATTN_HEADS / ModelConfig::NUM_KV_HEADS);     // 64 query rows per kv head and group
    if (per_group < 2) return;
    groups_.resize(DRK_MAX_PREFIX_GROUPS);
    const int n = cm_->common_prefix_groups(branches_.data(), B, per_group, 256, groups_.data(), DRK_MAX_PREFIX_GROUPS);
    groups_.resize((size_t)n);
}

// The scorer folds its whole new-score buffer into the scores on every step.  The rows of a branch
// that leaves the set must not be folded in again and again, nor be inherited by a later branch
// that gets the same id: they are cleared when the branch closes (in the NULL stream, then
// waited for: closing a branch is rare and happens between steps).
void KvStream::clear_mass_rows(int first_branch, int count)
{
    if (!scorer_ || !scorer_->d_new_scores() || count <= 0) return;
    const size_t stride = (size_t)cm_->table_stride();
    if (drk_device_synchronize() != DRK_OK ||
        drk_dev_memset_async(scorer_->d_new_scores() + (size_t)first_branch * stride, 0, (size_t)count * stride * sizeof(float),
                             nullptr) != DRK_OK ||
        drk_stream_synchronize(nullptr) != DRK_OK)
        LOG_ERROR("Conscientia", "KvStream: clearing attention masses: %s", drk_last_error());
}

void KvStream::close_branches()
{
    if (!branches_.empty()) clear_mass_rows(branches_.front(), (int)branches_.size());
    for (int id : branches_) cm_->release_branch(id);
    branches_.clear();
    pos_.clear();
    positions_on_device_ = false;
    shared_tokens_ = 0;
    groups_.clear();
    if (graph_) {                        // a captured step is tied to the branch set it was recorded for
        drk_graph_destroy(graph_);
        graph_ = nullptr;
    }
}

bool KvStream::host_begin(hipStream_t stream)
{
    const int B = (int)branches_.size();
    if (B == 0) return false;
    for (int i = 0; i < B; i++) {
        if (pos_[i] + 1 > max_context_len_) {
            LOG_ERROR("Conscientia", "KvStream: branch %d reached max_context_len %d", branches_[i], max_context_len_);
            return false;
        }
        if (!cm_->ensure_blocks_for(branches_[i], pos_[i])) {             // stream.cpp:297-301
            LOG_ERROR("Conscientia", "Block allocation failed at pos=%d (branch %d)", pos_[i], branches_[i]);
            return false;
        }
    }
    cm_->sync_block_table(stream);                                        // stream.cpp:302
    if (!positions_on_device_) {                                          // stream.cpp:304-305, once per branch set
        std::vector<int> len(B);
        for (int i = 0; i < B; i++) len[i] = pos_[i] + 1;
        if (drk_memcpy_h2d_async(d_pos_, pos_.data(), (size_t)B * sizeof(int), stream) != DRK_OK ||
            drk_memcpy_h2d_async(d_len_, len.data(), (size_t)B * sizeof(int), stream) != DRK_OK ||
            drk_stream_synchronize(stream) != DRK_OK) {                   // the host vectors go out of scope
            LOG_ERROR("Conscientia", "KvStream: position upload: %s", drk_last_error());
            return false;
        }
        positions_on_device_ = true;
    }
    return true;
}

void KvStream::host_end()
{
    for (size_t i = 0; i < branches_.size(); i++) {
        pos_[i]++;                                                        // stream.cpp:371-372
        cm_->set_seq_len(branches_[i], pos_[i]);
    }
}

bool KvStream::begin_decode_step(hipStream_t stream)
{
    first_layer_of_step_ = -1;
    plan_built_ = false;
    return host_begin(stream);
}

void KvStream::decode_layer(int fa_layer_idx, const KvLayerIO& io, hipStream_t stream)
{
    const int B = (int)branches_.size();
    if (B == 0) return;
    const BlockPool& pool = cm_->block_pool();
    const int hd = ModelConfig::HEAD_DIM, stride = cm_->table_stride();
    const int* tables = cm_->d_block_table(branches_[0]);
    const float scale = 1.0f / std::sqrt((float)hd);
    int max_len = 0;
    for (int p : pos_) max_len = p + 1 > max_len ? p + 1 : max_len;
    // a captured step is replayed while the branches grow: size the launch for the whole context
    if (max_context_len_ > max_len) max_len = max_context_len_;
    paged_qk_norm_rope_write_branches(io.qg, io.k, io.v, io.q_norm, io.k_norm, io.q_scratch, pool.pool_ptr(), tables, stride,
                                      d_pos_, B, fa_layer_idx, pool.max_blocks(), pool.block_size(), d_rope_table_,
                                      table_positions_, stream);
    const __half* gate = io.qg + hd;
    if (scorer_ && scorer_->d_new_scores()) {
        if (first_layer_of_step_ < 0) first_layer_of_step_ = fa_layer_idx;
        float* mass = scorer_->d_new_scores() + (size_t)branches_[0] * stride;
        // the step's unit descriptors where the kernel takes a plan, the gate on the merge
        const void* plan = step_plan(tables, stride, B, max_len, nullptr, 0, stream) ? d_plan_ : nullptr;
        paged_gqa_decode_attention_branches_scored(ws_decode_, plan, io.q_scratch, pool.pool_ptr(), tables, stride, d_len_, B,
                                                   max_len, gate, 2 * hd, io.attn_out, fa_layer_idx, pool.max_blocks(),
                                                   pool.block_size(), scale, mass, fa_layer_idx != first_layer_of_step_, stream);
    } else if (B >= shared_min_branches_ && !groups_.empty() && groups_[0].tok_end - groups_[0].tok_begin >= shared_min_tokens_) {
        // every range some of the branches share is streamed once for them, the gate rides on the merge
        if (step_plan(tables, stride, B, max_len, groups_.data(), (int)groups_.size(), stream))
            paged_gqa_decode_attention_planned(ws_decode_, d_plan_, io.q_scratch, pool.pool_ptr(), tables, stride, d_len_, B, max_len,
                                               groups_.data(), (int)groups_.size(), gate, 2 * hd, io.attn_out, fa_layer_idx,
                                               pool.max_blocks(), pool.block_size(), scale, stream);
        else
            paged_gqa_decode_attention_grouped(ws_decode_, io.q_scratch, pool.pool_ptr(), tables, stride, d_len_, B, max_len,
                                               groups_.data(), (int)groups_.size(), gate, 2 * hd, io.attn_out, fa_layer_idx,
                                               pool.max_blocks(), pool.block_size(), scale, stream);
    } else if (B >= shared_min_branches_ && shared_tokens_ >= shared_min_tokens_) {
        // the branches' common prefix is streamed once for all of them
        paged_gqa_decode_attention_shared(ws_decode_, io.q_scratch, pool.pool_ptr(), tables, stride, d_len_, B, max_len, shared_tokens_,
                                          io.attn_out, fa_layer_idx, pool.max_blocks(), pool.block_size(), scale, stream);
        if (drk_sigmoid_gate(io.attn_out, gate, io.attn_out, (size_t)B * ModelConfig::NUM_ATTN_HEADS, hd, 2 * (size_t)hd,
                             ModelConfig::IO_DTYPE, stream) != DRK_OK)
            LOG_ERROR("Conscientia", "sigmoid_gate: %s", drk_last_error());
    } else if (step_plan(tables, stride, B, max_len, nullptr, 0, stream)) {
        paged_gqa_decode_attention_planned(ws_decode_, d_plan_, io.q_scratch, pool.pool_ptr(), tables, stride, d_len_, B, max_len,
                                           nullptr, 0, gate, 2 * hd, io.attn_out, fa_layer_idx, pool.max_blocks(),
                                           pool.block_size(), scale, stream);
    } else {
        paged_gqa_decode_attention_gated_branches(ws_decode_, io.q_scratch, pool.pool_ptr(), tables, stride, d_len_, B, max_len, gate,
                                                  2 * hd, io.attn_out, fa_layer_idx, pool.max_blocks(), pool.block_size(),
                                                  scale, stream);
    }
}

// The step's unit descriptors: built by the first layer that asks, read by the others (the tables and lengths do not
// change within a step).  False where the kernels take no plan.
bool KvStream::step_plan(const int* tables, int stride, int B, int max_len, const drk_prefix_group* groups, int n_groups,
                         hipStream_t stream)
{
    if (!d_plan_ || B > 64) return false;
    if (plan_built_) return true;
    const BlockPool& pool = cm_->block_pool();
    if (!paged_decode_plan_build(d_plan_, plan_bytes_, tables, stride, d_len_, B, max_len, groups, n_groups, pool.max_blocks(),
                                 pool.block_size(), stream))
        return false;
    plan_built_ = true;
    return true;
}

void KvStream::end_decode_step(hipStream_t stream)
{
    const int B = (int)branches_.size();
    if (B == 0) return;
    if (scorer_ && first_layer_of_step_ >= 0) scorer_->apply_new_scores(stream);
    if (drk_positions_advance(d_pos_, d_len_, B, 1, stream) != DRK_OK)
        LOG_ERROR("Conscientia", "positions_advance: %s", drk_last_error());
    host_end();
}

bool KvStream::capture_decode_step(const std::function<void(hipStream_t)>& layers, hipStream_t stream)
{
    if (branches_.empty()) return false;
    if (graph_) {
        drk_graph_destroy(graph_);
        graph_ = nullptr;
    }
    // host part first: the capture must not contain table uploads or the position upload
    first_layer_of_step_ = -1;
    plan_built_ = false;
    if (!host_begin(stream)) return false;
    if (drk_graph_begin_capture(stream) != DRK_OK) {
        LOG_ERROR("Conscientia", "KvStream: begin capture: %s", drk_last_error());
        return false;
    }
    layers(stream);
    if (scorer_ && first_layer_of_step_ >= 0) scorer_->apply_new_scores(stream);
    drk_positions_advance(d_pos_, d_len_, (int)branches_.size(), 1, stream);
    if (drk_graph_end_capture(stream, &graph_) != DRK_OK) {
        LOG_ERROR("Conscientia", "KvStream: end capture: %s", drk_last_error());
        graph_ = nullptr;
        return false;
    }
    return true;                          // nothing ran yet: the first replay_decode_step() is this step
}

bool KvStream::replay_decode_step(hipStream_t stream)
{
    if (!graph_) return false;
    if (!host_begin(stream)) return false;
    if (scorer_) scorer_->wait_for_last_fold(stream);     // the recorded fold could not wait for a frame's by itself
    if (drk_graph_launch(graph_, stream) != DRK_OK) {
        LOG_ERROR("Conscientia", "KvStream: graph launch: %s", drk_last_error());
        return false;
    }
    if (scorer_ && scorer_->d_new_scores()) scorer_->note_fold_on(stream);
    host_end();
    return true;
}

} // namespace deusridet
