// importance_scorer.h -- per-block importance with exponential decay:
// score = score*decay + new.  Same interface as the reference's
// ImportanceScorer (src/memoria/importance_scorer.h:25-67).
#pragma once

#include <hip/hip_runtime_api.h>
#include <vector>

namespace deusridet {

class ImportanceScorer {
public:
    ImportanceScorer() = default;
    ~ImportanceScorer();
    ImportanceScorer(const ImportanceScorer&) = delete;
    ImportanceScorer& operator=(const ImportanceScorer&) = delete;

    // Device scores for max_blocks logical blocks, zeroed; own stream
    // (importance_scorer.cu:46-65).
    bool init(int max_blocks, float decay = 0.95f);
    // Host mirror only, no device memory: least_important()/score() work on what
    // load_host_scores() put there.  For tests and planning without a GPU.
    bool init_detached(int max_blocks, float decay = 0.95f);

    // scores[b] = scores[b]*decay + d_block_scores[b] for b < num_blocks, on the
    // scorer's stream, asynchronous (importance_scorer.cu:67-73).
    void update(const float* d_block_scores, int num_blocks);

    // Not in the reference (its scorer is never fed): a device buffer [max_blocks] for the
    // attention masses of one step, zeroed at init().  The scored attention call of
    // machina/paged_attention.h writes (first layer of a step) or accumulates (other layers)
    // into it; apply_new_scores() then folds it in with update()'s formula, on `stream` -- the
    // stream the attention ran on, so no cross-stream wait is needed.  sync_to_host() waits for
    // that stream too.  With a CacheManager of several branches the index is the table cell
    // branch * table_stride + logical block, so max_blocks must cover max_branches * table_stride.
    float* d_new_scores();
    void apply_new_scores(hipStream_t stream);
    // The same fold for cells [first, first + count) only, whose new scores are cleared with it: what a
    // perception frame does with the stream's own row while the rows of open decode branches keep the
    // masses of their last step (those were folded in by that step and must not be counted again).
    void apply_new_scores(int first, int count, hipStream_t stream);
    // The same for masses that live in a buffer of the caller's (count floats, cleared by the fold): a perception
    // frame gathers its masses there, so that a decode step's fold over the whole array, issued while the frame is
    // under way, neither reads half a frame nor counts it twice.
    void fold_masses(int first, int count, float* d_masses, hipStream_t stream);
    // Folds read and write the scores, so two of them must not run at once.  Each fold waits for the one
    // before it when that ran on another stream, and marks its own end for the next.  A fold recorded into a
    // graph cannot do either (the capture may not wait on work outside it): whoever replays such a graph calls
    // wait_for_last_fold(stream) before the launch and note_fold_on(stream) behind it.
    void wait_for_last_fold(hipStream_t stream);
    void note_fold_on(hipStream_t stream);

    // First minimum over the given logical block ids in list order, from the host
    // mirror (importance_scorer.cu:75-87).  -1 when n <= 0.
    int least_important(const int* gpu_resident, int n) const;
    float score(int logical_block) const;
    // Waits for the scorer's stream and copies the scores to the host mirror
    // (importance_scorer.cu:94-99).
    void sync_to_host();
    // Replace the host mirror (restoring a snapshot; no arithmetic).
    void load_host_scores(const float* scores, int n);

    void destroy();
    hipStream_t stream() const { return scorer_stream_; }
    int max_blocks() const { return max_blocks_; }

private:
    float* d_scores_ = nullptr;
    float* d_new_ = nullptr;
    hipStream_t last_apply_stream_ = nullptr;
    bool applied_ = false;
    void* fold_done_ = nullptr;          // event: end of the last fold that was launched (not captured)
    bool fold_marked_ = false;
    std::vector<float> h_scores_;
    int max_blocks_ = 0;
    float decay_ = 0.95f;
    hipStream_t scorer_stream_ = nullptr;
};

} // namespace deusridet
