// importance_scorer.cpp -- see importance_scorer.h.
#include "importance_scorer.h"
#include "../communis/log.h"
#include "drk_kv.h"

#include <cstring>

namespace deusridet {

ImportanceScorer::~ImportanceScorer() { destroy(); }

bool ImportanceScorer::init(int max_blocks, float decay)
{
    destroy();
    if (max_blocks < 1) return false;
    max_blocks_ = max_blocks;
    decay_ = decay;
    size_t bytes = (size_t)max_blocks * sizeof(float);
    void* p = nullptr;
    if (drk_dev_malloc(&p, bytes) != DRK_OK) {
        LOG_ERROR("Memoria", "ImportanceScorer: alloc failed: %s", drk_last_error());
        max_blocks_ = 0;
        return false;
    }
    d_scores_ = static_cast<float*>(p);
    void* s = nullptr;
    if (drk_stream_create(&s) != DRK_OK) {
        LOG_ERROR("Memoria", "ImportanceScorer: stream: %s", drk_last_error());
        destroy();
        return false;
    }
    scorer_stream_ = static_cast<hipStream_t>(s);
    drk_dev_memset_async(d_scores_, 0, bytes, scorer_stream_);
    h_scores_.assign(max_blocks, 0.0f);
    LOG_INFO("Memoria", "ImportanceScorer: %d blocks, decay=%.3f", max_blocks, decay);
    return true;
}

bool ImportanceScorer::init_detached(int max_blocks, float decay)
{
    destroy();
    if (max_blocks < 1) return false;
    max_blocks_ = max_blocks;
    decay_ = decay;
    h_scores_.assign(max_blocks, 0.0f);
    return true;
}

void ImportanceScorer::update(const float* d_block_scores, int num_blocks)
{
    if (!d_scores_ || num_blocks <= 0) return;
    if (num_blocks > max_blocks_) num_blocks = max_blocks_;
    if (drk_importance_update(d_scores_, d_block_scores, num_blocks, decay_, scorer_stream_) != DRK_OK)
        LOG_ERROR("Memoria", "ImportanceScorer: update: %s", drk_last_error());
}

float* ImportanceScorer::d_new_scores()
{
    if (!d_scores_) return nullptr;
    if (!d_new_) {
        void* p = nullptr;
        size_t bytes = (size_t)max_blocks_ * sizeof(float);
        if (drk_dev_malloc(&p, bytes) != DRK_OK) {
            LOG_ERROR("Memoria", "ImportanceScorer: alloc of the new-score buffer failed: %s", drk_last_error());
            return nullptr;
        }
        d_new_ = static_cast<float*>(p);
        drk_dev_memset_async(d_new_, 0, bytes, nullptr);
        drk_stream_synchronize(nullptr);
    }
    return d_new_;
}

namespace {
bool stream_is_capturing(hipStream_t stream)
{
    int capturing = 0;
    return stream && drk_stream_is_capturing(stream, &capturing) == DRK_OK && capturing;
}
}

void ImportanceScorer::wait_for_last_fold(hipStream_t stream)
{
    if (!fold_marked_ || stream == last_apply_stream_) return;
    if (drk_stream_wait_event(stream, fold_done_) != DRK_OK)
        LOG_ERROR("Memoria", "ImportanceScorer: waiting for the last fold: %s", drk_last_error());
}

void ImportanceScorer::note_fold_on(hipStream_t stream)
{
    if (!fold_done_ && drk_event_create(&fold_done_) != DRK_OK) {
        LOG_ERROR("Memoria", "ImportanceScorer: event: %s", drk_last_error());
        fold_done_ = nullptr;
    }
    last_apply_stream_ = stream;
    applied_ = true;
    fold_marked_ = fold_done_ && drk_event_record(fold_done_, stream) == DRK_OK;
}

void ImportanceScorer::apply_new_scores(hipStream_t stream)
{
    if (!d_scores_ || !d_new_) return;
    const bool captured = stream_is_capturing(stream);
    if (!captured) wait_for_last_fold(stream);
    if (drk_importance_update(d_scores_, d_new_, max_blocks_, decay_, stream) != DRK_OK)
        LOG_ERROR("Memoria", "ImportanceScorer: apply_new_scores: %s", drk_last_error());
    if (!captured) note_fold_on(stream);
}

void ImportanceScorer::apply_new_scores(int first, int count, hipStream_t stream)
{
    if (!d_new_ || first < 0 || first >= max_blocks_) return;
    fold_masses(first, count, d_new_ + first, stream);
}

void ImportanceScorer::fold_masses(int first, int count, float* d_masses, hipStream_t stream)
{
    if (!d_scores_ || !d_masses || first < 0 || count <= 0 || first >= max_blocks_) return;
    if (count > max_blocks_ - first) count = max_blocks_ - first;
    const bool captured = stream_is_capturing(stream);
    if (!captured) wait_for_last_fold(stream);
    if (drk_importance_fold_clear(d_scores_ + first, d_masses, count, decay_, stream) != DRK_OK)
        LOG_ERROR("Memoria", "ImportanceScorer: fold_masses: %s", drk_last_error());
    if (!captured) note_fold_on(stream);
}

int ImportanceScorer::least_important(const int* gpu_resident, int n) const
{
    if (n <= 0) return -1;
    int min_idx = gpu_resident[0];
    float min_score = score(min_idx);
    for (int i = 1; i < n; i++) {
        float s = score(gpu_resident[i]);
        if (s < min_score) {
            min_score = s;
            min_idx = gpu_resident[i];
        }
    }
    return min_idx;
}

float ImportanceScorer::score(int logical_block) const
{
    if (logical_block < 0 || logical_block >= max_blocks_) return 0.0f;
    return h_scores_[logical_block];
}

void ImportanceScorer::sync_to_host()
{
    if (!d_scores_) return;
    if (applied_) {
        drk_stream_synchronize(last_apply_stream_);
        applied_ = false;
    }
    if (drk_memcpy_d2h(h_scores_.data(), d_scores_, (size_t)max_blocks_ * sizeof(float), scorer_stream_) != DRK_OK)
        LOG_ERROR("Memoria", "ImportanceScorer: sync_to_host: %s", drk_last_error());
}

void ImportanceScorer::load_host_scores(const float* scores, int n)
{
    if (!scores || n <= 0) return;
    if (n > max_blocks_) n = max_blocks_;
    std::memcpy(h_scores_.data(), scores, (size_t)n * sizeof(float));
}

void ImportanceScorer::destroy()
{
    if (d_scores_) {
        drk_dev_free(d_scores_);
        d_scores_ = nullptr;
    }
    if (d_new_) {
        drk_dev_free(d_new_);
        d_new_ = nullptr;
    }
    applied_ = false;
    fold_marked_ = false;
    if (fold_done_) {
        drk_event_destroy(fold_done_);
        fold_done_ = nullptr;
    }
    if (scorer_stream_) {
        drk_stream_destroy(scorer_stream_);
        scorer_stream_ = nullptr;
    }
    h_scores_.clear();
    max_blocks_ = 0;
}

} // namespace deusridet
