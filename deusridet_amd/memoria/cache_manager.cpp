// cache_manager.cpp -- see cache_manager.h.  Host bookkeeping only; the device is
// reached through the C ABI (table upload, copy-on-write block copies).
#include "cache_manager.h"
#include <vector>
#include "kv_swapper.h"
#include "../communis/log.h"

#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <unordered_set>

namespace deusridet {

CacheManager::~CacheManager() { destroy(); }

bool CacheManager::setup_tables(int max_branches)
{
    if (max_branches < 1) max_branches = 1;
    max_branches_ = max_branches;
    // twice the physical blocks of logical space (cache_manager.cpp:37-39)
    max_logical_blocks_ = pool_.max_blocks() * 2;
    size_t cells = (size_t)max_branches_ * max_logical_blocks_;
    h_tables_.assign(cells, -1);
    location_.assign(cells, BlockLocation::INVALID);
    stamp_.assign(cells, 0);
    next_stamp_ = 1;
    evictable_.clear();
    refs_.assign(pool_.max_blocks(), {});
    held_.assign(cells, 0);
    held_cells_.clear();
    copy_pin_.assign(pool_.max_blocks(), 0);
    pending_copies_issued_.clear();
    deferred_release_.clear();
    ssd_paths_.assign(cells, std::string());
    seq_len_.assign(max_branches_, 0);
    alive_.assign(max_branches_, 0);
    alive_[0] = 1;
    dirty_lo_.assign(max_branches_, max_logical_blocks_);
    dirty_hi_.assign(max_branches_, 0);
    pending_copies_.clear();
    return true;
}

bool CacheManager::init(size_t kv_budget_bytes, const std::string& cache_dir, int block_size,
                        KVSwapper* swapper, ImportanceScorer* scorer, int max_branches)
{
    destroy();
    block_size_ = block_size;
    scorer_ = scorer;
    detached_ = false;
    swapper_ = swapper;
    cache_dir_ = cache_dir;
    if (!pool_.init(kv_budget_bytes, block_size)) return false;
    setup_tables(max_branches);
    // cache_manager.cpp:55-65: create the directory; without one the tier stays off
    if (!cache_dir_.empty()) {
        struct stat st;
        if (stat(cache_dir_.c_str(), &st) != 0 && mkdir(cache_dir_.c_str(), 0755) != 0) {
            LOG_WARN("Memoria", "Cannot create SSD cache dir: %s", cache_dir_.c_str());
            cache_dir_.clear();
        }
    }
    ssd_enabled_ = !cache_dir_.empty();

    size_t table_bytes = (size_t)max_branches_ * max_logical_blocks_ * sizeof(int);
    void* p = nullptr;
    if (drk_dev_malloc(&p, table_bytes) != DRK_OK) {
        LOG_ERROR("Memoria", "CacheManager: d_block_table alloc failed: %s", drk_last_error());
        destroy();
        return false;
    }
    d_tables_ = static_cast<int*>(p);
    pairs_capacity_ = 1024;
    if (drk_dev_malloc(&p, (size_t)pairs_capacity_ * 2 * sizeof(int)) != DRK_OK) {
        LOG_ERROR("Memoria", "CacheManager: copy staging alloc failed: %s", drk_last_error());
        destroy();
        return false;
    }
    d_pairs_ = static_cast<int*>(p);
    // -1 everywhere (cache_manager.cpp:53)
    if (drk_dev_memset_async(d_tables_, 0xFF, table_bytes, nullptr) != DRK_OK ||
        drk_stream_synchronize(nullptr) != DRK_OK) {
        LOG_ERROR("Memoria", "CacheManager: table init failed: %s", drk_last_error());
        destroy();
        return false;
    }
    LOG_INFO("Memoria", "CacheManager: %d phys blocks, %d max logical, %d branches, SSD=%s", pool_.max_blocks(),
             max_logical_blocks_, max_branches_, ssd_enabled_ ? cache_dir_.c_str() : "disabled");
    return true;
}

bool CacheManager::init_detached(int max_blocks, int block_size, ImportanceScorer* scorer, int max_branches)
{
    destroy();
    block_size_ = block_size;
    scorer_ = scorer;
    swapper_ = nullptr;
    cache_dir_.clear();
    ssd_enabled_ = false;
    detached_ = true;
    if (!pool_.init_detached(max_blocks, block_size)) return false;
    return setup_tables(max_branches);
}

void CacheManager::mark_dirty(int branch, int logical)
{
    dirty_lo_[branch] = std::min(dirty_lo_[branch], logical);
    dirty_hi_[branch] = std::max(dirty_hi_[branch], logical + 1);
}

// A resident cell is a candidate for eviction when its block has no other reference, the cell
// is not held (see hold_nolock) and no queued copy names the block.
void CacheManager::candidate_add_nolock(int c)
{
    if (!held_[c] && copy_pin_[h_tables_[c]] == 0) evictable_.insert({stamp_[c], c});
}

void CacheManager::candidate_remove_nolock(int c) { evictable_.erase({stamp_[c], c}); }

// The cell takes a reference on `phys` that alloc_block()/retain() has already
// counted in the pool.
void CacheManager::attach_nolock(int c, int phys, bool fresh_stamp)
{
    h_tables_[c] = phys;
    location_[c] = BlockLocation::GPU;
    if (fresh_stamp || stamp_[c] == 0) stamp_[c] = next_stamp_++;
    std::vector<int>& r = refs_[phys];
    if (r.size() == 1) candidate_remove_nolock(r[0]);            // the sole owner is now sharing
    r.push_back(c);
    if (r.size() == 1) candidate_add_nolock(c);
}

// The cell gives up its reference; the block is freed when it was the last.
void CacheManager::detach_nolock(int c)
{
    int phys = h_tables_[c];
    std::vector<int>& r = refs_[phys];
    if (r.size() == 1) candidate_remove_nolock(c);
    r.erase(std::remove(r.begin(), r.end(), c), r.end());
    // a block that a queued copy still reads or writes keeps its last reference until the copy has
    // been issued: nobody else may be handed the block (and fill it) before that
    if (r.empty() && copy_pin_[phys] > 0) deferred_release_.push_back(phys);
    else pool_.release(phys);
    if (r.size() == 1) candidate_add_nolock(r[0]);
    h_tables_[c] = -1;
}

// A cell that ensure_blocks_for has just made resident is about to be written by the caller's
// next launches, and may be the target of a copy that is still queued: until the next
// sync_block_table (which issues the copies) it must not be picked as a victim by a later
// allocation of the same step -- the reference never evicts the block it is about to write.
void CacheManager::hold_nolock(int c)
{
    if (held_[c]) return;
    held_[c] = 1;
    held_cells_.push_back(c);
    candidate_remove_nolock(c);
}

// The queued copies have been issued (or handed out): their blocks are ordinary blocks again,
// and so are the cells of the step.
void CacheManager::release_holds_nolock()
{
    std::vector<int> named;
    for (const auto& cp : pending_copies_issued_) {
        copy_pin_[cp.first]--;
        copy_pin_[cp.second]--;
        named.push_back(cp.first);
        named.push_back(cp.second);
    }
    pending_copies_issued_.clear();
    for (int phys : deferred_release_) pool_.release(phys);
    deferred_release_.clear();
    for (int c : held_cells_) held_[c] = 0;
    for (int c : held_cells_)
        if (location_[c] == BlockLocation::GPU && refs_[h_tables_[c]].size() == 1) candidate_add_nolock(c);
    held_cells_.clear();
    for (int phys : named)
        if (copy_pin_[phys] == 0 && refs_[phys].size() == 1) candidate_add_nolock(refs_[phys][0]);
}

// for_branch: the branch whose allocation needs room, or -1 for an explicit eviction request.
bool CacheManager::pick_victim_nolock(int& cell_out, int for_branch)
{
    const std::set<std::pair<uint64_t, int>>* from = &evictable_;
    std::set<std::pair<uint64_t, int>> last_resort;
    if (evictable_.empty()) {
        // Nothing but cells of the current step is left.  A branch that outgrows the pool loses its own
        // oldest blocks, as the reference's single sequence does (cache_manager.cpp:306-319); an explicit
        // request may take any of them; a block named by a queued copy, and another branch's block of this
        // step, are never taken.
        for (int c : held_cells_) {
            if (location_[c] != BlockLocation::GPU || refs_[h_tables_[c]].size() != 1 || copy_pin_[h_tables_[c]] > 0) continue;
            if (for_branch >= 0 && c / max_logical_blocks_ != for_branch) continue;
            last_resort.insert({stamp_[c], c});
        }
        if (last_resort.empty()) return false;
        from = &last_resort;
    }
    if (!scorer_) {                               // oldest first (cache_manager.cpp:203-204)
        cell_out = from->begin()->second;
        return true;
    }
    // least important; the first minimum in LRU order wins (cache_manager.cpp:188-201,
    // importance_scorer.cu:75-87)
    bool have = false;
    float best = 0.0f;
    for (const auto& e : *from) {
        float s = scorer_->score(e.second);       // by table cell; branch 0: the logical block index
        if (!have || s < best) {
            have = true;
            best = s;
            cell_out = e.second;
        }
    }
    return have;
}

int CacheManager::evict_nolock(int n, int for_branch)
{
    int evicted = 0;
    const bool to_ssd = ssd_enabled_ && swapper_ && swapper_->ready();
    // With the overflow tier every victim's swap-out is submitted first and all of them are waited
    // for once (the swapper pipelines them: one block's copy runs while its neighbour's file is
    // written).  A freed block cannot be handed out before that: the lock is held until then.
    std::vector<std::pair<int, char>> outcome;    // (cell, swap-out succeeded); the flags are written by the swapper's thread
    if (to_ssd) outcome.reserve(std::min((size_t)std::max(n, 0), evictable_.size() + held_cells_.size()));   // never reallocated: the flags are pointed at
    while (evicted < n) {
        int c;
        if (!pick_victim_nolock(c, for_branch)) break;
        int branch = c / max_logical_blocks_, logical = c % max_logical_blocks_;
        if (to_ssd) {                                                 // cache_manager.cpp:132-141
            outcome.push_back({c, 0});
            submit_swap_out_nolock(c, &outcome.back().second);
        }
        detach_nolock(c);                         // frees the block: it had one reference
        location_[c] = BlockLocation::INVALID;
        stamp_[c] = 0;
        mark_dirty(branch, logical);
        evicted++;
    }
    if (to_ssd && !outcome.empty()) {
        swapper_->drain();
        for (const auto& o : outcome) {
            const int c = o.first;
            if (o.second) {
                location_[c] = BlockLocation::SSD;
                ssd_paths_[c] = ssd_path_for(c);
            } else {
                LOG_WARN("Memoria", "SSD swap-out failed for block %d of branch %d, discarding", c % max_logical_blocks_,
                         c / max_logical_blocks_);
            }
        }
    }
    if (evicted > 0)
        LOG_INFO("Memoria", "Evicted %d blocks (SSD=%s), %d free now", evicted,
                 (ssd_enabled_ && swapper_ && swapper_->ready()) ? "yes" : "no", pool_.free_count());
    return evicted;
}

bool CacheManager::ensure_free_nolock(int n_free, int for_branch)
{
    while (pool_.free_count() < n_free) {         // the whole deficit in one batch (one wait for the overflow tier)
        if (evict_nolock(n_free - pool_.free_count(), for_branch) == 0) return false;
    }
    return true;
}

int CacheManager::alloc_phys_nolock(int for_branch)
{
    int phys = pool_.alloc_block();
    if (phys < 0) {                               // cache_manager.cpp:311-319
        if (!ensure_free_nolock(1, for_branch)) {
            LOG_ERROR("Memoria", "Cannot allocate a block: pool exhausted, eviction failed");
            return -1;
        }
        phys = pool_.alloc_block();
    }
    return phys;
}

bool CacheManager::ensure_nolock(int branch, int pos)
{
    if (branch < 0 || branch >= max_branches_ || !alive_[branch] || pos < 0) return false;
    int logical = pos / block_size_;
    if (logical >= max_logical_blocks_) {
        LOG_ERROR("Memoria", "Position %d exceeds max logical blocks (%d)", pos, max_logical_blocks_);
        return false;
    }
    int c = (int)cell(branch, logical);
    if (location_[c] == BlockLocation::GPU) {
        int phys = h_tables_[c];
        hold_nolock(c);                           // before any allocation below can look for a victim
        if (pool_.refcount(phys) > 1) {
            // copy-on-write: the write must not be seen by the other tables
            int fresh = alloc_phys_nolock(branch);
            if (fresh < 0) return false;
            pending_copies_.push_back({phys, fresh});
            pending_copies_issued_.push_back({phys, fresh});
            copy_pin_[phys]++;                    // neither block changes hands before the copy is issued
            copy_pin_[fresh]++;
            detach_nolock(c);                     // the old block keeps its other references
            attach_nolock(c, fresh, false);       // same place in the LRU order
            mark_dirty(branch, logical);
        }
        return true;
    }
    if (location_[c] == BlockLocation::SSD) {     // cache_manager.cpp:88-90
        if (!swap_from_ssd_nolock(c)) return false;
        hold_nolock(c);
        return true;
    }
    int phys = alloc_phys_nolock(branch);
    if (phys < 0) return false;
    attach_nolock(c, phys, true);                 // cache_manager.cpp:321-323
    hold_nolock(c);
    mark_dirty(branch, logical);
    return true;
}

// cache_manager.cpp:207-213; branch 0 keeps the reference's file names
std::string CacheManager::ssd_path_for(int c) const
{
    int branch = c / max_logical_blocks_, logical = c % max_logical_blocks_;
    std::string name = branch == 0 ? "block_" + std::to_string(logical) : "b" + std::to_string(branch) + "_block_" + std::to_string(logical);
    return cache_dir_ + "/" + name + ".kv";
}

// cache_manager.cpp:215-243: the request is queued; *ok is set by the swapper's thread before the
// request counts as complete (the caller drains before it reads the flag or lets the block go)
void CacheManager::submit_swap_out_nolock(int c, char* ok)
{
    SwapRequest req;
    req.direction = SwapDirection::GPU_TO_SSD;
    req.logical_block_idx = c;
    req.physical_block_id = h_tables_[c];
    req.ssd_path = ssd_path_for(c);
    req.callback = [ok](bool success) { *ok = success ? 1 : 0; };
    swapper_->drop_prefetch(c);                   // a stale prefetched image must not outlive the new file
    swapper_->submit(std::move(req));
}

// cache_manager.cpp:245-292.  The fresh block comes from the ordinary allocation path (which
// may evict, and swap out, another block first: requests are executed one after the other).
bool CacheManager::swap_from_ssd_nolock(int c)
{
    if (!swapper_ || !swapper_->ready()) return false;
    int phys = alloc_phys_nolock(c / max_logical_blocks_);
    if (phys < 0) return false;
    bool success = false;
    SwapRequest req;
    req.direction = SwapDirection::SSD_TO_GPU;
    req.logical_block_idx = c;
    req.physical_block_id = phys;
    req.ssd_path = ssd_paths_[c];
    req.callback = [&success](bool ok) { success = ok; };
    swapper_->submit(std::move(req));
    swapper_->drain();
    if (!success) {
        pool_.free_block(phys);
        return false;
    }
    attach_nolock(c, phys, true);                 // back of the LRU order (cache_manager.cpp:290)
    mark_dirty(c / max_logical_blocks_, c % max_logical_blocks_);
    return true;
}

bool CacheManager::ensure_blocks_for(int pos) { return ensure_blocks_for(0, pos); }
bool CacheManager::ensure_blocks_for_range(int pos_start, int M) { return ensure_blocks_for_range(0, pos_start, M); }

bool CacheManager::ensure_blocks_for(int branch, int pos)
{
    std::lock_guard<std::mutex> lock(mu_);
    return ensure_nolock(branch, pos);
}

bool CacheManager::ensure_blocks_for_range(int branch, int pos_start, int M)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (M <= 0) return true;
    int first = pos_start / block_size_, last = (pos_start + M - 1) / block_size_;
    for (int b = first; b <= last; b++)
        if (!ensure_nolock(branch, b * block_size_)) return false;
    return true;
}

const int* CacheManager::d_block_table(int branch) const
{
    if (!d_tables_ || branch < 0 || branch >= max_branches_) return nullptr;
    return d_tables_ + cell(branch, 0);
}

const int* CacheManager::h_block_table(int branch) const
{
    if (branch < 0 || branch >= max_branches_) return nullptr;
    return h_tables_.data() + cell(branch, 0);
}

// Copies whose source is written by an earlier queued copy (or whose target is
// touched by one) must not share a launch: the queue is cut into launches at
// such dependencies and the launches are stream-ordered.
void CacheManager::flush_copies(hipStream_t stream)
{
    size_t i = 0;
    const drk_kv_layout& g = pool_.layout();
    while (i < pending_copies_.size()) {
        std::unordered_set<int> written, read;
        std::vector<int> flat;
        while (i < pending_copies_.size() && (int)flat.size() / 2 < pairs_capacity_) {
            int s = pending_copies_[i].first, d = pending_copies_[i].second;
            if (written.count(s) || written.count(d) || read.count(d)) break;
            written.insert(d);
            read.insert(s);
            flat.push_back(s);
            flat.push_back(d);
            i++;
        }
        int n = (int)flat.size() / 2;
        if (n == 0) break;
        if (drk_memcpy_h2d_async(d_pairs_, flat.data(), flat.size() * sizeof(int), stream) != DRK_OK ||
            drk_kv_copy_blocks(&g, pool_.pool_raw(), d_pairs_, n, stream) != DRK_OK)
            LOG_ERROR("Memoria", "copy-on-write copy failed: %s", drk_last_error());
    }
    pending_copies_.clear();
}

void CacheManager::forget_stream(hipStream_t stream)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (swapper_) swapper_->remove_writer_stream(stream);
}

void CacheManager::sync_block_table(hipStream_t stream)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (swapper_ && swapper_->ready()) swapper_->add_writer_stream(stream);   // swaps order themselves behind this stream
    if (!detached_ && d_tables_) {
        flush_copies(stream);
        for (int b = 0; b < max_branches_; b++) {
            if (dirty_hi_[b] <= dirty_lo_[b]) continue;
            size_t off = cell(b, dirty_lo_[b]);
            size_t bytes = (size_t)(dirty_hi_[b] - dirty_lo_[b]) * sizeof(int);
            if (drk_memcpy_h2d_async(d_tables_ + off, h_tables_.data() + off, bytes, stream) != DRK_OK)
                LOG_ERROR("Memoria", "block table upload failed: %s", drk_last_error());
        }
    }
    for (int b = 0; b < max_branches_; b++) {
        dirty_lo_[b] = max_logical_blocks_;
        dirty_hi_[b] = 0;
    }
    if (!detached_) release_holds_nolock();       // the copies are issued: the step's cells are ordinary cells again
}

int CacheManager::seq_len(int branch) const
{
    std::lock_guard<std::mutex> lock(mu_);
    return (branch >= 0 && branch < max_branches_) ? seq_len_[branch] : 0;
}

void CacheManager::set_seq_len(int branch, int len)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (branch >= 0 && branch < max_branches_) seq_len_[branch] = len;
}

int CacheManager::num_logical_blocks(int branch) const
{
    return (seq_len(branch) + block_size_ - 1) / block_size_;
}

int CacheManager::fork_branch(int parent, int pos)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (parent < 0 || parent >= max_branches_ || !alive_[parent] || pos < 0) return -1;
    int id = -1;
    for (int i = 0; i < max_branches_; i++)
        if (!alive_[i]) { id = i; break; }
    if (id < 0) return -1;
    int nshared = (pos + block_size_ - 1) / block_size_;
    if (nshared > max_logical_blocks_) return -1;
    alive_[id] = 1;
    seq_len_[id] = pos;
    for (int l = 0; l < nshared; l++) {
        int pc = (int)cell(parent, l), cc = (int)cell(id, l);
        if (location_[pc] != BlockLocation::GPU) continue;   // a hole in the parent stays a hole
        int phys = h_tables_[pc];
        pool_.retain(phys);
        attach_nolock(cc, phys, true);
        mark_dirty(id, l);
    }
    return id;
}

void CacheManager::release_branch(int branch)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (branch < 0 || branch >= max_branches_ || !alive_[branch]) return;
    for (int l = 0; l < max_logical_blocks_; l++) {
        int c = (int)cell(branch, l);
        if (location_[c] == BlockLocation::SSD) {             // forget the swapped-out copy
            if (swapper_) swapper_->drop_prefetch(c);
            unlink(ssd_paths_[c].c_str());
            ssd_paths_[c].clear();
            location_[c] = BlockLocation::INVALID;
            continue;
        }
        if (location_[c] != BlockLocation::GPU) continue;
        detach_nolock(c);
        location_[c] = BlockLocation::INVALID;
        stamp_[c] = 0;
        mark_dirty(branch, l);
    }
    // a hold on a cell of this branch has nothing left to protect
    held_cells_.erase(std::remove_if(held_cells_.begin(), held_cells_.end(), [&](int c) {
                          if (c / max_logical_blocks_ != branch) return false;
                          held_[c] = 0;
                          return true;
                      }), held_cells_.end());
    seq_len_[branch] = 0;
    if (branch != 0) alive_[branch] = 0;
}

int CacheManager::common_prefix_tokens(const int* branches, int n) const
{
    std::lock_guard<std::mutex> lock(mu_);
    if (!branches || n <= 0) return 0;
    int min_len = 0x7fffffff;
    for (int i = 0; i < n; i++) {
        int b = branches[i];
        if (b < 0 || b >= max_branches_ || !alive_[b]) return 0;
        min_len = std::min(min_len, seq_len_[b]);
    }
    int limit = std::min(min_len / block_size_, max_logical_blocks_);
    int blocks = 0;
    for (; blocks < limit; blocks++) {
        int phys = h_tables_[cell(branches[0], blocks)];
        if (phys < 0) break;
        bool same = true;
        for (int i = 1; i < n && same; i++) same = h_tables_[cell(branches[i], blocks)] == phys;
        if (!same) break;
    }
    return blocks * block_size_;
}

int CacheManager::common_prefix_groups(const int* branches, int n, int max_group_branches, int min_tokens,
                                       drk_prefix_group* out, int max_groups) const
{
    std::lock_guard<std::mutex> lock(mu_);
    if (!branches || !out || n < 2 || max_groups <= 0 || max_group_branches < 2) return 0;
    for (int i = 0; i < n; i++) {
        const int b = branches[i];
        if (b < 0 || b >= max_branches_ || !alive_[b]) return 0;
    }
    // blocks neighbours i and i + 1 hold in common, from block 0 on (a missing page ends the run)
    std::vector<int> lcp((size_t)n - 1);
    for (int i = 0; i + 1 < n; i++) {
        const int limit = std::min(std::min(seq_len_[branches[i]], seq_len_[branches[i + 1]]) / block_size_, max_logical_blocks_);
        int k = 0;
        for (; k < limit; k++) {
            const int phys = h_tables_[cell(branches[i], k)];
            if (phys < 0 || h_tables_[cell(branches[i + 1], k)] != phys) break;
        }
        lcp[(size_t)i] = k;
    }
    const int min_blocks = std::max(1, (min_tokens + block_size_ - 1) / block_size_);
    struct Range { int lo, hi, base; };                       // positions [lo, hi) share blocks [0, base) through their ancestors
    std::vector<Range> queue{{0, n, 0}};
    int count = 0;
    for (size_t qi = 0; qi < queue.size() && count < max_groups; qi++) {      // breadth first: parents before children
        const Range r = queue[qi];
        if (r.hi - r.lo < 2) continue;
        int m = 0x7fffffff;
        for (int i = r.lo; i + 1 < r.hi; i++) m = std::min(m, lcp[(size_t)i]);
        int base = r.base;
        if (m - base >= min_blocks) {
            // the whole range shares blocks [base, m): one group, or several over the same blocks when it is too wide
            const int width = r.hi - r.lo;
            const int parts = (width + max_group_branches - 1) / max_group_branches;
            if (count + parts > max_groups) break;
            if (parts > 1) {
                // each part is a tree of its own from here on
                for (int p = 0; p < parts; p++) {
                    const int lo = r.lo + p * max_group_branches, hi = std::min(lo + max_group_branches, r.hi);
                    if (hi - lo < 2) continue;                     // a part of one branch: its tail reads the range
                    out[count++] = drk_prefix_group{lo, hi - lo, base * block_size_, m * block_size_};
                    queue.push_back({lo, hi, m});
                }
                continue;
            }
            out[count++] = drk_prefix_group{r.lo, width, base * block_size_, m * block_size_};
            base = m;
        }
        // neighbours that share more than the whole range does form the children
        int lo = r.lo;
        for (int i = r.lo; i + 1 <= r.hi; i++) {
            if (i + 1 == r.hi || lcp[(size_t)i] <= std::max(m, base)) {
                if (i + 1 - lo >= 2) queue.push_back({lo, i + 1, base});
                lo = i + 1;
            }
        }
    }
    return count;
}

bool CacheManager::branch_alive(int branch) const
{
    std::lock_guard<std::mutex> lock(mu_);
    return branch >= 0 && branch < max_branches_ && alive_[branch];
}

void CacheManager::touch_block(int branch, int logical_idx)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (branch < 0 || branch >= max_branches_ || logical_idx < 0 || logical_idx >= max_logical_blocks_) return;
    int c = (int)cell(branch, logical_idx);
    if (location_[c] != BlockLocation::GPU) return;
    bool sole = refs_[h_tables_[c]].size() == 1;
    if (sole) candidate_remove_nolock(c);
    stamp_[c] = next_stamp_++;
    if (sole) candidate_add_nolock(c);
}

BlockLocation CacheManager::block_location(int branch, int logical_idx) const
{
    std::lock_guard<std::mutex> lock(mu_);
    if (branch < 0 || branch >= max_branches_ || logical_idx < 0 || logical_idx >= max_logical_blocks_)
        return BlockLocation::INVALID;
    return location_[cell(branch, logical_idx)];
}

int CacheManager::evict_blocks(int n)
{
    std::lock_guard<std::mutex> lock(mu_);
    return evict_nolock(n, -1);
}

bool CacheManager::ensure_free_blocks(int n_free)
{
    std::lock_guard<std::mutex> lock(mu_);
    return ensure_free_nolock(n_free, -1);
}

void CacheManager::prefetch_block(int branch, int logical_idx)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (branch < 0 || branch >= max_branches_ || logical_idx < 0 || logical_idx >= max_logical_blocks_) return;
    int c = (int)cell(branch, logical_idx);
    if (location_[c] != BlockLocation::SSD || !swapper_ || !swapper_->ready()) return;
    swapper_->prefetch(c, ssd_paths_[c]);         // fire and forget (cache_manager.cpp:171-178)
}

int CacheManager::ssd_blocks_used() const
{
    std::lock_guard<std::mutex> lock(mu_);
    int n = 0;
    for (BlockLocation loc : location_)
        if (loc == BlockLocation::SSD) n++;
    return n;
}

int CacheManager::gpu_blocks_used() const { return pool_.max_blocks() - pool_.free_count(); }

std::vector<std::pair<int, int>> CacheManager::lru_snapshot() const
{
    std::lock_guard<std::mutex> lock(mu_);
    std::vector<std::pair<uint64_t, int>> order;
    for (size_t c = 0; c < stamp_.size(); c++)
        if (stamp_[c]) order.push_back({stamp_[c], (int)c});
    std::sort(order.begin(), order.end());
    std::vector<std::pair<int, int>> out;
    out.reserve(order.size());
    for (const auto& e : order) out.push_back({e.second / max_logical_blocks_, e.second % max_logical_blocks_});
    return out;
}

std::vector<std::pair<int, int>> CacheManager::take_pending_copies()
{
    std::lock_guard<std::mutex> lock(mu_);
    std::vector<std::pair<int, int>> out;
    out.swap(pending_copies_);
    release_holds_nolock();                       // detached: handing the copies out is this manager's "issued"
    return out;
}

void CacheManager::destroy()
{
    if (d_tables_) {
        drk_dev_free(d_tables_);
        d_tables_ = nullptr;
    }
    if (d_pairs_) {
        drk_dev_free(d_pairs_);
        d_pairs_ = nullptr;
    }
    pool_.destroy();
    h_tables_.clear();
    location_.clear();
    stamp_.clear();
    evictable_.clear();
    refs_.clear();
    held_.clear();
    held_cells_.clear();
    copy_pin_.clear();
    pending_copies_issued_.clear();
    deferred_release_.clear();
    seq_len_.clear();
    alive_.clear();
    dirty_lo_.clear();
    dirty_hi_.clear();
    pending_copies_.clear();
    max_logical_blocks_ = 0;
    max_branches_ = 0;
}

} // namespace deusridet
