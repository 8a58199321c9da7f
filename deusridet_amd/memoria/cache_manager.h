// cache_manager.h -- block tables, allocation, eviction and (new) branches over
// one BlockPool.  Same interface as the reference's CacheManager
// (src/memoria/cache_manager.h:52-169) with HIP vocabulary types; the calls the
// reference has act on branch 0, its single consciousness stream.
//
// Added on top of the reference (it describes them in
// docs/en/architecture/02-memoria.md:25-26 and 03-cogitatio.md:3-5 but has no
// code for them):
//   - branches: fork_branch() gives a decode branch its own block table whose
//     prefix entries point at the parent's physical blocks (refcount + 1 each);
//   - copy-on-write: ensure_blocks_for() on a block that other tables also
//     reference allocates a fresh block, queues a device copy of every layer and
//     remaps the entry; the copies are issued by sync_block_table(), ahead of the
//     table upload, on the caller's stream;
//   - a cell that ensure_blocks_for() has made resident is not a victim until the next
//     sync_block_table(): a later allocation of the same step never takes the block the
//     caller is about to write, or the target of a copy that is still queued;
//   - refcount-aware eviction: an entry whose block is shared is pinned; victims
//     are taken in LRU order (allocation order, moved to the back by
//     touch_block()) or by lowest importance when a scorer is attached;
//   - sync_block_table() uploads only the table ranges that changed (the
//     reference re-sends the whole table every step, cache_manager.cpp:108-112).
//
// Overflow tier: with a cache_dir and a KVSwapper (initialised by the caller on
// block_pool() after init(), as the reference's two-step set-up implies), an
// evicted block is written to <cache_dir>/block_<logical>.kv (branch 0; other
// branches: b<branch>_block_<logical>.kv) and its entry becomes SSD;
// ensure_blocks_for() on such an entry brings it back into a fresh physical block
// (cache_manager.cpp:118-156, 207-292).  Without them blocks are discarded
// (cache_manager.cpp:143-147).  Only unshared blocks are ever evicted, so a block
// on SSD belongs to exactly one table entry; fork_branch() treats it as a hole.
#pragma once
#include "drk_kv.h"

#include "block_pool.h"
#include "importance_scorer.h"
#include <cstdint>
#include <mutex>
#include <set>
#include <string>
#include <utility>
#include <vector>

namespace deusridet {

class KVSwapper;

enum class BlockLocation : int8_t {   // cache_manager.h:42-46
    GPU = 0,
    SSD = -2,
    INVALID = -1
};

class CacheManager {
public:
    CacheManager() = default;
    ~CacheManager();
    CacheManager(const CacheManager&) = delete;
    CacheManager& operator=(const CacheManager&) = delete;

    // cache_manager.cpp:24-71.  max_branches (new) sizes the per-branch tables.
    bool init(size_t kv_budget_bytes, const std::string& cache_dir = "",
              int block_size = PagedKVConfig::BLOCK_SIZE, KVSwapper* swapper = nullptr,
              ImportanceScorer* scorer = nullptr, int max_branches = 1);
    // Bookkeeping only (no device memory): copies are queued but never issued;
    // take_pending_copies() hands them to the caller.
    bool init_detached(int max_blocks, int block_size, ImportanceScorer* scorer = nullptr, int max_branches = 1);

    // ---- token-level API (branch 0 = the reference's sequence) ------------
    bool ensure_blocks_for(int pos);                         // cache_manager.cpp:73-95
    bool ensure_blocks_for_range(int pos_start, int M);      // cache_manager.cpp:97-106
    bool ensure_blocks_for(int branch, int pos);
    bool ensure_blocks_for_range(int branch, int pos_start, int M);

    // ---- block tables -------------------------------------------------------
    const int* d_block_table() const { return d_tables_; }   // branch 0
    const int* d_block_table(int branch) const;
    const int* d_block_tables() const { return d_tables_; }  // [max_branches][table_stride()]
    int  table_stride() const { return max_logical_blocks_; }
    // Issue queued copy-on-write copies, then upload changed table ranges, both on
    // `stream`, asynchronously (cache_manager.cpp:108-112).
    void sync_block_table(hipStream_t stream = 0);
    // With an overflow tier every stream passed to sync_block_table() is remembered (swaps order themselves behind
    // it); call this before such a stream is destroyed.
    void forget_stream(hipStream_t stream);
    const int* h_block_table(int branch = 0) const;

    int  seq_len() const { return seq_len(0); }
    void set_seq_len(int len) { set_seq_len(0, len); }
    int  seq_len(int branch) const;
    void set_seq_len(int branch, int len);
    int  num_logical_blocks() const { return num_logical_blocks(0); }   // cache_manager.cpp:114-116
    int  num_logical_blocks(int branch) const;

    // ---- branches (new) -----------------------------------------------------
    // New branch sharing the parent's resident blocks that hold tokens [0, pos);
    // seq_len(child) = pos.  Lowest free id, or -1 (no free id / bad arguments).
    int  fork_branch(int parent, int pos);
    // Drop every reference the branch holds (ascending logical order) and free its
    // id; branch 0 stays alive but empty.
    void release_branch(int branch);
    bool branch_alive(int branch) const;
    int  max_branches() const { return max_branches_; }
    // Tokens [0, n) whose pages are the same physical blocks in every listed branch
    // (whole blocks only, capped by the shortest seq_len): what
    // paged_gqa_decode_attention_shared() may stream once for all of them.
    int  common_prefix_tokens(const int* branches, int n) const;
    // The fork tree of the listed branches (consecutive ids: their table rows are one [n, stride] array) as
    // the shared ranges paged_gqa_decode_attention_grouped() takes: group = branches [first_branch,
    // first_branch + n_branches) (positions in `branches`) hold tokens [tok_begin, tok_end) in the same
    // physical blocks.  Ranges are whole blocks, at least min_tokens long, over at most max_group_branches
    // neighbours (a wider set is cut into several groups over the same range); parents come before their
    // children, so that cutting the list short (max_groups) leaves a valid tree.  Only neighbours in the list
    // are compared: fork branches that belong together one after the other.  Returns the number of groups.
    int  common_prefix_groups(const int* branches, int n, int max_group_branches, int min_tokens,
                              drk_prefix_group* out, int max_groups) const;
    // Recency update: move the entry to the back of the LRU order.
    void touch_block(int branch, int logical_idx);
    int  refcount(int phys_block) const { return pool_.refcount(phys_block); }
    BlockLocation block_location(int branch, int logical_idx) const;

    // ---- eviction -------------------------------------------------------------
    int  evict_blocks(int n);                  // cache_manager.cpp:118-156
    bool ensure_free_blocks(int n_free);       // cache_manager.cpp:158-164
    void prefetch_block(int logical_idx) { prefetch_block(0, logical_idx); }   // cache_manager.cpp:166-179
    void prefetch_block(int branch, int logical_idx);

    BlockPool& block_pool() { return pool_; }
    const BlockPool& block_pool() const { return pool_; }

    int gpu_blocks_used() const;               // cache_manager.cpp:294-296
    int ssd_blocks_used() const;               // cache_manager.cpp:298-304
    int free_blocks() const { return pool_.free_count(); }

    // LRU order, oldest first, as (branch, logical) pairs (tests, state dumps).
    std::vector<std::pair<int, int>> lru_snapshot() const;
    // Queued (src, dst) block copies not yet issued; clears the queue.
    std::vector<std::pair<int, int>> take_pending_copies();

    void destroy();

private:
    BlockPool pool_;
    ImportanceScorer* scorer_ = nullptr;       // not owned (cache_manager.h:129-130)
    KVSwapper* swapper_ = nullptr;             // not owned
    std::string cache_dir_;
    bool ssd_enabled_ = false;
    std::vector<std::string> ssd_paths_;       // per cell, set while the block is on SSD
    int max_logical_blocks_ = 0;
    int max_branches_ = 0;
    int block_size_ = PagedKVConfig::BLOCK_SIZE;
    bool detached_ = false;

    // cell = branch * max_logical_blocks_ + logical
    std::vector<int> h_tables_;                // physical id or -1 (cache_manager.h:132-135)
    std::vector<BlockLocation> location_;      // cache_manager.h:139
    std::vector<uint64_t> stamp_;              // LRU position of a resident cell, 0 = none
    uint64_t next_stamp_ = 1;
    std::set<std::pair<uint64_t, int>> evictable_;   // resident cells whose block has one reference
    std::vector<std::vector<int>> refs_;       // physical block -> cells that reference it
    std::vector<char> held_;                   // cell was ensured since the last sync_block_table: not a victim
    std::vector<int> held_cells_;
    std::vector<int> copy_pin_;                // physical block -> queued copies that name it (source or target)
    std::vector<std::pair<int, int>> pending_copies_issued_;   // the pairs behind copy_pin_, until the holds are released
    std::vector<int> deferred_release_;        // blocks whose last reference went while a queued copy named them
    std::vector<int> seq_len_;
    std::vector<char> alive_;
    std::vector<int> dirty_lo_, dirty_hi_;     // per branch, [lo, hi) of changed table entries
    std::vector<std::pair<int, int>> pending_copies_;

    int* d_tables_ = nullptr;
    int* d_pairs_ = nullptr;                   // staging for copy pairs
    int  pairs_capacity_ = 0;

    mutable std::mutex mu_;

    size_t cell(int branch, int logical) const { return (size_t)branch * max_logical_blocks_ + logical; }
    bool setup_tables(int max_branches);
    void mark_dirty(int branch, int logical);
    bool ensure_nolock(int branch, int pos);
    int  alloc_phys_nolock(int for_branch);
    int  evict_nolock(int n, int for_branch);
    bool ensure_free_nolock(int n_free, int for_branch);
    bool pick_victim_nolock(int& cell_out, int for_branch);
    std::string ssd_path_for(int cell_idx) const;
    void submit_swap_out_nolock(int cell_idx, char* ok);
    void candidate_add_nolock(int cell_idx);
    void candidate_remove_nolock(int cell_idx);
    void hold_nolock(int cell_idx);
    void release_holds_nolock();
    bool swap_from_ssd_nolock(int cell_idx);
    void attach_nolock(int cell_idx, int phys, bool fresh_stamp);
    void detach_nolock(int cell_idx);
    void flush_copies(hipStream_t stream);
};

} // namespace deusridet
