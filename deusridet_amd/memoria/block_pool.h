// block_pool.h -- GPU KV-cache block pool: one device slab, fixed-size blocks, a
// LIFO free stack.  Same interface as the reference's BlockPool
// (src/memoria/block_pool.h:58-123) with HIP vocabulary types, plus reference
// counts per physical block (the reference's design names them,
// docs/en/architecture/02-memoria.md:25-26, but does not implement them).
//
// Pool layout, per FA layer and physical block (block_pool.h:10-12 of the
// reference; bytes in drk_kv.h): K [NUM_KV_HEADS, block_size, HEAD_DIM] then
// V [NUM_KV_HEADS, block_size, HEAD_DIM]; an INT8 pool adds two fp16 scale
// planes [NUM_KV_HEADS, block_size] after V.
//
// Geometry comes from ModelConfig's runtime statics at init() time (the
// reference hard-codes NUM_KV_HEADS = 4 and HEAD_DIM = 256 in PagedKVConfig,
// block_pool.h:34-38, and reads NUM_FA_LAYERS from ModelConfig).
#pragma once

#include "../machina/model.h"
#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>
#include <cstdint>
#include <mutex>
#include <vector>

namespace deusridet {

struct PagedKVConfig {
    static constexpr int BLOCK_SIZE = 256;   // default tokens per block (block_pool.h:35)
    // Bytes of one block across all FA layers for the current ModelConfig
    // (block_pool.h:49-51).
    static size_t block_total_bytes(int block_size = BLOCK_SIZE);
};

class BlockPool {
public:
    BlockPool() = default;
    ~BlockPool();
    BlockPool(const BlockPool&) = delete;
    BlockPool& operator=(const BlockPool&) = delete;

    // Allocate the device pool for the given budget; max_blocks = budget /
    // bytes-per-block.  false when fewer than 4 blocks fit or the allocation fails
    // (block_pool.cpp:18-61).  The slab is zero-filled.
    bool init(size_t budget_bytes, int block_size = PagedKVConfig::BLOCK_SIZE);

    // Bookkeeping only: the same allocator over max_blocks ids with no device
    // memory behind it (pool_ptr() stays null).  For capacity planning and tests
    // that run without a GPU.
    bool init_detached(int max_blocks, int block_size = PagedKVConfig::BLOCK_SIZE);

    int  alloc_block();               // id >= 0 with refcount 1, or -1 when exhausted
    void free_block(int block_id);    // unconditional: refcount -> 0, id pushed on the stack
    int  free_count() const;
    int  max_blocks() const { return max_blocks_; }
    int  block_size() const { return block_size_; }

    // Reference counts (not in the reference).  release() frees the block when the
    // count reaches 0 and returns the new count.
    int  retain(int block_id);
    int  release(int block_id);
    int  refcount(int block_id) const;

    __half* pool_ptr() const { return reinterpret_cast<__half*>(pool_); }
    void*   pool_raw() const { return pool_; }
    __half* k_ptr(int fa_layer_idx, int block_id) const;
    __half* v_ptr(int fa_layer_idx, int block_id) const;
    size_t  k_offset(int fa_layer_idx, int block_id) const;   // bytes from pool base
    size_t  v_offset(int fa_layer_idx, int block_id) const;
    size_t  total_bytes() const { return total_bytes_; }

    const drk_kv_layout& layout() const { return layout_; }

    // Snapshot of the free stack, bottom first (for tests and state dumps).
    std::vector<int> free_stack_snapshot() const;

    void destroy();

private:
    bool setup(int max_blocks, int block_size);

    void* pool_ = nullptr;
    int max_blocks_ = 0;
    int block_size_ = PagedKVConfig::BLOCK_SIZE;
    size_t total_bytes_ = 0;
    size_t layer_stride_ = 0;   // bytes
    size_t block_stride_ = 0;   // bytes
    size_t kv_plane_ = 0;       // bytes
    drk_kv_layout layout_{};
    std::vector<int> free_stack_;   // LIFO (block_pool.h:118-119)
    std::vector<int> refcount_;
    mutable std::mutex mu_;
};

} // namespace deusridet
