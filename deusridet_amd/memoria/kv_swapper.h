// kv_swapper.h -- overflow tier for KV blocks: GPU <-> pinned host staging <-> file.
// Same interface as the reference's KVSwapper (src/memoria/kv_swapper.h:34-114):
// requests are queued to one background I/O thread; swap-out gathers every layer of a
// block into a staging buffer and writes one consolidated file, swap-in reads it back
// and scatters it into a (possibly different) physical block; prefetch reads a file
// into a host-side cache ahead of time so that the later swap-in skips the disk.
//
// Re-thought for a discrete GPU:
//   - a block's layers lie layer_stride apart in the pool; they move as ONE strided
//     2-D copy per block (drk_kv_block_to_host / _from_host) instead of the reference's
//     2 x layers separate copies (kv_swapper.cpp:183-198, 268-283);
//   - the staging buffers are pinned allocations (never registrations of existing memory);
//   - no POSIX_FADV_DONTNEED: on Tegra the page cache competes with the GPU for the same
//     DRAM (kv_swapper.cpp:214-217); here it is host memory the GPU does not allocate
//     from, and keeping recently written blocks in it makes a swap-in after a swap-out cheap.
// The file image is [layer][K plane | V plane (| K scales | V scales)], byte for byte the
// reference's .kv layout for its fp16 pool.
#pragma once

#include "block_pool.h"
#include <condition_variable>
#include <functional>
#include <mutex>
#include <queue>
#include <string>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace deusridet {

enum class SwapDirection { GPU_TO_SSD, SSD_TO_GPU };

struct SwapRequest {                       // kv_swapper.h:38-44
    SwapDirection direction;
    int logical_block_idx;                 // key of the prefetch cache (CacheManager passes its table cell)
    int physical_block_id;                 // GPU block (source for out, target for in); -1 = prefetch only
    std::string ssd_path;
    std::function<void(bool)> callback;    // completion (success), called on the I/O thread
};

class KVSwapper {
public:
    KVSwapper() = default;
    ~KVSwapper();
    KVSwapper(const KVSwapper&) = delete;
    KVSwapper& operator=(const KVSwapper&) = delete;

    // kv_swapper.cpp:32-69.  The pool must have device memory.
    bool init(BlockPool& pool, const std::string& ssd_dir, int staging_blocks = 2);
    bool ready() const { return running_; }

    void submit(SwapRequest req);          // non-blocking
    void drain();                          // wait until every submitted request has completed
    void shutdown();
    int  pending() const;

    void prefetch(int logical_block_idx, const std::string& ssd_path);
    bool is_prefetched(int logical_block_idx) const;
    void drop_prefetch(int logical_block_idx);

    size_t block_bytes() const { return staging_buf_size_; }

private:
    BlockPool* pool_ = nullptr;
    std::string ssd_dir_;
    std::vector<void*> staging_bufs_;
    size_t staging_buf_size_ = 0;
    std::unordered_map<int, std::vector<char>> prefetch_cache_;
    std::unordered_set<int> prefetch_pending_;
    std::thread io_thread_;
    std::queue<SwapRequest> queue_;
    int in_flight_ = 0;                    // requests taken off the queue and not finished yet
    mutable std::mutex mu_;
    std::condition_variable cv_;
    bool running_ = false;
    hipStream_t copy_stream_ = nullptr;

    void io_loop();
    bool swap_out(const SwapRequest& req);
    bool swap_in(const SwapRequest& req);
};

} // namespace deusridet
