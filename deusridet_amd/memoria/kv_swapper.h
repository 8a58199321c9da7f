// kv_swapper.h -- overflow tier for KV blocks: GPU <-> pinned host staging <-> file.
// The interface is the reference's KVSwapper (src/memoria/kv_swapper.h:34-114: init, submit,
// drain, shutdown, pending, prefetch, is_prefetched, drop_prefetch, SwapRequest); what is
// behind it is built for a discrete GPU:
//
//   - a block's layers lie layer_stride apart in the pool and move as ONE strided 2-D copy
//     (drk_kv_block_to_host / _from_host) instead of 2 x layers copies (kv_swapper.cpp:183-198);
//   - the staging slots are pinned allocations and work as a pipeline: every request has a
//     device phase (an asynchronous copy on the swapper's own stream, marked by an event) and
//     a file phase, and the worker starts the next request's first phase before it finishes
//     the previous request's second, so the PCIe copy of one block overlaps the file I/O of
//     its neighbour.  Requests still complete, and call back, in the order they were submitted;
//   - no device-wide synchronisation: submit() records an event on every stream that has
//     been announced as a user of the pool (add_writer_stream; CacheManager announces the
//     stream of every sync_block_table) and the copy waits for those events only -- the
//     kernels that wrote, or still read, the block were enqueued before the request was made.
//     Without any announced stream the worker falls back to waiting for the whole device;
//   - no POSIX_FADV_DONTNEED: on Tegra the page cache takes DRAM from the GPU
//     (kv_swapper.cpp:214-217); here it is host memory, and a swap-in soon after a swap-out is
//     served from it.
// The file image is [layer][K plane | V plane (| K scales | V scales)], byte for byte the
// reference's .kv layout for its fp16 pool.
#pragma once

#include "block_pool.h"
#include <condition_variable>
#include <deque>
#include <functional>
#include <mutex>
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
    std::function<void(bool)> callback;    // completion (success), called on the worker thread
};

class KVSwapper {
public:
    KVSwapper() = default;
    ~KVSwapper();
    KVSwapper(const KVSwapper&) = delete;
    KVSwapper& operator=(const KVSwapper&) = delete;

    // kv_swapper.cpp:32-69.  The pool must have device memory.  staging_blocks = depth of the pipeline.
    bool init(BlockPool& pool, const std::string& ssd_dir, int staging_blocks = 2);
    bool ready() const { return running_; }

    void submit(SwapRequest req);          // non-blocking; on a swapper that is not running the callback gets false at once
    void drain();                          // until every submitted request has completed
    void shutdown();
    int  pending() const;

    void prefetch(int logical_block_idx, const std::string& ssd_path);
    bool is_prefetched(int logical_block_idx) const;
    void drop_prefetch(int logical_block_idx);

    // A stream whose kernels write or read the pool: requests submitted from now on wait for what
    // that stream had been given when they were submitted.  Idempotent.
    void add_writer_stream(hipStream_t stream);
    // Before such a stream is destroyed: later requests must not record events on a dead handle.
    void remove_writer_stream(hipStream_t stream);

    size_t block_bytes() const { return block_bytes_; }

private:
    struct Ticket {                        // a request and the events it has to wait for
        SwapRequest req;
        std::vector<void*> after;
    };
    struct Flight {                        // a request whose copy has been issued
        Ticket t;
        int slot = -1;
        bool ok = true;
    };

    BlockPool* pool_ = nullptr;
    std::string ssd_dir_;
    size_t block_bytes_ = 0;
    std::vector<void*> slots_;             // pinned staging, one block each
    std::vector<void*> slot_done_;         // event per slot: its copy has finished
    std::vector<hipStream_t> writers_;
    hipStream_t copy_stream_ = nullptr;

    std::unordered_map<int, std::vector<char>> host_cache_;   // prefetched images by logical_block_idx
    std::unordered_set<int> prefetching_;

    std::thread worker_;
    std::deque<Ticket> queue_;
    int unfinished_ = 0;                   // submitted and not completed yet
    mutable std::mutex mu_;
    std::condition_variable cv_;
    bool running_ = false;

    void run();
    bool begin(Flight& f);                 // first phase; false = failed, nothing in flight
    void finish(Flight& f);                // second phase + callback
    void complete(Ticket& t, bool ok);
    void wait_for_users(Ticket& t);
    bool fill_from_host(const SwapRequest& req, void* staging);
};

} // namespace deusridet
