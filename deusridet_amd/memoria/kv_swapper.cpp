// kv_swapper.cpp -- see kv_swapper.h.  Device memory is reached through the C ABI only.
#include "kv_swapper.h"
#include "../communis/log.h"

#include <algorithm>
#include <cstring>
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

namespace deusridet {

namespace {

bool write_file(const std::string& path, const void* data, size_t n)
{
    int fd = open(path.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0644);
    if (fd < 0) return false;
    const char* p = static_cast<const char*>(data);
    bool ok = true;
    while (n > 0 && ok) {
        ssize_t w = write(fd, p, n);
        if (w <= 0) ok = false;
        else { p += w; n -= (size_t)w; }
    }
    close(fd);
    return ok;
}

bool read_file(const std::string& path, void* data, size_t n)
{
    int fd = open(path.c_str(), O_RDONLY);
    if (fd < 0) return false;
    char* p = static_cast<char*>(data);
    bool ok = true;
    while (n > 0 && ok) {
        ssize_t r = read(fd, p, n);
        if (r <= 0) ok = false;
        else { p += r; n -= (size_t)r; }
    }
    close(fd);
    return ok;
}

} // namespace

KVSwapper::~KVSwapper() { shutdown(); }

bool KVSwapper::init(BlockPool& pool, const std::string& ssd_dir, int staging_blocks)
{
    shutdown();
    if (!pool.pool_raw() || ssd_dir.empty() || staging_blocks < 1) {
        LOG_ERROR("Memoria", "KVSwapper: needs a device pool, a directory and at least one staging block");
        return false;
    }
    pool_ = &pool;
    ssd_dir_ = ssd_dir;
    block_bytes_ = drk_kv_block_total_bytes(&pool.layout());           // one block across all layers
    struct stat st;
    if (stat(ssd_dir_.c_str(), &st) != 0 && mkdir(ssd_dir_.c_str(), 0755) != 0) {
        LOG_ERROR("Memoria", "KVSwapper: cannot create %s", ssd_dir_.c_str());
        shutdown();
        return false;
    }
    void* s = nullptr;
    if (drk_stream_create(&s) != DRK_OK) {
        LOG_ERROR("Memoria", "KVSwapper: stream: %s", drk_last_error());
        shutdown();
        return false;
    }
    copy_stream_ = static_cast<hipStream_t>(s);
    for (int i = 0; i < staging_blocks; i++) {
        void* host = nullptr;
        void* ev = nullptr;
        if (drk_host_malloc(&host, block_bytes_) != DRK_OK || drk_event_create(&ev) != DRK_OK) {
            LOG_ERROR("Memoria", "KVSwapper: staging slot %d: %s", i, drk_last_error());
            if (host) drk_host_free(host);
            shutdown();
            return false;
        }
        slots_.push_back(host);
        slot_done_.push_back(ev);
    }
    running_ = true;
    worker_ = std::thread(&KVSwapper::run, this);
    LOG_INFO("Memoria", "KVSwapper: %d staging slots x %.1f MB, dir=%s", staging_blocks, block_bytes_ / 1048576.0,
             ssd_dir_.c_str());
    return true;
}

void KVSwapper::add_writer_stream(hipStream_t stream)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (std::find(writers_.begin(), writers_.end(), stream) == writers_.end()) writers_.push_back(stream);
}

void KVSwapper::remove_writer_stream(hipStream_t stream)
{
    std::lock_guard<std::mutex> lock(mu_);
    writers_.erase(std::remove(writers_.begin(), writers_.end(), stream), writers_.end());
}

// Called on the requester's thread: the events mark what the pool's users have been given up
// to now -- everything that wrote, or may still read, the block of this request.
void KVSwapper::submit(SwapRequest req)
{
    Ticket t;
    t.req = std::move(req);
    {
        std::unique_lock<std::mutex> lock(mu_);
        if (!running_) {                              // no worker would ever take it: fail it here
            lock.unlock();
            LOG_ERROR("Memoria", "KVSwapper: submit() on a swapper that is not running (block %d)", t.req.logical_block_idx);
            if (t.req.callback) t.req.callback(false);
            return;
        }
        if (t.req.physical_block_id >= 0) {
            for (hipStream_t w : writers_) {
                int capturing = 0;
                if (drk_stream_is_capturing(w, &capturing) != DRK_OK || capturing) continue;   // work under capture is not running
                void* ev = nullptr;
                if (drk_event_create(&ev) == DRK_OK && drk_event_record(ev, w) == DRK_OK) t.after.push_back(ev);
                else if (ev) drk_event_destroy(ev);
            }
        }
        queue_.push_back(std::move(t));
        unfinished_++;
    }
    cv_.notify_all();
}

// The reference waits for an empty queue only (kv_swapper.cpp:80-83), which can return while the
// last request is still being executed; here a request counts until its callback has returned.
void KVSwapper::drain()
{
    std::unique_lock<std::mutex> lock(mu_);
    cv_.wait(lock, [this] { return unfinished_ == 0 || !running_; });
}

void KVSwapper::shutdown()
{
    {
        std::lock_guard<std::mutex> lock(mu_);
        running_ = false;
    }
    cv_.notify_all();
    if (worker_.joinable()) worker_.join();          // the worker empties the queue before it leaves
    // what a worker that never started (init failed half-way) or a late submit() left behind fails here
    std::deque<Ticket> left;
    {
        std::lock_guard<std::mutex> lock(mu_);
        left.swap(queue_);
    }
    for (Ticket& t : left) complete(t, false);
    {
        std::lock_guard<std::mutex> lock(mu_);
        unfinished_ = 0;
    }
    for (void* h : slots_)
        if (h) drk_host_free(h);
    for (void* e : slot_done_)
        if (e) drk_event_destroy(e);
    slots_.clear();
    slot_done_.clear();
    writers_.clear();
    host_cache_.clear();
    prefetching_.clear();
    if (copy_stream_) {
        drk_stream_destroy(copy_stream_);
        copy_stream_ = nullptr;
    }
    pool_ = nullptr;
}

int KVSwapper::pending() const
{
    std::lock_guard<std::mutex> lock(mu_);
    return unfinished_;
}

void KVSwapper::prefetch(int logical_block_idx, const std::string& ssd_path)
{
    {
        std::lock_guard<std::mutex> lock(mu_);
        if (host_cache_.count(logical_block_idx) || !prefetching_.insert(logical_block_idx).second) return;
    }
    SwapRequest req;
    req.direction = SwapDirection::SSD_TO_GPU;
    req.logical_block_idx = logical_block_idx;
    req.physical_block_id = -1;                      // file -> host cache only
    req.ssd_path = ssd_path;
    req.callback = nullptr;
    submit(std::move(req));
}

bool KVSwapper::is_prefetched(int logical_block_idx) const
{
    std::lock_guard<std::mutex> lock(mu_);
    return host_cache_.count(logical_block_idx) > 0;
}

void KVSwapper::drop_prefetch(int logical_block_idx)
{
    std::lock_guard<std::mutex> lock(mu_);
    host_cache_.erase(logical_block_idx);
    prefetching_.erase(logical_block_idx);
}

void KVSwapper::complete(Ticket& t, bool ok)
{
    for (void* ev : t.after) drk_event_destroy(ev);
    t.after.clear();
    if (t.req.callback) t.req.callback(ok);
    {
        std::lock_guard<std::mutex> lock(mu_);
        unfinished_--;
    }
    cv_.notify_all();
}

// the copy stream goes behind what the pool's users had been given when the request was made
void KVSwapper::wait_for_users(Ticket& t)
{
    if (t.after.empty()) {
        // nobody announced a stream: the conservative order is the whole device
        if (drk_device_synchronize() != DRK_OK) LOG_ERROR("Memoria", "KVSwapper: device synchronize: %s", drk_last_error());
        return;
    }
    for (void* ev : t.after)
        if (drk_stream_wait_event(copy_stream_, ev) != DRK_OK) {
            LOG_ERROR("Memoria", "KVSwapper: stream wait: %s", drk_last_error());
            drk_event_synchronize(ev);
        }
}

// staging <- the block's image, from the host cache when a prefetch put it there, else from its file
bool KVSwapper::fill_from_host(const SwapRequest& req, void* staging)
{
    {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = host_cache_.find(req.logical_block_idx);
        if (it != host_cache_.end()) {               // no disk I/O (kv_swapper.cpp:236-243)
            std::memcpy(staging, it->second.data(), block_bytes_);
            host_cache_.erase(it);
            prefetching_.erase(req.logical_block_idx);
            return true;
        }
    }
    if (!read_file(req.ssd_path, staging, block_bytes_)) {
        LOG_ERROR("Memoria", "KVSwapper: read of %s failed", req.ssd_path.c_str());
        return false;
    }
    return true;
}

// First phase: the asynchronous copy of the request, marked by the slot's event.
bool KVSwapper::begin(Flight& f)
{
    const SwapRequest& req = f.t.req;
    void* staging = slots_[f.slot];
    int rc;
    if (req.direction == SwapDirection::GPU_TO_SSD) {
        wait_for_users(f.t);
        rc = drk_kv_block_to_host(&pool_->layout(), pool_->pool_raw(), req.physical_block_id, staging, copy_stream_);
    } else {
        if (!fill_from_host(req, staging)) return false;
        wait_for_users(f.t);
        rc = drk_kv_block_from_host(&pool_->layout(), pool_->pool_raw(), req.physical_block_id, staging, copy_stream_);
    }
    if (rc != DRK_OK || drk_event_record(slot_done_[f.slot], copy_stream_) != DRK_OK) {
        LOG_ERROR("Memoria", "KVSwapper: copy of block %d: %s", req.physical_block_id, drk_last_error());
        drk_stream_synchronize(copy_stream_);         // whatever was issued no longer touches the slot afterwards
        return false;
    }
    return true;
}

// Second phase: wait for the copy; a swap-out then writes its file.
void KVSwapper::finish(Flight& f)
{
    const SwapRequest& req = f.t.req;
    bool ok = drk_event_synchronize(slot_done_[f.slot]) == DRK_OK;
    if (!ok) LOG_ERROR("Memoria", "KVSwapper: copy of block %d did not complete: %s", req.physical_block_id, drk_last_error());
    if (ok && req.direction == SwapDirection::GPU_TO_SSD) {
        ok = write_file(req.ssd_path, slots_[f.slot], block_bytes_);
        if (!ok) LOG_ERROR("Memoria", "KVSwapper: write of %s failed", req.ssd_path.c_str());
    }
    complete(f.t, ok);
}

void KVSwapper::run()
{
    std::deque<Flight> flying;                        // copies issued, oldest first
    std::vector<int> free_slots;
    for (int i = (int)slots_.size() - 1; i >= 0; i--) free_slots.push_back(i);

    auto finish_oldest = [&] {
        Flight f = std::move(flying.front());
        flying.pop_front();
        finish(f);
        free_slots.push_back(f.slot);
    };

    for (;;) {
        Ticket t;
        bool start = false;
        {
            std::unique_lock<std::mutex> lock(mu_);
            if (flying.empty()) cv_.wait(lock, [this] { return !queue_.empty() || !running_; });
            if (!queue_.empty() && !free_slots.empty()) {
                t = std::move(queue_.front());
                queue_.pop_front();
                start = true;
            } else if (flying.empty()) {
                break;                                // shut down and nothing left to do
            }
        }
        if (!start) {                                 // no request, or no slot: retire the oldest copy
            finish_oldest();
            continue;
        }
        const bool reads_file = t.req.direction == SwapDirection::SSD_TO_GPU;
        if (reads_file) {
            // a file this request reads may be one a flying swap-out has yet to write
            while (!flying.empty() && std::any_of(flying.begin(), flying.end(), [](const Flight& f) {
                       return f.t.req.direction == SwapDirection::GPU_TO_SSD; }))
                finish_oldest();
        }
        if (reads_file && t.req.physical_block_id < 0) {
            // prefetch: file -> host cache, no device phase and no slot
            std::vector<char> image(block_bytes_);
            bool ok = read_file(t.req.ssd_path, image.data(), block_bytes_);
            {
                std::lock_guard<std::mutex> lock(mu_);
                if (prefetching_.erase(t.req.logical_block_idx) && ok)      // dropped in the meantime: discard
                    host_cache_[t.req.logical_block_idx] = std::move(image);
            }
            if (!ok) LOG_ERROR("Memoria", "KVSwapper: prefetch of %s failed", t.req.ssd_path.c_str());
            while (!flying.empty()) finish_oldest();      // completion order is submission order
            complete(t, ok);
            continue;
        }
        Flight f;
        f.t = std::move(t);
        f.slot = free_slots.back();
        free_slots.pop_back();
        if (begin(f)) {
            flying.push_back(std::move(f));
        } else {
            free_slots.push_back(f.slot);
            while (!flying.empty()) finish_oldest();      // the older requests call back first
            complete(f.t, false);
        }
    }
}

} // namespace deusridet
