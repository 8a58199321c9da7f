// kv_swapper.cpp -- see kv_swapper.h.  Device memory is reached through the C ABI only.
#include "kv_swapper.h"
#include "../communis/log.h"

#include <cstring>
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

namespace deusridet {

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
    staging_buf_size_ = drk_kv_block_total_bytes(&pool.layout());      // one block across all layers
    staging_bufs_.assign(staging_blocks, nullptr);
    for (int i = 0; i < staging_blocks; i++) {
        if (drk_host_malloc(&staging_bufs_[i], staging_buf_size_) != DRK_OK) {
            LOG_ERROR("Memoria", "KVSwapper: staging alloc failed: %s", drk_last_error());
            shutdown();
            return false;
        }
    }
    void* s = nullptr;
    if (drk_stream_create(&s) != DRK_OK) {
        LOG_ERROR("Memoria", "KVSwapper: stream: %s", drk_last_error());
        shutdown();
        return false;
    }
    copy_stream_ = static_cast<hipStream_t>(s);
    struct stat st;
    if (stat(ssd_dir_.c_str(), &st) != 0 && mkdir(ssd_dir_.c_str(), 0755) != 0) {
        LOG_ERROR("Memoria", "KVSwapper: cannot create %s", ssd_dir_.c_str());
        shutdown();
        return false;
    }
    running_ = true;
    io_thread_ = std::thread(&KVSwapper::io_loop, this);
    LOG_INFO("Memoria", "KVSwapper: %d staging bufs x %.1f MB, dir=%s", staging_blocks, staging_buf_size_ / 1048576.0,
             ssd_dir_.c_str());
    return true;
}

void KVSwapper::submit(SwapRequest req)
{
    {
        std::lock_guard<std::mutex> lock(mu_);
        queue_.push(std::move(req));
    }
    cv_.notify_all();
}

// The reference waits for an empty queue only (kv_swapper.cpp:80-83), which can return
// while the last request is still being executed; here the request in execution counts.
void KVSwapper::drain()
{
    std::unique_lock<std::mutex> lock(mu_);
    cv_.wait(lock, [this] { return (queue_.empty() && in_flight_ == 0) || !running_; });
}

void KVSwapper::shutdown()
{
    {
        std::lock_guard<std::mutex> lock(mu_);
        running_ = false;
    }
    cv_.notify_all();
    if (io_thread_.joinable()) io_thread_.join();
    for (void* buf : staging_bufs_)
        if (buf) drk_host_free(buf);
    staging_bufs_.clear();
    prefetch_cache_.clear();
    prefetch_pending_.clear();
    if (copy_stream_) {
        drk_stream_destroy(copy_stream_);
        copy_stream_ = nullptr;
    }
    pool_ = nullptr;
}

int KVSwapper::pending() const
{
    std::lock_guard<std::mutex> lock(mu_);
    return static_cast<int>(queue_.size()) + in_flight_;
}

void KVSwapper::prefetch(int logical_block_idx, const std::string& ssd_path)
{
    {
        std::lock_guard<std::mutex> lock(mu_);
        if (prefetch_cache_.count(logical_block_idx) || prefetch_pending_.count(logical_block_idx)) return;
        prefetch_pending_.insert(logical_block_idx);
    }
    SwapRequest req;
    req.direction = SwapDirection::SSD_TO_GPU;
    req.logical_block_idx = logical_block_idx;
    req.physical_block_id = -1;            // prefetch only: file -> host cache
    req.ssd_path = ssd_path;
    req.callback = nullptr;
    submit(std::move(req));
}

bool KVSwapper::is_prefetched(int logical_block_idx) const
{
    std::lock_guard<std::mutex> lock(mu_);
    return prefetch_cache_.count(logical_block_idx) > 0;
}

void KVSwapper::drop_prefetch(int logical_block_idx)
{
    std::lock_guard<std::mutex> lock(mu_);
    prefetch_cache_.erase(logical_block_idx);
    prefetch_pending_.erase(logical_block_idx);
}

void KVSwapper::io_loop()
{
    while (true) {
        SwapRequest req;
        {
            std::unique_lock<std::mutex> lock(mu_);
            cv_.wait(lock, [this] { return !queue_.empty() || !running_; });
            if (!running_ && queue_.empty()) break;
            req = std::move(queue_.front());
            queue_.pop();
            in_flight_++;
        }
        bool ok = req.direction == SwapDirection::GPU_TO_SSD ? swap_out(req) : swap_in(req);
        if (req.callback) req.callback(ok);
        {
            std::lock_guard<std::mutex> lock(mu_);
            in_flight_--;
        }
        cv_.notify_all();
    }
}

static bool write_all(int fd, const char* p, size_t n)
{
    while (n > 0) {
        ssize_t w = write(fd, p, n);
        if (w <= 0) return false;
        p += w;
        n -= (size_t)w;
    }
    return true;
}

static bool read_all(int fd, char* p, size_t n)
{
    while (n > 0) {
        ssize_t r = read(fd, p, n);
        if (r <= 0) return false;
        p += r;
        n -= (size_t)r;
    }
    return true;
}

bool KVSwapper::swap_out(const SwapRequest& req)
{
    void* staging = staging_bufs_[0];
    // kernels that wrote the block may still be running on the caller's streams
    if (drk_device_synchronize() != DRK_OK) {
        LOG_ERROR("Memoria", "KVSwapper: device synchronize failed: %s", drk_last_error());
        return false;
    }
    if (drk_kv_block_to_host(&pool_->layout(), pool_->pool_raw(), req.physical_block_id, staging, copy_stream_) != DRK_OK ||
        drk_stream_synchronize(copy_stream_) != DRK_OK) {
        LOG_ERROR("Memoria", "KVSwapper: device -> host copy of block %d failed: %s", req.physical_block_id,
                  drk_last_error());
        return false;
    }
    int fd = open(req.ssd_path.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0644);
    if (fd < 0) {
        LOG_ERROR("Memoria", "KVSwapper: open(%s) for write failed", req.ssd_path.c_str());
        return false;
    }
    bool ok = write_all(fd, static_cast<const char*>(staging), staging_buf_size_);
    close(fd);
    if (!ok) LOG_ERROR("Memoria", "KVSwapper: write of %s failed", req.ssd_path.c_str());
    return ok;
}

bool KVSwapper::swap_in(const SwapRequest& req)
{
    const size_t total = staging_buf_size_;
    const bool is_prefetch = req.physical_block_id < 0;
    void* staging = staging_bufs_[0];
    bool from_cache = false;
    if (!is_prefetch) {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = prefetch_cache_.find(req.logical_block_idx);
        if (it != prefetch_cache_.end()) {              // prefetch hit: no disk I/O (kv_swapper.cpp:236-243)
            std::memcpy(staging, it->second.data(), total);
            prefetch_cache_.erase(it);
            prefetch_pending_.erase(req.logical_block_idx);
            from_cache = true;
        }
    }
    if (!from_cache) {
        int fd = open(req.ssd_path.c_str(), O_RDONLY);
        if (fd < 0) {
            LOG_ERROR("Memoria", "KVSwapper: open(%s) for read failed", req.ssd_path.c_str());
            if (is_prefetch) drop_prefetch(req.logical_block_idx);
            return false;
        }
        bool ok = read_all(fd, static_cast<char*>(staging), total);
        close(fd);
        if (!ok) {
            LOG_ERROR("Memoria", "KVSwapper: read of %s failed", req.ssd_path.c_str());
            if (is_prefetch) drop_prefetch(req.logical_block_idx);
            return false;
        }
        if (is_prefetch) {
            std::vector<char> buf(static_cast<const char*>(staging), static_cast<const char*>(staging) + total);
            std::lock_guard<std::mutex> lock(mu_);
            if (prefetch_pending_.erase(req.logical_block_idx))      // dropped in the meantime: discard
                prefetch_cache_[req.logical_block_idx] = std::move(buf);
            return true;
        }
    }
    if (drk_kv_block_from_host(&pool_->layout(), pool_->pool_raw(), req.physical_block_id, staging, copy_stream_) != DRK_OK ||
        drk_stream_synchronize(copy_stream_) != DRK_OK) {
        LOG_ERROR("Memoria", "KVSwapper: host -> device copy into block %d failed: %s", req.physical_block_id,
                  drk_last_error());
        return false;
    }
    return true;
}

} // namespace deusridet
