// block_pool.cpp -- see block_pool.h.  Device memory is reached through the C
// ABI (drk_dev_*), never through HIP directly.
#include "block_pool.h"
#include "../communis/log.h"

namespace deusridet {

int ModelConfig::NUM_ATTN_HEADS = 24;
int ModelConfig::NUM_KV_HEADS = 4;
int ModelConfig::HEAD_DIM = 256;
int ModelConfig::NUM_KV_GROUPS = 6;
int ModelConfig::NUM_FA_LAYERS = 16;
float ModelConfig::RMS_EPS = 1e-6f;
float ModelConfig::ROPE_THETA = 1.0e7f;
int ModelConfig::ROTARY_DIM = 64;
int ModelConfig::KV_DTYPE = DRK_F16;
int ModelConfig::IO_DTYPE = DRK_F16;

bool ModelConfig::set_attention_geometry(int num_fa_layers, int num_attn_heads, int num_kv_heads, int head_dim,
                                         int kv_dtype, int io_dtype)
{
    if (io_dtype < 0) io_dtype = (kv_dtype == DRK_BF16 || kv_dtype == DRK_F16) ? kv_dtype : DRK_BF16;
    drk_kv_layout g{num_fa_layers, num_kv_heads, num_attn_heads, head_dim, 16, 4, kv_dtype, 0};
    if (drk_kv_layout_check(&g) != DRK_OK || (io_dtype != DRK_F16 && io_dtype != DRK_BF16)) {
        LOG_ERROR("Machina", "ModelConfig: bad attention geometry: %s", drk_last_error());
        return false;
    }
    NUM_FA_LAYERS = num_fa_layers;
    NUM_ATTN_HEADS = num_attn_heads;
    NUM_KV_HEADS = num_kv_heads;
    HEAD_DIM = head_dim;
    NUM_KV_GROUPS = num_attn_heads / num_kv_heads;
    KV_DTYPE = kv_dtype;
    IO_DTYPE = io_dtype;
    return true;
}

bool ModelConfig::set_rope(int rotary_dim, float theta, float rms_eps)
{
    const int q = rotary_dim / 16;
    if (rotary_dim < 16 || rotary_dim > HEAD_DIM || (rotary_dim % 16) || (q & (q - 1)) || !(theta > 0.0f) || !(rms_eps >= 0.0f)) {
        LOG_ERROR("Machina", "ModelConfig: rotary_dim %d / theta %g / eps %g not usable with head_dim %d", rotary_dim,
                  (double)theta, (double)rms_eps, HEAD_DIM);
        return false;
    }
    ROTARY_DIM = rotary_dim;
    ROPE_THETA = theta;
    RMS_EPS = rms_eps;
    return true;
}

drk_kv_layout ModelConfig::layout(int max_phys_blocks, int block_size)
{
    return drk_kv_layout{NUM_FA_LAYERS, NUM_KV_HEADS, NUM_ATTN_HEADS, HEAD_DIM, block_size,
                         max_phys_blocks, KV_DTYPE, 0};
}

size_t PagedKVConfig::block_total_bytes(int block_size)
{
    drk_kv_layout g = ModelConfig::layout(1, block_size);
    return (size_t)g.num_layers * drk_kv_block_stride_bytes(&g);
}

BlockPool::~BlockPool() { destroy(); }

bool BlockPool::setup(int max_blocks, int block_size)
{
    block_size_ = block_size;
    max_blocks_ = max_blocks;
    layout_ = ModelConfig::layout(max_blocks, block_size);
    if (drk_kv_layout_check(&layout_) != DRK_OK) {
        LOG_ERROR("Memoria", "BlockPool: %s", drk_last_error());
        max_blocks_ = 0;
        return false;
    }
    kv_plane_ = drk_kv_plane_bytes(&layout_);
    block_stride_ = drk_kv_block_stride_bytes(&layout_);
    layer_stride_ = drk_kv_layer_stride_bytes(&layout_);
    total_bytes_ = drk_kv_pool_bytes(&layout_);
    // all blocks available, pushed in reverse so that allocation yields 0, 1, 2 ...
    // (block_pool.cpp:51-55)
    free_stack_.resize(max_blocks_);
    for (int i = 0; i < max_blocks_; i++) free_stack_[i] = max_blocks_ - 1 - i;
    refcount_.assign(max_blocks_, 0);
    return true;
}

bool BlockPool::init(size_t budget_bytes, int block_size)
{
    destroy();
    if (block_size < 1) {
        LOG_ERROR("Memoria", "BlockPool: block_size %d", block_size);
        return false;
    }
    size_t block_total = PagedKVConfig::block_total_bytes(block_size);
    if (block_total == 0) {
        LOG_ERROR("Memoria", "BlockPool: %s", drk_last_error());
        return false;
    }
    size_t n = budget_bytes / block_total;
    if (n > 0x7fffffffu) n = 0x7fffffffu;
    if (n < 4) {   // block_pool.cpp:32-36
        LOG_ERROR("Memoria", "BlockPool: budget %.1f MB too small (need >= 4 blocks x %.1f MB)",
                  budget_bytes / 1048576.0, block_total / 1048576.0);
        return false;
    }
    if (!setup((int)n, block_size)) return false;
    if (drk_dev_malloc(&pool_, total_bytes_) != DRK_OK) {
        LOG_ERROR("Memoria", "BlockPool: device allocation of %.1f MB failed: %s", total_bytes_ / 1048576.0,
                  drk_last_error());
        pool_ = nullptr;
        destroy();
        return false;
    }
    if (drk_dev_memset_async(pool_, 0, total_bytes_, nullptr) != DRK_OK || drk_stream_synchronize(nullptr) != DRK_OK) {
        LOG_ERROR("Memoria", "BlockPool: zero-fill failed: %s", drk_last_error());
        destroy();
        return false;
    }
    LOG_INFO("Memoria", "BlockPool: %d blocks x %d tokens = %dK max, %.1f MB GPU", max_blocks_, block_size_,
             (int)((long)max_blocks_ * block_size_ / 1024), total_bytes_ / 1048576.0);
    return true;
}

bool BlockPool::init_detached(int max_blocks, int block_size)
{
    destroy();
    if (max_blocks < 1 || block_size < 1) return false;
    return setup(max_blocks, block_size);
}

int BlockPool::alloc_block()
{
    std::lock_guard<std::mutex> lock(mu_);
    if (free_stack_.empty()) return -1;
    int id = free_stack_.back();
    free_stack_.pop_back();
    refcount_[id] = 1;
    return id;
}

void BlockPool::free_block(int block_id)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (block_id < 0 || block_id >= max_blocks_) return;
    refcount_[block_id] = 0;
    free_stack_.push_back(block_id);
}

int BlockPool::free_count() const
{
    std::lock_guard<std::mutex> lock(mu_);
    return static_cast<int>(free_stack_.size());
}

int BlockPool::retain(int block_id)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (block_id < 0 || block_id >= max_blocks_) return -1;
    return ++refcount_[block_id];
}

int BlockPool::release(int block_id)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (block_id < 0 || block_id >= max_blocks_) return -1;
    int c = --refcount_[block_id];
    if (c <= 0) {
        refcount_[block_id] = 0;
        free_stack_.push_back(block_id);
        return 0;
    }
    return c;
}

int BlockPool::refcount(int block_id) const
{
    std::lock_guard<std::mutex> lock(mu_);
    if (block_id < 0 || block_id >= max_blocks_) return 0;
    return refcount_[block_id];
}

__half* BlockPool::k_ptr(int fa_layer_idx, int block_id) const
{
    return reinterpret_cast<__half*>(static_cast<char*>(pool_) + k_offset(fa_layer_idx, block_id));
}
__half* BlockPool::v_ptr(int fa_layer_idx, int block_id) const
{
    return reinterpret_cast<__half*>(static_cast<char*>(pool_) + v_offset(fa_layer_idx, block_id));
}
size_t BlockPool::k_offset(int fa_layer_idx, int block_id) const
{
    return (size_t)fa_layer_idx * layer_stride_ + (size_t)block_id * block_stride_;
}
size_t BlockPool::v_offset(int fa_layer_idx, int block_id) const
{
    return k_offset(fa_layer_idx, block_id) + kv_plane_;
}

std::vector<int> BlockPool::free_stack_snapshot() const
{
    std::lock_guard<std::mutex> lock(mu_);
    return free_stack_;
}

void BlockPool::destroy()
{
    if (pool_) {
        drk_dev_free(pool_);
        pool_ = nullptr;
    }
    free_stack_.clear();
    refcount_.clear();
    max_blocks_ = 0;
    total_bytes_ = 0;
}

} // namespace deusridet
