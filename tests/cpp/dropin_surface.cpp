// dropin_surface.cpp -- compile-and-link check of the C++ host surface.
//
// Every method and free function a caller of DeusRidet's Memoria / Machina KV path uses is
// called here with the argument lists, default arguments and return types that caller code
// is written against (the reference's src/memoria/block_pool.h:58-123,
// cache_manager.h:52-169, importance_scorer.h:25-67, kv_swapper.h:34-114,
// cache_kernels.h:44-74, src/machina/paged_attention.h:27-106; the call sites are
// src/conscientia/stream.cpp:151-156, 187-204, 297-334 and
// src/actus/awaken_consciousness.cpp:82-100).  Nothing is declared here: the file
// includes this library's headers only, so it compiles exactly when they offer that
// surface, and links exactly when libdeusridet_memoria.so exports it.  It is never run:
// the test that builds it has no GPU.
#include "conscientia/kv_stream.h"
#include "machina/layer.h"
#include "machina/paged_attention.h"
#include "memoria/block_pool.h"
#include "memoria/cache_kernels.h"
#include "memoria/cache_manager.h"
#include "memoria/importance_scorer.h"
#include "memoria/kv_swapper.h"

#include <string>
#include <type_traits>

using namespace deusridet;

static_assert(!std::is_copy_constructible<BlockPool>::value && !std::is_copy_assignable<BlockPool>::value,
              "BlockPool is non-copyable");
static_assert(!std::is_copy_constructible<CacheManager>::value, "CacheManager is non-copyable");
static_assert(std::is_same<std::underlying_type<BlockLocation>::type, int8_t>::value, "BlockLocation : int8_t");
static_assert((int)BlockLocation::GPU == 0 && (int)BlockLocation::SSD == -2 && (int)BlockLocation::INVALID == -1,
              "BlockLocation values");
static_assert(PagedKVConfig::BLOCK_SIZE == 256, "default tokens per block");

// block_pool.h:58-123
bool surface_block_pool(BlockPool& pool, size_t budget)
{
    bool ok = pool.init(budget);                       // block_size defaults to 256
    ok = pool.init(budget, 16) && ok;
    int id = pool.alloc_block();
    pool.free_block(id);
    int n = pool.free_count() + pool.max_blocks() + pool.block_size();
    __half* base = pool.pool_ptr();
    __half* k = pool.k_ptr(0, id);
    __half* v = pool.v_ptr(0, id);
    size_t off = pool.k_offset(0, id) + pool.v_offset(0, id) + pool.total_bytes() + PagedKVConfig::block_total_bytes();
    pool.destroy();
    return ok && n >= 0 && base && k && v && off > 0;
}

// importance_scorer.h:25-67
float surface_scorer(ImportanceScorer& sc, const float* d_new, const int* resident, int n)
{
    bool ok = sc.init(1024);                           // decay defaults to 0.95
    ok = sc.init(1024, 0.9f) && ok;
    sc.update(d_new, n);
    int least = sc.least_important(resident, n);
    sc.sync_to_host();
    float s = sc.score(least);
    sc.destroy();
    return ok ? s : 0.0f;
}

// kv_swapper.h:34-114
int surface_swapper(KVSwapper& sw, BlockPool& pool)
{
    bool ok = sw.init(pool, "/tmp/deusridet_cache");   // staging_blocks defaults to 2
    SwapRequest req;
    req.direction = SwapDirection::GPU_TO_SSD;
    req.logical_block_idx = 3;
    req.physical_block_id = 1;
    req.ssd_path = "/tmp/deusridet_cache/block_3.kv";
    req.callback = [](bool) {};
    sw.submit(req);
    sw.drain();
    sw.prefetch(3, req.ssd_path);
    bool have = sw.is_prefetched(3);
    sw.drop_prefetch(3);
    int left = sw.pending();
    sw.shutdown();
    return ok && have ? left : -1;
}

// cache_manager.h:52-169; awaken_consciousness.cpp:82-100; stream.cpp:151-156, 297-305, 371-372
int surface_cache_manager(CacheManager& cache, KVSwapper* swapper, ImportanceScorer* scorer, hipStream_t stream)
{
    size_t kv_budget = (size_t)14 << 30;
    bool ok = cache.init(kv_budget, "/tmp/deusridet_cache");           // block_size, swapper, scorer defaulted
    ok = cache.init(kv_budget) && ok;
    ok = cache.init(kv_budget, std::string("/tmp/deusridet_cache"), 256, swapper, scorer) && ok;
    int current_pos = cache.seq_len();
    ok = cache.ensure_blocks_for_range(current_pos, 2048) && ok;
    cache.sync_block_table(stream);
    ok = cache.ensure_blocks_for(current_pos) && ok;
    cache.sync_block_table();                                           // stream defaults to 0
    const int* blk_tbl = cache.d_block_table();
    cache.set_seq_len(current_pos + 1);
    int n = cache.num_logical_blocks() + cache.evict_blocks(4);
    ok = cache.ensure_free_blocks(8) && ok;
    cache.prefetch_block(0);
    BlockPool& pool = cache.block_pool();
    n += pool.max_blocks() + pool.block_size();
    n += cache.gpu_blocks_used() + cache.ssd_blocks_used() + cache.free_blocks();
    cache.destroy();
    return ok && blk_tbl ? n : -1;
}

// cache_kernels.h:44-74
void surface_cache_kernels(__half* flat, __half* kv_pool, const int* block_table, hipStream_t stream)
{
    invoke_extract_kv_from_pages(flat, kv_pool, block_table, 0, 512, 16, 4, 256, 256, 1024, stream);
    invoke_inject_kv_to_pages(kv_pool, flat, block_table, 0, 512, 16, 4, 256, 256, 1024, stream);
}

// paged_attention.h:27-106 as stream.cpp:187-204, 319-334 and paged_attention.cu:355-366, 617-630 call them
void surface_paged_attention(const __half* x, const FullAttentionWeights& attn, InferenceState& state, CacheManager& cache,
                             const __half* k_buf, const __half* v_buf, const __half* q_ptr)
{
    hipStream_t stream = state.compute_stream;
    const int max_phys = cache.block_pool().max_blocks();
    const int blk_size = cache.block_pool().block_size();
    __half* kv_pool = cache.block_pool().pool_ptr();
    const int* blk_tbl = cache.d_block_table();
    int fa_layer_idx = 0, current_pos = 100, seq_len = current_pos + 1, pos_start = 0, chunk = 2048;
    float scale = 0.0625f;

    paged_kv_cache_write(k_buf, v_buf, kv_pool, blk_tbl, fa_layer_idx, state.d_pos, max_phys, blk_size, stream);
    paged_kv_cache_write(k_buf, v_buf, kv_pool, blk_tbl, fa_layer_idx, state.d_pos, max_phys, blk_size);   // stream = 0
    paged_kv_cache_write_batch(k_buf, v_buf, kv_pool, blk_tbl, fa_layer_idx, pos_start, chunk, max_phys, blk_size, stream);
    paged_kv_cache_write_batch(k_buf, v_buf, kv_pool, blk_tbl, fa_layer_idx, pos_start, chunk, max_phys, blk_size);
    paged_gqa_decode_attention(q_ptr, kv_pool, blk_tbl, state.attn_out, fa_layer_idx, seq_len, max_phys, blk_size, scale, stream);
    paged_gqa_decode_attention(q_ptr, kv_pool, blk_tbl, state.attn_out, fa_layer_idx, seq_len, max_phys, blk_size, scale);

    full_attention_forward_paged(x, attn, kv_pool, blk_tbl, fa_layer_idx, current_pos, seq_len, max_phys, blk_size, state, stream);
    full_attention_forward_paged(x, attn, kv_pool, blk_tbl, fa_layer_idx, current_pos, seq_len, max_phys, blk_size, state);
    full_attention_forward_paged_prefill(x, attn, kv_pool, blk_tbl, fa_layer_idx, pos_start, chunk, pos_start + chunk, max_phys,
                                         blk_size, state, stream);
    full_attention_forward_paged_prefill(x, attn, kv_pool, blk_tbl, fa_layer_idx, pos_start, chunk, pos_start + chunk, max_phys,
                                         blk_size, state);
}

// layer.h:77-79, 124-140 as paged_attention.cu:348-370 calls them
void surface_layer_steps(__half* q_ptr, __half* k_buf, const FullAttentionWeights& attn, InferenceState& state,
                         const __half* gate_ptr, hipStream_t stream)
{
    using MC = ModelConfig;
    head_norm(q_ptr, attn.q_norm, q_ptr, MC::NUM_ATTN_HEADS, MC::HEAD_DIM, MC::RMS_EPS, stream);
    head_norm(k_buf, attn.k_norm, k_buf, MC::NUM_KV_HEADS, MC::HEAD_DIM, MC::RMS_EPS, stream);
    apply_rope(q_ptr, k_buf, MC::NUM_ATTN_HEADS, MC::NUM_KV_HEADS, MC::HEAD_DIM, MC::ROTARY_DIM, state.d_pos, MC::ROPE_THETA, stream);
    sigmoid_gate(state.attn_out, gate_ptr, state.attn_out, MC::NUM_ATTN_HEADS * MC::HEAD_DIM, stream);
    int groups = MC::NUM_KV_GROUPS + MC::NUM_FA_LAYERS;
    (void)groups;
}

int main() { return 0; }
