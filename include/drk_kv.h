/*
 * drk_kv.h -- C ABI of the MI355X (gfx950) paged-KV hot path.
 *
 * This is the only layer that touches HIP.  The C++ host interface that mirrors
 * DeusRidet's Memoria/Machina classes (deusridet_amd/memoria/, machina/) is
 * written against these entry points and nothing else; any other language binds
 * the same symbols (cgo, JNI, ctypes ...).
 *
 * Conventions
 *   - every call returns DRK_OK (0) or a negative DRK_ERR_* code; the text of the
 *     last error on the calling thread is at drk_last_error();
 *   - pointers named d_* / pool / q / out / src_* / workspace are DEVICE pointers;
 *     h_* are host pointers;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     every launch is asynchronous on it, nothing here synchronises unless it
 *     says so, and no kernel entry point allocates or frees memory;
 *   - geometry travels in a drk_kv_layout (the reference spreads it over
 *     PagedKVConfig constexprs, block_pool.h:34-52, and ModelConfig statics,
 *     model.h:39-42, 73);
 *   - citations are file:line in the DeusRidet tree.
 */
#ifndef DRK_KV_H
#define DRK_KV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DRK_OK               0
#define DRK_ERR_INVALID     -1   /* bad argument / shape the kernels do not take */
#define DRK_ERR_HIP         -2   /* a HIP runtime call failed                     */
#define DRK_ERR_UNSUPPORTED -3   /* geometry outside the compiled set             */
#define DRK_ERR_WORKSPACE   -4   /* workspace missing or too small                */

/* storage type of the pool / element type of Q, out and append sources */
enum { DRK_F16 = 0, DRK_BF16 = 1, DRK_INT8 = 2, DRK_FP8_E4M3 = 3 };

/*
 * Pool layout (bytes), the contract shared by every kernel and by the host
 * classes (block_pool.cpp:23-39, 81-95; paged_attention.cu:36-64;
 * cache_kernels.cu:71-84):
 *   E            = 2 (F16, BF16) or 1 (INT8, FP8_E4M3)
 *   kv_plane     = num_kv_heads * block_size * head_dim * E
 *   scale_plane  = INT8 ? num_kv_heads * block_size * 2 : 0      (fp16 scales)
 *   block_stride = 2*kv_plane + 2*scale_plane
 *   layer_stride = max_phys_blocks * block_stride
 *   K(l,b,h,p,d) = l*layer_stride + b*block_stride + ((h*block_size+p)*head_dim+d)*E
 *   V(l,b,h,p,d) = K(l,b,h,p,d) + kv_plane
 *   Kscale(l,b,h,p) = l*layer_stride + b*block_stride + 2*kv_plane + (h*block_size+p)*2
 *   Vscale(l,b,h,p) = Kscale(l,b,h,p) + scale_plane
 */
typedef struct drk_kv_layout {
    int32_t num_layers;       /* ModelConfig::NUM_FA_LAYERS  (model.h:73)        */
    int32_t num_kv_heads;     /* ModelConfig::NUM_KV_HEADS   (model.h:40)        */
    int32_t num_q_heads;      /* ModelConfig::NUM_ATTN_HEADS (model.h:39)        */
    int32_t head_dim;         /* ModelConfig::HEAD_DIM       (model.h:41)        */
    int32_t block_size;       /* tokens per block (block_pool.h:35, runtime)     */
    int32_t max_phys_blocks;  /* BlockPool::max_blocks()     (block_pool.h:80)   */
    int32_t dtype;            /* DRK_*: storage type of the pool                 */
    int32_t reserved;         /* must be 0                                       */
} drk_kv_layout;

/* ---- library ---------------------------------------------------------- */
int         drk_abi_version(void);
const char *drk_last_error(void);
const char *drk_strerror(int code);
int         drk_device_count(int *count);

/* ---- layout arithmetic (host only, no GPU needed) --------------------- */
/* block_pool.cpp:23-39: strides; block_pool.cpp:28-32: budget -> max_blocks */
int drk_kv_layout_check(const drk_kv_layout *g);
size_t drk_kv_elem_bytes(const drk_kv_layout *g);
size_t drk_kv_plane_bytes(const drk_kv_layout *g);
size_t drk_kv_block_stride_bytes(const drk_kv_layout *g);
size_t drk_kv_layer_stride_bytes(const drk_kv_layout *g);
size_t drk_kv_pool_bytes(const drk_kv_layout *g);
/* BlockPool::k_offset / v_offset, block_pool.cpp:89-95 */
size_t drk_kv_k_offset(const drk_kv_layout *g, int layer, int block);
size_t drk_kv_v_offset(const drk_kv_layout *g, int layer, int block);
int    drk_kv_max_blocks_for_budget(const drk_kv_layout *g, size_t budget_bytes);

/* ---- device memory plumbing for the host classes ---------------------- */
/* cudaMalloc/cudaMemset/cudaFree in BlockPool::init/destroy
 * (block_pool.cpp:42-49, 97-101) and CacheManager::init (cache_manager.cpp:46-53);
 * cudaMemcpyAsync in CacheManager::sync_block_table (cache_manager.cpp:108-112). */
int drk_dev_malloc(void **d_ptr, size_t bytes);
int drk_dev_free(void *d_ptr);
int drk_dev_memset_async(void *d_ptr, int byte, size_t bytes, void *stream);
int drk_memcpy_h2d_async(void *d_dst, const void *h_src, size_t bytes, void *stream);
int drk_memcpy_d2d_async(void *d_dst, const void *d_src, size_t bytes, void *stream);
int drk_memcpy_d2h(void *h_dst, const void *d_src, size_t bytes, void *stream); /* syncs */
/* d_pos[i] += delta and d_seq_lens[i] += delta for i < n (either may be NULL), in the stream:
 * lets a captured decode step move its own positions on. */
int drk_positions_advance(int32_t *d_pos, int32_t *d_seq_lens, int n, int delta, void *stream);
/* Capture what is enqueued on `stream` between begin and end into an executable graph
 * (thread-local capture mode; a stream of its own, not the NULL stream), launch it, destroy it.  None of the append / attention entry
 * points allocates, memsets or synchronises, so a whole decode step can be captured. */
int drk_graph_begin_capture(void *stream);
int drk_graph_end_capture(void *stream, void **graph_exec);
int drk_graph_launch(void *graph_exec, void *stream);
int drk_graph_destroy(void *graph_exec);
/* Waits for all work on every stream of the current device. */
int drk_device_synchronize(void);
/* Pinned host memory (allocated pinned, for staging buffers). */
int drk_host_malloc(void **h_ptr, size_t bytes);
int drk_host_free(void *h_ptr);
/* One physical block, all layers, to / from a contiguous host image of
 * drk_kv_block_total_bytes(): [layer][K plane | V plane (| K scales | V scales)], the
 * order KVSwapper writes its .kv files in (kv_swapper.cpp:183-198, 268-283).
 * Asynchronous on `stream`; the host side should be pinned. */
size_t drk_kv_block_total_bytes(const drk_kv_layout *g);
int drk_kv_block_to_host(const drk_kv_layout *g, const void *pool, int blk, void *h_dst, void *stream);
int drk_kv_block_from_host(const drk_kv_layout *g, void *pool, int blk, const void *h_src, void *stream);
int drk_stream_create(void **stream);
int drk_stream_destroy(void *stream);
int drk_stream_synchronize(void *stream);
/* *capturing = 1 while `stream` records into a graph (hipStreamIsCapturing); NULL stream: 0. */
int drk_stream_is_capturing(void *stream, int *capturing);
/* Events without timing: drk_event_record marks what `stream` has been given so far,
 * drk_stream_wait_event makes another stream wait for exactly that (cudaEventRecord /
 * cudaStreamWaitEvent in the reference's vocabulary, model.h:292-293), drk_event_synchronize
 * blocks the host until it has happened. */
int drk_event_create(void **event);
int drk_event_destroy(void *event);
int drk_event_record(void *event, void *stream);
int drk_event_synchronize(void *event);
int drk_stream_wait_event(void *stream, void *event);

/* ---- append into pages ------------------------------------------------ */
/* paged_kv_cache_write, paged_attention.cu:73-115: one token at *d_pos.
 * src_k/src_v [num_kv_heads, head_dim] of src_dtype (F16/BF16); an INT8/FP8 pool
 * quantises on the way in (round-half-even). */
int drk_kv_append_token(const drk_kv_layout *g, void *pool, const int32_t *d_block_table,
                        int layer, const int32_t *d_pos, const void *src_k,
                        const void *src_v, int src_dtype, void *stream);
/* paged_kv_cache_write_batch, paged_attention.cu:123-167: M consecutive tokens
 * from src [M, num_kv_heads, head_dim].  layer_count > 1 appends the same
 * positions for layers layer..layer+layer_count-1 in one launch from
 * src [layer_count, M, num_kv_heads, head_dim]. */
int drk_kv_append_batch(const drk_kv_layout *g, void *pool, const int32_t *d_block_table,
                        int layer, int layer_count, int pos_start, int M,
                        const void *src_k, const void *src_v, int src_dtype, void *stream);
/* One token for each of B branches in one launch (no reference counterpart; the
 * reference has one sequence).  d_tables [B, table_stride], d_pos [B],
 * src [layer_count, B, num_kv_heads, head_dim]. */
int drk_kv_append_branches(const drk_kv_layout *g, void *pool, const int32_t *d_tables,
                           int table_stride, const int32_t *d_pos, int B, int layer,
                           int layer_count, const void *src_k, const void *src_v,
                           int src_dtype, void *stream);

/* ---- gather / scatter ------------------------------------------------- */
/* invoke_extract_kv_from_pages, cache_kernels.cu:30-87, 147-166:
 * dst [num_layers][2][num_tokens][num_kv_heads][head_dim] in the pool's storage
 * type; INT8 pools also fill d_dst_scales [num_layers][2][num_tokens][num_kv_heads]
 * fp16 when it is not NULL.  A hole (table entry < 0) is zero-filled. */
int drk_kv_extract(const drk_kv_layout *g, void *d_dst, void *d_dst_scales, const void *pool,
                   const int32_t *d_block_table, int start_token, int num_tokens,
                   int num_layers, void *stream);
/* invoke_inject_kv_to_pages, cache_kernels.cu:93-141, 168-187; a hole is skipped. */
int drk_kv_inject(const drk_kv_layout *g, void *pool, const void *d_src, const void *d_src_scales,
                  const int32_t *d_block_table, int start_token, int num_tokens,
                  int num_layers, void *stream);
/* Copy-on-write: copy every layer of physical block src to dst for n pairs
 * (no reference counterpart; intent docs/en/architecture/02-memoria.md:25-26).
 * d_pairs [n][2] = (src, dst). */
int drk_kv_copy_blocks(const drk_kv_layout *g, void *pool, const int32_t *d_pairs, int n,
                       void *stream);

/* ---- paged GQA decode attention --------------------------------------- */
/* Kernels: head_dim 128 or 256 with 1..16 query heads per kv head and block_size % 16 == 0 run
 * on the persistent tiled kernel (every storage type; the reference's own 24 Q / 4 KV x 256,
 * block 256 included; 64 branches per launch, more branches take several launches); any other geometry (head_dim a
 * multiple of 64 up to 512, group size <= 16) on a portable one.
 * Bytes of workspace the split-K decode needs for B branches of at most max_seq_len tokens: */
size_t drk_decode_workspace_bytes(const drk_kv_layout *g, int B, int max_seq_len);
/* Same for an explicit split_tokens: B*num_q_heads*ceil(max_seq_len/split)*(head_dim+2)*4. */
size_t drk_decode_workspace_bytes_for_split(const drk_kv_layout *g, int B, int max_seq_len,
                                            int split_tokens);
/* The split (tokens per workgroup, a multiple of 64) the library picks when
 * split_tokens == 0. */
int drk_decode_default_split(const drk_kv_layout *g, int B, int max_seq_len);
/* paged_gqa_decode_attention, paged_attention.cu:179-282: one sequence.
 * q/out [num_q_heads, head_dim] of io_dtype (F16/BF16). */
int drk_paged_decode_attention(const drk_kv_layout *g, const void *q, const void *pool,
                               const int32_t *d_block_table, void *out, int layer,
                               int seq_len, float scale, int io_dtype, void *workspace,
                               size_t workspace_bytes, void *stream);
/* B branches in one launch: d_tables [B, table_stride], d_seq_lens [B] (device),
 * q/out [B, num_q_heads, head_dim]; max_seq_len >= every d_seq_lens[b] sizes the
 * grid.  split_tokens = 0 lets the library choose; otherwise a multiple of 64, at most 16 384 on the tiled
 * kernel (larger values are refused with DRK_ERR_INVALID). */
int drk_paged_decode_attention_branches(const drk_kv_layout *g, const void *q, const void *pool,
                                        const int32_t *d_tables, int table_stride,
                                        const int32_t *d_seq_lens, int B, int max_seq_len,
                                        void *out, int layer, float scale, int io_dtype,
                                        int split_tokens, void *workspace,
                                        size_t workspace_bytes, void *stream);

/* The same call for callers that cannot allocate or carry a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference.  The split-K partials live in a file-scope device array of
 * DRK_STATIC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends;
 * the call allocates and frees nothing, picks the split itself, and fails with
 * DRK_ERR_WORKSPACE when drk_decode_workspace_bytes(g, B, max_seq_len) exceeds that size
 * (config 2's 8 x 32k needs 8.8 MB; 16 branches x 32 query heads x 128 at 32k, 17.6 MB).
 * Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams,
 * two threads) race on the partials -- serialise them, or use the call above with a
 * workspace per stream.  Nothing in the array needs clearing between calls.  The first call
 * on each device looks the array's address up (hipGetSymbolAddress): make it outside a
 * stream capture. */
#define DRK_STATIC_SCRATCH_BYTES (32u << 20)
int drk_paged_decode_attention_branches_static(const drk_kv_layout *g, const void *q, const void *pool,
                                               const int32_t *d_tables, int table_stride,
                                               const int32_t *d_seq_lens, int B, int max_seq_len,
                                               void *out, int layer, float scale, int io_dtype,
                                               void *stream);

/* Branches that share a prefix (no reference counterpart; intent
 * docs/en/architecture/03-cogitatio.md:3-5, 18-22: decode branches over one
 * persistent Conscientia prefix).  The caller promises that the pages holding
 * tokens [0, shared_tokens) are the same physical blocks in all B table rows and
 * that every d_seq_lens[b] >= shared_tokens (CacheManager::common_prefix_tokens
 * computes it).  Those pages are then streamed from HBM once for all B branches
 * instead of once per branch.  shared_tokens is rounded down to a multiple of 64;
 * 0, or a geometry the tiled decode kernel does not take, gives exactly
 * drk_paged_decode_attention_branches (every storage type has the shared pass).  Results equal the per-branch call up to
 * summation order.  drk_decode_shared_workspace_bytes(g, B, max_seq_len, s) is enough for every call with these B and
 * max_seq_len and any shared_tokens up to s. */
size_t drk_decode_shared_workspace_bytes(const drk_kv_layout *g, int B, int max_seq_len, int shared_tokens);
int drk_paged_decode_attention_shared(const drk_kv_layout *g, const void *q, const void *pool,
                                      const int32_t *d_tables, int table_stride,
                                      const int32_t *d_seq_lens, int B, int max_seq_len,
                                      int shared_tokens, void *out, int layer, float scale,
                                      int io_dtype, void *workspace, size_t workspace_bytes,
                                      void *stream);

/* Branches that share pages as a tree (no reference counterpart; intent
 * docs/en/architecture/03-cogitatio.md:8-22: the Action / Speech / Thinking / Daydream branches fork from one
 * context and from one another; src/conscientia/scheduler.h:53-56).  A group says: branches
 * [first_branch, first_branch + n_branches) hold tokens [tok_begin, tok_end) in the same physical blocks, and every
 * one of them is at least tok_end tokens long (CacheManager::common_prefix_groups computes the groups from the
 * tables).  For every branch the groups it belongs to must follow one another from token 0 without gap or overlap
 * -- a fork tree: the whole set over the persistent prefix, subsets over what they wrote before they split again --
 * and a group takes at most 64 / (num_q_heads / num_kv_heads) branches.  Group boundaries are rounded down to
 * multiples of 64 tokens; what a group loses at its end is read by the group or the private tail behind it.  All
 * shared and private pages are streamed once, in ONE launch whose workgroups take equal shares of the bytes, and
 * one merge.  head_dim 128, block_size % 16 == 0, at most 64 branches, at most 16 query heads per kv head, every
 * storage type; DRK_ERR_UNSUPPORTED otherwise (use drk_paged_decode_attention_shared / _branches).  gate may be
 * NULL; otherwise as in drk_paged_decode_attention_gated.  Results equal the per-branch call up to summation order.
 * Workspace: drk_decode_grouped_workspace_bytes for these very groups, or _max for any tree nested at most
 * max_depth groups deep (what a caller reserves once). */
#define DRK_MAX_PREFIX_GROUPS 16
typedef struct drk_prefix_group {
    int32_t first_branch, n_branches;
    int32_t tok_begin, tok_end;
} drk_prefix_group;
size_t drk_decode_grouped_workspace_bytes(const drk_kv_layout *g, int B, int max_seq_len,
                                          const drk_prefix_group *groups, int n_groups);
size_t drk_decode_grouped_workspace_bytes_max(const drk_kv_layout *g, int B, int max_seq_len, int max_depth);
int drk_paged_decode_attention_grouped(const drk_kv_layout *g, const void *q, const void *pool,
                                       const int32_t *d_tables, int table_stride,
                                       const int32_t *d_seq_lens, int B, int max_seq_len,
                                       const drk_prefix_group *groups, int n_groups, void *out,
                                       int layer, float scale, int io_dtype, const void *gate,
                                       size_t gate_stride, void *workspace, size_t workspace_bytes,
                                       void *stream);

/* The layers of one decode step read the same tables and lengths: the tiled decode kernels' per-workgroup
 * unit descriptors (which 64-token tile of which branch and kv head, where its pages lie) can be built once
 * per step instead of once per layer (no reference counterpart; the reference's kernel takes one workgroup per
 * (head, branch) and needs none).  drk_decode_plan_build writes them to d_plan -- a launch of its own that reads
 * d_tables and d_seq_lens only -- and drk_paged_decode_attention_planned is drk_paged_decode_attention_grouped
 * (n_groups = 0: drk_paged_decode_attention_gated, gate may be NULL) reading them.  The caller promises that the
 * plan was built with the same g (any layer), d_tables contents, d_seq_lens contents, B, max_seq_len and groups,
 * and with the debug switches of drk_debug.h unchanged; the results are then bit for bit those of the unplanned
 * call.  At most 64 branches, head_dim 128 or 256 with block_size % 16 == 0 (drk_decode_plan_bytes returns 0
 * otherwise and both calls DRK_ERR_UNSUPPORTED).  drk_decode_plan_bytes: up to 12.6 MB; 16-byte aligned. */
size_t drk_decode_plan_bytes(const drk_kv_layout *g, int B, int max_seq_len, int n_groups);
int drk_decode_plan_build(const drk_kv_layout *g, const int32_t *d_tables, int table_stride,
                          const int32_t *d_seq_lens, int B, int max_seq_len,
                          const drk_prefix_group *groups, int n_groups, void *d_plan, size_t plan_bytes,
                          void *stream);
int drk_paged_decode_attention_planned(const drk_kv_layout *g, const void *q, const void *pool,
                                       const int32_t *d_tables, int table_stride,
                                       const int32_t *d_seq_lens, int B, int max_seq_len,
                                       const drk_prefix_group *groups, int n_groups, const void *d_plan,
                                       void *out, int layer, float scale, int io_dtype, const void *gate,
                                       size_t gate_stride, void *workspace, size_t workspace_bytes,
                                       void *stream);
/* One layer of a decode step in one call: drk_kv_append_branches of one token per branch at position
 * d_seq_lens[b] - 1 (write then attend: the lengths already count the new token; new_k / new_v are
 * [B, num_kv_heads, head_dim] of src_dtype), then drk_paged_decode_attention_planned.  With 16-bit pages, src_dtype
 * equal to the pool's type and 16-byte aligned sources it is ONE launch, with or without groups: the workgroup that
 * owns a branch's last tile writes the new rows before it reads the tile, which takes the append's launch out of
 * every layer; otherwise the append is launched by itself first.  Same bytes in the pool and same output bits as
 * the two calls (tested).  As for any append, the page that receives a branch's new token must be mapped by that
 * branch alone (copy-on-write done: CacheManager::ensure_blocks_for sees to it) -- here also because no other
 * workgroup may be reading it.  The plan must have been built from these lengths. */
int drk_kv_append_decode_planned(const drk_kv_layout *g, void *pool, const int32_t *d_tables,
                                 int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len,
                                 const drk_prefix_group *groups, int n_groups, const void *d_plan,
                                 const void *new_k, const void *new_v, int src_dtype, const void *q, void *out,
                                 int layer, float scale, int io_dtype, const void *gate, size_t gate_stride,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* ---- paged causal prefill attention ------------------------------------ */
/* paged_prefill_attention_kernel, paged_attention.cu:465-554, 621-630:
 * q/out [M, num_q_heads, head_dim]; row t attends to tokens 0..pos_start+t (the
 * chunk's own K/V must already be in the pages: write, then attend).
 * head_dim 128 or 256 with block_size % 16 == 0 (any storage type, any number of query
 * heads per KV head up to 128) runs on the MFMA prefill kernel, which needs no workspace.
 * A chunk of up to 512 rows behind 2 048 tokens or more (1 024 behind 4 096) is spread over
 * the whole chip instead -- the same kernel with the context split as in
 * drk_paged_decode_attention_shared, rows = the chunk's tokens, then a merge -- when the
 * workspace drk_prefill_workspace_bytes reports for it is passed (16-byte aligned, up to
 * ~35 MB at 32 query heads x 128); without it the unsplit kernel does the work, up to 30
 * times slower for a chunk of a few tokens behind a long context.  Head_dim 256 on 16-bit pages
 * (blocks of 16 * 2^k tokens) does not take that path: its chunk kernel cuts the walks of a round
 * that does not fill the chip into up to 32 pieces each and merges them, with the same workspace
 * call (up to 33.8 MB).  Anything else runs row by row through the portable decode kernel, which
 * needs the workspace. */
size_t drk_prefill_workspace_bytes(const drk_kv_layout *g, int pos_start, int M);
/* The most drk_prefill_workspace_bytes reports for any chunk of up to max_rows rows that
 * ends at or before max_seq_len tokens: what a caller reserves once, up front.  (Both sizes follow the
 * debug switches of drk_debug.h as they stand at the time of the call: reserve after setting them.)
 * scale must be positive: DRK_ERR_INVALID otherwise. */
size_t drk_prefill_workspace_bytes_max(const drk_kv_layout *g, int max_seq_len, int max_rows);
int drk_paged_prefill_attention(const drk_kv_layout *g, const void *q, const void *pool,
                                const int32_t *d_block_table, void *out, int layer,
                                int pos_start, int M, float scale, int io_dtype,
                                void *workspace, size_t workspace_bytes, void *stream);

/* ---- the layer steps either side of the page kernels --------------------- */
/* full_attention_forward_paged / _paged_prefill, paged_attention.cu:314-376, 563-638:
 * split of the interleaved Q|gate projection, per-head RMSNorm, partial half-half
 * RoPE, [page write, attention], sigmoid gate.  All tensors hold 16-bit elements of
 * type dtype (DRK_F16 / DRK_BF16); head_dim is a power of two in [8, 512];
 * rotary_dim = 16 * 2^k <= head_dim.  Rows are heads of head_dim elements.
 *
 * A rope table is float [table_positions][rotary_dim/2][2] = (cos, sin) of
 * pos * theta^(-2 pair / rotary_dim), formed in fp32 as rope_kernel does
 * (layer_attention.cu:42-48).  Entry points that take one use it for positions inside
 * it and evaluate the same expressions in the kernel for any other (or when it is NULL). */
int drk_rope_table_fill(float *d_table, int n_pos, int rotary_dim, float theta, void *stream);
/* head_norm, layer_attention.cu:86-135: out = (x * rsqrt(mean(x^2) + eps)) * weight per row */
int drk_head_norm(const void *x, const void *weight, void *out, int num_rows, int head_dim,
                  float eps, int dtype, void *stream);
/* apply_rope, layer_attention.cu:32-79 (T = 1, position *d_pos) and
 * paged_rope_batch_kernel, paged_attention.cu:412-451 (T tokens at pos_start + t): in place
 * on q [T, num_q_heads, head_dim] and k [T, num_kv_heads, head_dim].  d_pos != NULL: one
 * position per token (decode branches), read on the device. */
int drk_apply_rope(void *q, void *k, int T, int num_q_heads, int num_kv_heads, int head_dim,
                   int rotary_dim, const int32_t *d_pos, int pos_start, float theta,
                   const float *d_rope_table, int table_positions, int dtype, void *stream);
/* paged_split_q_gate[_batch_kernel], paged_attention.cu:288-298, 386-404:
 * qg [T, num_heads, 2 * head_dim] -> q, gate [T, num_heads, head_dim] */
int drk_split_q_gate(const void *qg, void *q, void *gate, int T, int num_heads, int head_dim,
                     void *stream);
/* sigmoid_gate, layer.cu:406-439: out = x * sigmoid(gate); x, out [num_rows, head_dim]
 * (may alias), gate rows gate_stride elements apart (head_dim when gate is its own tensor,
 * 2 * head_dim when it still sits in the Q|gate projection: pass qg + head_dim) */
int drk_sigmoid_gate(const void *x, const void *gate, void *out, size_t num_rows, int head_dim,
                     size_t gate_stride, int dtype, void *stream);
/* Steps 1b-5 of full_attention_forward_paged (paged_attention.cu:331-360; batch form
 * 589-619) in ONE launch, no reference counterpart as a single function: reads the raw
 * projections qg [T, QH, 2*D], k, v [T, KVH, D] and the norm weights [D]; writes
 * q_out [T, QH, D] = rope(norm(q)); appends rope(norm(k)) and v into the pages of layer
 * `layer` (quantising for int8 / fp8 pools exactly as drk_kv_append_* does).  The gate
 * halves of qg are left where they are (see drk_sigmoid_gate / the _gated attention
 * calls).  d_pos != NULL: token t is the new token of branch t at d_pos[t] with table row
 * t (as drk_kv_append_branches); NULL: positions pos_start + t of one table (as
 * drk_kv_append_batch).  Equals split + head_norm x2 + apply_rope + append bit for bit. */
int drk_qk_norm_rope_append(const drk_kv_layout *g, void *pool, const int32_t *d_tables,
                            int table_stride, const int32_t *d_pos, int pos_start, int T, int layer,
                            const void *qg, const void *k, const void *v, const void *q_norm_w,
                            const void *k_norm_w, float eps, int rotary_dim, float theta,
                            const float *d_rope_table, int table_positions, void *q_out,
                            int src_dtype, void *stream);
/* Attention with the sigmoid gate folded into the epilogue (steps 6+7 / 8+9 of the
 * wrappers above): out = f16(f16(attention) * sigmoid(gate)), the same two roundings the
 * separate kernels make.  gate rows [B or M][num_q_heads] are gate_stride elements apart
 * and 16-byte aligned.  As in the reference, a row no token took part in is gated too
 * (out must then hold defined values). */
int drk_paged_decode_attention_gated(const drk_kv_layout *g, const void *q, const void *pool,
                                     const int32_t *d_tables, int table_stride,
                                     const int32_t *d_seq_lens, int B, int max_seq_len, void *out,
                                     int layer, float scale, int io_dtype, const void *gate,
                                     size_t gate_stride, void *workspace, size_t workspace_bytes,
                                     void *stream);
int drk_paged_prefill_attention_gated(const drk_kv_layout *g, const void *q, const void *pool,
                                      const int32_t *d_block_table, void *out, int layer,
                                      int pos_start, int M, float scale, int io_dtype,
                                      const void *gate, size_t gate_stride, void *workspace,
                                      size_t workspace_bytes, void *stream);

/* ---- importance scores -------------------------------------------------- */
/* Decode attention (as drk_paged_decode_attention_branches) that also reports the attention
 * mass every block received: d_block_mass[b * mass_stride + lb] = sum over the tokens of
 * logical block lb of branch b and over all query heads of the softmax probability (so a
 * branch's blocks sum to num_q_heads).  This is the per-block "new importance value from
 * attention" that ImportanceScorer::update consumes (importance_scorer.h:37-41; the
 * reference never computes it: its scorer is unwired).  accumulate != 0 adds to what
 * d_block_mass holds (sum over the layers of a step); 0 overwrites, and zeroes the entries
 * of blocks past a branch's length.  mass_stride >= ceil(max_seq_len / block_size); with
 * mass_stride = CacheManager::table_stride() the array is indexed like the block tables.
 * Geometry: head_dim 128 or 256, at most 16 query heads per kv head, block_size % 16 == 0,
 * B <= 64. */
size_t drk_decode_mass_workspace_bytes(const drk_kv_layout *g, int B, int max_seq_len);
int drk_paged_decode_attention_mass(const drk_kv_layout *g, const void *q, const void *pool,
                                    const int32_t *d_tables, int table_stride,
                                    const int32_t *d_seq_lens, int B, int max_seq_len, void *out,
                                    int layer, float scale, int io_dtype, float *d_block_mass,
                                    int mass_stride, int accumulate, void *workspace,
                                    size_t workspace_bytes, void *stream);
/* The same with the two things a layer step of the reference model does around it folded in (no reference
 * counterpart): d_plan, or NULL -- the step's unit descriptors from drk_decode_plan_build (built without groups),
 * read instead of rebuilt by every layer's launch; gate, or NULL -- out = attention * sigmoid(gate) applied in the
 * merge, as drk_paged_decode_attention_gated does (rows gate_stride elements apart).  Same output bits as
 * drk_paged_decode_attention_mass followed by drk_sigmoid_gate, same masses. */
int drk_paged_decode_attention_mass_gated(const drk_kv_layout *g, const void *q, const void *pool,
                                          const int32_t *d_tables, int table_stride,
                                          const int32_t *d_seq_lens, int B, int max_seq_len,
                                          const void *d_plan, void *out, int layer, float scale,
                                          int io_dtype, const void *gate, size_t gate_stride,
                                          float *d_block_mass, int mass_stride, int accumulate,
                                          void *workspace, size_t workspace_bytes, void *stream);
/* The attention mass a perception frame gives to every block of the context: for the chunk of M
 * query tokens at pos_start (rows and visibility as in drk_paged_prefill_attention),
 *   d_block_mass[lb] (+)= sum over the chunk's tokens, all query heads, and the tokens of logical
 *   block lb of the row's softmax probability
 * so the entries add up to M * num_q_heads.  "After each Prefill frame, record cumulative attention
 * weight received by each KV block" (docs/en/architecture/02-memoria.md:40-44); the reference's
 * scorer takes such an array (importance_scorer.h:37-41) and nothing in the reference fills it.
 * A separate pass after the frame's attention, as the reference schedules it: it reads Q and K
 * only (K twice), takes no workspace and writes no attention output.  accumulate != 0 adds to
 * d_block_mass (sum over layers); 0 clears its mass_len entries first.  mass_len >=
 * ceil((pos_start + M) / block_size).  The sums are made with float atomics: they differ in
 * the last bits from run to run.  Geometry: head_dim 128 or 256, block_size % 16 == 0. */
int drk_paged_prefill_attention_mass(const drk_kv_layout *g, const void *q, const void *pool,
                                     const int32_t *d_block_table, int layer, int pos_start, int M,
                                     float scale, int io_dtype, float *d_block_mass, int mass_len,
                                     int accumulate, void *stream);
/* The two halves of the same measurement without the second walk over the keys (no reference counterpart).
 * drk_paged_prefill_attention_lse is drk_paged_prefill_attention_gated (gate may be NULL here) that also writes
 * every row's log2-sum-exp of its scaled scores to d_row_lse[M * num_q_heads] (+inf for a row without a visible
 * token) -- the chunk kernels know it where a row's walk ends.  drk_paged_prefill_attention_mass_lse is the mass
 * pass given those values: it reads K once.  It may run on another stream behind an event (it reads q, the pages
 * and d_row_lse; nothing the attention call wrote except d_row_lse).  Head_dim 128 or 256, block_size % 16 == 0;
 * DRK_ERR_UNSUPPORTED otherwise.  Over 16-bit pages, and over 8-bit pages at head_dim 128 (blocks of 16 * 2^k tokens
 * either way), the pass scores the way the attention call did and a row's masses sum to 1 within 1e-6;
 * over 8-bit pages at head_dim 256, and with other block sizes, the two calls round Q differently for some chunk
 * lengths (the long-chunk kernels fold the scale into Q in its 16-bit type) and the sum is 1 within 2e-3.  d_row_lse must come from the attention call for the same
 * chunk with the library's debug switches unchanged in between. */
int drk_paged_prefill_attention_lse(const drk_kv_layout *g, const void *q, const void *pool,
                                    const int32_t *d_block_table, void *out, int layer, int pos_start, int M,
                                    float scale, int io_dtype, const void *gate, size_t gate_stride,
                                    float *d_row_lse, void *workspace, size_t workspace_bytes, void *stream);
int drk_paged_prefill_attention_mass_lse(const drk_kv_layout *g, const void *q, const void *pool,
                                         const int32_t *d_block_table, int layer, int pos_start, int M,
                                         float scale, int io_dtype, const float *d_row_lse, float *d_block_mass,
                                         int mass_len, int accumulate, void *stream);
/* importance_update_kernel, importance_scorer.cu:27-36, 67-73 */
int drk_importance_update(float *d_scores, const float *d_new_scores, int n, float decay,
                          void *stream);
/* The same fold over a range whose new scores are spent with it: d_new_scores[0..n) is zero afterwards (no
 * reference counterpart: the reference's scorer is never fed).  One launch, no memset node: may be captured. */
int drk_importance_fold_clear(float *d_scores, float *d_new_scores, int n, float decay, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DRK_KV_H */
