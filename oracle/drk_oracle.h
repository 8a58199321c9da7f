/*
 * drk_oracle.h -- CPU restatement of the DeusRidet Memoria/Machina paged-KV path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code; only tests, the smoke check and the benchmark's CPU-baseline
 * leg may use it, and there only as the checker or as the timed CPU baseline.
 *
 * Every function cites the reference file:line (relative to the DeusRidet tree)
 * whose behaviour it restates.  Parts that have no counterpart in the reference
 * (branches, refcounts, copy-on-write, int8/fp8 codecs, split-K) are marked
 * "builder-specified"; what pins them is stated in drk_oracle.c's header.
 */
#ifndef DRK_ORACLE_H
#define DRK_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element / storage types of the pool */
enum { ORC_F16 = 0, ORC_BF16 = 1, ORC_INT8 = 2, ORC_FP8 = 3 };

typedef struct orc_layout {
    int32_t L;     /* full-attention layers                */
    int32_t KVH;   /* KV heads                             */
    int32_t QH;    /* query heads                          */
    int32_t D;     /* head dim                             */
    int32_t bs;    /* tokens per block                     */
    int32_t NB;    /* physical blocks (max_phys_blocks)    */
    int32_t dtype; /* ORC_*                                */
} orc_layout;

/* ---- scalar conversions (pinned against numpy.float16 / torch casts) ---- */
float    orc_h2f(uint16_t h);
uint16_t orc_f2h(float f);            /* round-to-nearest-even              */
float    orc_bf2f(uint16_t b);
uint16_t orc_f2bf(float f);           /* round-to-nearest-even              */
uint8_t  orc_f2fp8(float f);          /* OCP E4M3FN, RNE, saturating        */
float    orc_fp82f(uint8_t c);

/* ---- pool addressing, in BYTES (block_pool.cpp:23-39, 81-95) ------------ */
size_t orc_elem_bytes(const orc_layout *g);
size_t orc_kv_plane_bytes(const orc_layout *g);
size_t orc_block_stride_bytes(const orc_layout *g);
size_t orc_layer_stride_bytes(const orc_layout *g);
size_t orc_pool_bytes(const orc_layout *g);
size_t orc_k_off(const orc_layout *g, int layer, int blk, int h, int p, int d);
size_t orc_v_off(const orc_layout *g, int layer, int blk, int h, int p, int d);
size_t orc_kscale_off(const orc_layout *g, int layer, int blk, int h, int p);
size_t orc_vscale_off(const orc_layout *g, int layer, int blk, int h, int p);
int    orc_max_blocks_for_budget(const orc_layout *g, size_t budget_bytes);

/* ---- append / gather (paged_attention.cu:73-167, cache_kernels.cu:30-141) */
/* src element type: ORC_F16 or ORC_BF16; when the pool is INT8/FP8 the rows are
 * quantised on the way in. */
void orc_append_token(const orc_layout *g, void *pool, const int32_t *table,
                      int layer, int pos, const uint16_t *src_k,
                      const uint16_t *src_v, int src_dtype);
void orc_append_batch(const orc_layout *g, void *pool, const int32_t *table,
                      int layer, int pos_start, int M, const uint16_t *src_k,
                      const uint16_t *src_v, int src_dtype);
void orc_extract(const orc_layout *g, void *dst, void *dst_scales,
                 const void *pool, const int32_t *table, int start_token,
                 int num_tokens, int num_layers);
void orc_inject(const orc_layout *g, void *pool, const void *src,
                const void *src_scales, const int32_t *table, int start_token,
                int num_tokens, int num_layers);
void orc_copy_block(const orc_layout *g, void *pool, int src_blk, int dst_blk);
/* the .kv file image of one block, all layers (kv_swapper.cpp:183-198, 268-283) */
void orc_block_image(const orc_layout *g, const void *pool, int blk, void *out);
void orc_block_from_image(const orc_layout *g, void *pool, int blk, const void *image);

/* ---- codecs (builder-specified; precedent layer_int8_dual.cu:239-293) ---- */
/* one row of D elements -> D int8 codes + one fp16 scale */
void orc_quant_row_int8(const uint16_t *x, int D, int src_dtype, int8_t *codes,
                        uint16_t *scale_h);
void orc_quant_row_fp8(const uint16_t *x, int D, int src_dtype, uint8_t *codes);

/* ---- attention (paged_attention.cu:179-269, 465-554) --------------------- */
/* Q/out element type io_dtype (F16/BF16).  Holes (table entry < 0) are skipped.
 * Returns the number of tokens that took part. */
int orc_decode_ref_order(const orc_layout *g, const uint16_t *Q, const void *pool,
                         const int32_t *table, uint16_t *out, int layer,
                         int seq_len, float scale, int io_dtype);
/* fp64 textbook softmax(QK^T*scale)V; writes doubles [QH][D] */
int orc_decode_f64(const orc_layout *g, const uint16_t *Q, const void *pool,
                   const int32_t *table, double *out, int layer, int seq_len,
                   double scale, int io_dtype);
void orc_prefill_ref_order(const orc_layout *g, const uint16_t *Q,
                           const void *pool, const int32_t *table, uint16_t *out,
                           int layer, int pos_start, int M, float scale,
                           int io_dtype);
void orc_prefill_f64(const orc_layout *g, const uint16_t *Q, const void *pool,
                     const int32_t *table, double *out, int layer, int pos_start,
                     int M, double scale, int io_dtype);
/* split-K partials + merge (asr_ops_attn.cu:29-108 algebra) */
void orc_decode_splitk(const orc_layout *g, const uint16_t *Q, const void *pool,
                       const int32_t *table, uint16_t *out, int layer,
                       int seq_len, float scale, int io_dtype, int split_tokens);
/* multi-threaded (OpenMP over q heads / branches) variants for the timed CPU
 * baseline */
void orc_decode_branches(const orc_layout *g, const uint16_t *Q, const void *pool,
                         const int32_t *tables, int table_stride,
                         const int32_t *seq_lens, int B, uint16_t *out, int layer,
                         float scale, int io_dtype, int threads);

/* attention mass per (branch, logical block), fp64; builder-specified, see drk_oracle.c */
void orc_block_attention_mass(const orc_layout *g, const uint16_t *Q, const void *pool,
                              const int32_t *tables, int table_stride,
                              const int32_t *seq_lens, int B, int layer, double scale,
                              int io_dtype, double *mass, int mass_stride);

/* ---- importance scorer (importance_scorer.cu:27-36, 75-87) --------------- */
void orc_importance_update(float *scores, const float *new_scores, int n,
                           float decay);
int  orc_least_important(const float *scores, const int *ids, int n);

/* ---- the layer steps either side of the kernels --------------------------
 * (full_attention_forward_paged, paged_attention.cu:314-376: split Q|gate,
 * per-head RMSNorm, partial RoPE, [write, attend], sigmoid gate).  16-bit
 * elements of type dtype (ORC_F16 / ORC_BF16). */
/* paged_attention.cu:288-298, 386-404: qg [T][H][2D] -> q, gate [T][H][D] */
void orc_split_q_gate(const uint16_t *qg, uint16_t *q, uint16_t *gate, int T,
                      int H, int D);
/* layer_attention.cu:86-135: rows of D elements, one weight vector [D] */
void orc_head_norm(const uint16_t *x, const uint16_t *w, uint16_t *out,
                   int rows, int D, float eps, int dtype);
/* layer_attention.cu:32-55: table[pos][pair] = (cos, sin) of pos * theta^(-2 pair / rd) */
void orc_rope_table(float *table, int n_pos, int rotary_dim, float theta);
/* layer_attention.cu:57-79 / paged_attention.cu:412-451: rotate pairs
 * (i, i + rd/2) of every head of token t at position pos[t], in place */
void orc_apply_rope(uint16_t *x, int T, int H, int D, int rotary_dim,
                    const int32_t *pos, const float *table, int dtype);
/* layer.cu:406-431: out = x * sigmoid(gate) */
void orc_sigmoid_gate(const uint16_t *x, const uint16_t *gate, uint16_t *out,
                      size_t n, int dtype);

/* ---- host bookkeeping: pool + cache manager ------------------------------ */
typedef struct orc_cm orc_cm;
orc_cm *orc_cm_create(int NB, int bs, int max_branches);
void    orc_cm_destroy(orc_cm *c);
/* BlockPool (block_pool.cpp:63-80) */
int  orc_cm_alloc_block(orc_cm *c);
void orc_cm_free_block(orc_cm *c, int id);
int  orc_cm_free_count(const orc_cm *c);
int  orc_cm_refcount(const orc_cm *c, int id);
int  orc_cm_free_stack(const orc_cm *c, int32_t *out, int cap);
/* CacheManager (cache_manager.cpp:73-164, 185-205, 294-326) + branches */
int  orc_cm_ensure(orc_cm *c, int branch, int pos);              /* 1/0 */
int  orc_cm_ensure_range(orc_cm *c, int branch, int pos_start, int M);
int  orc_cm_evict_blocks(orc_cm *c, int n);
int  orc_cm_ensure_free_blocks(orc_cm *c, int n_free);           /* 1/0 */
int  orc_cm_fork(orc_cm *c, int parent, int pos);                /* id or -1 */
void orc_cm_release(orc_cm *c, int branch);
void orc_cm_touch(orc_cm *c, int branch, int logical);
void orc_cm_set_scores(orc_cm *c, const float *scores, int n);   /* NULL = off */
int  orc_cm_max_logical(const orc_cm *c);
int  orc_cm_gpu_blocks_used(const orc_cm *c);
const int32_t *orc_cm_table(const orc_cm *c, int branch);
const int8_t  *orc_cm_location(const orc_cm *c, int branch);
int  orc_cm_seq_len(const orc_cm *c, int branch);
void orc_cm_set_seq_len(orc_cm *c, int branch, int len);
int  orc_cm_lru(const orc_cm *c, int32_t *branch_out, int32_t *logical_out, int cap);
/* copy-on-write copies queued since the last drain: pairs (src,dst) */
int  orc_cm_drain_copies(orc_cm *c, int32_t *src_out, int32_t *dst_out, int cap);

#ifdef __cplusplus
}
#endif
#endif
