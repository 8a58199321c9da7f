/*
 * drk_oracle.c -- CPU restatement of the DeusRidet Memoria/Machina paged-KV path.
 *
 * TEST INFRASTRUCTURE ONLY (see drk_oracle.h).  Plain C, scalar, written for
 * clarity; compiled with -ffp-contract=off so every fp32 operation rounds once.
 *
 * What pins each part (the reference has no test, fixture or golden vector for
 * this path, and its host classes need CUDA headers this image lacks, so it is
 * not buildable here):
 *   - conversions: exhaustive against numpy.float16 and torch bf16/float8 casts;
 *   - addressing: closed form + brute-force fill/read-back on tiny geometry;
 *   - free stack / table / eviction: closed-form sequences and invariants;
 *   - append / extract / inject: pure copies, round trips, M x single == batch;
 *   - attention: fp64 numpy softmax(QK^T)V on independently gathered K/V,
 *     seq_len==1 => out==V[0], equal K rows => mean(V), split-K == unsplit;
 *   - int8 codec: numpy restatement (np.rint is round-half-even) + enumerated ties;
 *   - fp8 codec: torch.float8_e4m3fn casts for |x|<=448, saturation by spec;
 *   - branches / refcount / COW: model-based check against a naive simulator in
 *     which every branch owns a private copy of its K/V;
 *   - head norm / RoPE / gate: fp64 numpy closed forms (x / sqrt(mean(x^2) + eps) * w,
 *     plane rotation by pos * theta^(-2i/rd), x * logistic(g)) to one unit in the
 *     last place of the 16-bit type, rotation by position 0 == identity, rotations
 *     keep each pair's length;
 *   - fixtures written without this file (tests/golden: the E4M3FN table with encode
 *     cases, int8 rows in IEEE arithmetic, a free-stack trace, fp64 attention of the
 *     512-token fp16 configuration).
 * Parity of the *reference decode kernel's exact fp16 output bits* (it is built
 * with --use_fast_math) is unpinned: the tolerance in the tests is against fp64.
 */
#include "drk_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ======================================================================== */
/* scalar conversions                                                       */
/* ======================================================================== */

static uint32_t f_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float bits_f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float orc_h2f(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    int e = (h >> 10) & 0x1f;
    uint32_t m = h & 0x3ffu;
    if (e == 0x1f) return bits_f(sign | 0x7f800000u | (m << 13));
    if (e == 0) {
        float v = ldexpf((float)m, -24);
        return sign ? -v : v;
    }
    return bits_f(sign | ((uint32_t)(e - 15 + 127) << 23) | (m << 13));
}

uint16_t orc_f2h(float f)
{
    uint32_t u = f_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    double a = fabs((double)f);
    if (isnan(f)) return (uint16_t)(sign | 0x7e00u);
    if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u);
    if (a < ldexp(1.0, -14)) {
        int q = (int)nearbyint(a * ldexp(1.0, 24));      /* 0..1024 */
        return (uint16_t)(sign | (uint16_t)q);
    }
    int e = ilogb(a);
    double m = ldexp(a, -e);                               /* [1,2) */
    int q = (int)nearbyint((m - 1.0) * 1024.0);
    if (q == 1024) { e += 1; q = 0; }
    return (uint16_t)(sign | (uint16_t)((e + 15) << 10) | (uint16_t)q);
}

float orc_bf2f(uint16_t b) { return bits_f((uint32_t)b << 16); }

uint16_t orc_f2bf(float f)
{
    uint32_t u = f_bits(f);
    if (isnan(f)) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* OCP E4M3FN: bias 7, 3 mantissa bits, max 448 (0x7E), 0x7F = NaN, no inf.
 * Builder-specified: round-half-even; every finite |x| >= 448 and +-inf
 * saturate to +-448; NaN -> sign|0x7F. */
uint8_t orc_f2fp8(float f)
{
    uint8_t sign = (uint8_t)((f_bits(f) >> 24) & 0x80u);
    double a = fabs((double)f);
    if (isnan(f)) return (uint8_t)(sign | 0x7fu);
    if (a >= 448.0) return (uint8_t)(sign | 0x7eu);
    if (a < ldexp(1.0, -6)) {
        int q = (int)nearbyint(a * 512.0);                 /* 0..8 */
        return (uint8_t)(sign | (uint8_t)q);
    }
    int e = ilogb(a);
    double m = ldexp(a, -e);
    int q = (int)nearbyint((m - 1.0) * 8.0);
    if (q == 8) { e += 1; q = 0; }
    int code = ((e + 7) << 3) | q;
    if (code > 0x7e) code = 0x7e;
    return (uint8_t)(sign | (uint8_t)code);
}

float orc_fp82f(uint8_t c)
{
    int e = (c >> 3) & 0xf, m = c & 7;
    float v;
    if (e == 0xf && m == 7) return bits_f(((uint32_t)(c & 0x80u) << 24) | 0x7fc00000u);
    if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (c & 0x80u) ? -v : v;
}

static float elem_to_f(uint16_t x, int dtype)
{
    return dtype == ORC_BF16 ? orc_bf2f(x) : orc_h2f(x);
}
static uint16_t f_to_elem(float f, int dtype)
{
    return dtype == ORC_BF16 ? orc_f2bf(f) : orc_f2h(f);
}

/* ======================================================================== */
/* addressing -- block_pool.cpp:23-39 (strides), 81-95 (k_ptr/v_ptr/offsets); */
/* device twin paged_attention.cu:36-64; cache_kernels.cu:71-84.             */
/* INT8 appends two fp16 scale planes [KVH][bs] (K then V) after the V codes  */
/* of each (layer, block) -- builder-specified.                               */
/* ======================================================================== */

size_t orc_elem_bytes(const orc_layout *g)
{
    return (g->dtype == ORC_F16 || g->dtype == ORC_BF16) ? 2 : 1;
}
size_t orc_kv_plane_bytes(const orc_layout *g)
{
    return (size_t)g->KVH * g->bs * g->D * orc_elem_bytes(g);
}
static size_t scale_plane_bytes(const orc_layout *g)
{
    return g->dtype == ORC_INT8 ? (size_t)g->KVH * g->bs * 2 : 0;
}
size_t orc_block_stride_bytes(const orc_layout *g)
{
    return 2 * orc_kv_plane_bytes(g) + 2 * scale_plane_bytes(g);
}
size_t orc_layer_stride_bytes(const orc_layout *g)
{
    return (size_t)g->NB * orc_block_stride_bytes(g);
}
size_t orc_pool_bytes(const orc_layout *g)
{
    return (size_t)g->L * orc_layer_stride_bytes(g);
}
size_t orc_k_off(const orc_layout *g, int layer, int blk, int h, int p, int d)
{
    return (size_t)layer * orc_layer_stride_bytes(g)
         + (size_t)blk * orc_block_stride_bytes(g)
         + (((size_t)h * g->bs + p) * g->D + d) * orc_elem_bytes(g);
}
size_t orc_v_off(const orc_layout *g, int layer, int blk, int h, int p, int d)
{
    return orc_k_off(g, layer, blk, h, p, d) + orc_kv_plane_bytes(g);
}
size_t orc_kscale_off(const orc_layout *g, int layer, int blk, int h, int p)
{
    return (size_t)layer * orc_layer_stride_bytes(g)
         + (size_t)blk * orc_block_stride_bytes(g)
         + 2 * orc_kv_plane_bytes(g) + ((size_t)h * g->bs + p) * 2;
}
size_t orc_vscale_off(const orc_layout *g, int layer, int blk, int h, int p)
{
    return orc_kscale_off(g, layer, blk, h, p) + scale_plane_bytes(g);
}
/* block_pool.cpp:28-32: max_blocks = budget / (num_fa * block_stride bytes) */
int orc_max_blocks_for_budget(const orc_layout *g, size_t budget_bytes)
{
    size_t per_block = (size_t)g->L * orc_block_stride_bytes(g);
    return (int)(budget_bytes / per_block);
}

/* The consolidated image of one physical block that KVSwapper::swap_out writes to its
 * .kv file (kv_swapper.cpp:183-198): for every layer the block's K plane, then its V
 * plane (then, for int8 pools, the two scale planes) -- i.e. the block's bytes of each
 * layer, layers in order. */
void orc_block_image(const orc_layout *g, const void *pool, int blk, void *out)
{
    size_t bs = orc_block_stride_bytes(g), ls = orc_layer_stride_bytes(g);
    for (int l = 0; l < g->L; l++)
        memcpy((uint8_t *)out + (size_t)l * bs, (const uint8_t *)pool + (size_t)l * ls + (size_t)blk * bs, bs);
}

void orc_block_from_image(const orc_layout *g, void *pool, int blk, const void *image)
{
    size_t bs = orc_block_stride_bytes(g), ls = orc_layer_stride_bytes(g);
    for (int l = 0; l < g->L; l++)
        memcpy((uint8_t *)pool + (size_t)l * ls + (size_t)blk * bs, (const uint8_t *)image + (size_t)l * bs, bs);
}

/* ======================================================================== */
/* codecs                                                                   */
/* ======================================================================== */

/* Symmetric int8, one fp16 scale per row (= per token, per head).
 * Precedent layer_int8_dual.cu:239-293: scale = absmax/127 (fp32),
 * rcp = scale>0 ? 1/scale : 0, q = clamp(rint(x*rcp), -127, 127).
 * Builder-specified: the scale is stored as fp16 (RNE; +inf -> 65504) and the
 * reciprocal is taken of the *stored* scale, so dequant (code*scale) uses the
 * same number. */
void orc_quant_row_int8(const uint16_t *x, int D, int src_dtype, int8_t *codes,
                        uint16_t *scale_h)
{
    float amax = 0.0f;
    for (int d = 0; d < D; d++) {
        float v = fabsf(elem_to_f(x[d], src_dtype));
        if (v > amax) amax = v;
    }
    float s32 = amax / 127.0f;
    uint16_t sh = orc_f2h(s32);
    if ((sh & 0x7fffu) == 0x7c00u) sh = 0x7bffu;
    float sf = orc_h2f(sh);
    float rcp = sf > 0.0f ? 1.0f / sf : 0.0f;
    for (int d = 0; d < D; d++) {
        float v = elem_to_f(x[d], src_dtype) * rcp;
        float r = nearbyintf(v);                  /* default mode: half-even */
        if (r > 127.0f) r = 127.0f;
        if (r < -127.0f) r = -127.0f;
        codes[d] = (int8_t)(int)r;
    }
    *scale_h = sh;
}

void orc_quant_row_fp8(const uint16_t *x, int D, int src_dtype, uint8_t *codes)
{
    for (int d = 0; d < D; d++) codes[d] = orc_f2fp8(elem_to_f(x[d], src_dtype));
}

/* ======================================================================== */
/* append -- paged_attention.cu:73-102 (one token), 123-153 (batch)          */
/* A hole (table entry < 0) is skipped (the reference would index out of     */
/* bounds there; inject_kv_to_pages_kernel, cache_kernels.cu:120, skips).    */
/* ======================================================================== */

static void put_row(const orc_layout *g, uint8_t *pool, int layer, int blk, int h,
                    int p, int is_v, const uint16_t *row, int src_dtype)
{
    size_t off = is_v ? orc_v_off(g, layer, blk, h, p, 0)
                      : orc_k_off(g, layer, blk, h, p, 0);
    if (g->dtype == ORC_F16 || g->dtype == ORC_BF16) {
        memcpy(pool + off, row, (size_t)g->D * 2);
    } else if (g->dtype == ORC_INT8) {
        uint16_t sh;
        orc_quant_row_int8(row, g->D, src_dtype, (int8_t *)(pool + off), &sh);
        size_t so = is_v ? orc_vscale_off(g, layer, blk, h, p)
                         : orc_kscale_off(g, layer, blk, h, p);
        memcpy(pool + so, &sh, 2);
    } else {
        orc_quant_row_fp8(row, g->D, src_dtype, pool + off);
    }
}

void orc_append_token(const orc_layout *g, void *pool, const int32_t *table,
                      int layer, int pos, const uint16_t *src_k,
                      const uint16_t *src_v, int src_dtype)
{
    int logical = pos / g->bs, p = pos % g->bs;
    int blk = table[logical];
    if (blk < 0) return;
    for (int h = 0; h < g->KVH; h++) {
        put_row(g, (uint8_t *)pool, layer, blk, h, p, 0, src_k + (size_t)h * g->D, src_dtype);
        put_row(g, (uint8_t *)pool, layer, blk, h, p, 1, src_v + (size_t)h * g->D, src_dtype);
    }
}

void orc_append_batch(const orc_layout *g, void *pool, const int32_t *table,
                      int layer, int pos_start, int M, const uint16_t *src_k,
                      const uint16_t *src_v, int src_dtype)
{
    size_t tok = (size_t)g->KVH * g->D;
    for (int t = 0; t < M; t++)
        orc_append_token(g, pool, table, layer, pos_start + t, src_k + t * tok,
                         src_v + t * tok, src_dtype);
}

/* ======================================================================== */
/* extract / inject -- cache_kernels.cu:30-87, 93-141                        */
/* flat layout [layer][K|V][token][head][dim] (+ [layer][K|V][token][head]   */
/* fp16 scales for INT8).  Hole => zero-fill (extract) / skip (inject).      */
/* ======================================================================== */

void orc_extract(const orc_layout *g, void *dst_, void *dst_scales_,
                 const void *pool_, const int32_t *table, int start_token,
                 int num_tokens, int num_layers)
{
    uint8_t *dst = (uint8_t *)dst_;
    uint8_t *dsc = (uint8_t *)dst_scales_;
    const uint8_t *pool = (const uint8_t *)pool_;
    size_t rb = (size_t)g->D * orc_elem_bytes(g);
    for (int l = 0; l < num_layers; l++)
        for (int kv = 0; kv < 2; kv++)
            for (int t = 0; t < num_tokens; t++)
                for (int h = 0; h < g->KVH; h++) {
                    size_t fi = (((size_t)l * 2 + kv) * num_tokens + t) * g->KVH + h;
                    int gt = start_token + t;
                    int blk = table[gt / g->bs], p = gt % g->bs;
                    if (blk < 0) {
                        memset(dst + fi * rb, 0, rb);
                        if (dsc && g->dtype == ORC_INT8) memset(dsc + fi * 2, 0, 2);
                        continue;
                    }
                    size_t off = kv ? orc_v_off(g, l, blk, h, p, 0) : orc_k_off(g, l, blk, h, p, 0);
                    memcpy(dst + fi * rb, pool + off, rb);
                    if (dsc && g->dtype == ORC_INT8) {
                        size_t so = kv ? orc_vscale_off(g, l, blk, h, p) : orc_kscale_off(g, l, blk, h, p);
                        memcpy(dsc + fi * 2, pool + so, 2);
                    }
                }
}

void orc_inject(const orc_layout *g, void *pool_, const void *src_,
                const void *src_scales_, const int32_t *table, int start_token,
                int num_tokens, int num_layers)
{
    uint8_t *pool = (uint8_t *)pool_;
    const uint8_t *src = (const uint8_t *)src_;
    const uint8_t *ssc = (const uint8_t *)src_scales_;
    size_t rb = (size_t)g->D * orc_elem_bytes(g);
    for (int l = 0; l < num_layers; l++)
        for (int kv = 0; kv < 2; kv++)
            for (int t = 0; t < num_tokens; t++)
                for (int h = 0; h < g->KVH; h++) {
                    size_t fi = (((size_t)l * 2 + kv) * num_tokens + t) * g->KVH + h;
                    int gt = start_token + t;
                    int blk = table[gt / g->bs], p = gt % g->bs;
                    if (blk < 0) continue;
                    size_t off = kv ? orc_v_off(g, l, blk, h, p, 0) : orc_k_off(g, l, blk, h, p, 0);
                    memcpy(pool + off, src + fi * rb, rb);
                    if (ssc && g->dtype == ORC_INT8) {
                        size_t so = kv ? orc_vscale_off(g, l, blk, h, p) : orc_kscale_off(g, l, blk, h, p);
                        memcpy(pool + so, ssc + fi * 2, 2);
                    }
                }
}

/* copy-on-write device copy: every layer's (K,V[,scales]) of one block.
 * Builder-specified (intent docs/en/architecture/02-memoria.md:25-26). */
void orc_copy_block(const orc_layout *g, void *pool_, int src_blk, int dst_blk)
{
    uint8_t *pool = (uint8_t *)pool_;
    size_t bsb = orc_block_stride_bytes(g), lsb = orc_layer_stride_bytes(g);
    for (int l = 0; l < g->L; l++)
        memcpy(pool + l * lsb + (size_t)dst_blk * bsb, pool + l * lsb + (size_t)src_blk * bsb, bsb);
}

/* ======================================================================== */
/* attention                                                                */
/* ======================================================================== */

/* dequantised K or V row as fp32 */
static void load_row(const orc_layout *g, const uint8_t *pool, int layer, int blk,
                     int h, int p, int is_v, float *row)
{
    size_t off = is_v ? orc_v_off(g, layer, blk, h, p, 0) : orc_k_off(g, layer, blk, h, p, 0);
    int D = g->D;
    if (g->dtype == ORC_F16 || g->dtype == ORC_BF16) {
        const uint16_t *e = (const uint16_t *)(pool + off);
        for (int d = 0; d < D; d++) row[d] = elem_to_f(e[d], g->dtype);
    } else if (g->dtype == ORC_INT8) {
        size_t so = is_v ? orc_vscale_off(g, layer, blk, h, p) : orc_kscale_off(g, layer, blk, h, p);
        uint16_t sh; memcpy(&sh, pool + so, 2);
        float sf = orc_h2f(sh);
        const int8_t *c = (const int8_t *)(pool + off);
        for (int d = 0; d < D; d++) row[d] = (float)c[d] * sf;
    } else {
        const uint8_t *c = pool + off;
        for (int d = 0; d < D; d++) row[d] = orc_fp82f(c[d]);
    }
}

/* The reference's dot product order (paged_attention.cu:231-246): per-lane
 * product q[d]*k[d]; 32-lane xor butterfly (offsets 16,8,4,2,1) inside each
 * warp; lane 0 of each warp stores its sum; thread 0 adds the warp sums in
 * order and multiplies by scale. */
static float ref_dot(const float *q, const float *k, int D, float scale)
{
    float sum = 0.0f;
    for (int w = 0; w < (D + 31) / 32; w++) {
        float lane[32];
        for (int i = 0; i < 32; i++) {
            int d = w * 32 + i;
            lane[i] = d < D ? q[d] * k[d] : 0.0f;
        }
        for (int off = 16; off > 0; off /= 2) {
            float nxt[32];
            for (int i = 0; i < 32; i++) nxt[i] = lane[i] + lane[i ^ off];
            memcpy(lane, nxt, sizeof lane);
        }
        sum += lane[0];
    }
    return sum * scale;
}

/* One query head over tokens [t0, t1) in the reference's sequential
 * online-softmax order (paged_attention.cu:212-263): m=-FLT_MAX, l=0, o=0;
 * per token m'=max(m,s), alpha=exp(m-m'), p=exp(s-m'), o=o*alpha+v*p,
 * l=l*alpha+p.  expf stands in for the reference's __expf.  Leaves (o,m,l)
 * unnormalised so the same routine serves split-K.  Returns tokens seen. */
static int head_partial(const orc_layout *g, const float *q, const uint8_t *pool,
                        const int32_t *table, int layer, int kvh, int t0, int t1,
                        float scale, float *o, float *m_out, float *l_out)
{
    int D = g->D, seen = 0;
    float m = -FLT_MAX, l = 0.0f;
    float *krow = (float *)malloc(sizeof(float) * D * 2), *vrow = krow + D;
    for (int d = 0; d < D; d++) o[d] = 0.0f;
    for (int t = t0; t < t1; t++) {
        int blk = table[t / g->bs];
        if (blk < 0) continue;
        load_row(g, pool, layer, blk, kvh, t % g->bs, 0, krow);
        load_row(g, pool, layer, blk, kvh, t % g->bs, 1, vrow);
        float s = ref_dot(q, krow, D, scale);
        float m_new = fmaxf(m, s);
        float alpha = expf(m - m_new);
        float p = expf(s - m_new);
        for (int d = 0; d < D; d++) o[d] = o[d] * alpha + vrow[d] * p;
        l = l * alpha + p;
        m = m_new;
        seen++;
    }
    free(krow);
    *m_out = m; *l_out = l;
    return seen;
}

/* paged_gqa_decode_attention_kernel, paged_attention.cu:179-269.
 * kv head of query head h = h / (QH/KVH) (line 194); out written only when
 * l > 0 (line 266). */
int orc_decode_ref_order(const orc_layout *g, const uint16_t *Q, const void *pool,
                         const int32_t *table, uint16_t *out, int layer,
                         int seq_len, float scale, int io_dtype)
{
    int D = g->D, groups = g->QH / g->KVH, seen = 0;
    float *q = (float *)malloc(sizeof(float) * D * 2), *o = q + D;
    for (int h = 0; h < g->QH; h++) {
        float m, l;
        for (int d = 0; d < D; d++) q[d] = elem_to_f(Q[(size_t)h * D + d], io_dtype);
        seen = head_partial(g, q, (const uint8_t *)pool, table, layer, h / groups,
                            0, seq_len, scale, o, &m, &l);
        if (l > 0.0f)
            for (int d = 0; d < D; d++) out[(size_t)h * D + d] = f_to_elem(o[d] / l, io_dtype);
    }
    free(q);
    return seen;
}

/* fp64 textbook attention: two passes (max, then exp/sum), no online rescale. */
static void head_f64(const orc_layout *g, const uint16_t *Qh, const uint8_t *pool,
                     const int32_t *table, int layer, int kvh, int seq_len,
                     double scale, int io_dtype, double *out, int *seen_out)
{
    int D = g->D, n = 0;
    double *s = (double *)malloc(sizeof(double) * (seq_len > 0 ? seq_len : 1));
    float *row = (float *)malloc(sizeof(float) * D);
    double mx = -INFINITY, denom = 0.0;
    for (int t = 0; t < seq_len; t++) {
        int blk = table[t / g->bs];
        if (blk < 0) { s[t] = -INFINITY; continue; }
        load_row(g, pool, layer, blk, kvh, t % g->bs, 0, row);
        double acc = 0.0;
        for (int d = 0; d < D; d++) acc += (double)elem_to_f(Qh[d], io_dtype) * (double)row[d];
        s[t] = acc * scale;
        if (s[t] > mx) mx = s[t];
        n++;
    }
    for (int d = 0; d < D; d++) out[d] = 0.0;
    for (int t = 0; t < seq_len; t++) {
        if (s[t] == -INFINITY) continue;
        int blk = table[t / g->bs];
        double p = exp(s[t] - mx);
        denom += p;
        load_row(g, pool, layer, blk, kvh, t % g->bs, 1, row);
        for (int d = 0; d < D; d++) out[d] += p * (double)row[d];
    }
    if (denom > 0.0) for (int d = 0; d < D; d++) out[d] /= denom;
    free(s); free(row);
    *seen_out = n;
}

int orc_decode_f64(const orc_layout *g, const uint16_t *Q, const void *pool,
                   const int32_t *table, double *out, int layer, int seq_len,
                   double scale, int io_dtype)
{
    int groups = g->QH / g->KVH, seen = 0;
    for (int h = 0; h < g->QH; h++)
        head_f64(g, Q + (size_t)h * g->D, (const uint8_t *)pool, table, layer,
                 h / groups, seq_len, scale, io_dtype, out + (size_t)h * g->D, &seen);
    return seen;
}

/* paged_prefill_attention_kernel, paged_attention.cu:465-554: row t of the
 * chunk is the decode loop with causal_len = pos_start + t + 1 (line 481);
 * Q/out are [M][QH][D] (lines 483-485, 552). */
void orc_prefill_ref_order(const orc_layout *g, const uint16_t *Q,
                           const void *pool, const int32_t *table, uint16_t *out,
                           int layer, int pos_start, int M, float scale,
                           int io_dtype)
{
    size_t row = (size_t)g->QH * g->D;
    for (int t = 0; t < M; t++)
        orc_decode_ref_order(g, Q + t * row, pool, table, out + t * row, layer,
                             pos_start + t + 1, scale, io_dtype);
}

void orc_prefill_f64(const orc_layout *g, const uint16_t *Q, const void *pool,
                     const int32_t *table, double *out, int layer, int pos_start,
                     int M, double scale, int io_dtype)
{
    size_t row = (size_t)g->QH * g->D;
    /* rows are independent (each call allocates its own scratch): the threads only shorten the tests */
#pragma omp parallel for schedule(dynamic, 4)
    for (int t = 0; t < M; t++)
        orc_decode_f64(g, Q + t * row, pool, table, out + t * row, layer,
                       pos_start + t + 1, scale, io_dtype);
}

/* Split-K: partial (o, m, l) per run of split_tokens tokens, merged with the
 * max-rescaled algebra of contiguous_split_k_merge_kernel
 * (asr_ops_attn.cu:84-108).  An empty or all-hole partition carries l = 0 and
 * contributes nothing; out = l>0 ? acc/l : unchanged. */
void orc_decode_splitk(const orc_layout *g, const uint16_t *Q, const void *pool,
                       const int32_t *table, uint16_t *out, int layer,
                       int seq_len, float scale, int io_dtype, int split_tokens)
{
    int D = g->D, groups = g->QH / g->KVH;
    int nsplit = (seq_len + split_tokens - 1) / split_tokens;
    float *q = (float *)malloc(sizeof(float) * D * 3), *o = q + D, *acc = q + 2 * D;
    for (int h = 0; h < g->QH; h++) {
        float M = -FLT_MAX, Lsum = 0.0f;
        for (int d = 0; d < D; d++) { q[d] = elem_to_f(Q[(size_t)h * D + d], io_dtype); acc[d] = 0.0f; }
        for (int s = 0; s < nsplit; s++) {
            int t0 = s * split_tokens, t1 = t0 + split_tokens;
            float pm, pl;
            if (t1 > seq_len) t1 = seq_len;
            head_partial(g, q, (const uint8_t *)pool, table, layer, h / groups, t0, t1, scale, o, &pm, &pl);
            if (!(pl > 0.0f)) continue;
            if (pm > M) {
                float sc = expf(M - pm);
                for (int d = 0; d < D; d++) acc[d] = acc[d] * sc + o[d];
                Lsum = Lsum * sc + pl; M = pm;
            } else {
                float sc = expf(pm - M);
                for (int d = 0; d < D; d++) acc[d] += o[d] * sc;
                Lsum += pl * sc;
            }
        }
        if (Lsum > 0.0f)
            for (int d = 0; d < D; d++) out[(size_t)h * D + d] = f_to_elem(acc[d] / Lsum, io_dtype);
    }
    free(q);
}

/* Multi-branch decode (builder-specified batching of the kernel above): branch
 * b uses table row b and seq_lens[b]; Q/out are [B][QH][D].  OpenMP over
 * (branch, q head) when threads > 1 -- this is the timed CPU baseline. */
void orc_decode_branches(const orc_layout *g, const uint16_t *Q, const void *pool,
                         const int32_t *tables, int table_stride,
                         const int32_t *seq_lens, int B, uint16_t *out, int layer,
                         float scale, int io_dtype, int threads)
{
    int D = g->D, groups = g->QH / g->KVH, total = B * g->QH;
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads > 0 ? threads : 1)
#endif
    for (int w = 0; w < total; w++) {
        int b = w / g->QH, h = w % g->QH;
        float *q = (float *)malloc(sizeof(float) * D * 2), *o = q + D, m, l;
        const uint16_t *Qh = Q + ((size_t)b * g->QH + h) * D;
        for (int d = 0; d < D; d++) q[d] = elem_to_f(Qh[d], io_dtype);
        head_partial(g, q, (const uint8_t *)pool, tables + (size_t)b * table_stride,
                     layer, h / groups, 0, seq_lens[b], scale, o, &m, &l);
        if (l > 0.0f)
            for (int d = 0; d < D; d++)
                out[((size_t)b * g->QH + h) * D + d] = f_to_elem(o[d] / l, io_dtype);
        free(q);
    }
}

/* Attention mass per (branch, logical block): sum over the block's tokens and over all
 * query heads of the softmax probability, in fp64 (builder-specified; it is the "new
 * importance value from attention" of importance_scorer.h:37-41, which the reference
 * never computes).  mass [B][mass_stride], entries past a branch's blocks are set to 0. */
void orc_block_attention_mass(const orc_layout *g, const uint16_t *Q, const void *pool,
                              const int32_t *tables, int table_stride, const int32_t *seq_lens,
                              int B, int layer, double scale, int io_dtype, double *mass,
                              int mass_stride)
{
    int D = g->D, groups = g->QH / g->KVH;
    float *row = (float *)malloc(sizeof(float) * D);
    for (int b = 0; b < B; b++) {
        const int32_t *table = tables + (size_t)b * table_stride;
        int n = seq_lens[b];
        double *s = (double *)malloc(sizeof(double) * (n > 0 ? n : 1));
        for (int lb = 0; lb < mass_stride; lb++) mass[(size_t)b * mass_stride + lb] = 0.0;
        for (int h = 0; h < g->QH; h++) {
            const uint16_t *Qh = Q + ((size_t)b * g->QH + h) * D;
            double mx = -INFINITY, denom = 0.0;
            for (int t = 0; t < n; t++) {
                int blk = table[t / g->bs];
                if (blk < 0) { s[t] = -INFINITY; continue; }
                load_row(g, (const uint8_t *)pool, layer, blk, h / groups, t % g->bs, 0, row);
                double acc = 0.0;
                for (int d = 0; d < D; d++) acc += (double)elem_to_f(Qh[d], io_dtype) * (double)row[d];
                s[t] = acc * scale;
                if (s[t] > mx) mx = s[t];
            }
            for (int t = 0; t < n; t++) if (s[t] != -INFINITY) denom += exp(s[t] - mx);
            if (!(denom > 0.0)) continue;
            for (int t = 0; t < n; t++)
                if (s[t] != -INFINITY) mass[(size_t)b * mass_stride + t / g->bs] += exp(s[t] - mx) / denom;
        }
        free(s);
    }
    free(row);
}

/* ======================================================================== */
/* layer steps either side of the kernels                                   */
/* ======================================================================== */

/* paged_split_q_gate, paged_attention.cu:288-298 (batch form 386-404) */
void orc_split_q_gate(const uint16_t *qg, uint16_t *q, uint16_t *gate, int T, int H, int D)
{
    for (int t = 0; t < T; t++)
        for (int h = 0; h < H; h++)
            for (int d = 0; d < D; d++) {
                q[((size_t)t * H + h) * D + d] = qg[((size_t)t * H + h) * 2 * D + d];
                gate[((size_t)t * H + h) * D + d] = qg[((size_t)t * H + h) * 2 * D + D + d];
            }
}

/* head_norm_kernel, layer_attention.cu:86-127: sum of squares in fp32,
 * inv_rms = rsqrt(ss / D + eps), out = fp16((x * inv_rms) * w).
 * The reference's summation order is a property of its 128/256-thread launch and
 * rsqrtf is an approximation under --use_fast_math; the order fixed here is the
 * one the HIP kernels use so that both sides agree to the bit: D/8 partial sums
 * of 8 consecutive elements each (fused multiply-adds), folded by an xor
 * butterfly with strides D/16, ..., 2, 1; then 1 / sqrt(.) correctly rounded. */
void orc_head_norm(const uint16_t *x, const uint16_t *w, uint16_t *out, int rows, int D, float eps, int dtype)
{
    const int nl = D / 8;
    float part[64];
    for (int r = 0; r < rows; r++) {
        const uint16_t *xr = x + (size_t)r * D;
        for (int l = 0; l < nl; l++) {
            float s = 0.0f;
            for (int i = 0; i < 8; i++) {
                const float v = elem_to_f(xr[l * 8 + i], dtype);
                s = fmaf(v, v, s);
            }
            part[l] = s;
        }
        for (int off = nl >> 1; off > 0; off >>= 1) {
            float nxt[64];
            for (int l = 0; l < nl; l++) nxt[l] = part[l] + part[l ^ off];
            memcpy(part, nxt, sizeof(float) * (size_t)nl);
        }
        const float inv_rms = 1.0f / sqrtf(part[0] / (float)D + eps);
        for (int d = 0; d < D; d++) {
            const float v = elem_to_f(xr[d], dtype) * inv_rms;
            out[(size_t)r * D + d] = f_to_elem(v * elem_to_f(w[d], dtype), dtype);
        }
    }
}

/* rope_kernel, layer_attention.cu:42-48: freq = 1 / powf(theta, 2 pair / rd),
 * angle = pos * freq, all in fp32 */
void orc_rope_table(float *table, int n_pos, int rotary_dim, float theta)
{
    const int np = rotary_dim / 2;
    for (int pos = 0; pos < n_pos; pos++)
        for (int pair = 0; pair < np; pair++) {
            const float freq = 1.0f / powf(theta, (2.0f * (float)pair) / (float)rotary_dim);
            const float angle = (float)pos * freq;
            table[((size_t)pos * np + pair) * 2] = cosf(angle);
            table[((size_t)pos * np + pair) * 2 + 1] = sinf(angle);
        }
}

/* rope_kernel, layer_attention.cu:50-69 (half-half pairing (i, i + rd/2));
 * nvcc contracts x0*c - x1*s and x1*c + x0*s into one product and one fused
 * multiply-add each; the form fixed here rounds the second product first. */
void orc_apply_rope(uint16_t *x, int T, int H, int D, int rotary_dim, const int32_t *pos, const float *table,
                    int dtype)
{
    const int np = rotary_dim / 2;
    for (int t = 0; t < T; t++)
        for (int h = 0; h < H; h++) {
            uint16_t *row = x + ((size_t)t * H + h) * D;
            for (int pair = 0; pair < np; pair++) {
                const float c = table[((size_t)pos[t] * np + pair) * 2], s = table[((size_t)pos[t] * np + pair) * 2 + 1];
                const float x0 = elem_to_f(row[pair], dtype), x1 = elem_to_f(row[pair + np], dtype);
                row[pair] = f_to_elem(fmaf(x0, c, -(x1 * s)), dtype);
                row[pair + np] = f_to_elem(fmaf(x1, c, x0 * s), dtype);
            }
        }
}

/* sigmoid_gate_kernel, layer.cu:406-431: v / (1 + exp(-g)) */
void orc_sigmoid_gate(const uint16_t *x, const uint16_t *gate, uint16_t *out, size_t n, int dtype)
{
    for (size_t i = 0; i < n; i++) {
        const float v = elem_to_f(x[i], dtype), g = elem_to_f(gate[i], dtype);
        out[i] = f_to_elem(v / (1.0f + expf(-g)), dtype);
    }
}

/* ======================================================================== */
/* importance scorer -- importance_scorer.cu:27-36 (update), 75-87 (argmin)  */
/* ======================================================================== */

/* nvcc's default (-fmad=true) contracts score*decay + new into one fused
 * multiply-add, so the restatement uses fmaf: one rounding. */
void orc_importance_update(float *scores, const float *new_scores, int n, float decay)
{
    for (int b = 0; b < n; b++) scores[b] = fmaf(scores[b], decay, new_scores[b]);
}

int orc_least_important(const float *scores, const int *ids, int n)
{
    if (n <= 0) return -1;
    int min_idx = ids[0];
    float min_score = scores[min_idx];
    for (int i = 1; i < n; i++)
        if (scores[ids[i]] < min_score) { min_score = scores[ids[i]]; min_idx = ids[i]; }
    return min_idx;
}

/* ======================================================================== */
/* host bookkeeping                                                          */
/* ======================================================================== */

struct orc_cm {
    int NB, bs, max_logical, max_branches;
    /* BlockPool: LIFO free stack (block_pool.cpp:51-55, 63-75) */
    int32_t *free_stack; int free_n;
    int32_t *refcount;                       /* builder-specified */
    /* per branch (branch 0 = the reference's single sequence) */
    int32_t *table;                          /* [max_branches][max_logical] */
    int8_t  *loc;                            /* 0 GPU, -1 INVALID (cache_manager.h:42-46) */
    int32_t *seq_len; int8_t *alive;
    /* lru_order_ deque (cache_manager.h:139): front = oldest */
    int32_t *lru_b, *lru_l; int lru_n;
    /* optional scores indexed by table cell = branch * max_logical + logical block; for branch 0,
     * the reference's one sequence, that is its logical block index (cache_manager.cpp:188-201) */
    float *scores; int nscores;
    /* queued COW copies */
    int32_t *cp_src, *cp_dst; int cp_n, cp_cap;
    /* builder-specified protection of the current step: a cell that ensure() made resident is held
     * until the queued copies are drained; a block named by a queued copy is pinned; a pinned block
     * that loses its last reference is freed only at the drain */
    int8_t *held;                            /* per cell */
    int32_t *pin;                            /* per physical block */
    int32_t *deferred; int deferred_n;
};

orc_cm *orc_cm_create(int NB, int bs, int max_branches)
{
    orc_cm *c = (orc_cm *)calloc(1, sizeof *c);
    c->NB = NB; c->bs = bs; c->max_branches = max_branches;
    c->max_logical = 2 * NB;                              /* cache_manager.cpp:39 */
    c->free_stack = (int32_t *)malloc(sizeof(int32_t) * NB);
    for (int i = 0; i < NB; i++) c->free_stack[i] = NB - 1 - i;   /* block_pool.cpp:53-55 */
    c->free_n = NB;
    c->refcount = (int32_t *)calloc(NB, sizeof(int32_t));
    size_t cells = (size_t)max_branches * c->max_logical;
    c->table = (int32_t *)malloc(sizeof(int32_t) * cells);
    c->loc = (int8_t *)malloc(cells);
    for (size_t i = 0; i < cells; i++) { c->table[i] = -1; c->loc[i] = -1; }
    c->seq_len = (int32_t *)calloc(max_branches, sizeof(int32_t));
    c->alive = (int8_t *)calloc(max_branches, 1);
    c->alive[0] = 1;
    c->lru_b = (int32_t *)malloc(sizeof(int32_t) * cells);
    c->lru_l = (int32_t *)malloc(sizeof(int32_t) * cells);
    c->cp_cap = 1024;
    c->cp_src = (int32_t *)malloc(sizeof(int32_t) * c->cp_cap);
    c->cp_dst = (int32_t *)malloc(sizeof(int32_t) * c->cp_cap);
    c->held = (int8_t *)calloc(cells, 1);
    c->pin = (int32_t *)calloc(NB, sizeof(int32_t));
    c->deferred = (int32_t *)malloc(sizeof(int32_t) * NB);
    return c;
}

void orc_cm_destroy(orc_cm *c)
{
    if (!c) return;
    free(c->free_stack); free(c->refcount); free(c->table); free(c->loc);
    free(c->seq_len); free(c->alive); free(c->lru_b); free(c->lru_l);
    free(c->scores); free(c->cp_src); free(c->cp_dst); free(c->held); free(c->pin); free(c->deferred); free(c);
}

/* block_pool.cpp:63-69 */
int orc_cm_alloc_block(orc_cm *c)
{
    if (c->free_n == 0) return -1;
    int id = c->free_stack[--c->free_n];
    c->refcount[id] = 1;
    return id;
}
/* block_pool.cpp:71-74 */
void orc_cm_free_block(orc_cm *c, int id)
{
    c->refcount[id] = 0;
    c->free_stack[c->free_n++] = id;
}
int orc_cm_free_count(const orc_cm *c) { return c->free_n; }
int orc_cm_refcount(const orc_cm *c, int id) { return c->refcount[id]; }
int orc_cm_free_stack(const orc_cm *c, int32_t *out, int cap)
{
    int n = c->free_n < cap ? c->free_n : cap;
    memcpy(out, c->free_stack, sizeof(int32_t) * n);
    return c->free_n;
}

static void drop_ref(orc_cm *c, int phys)
{
    if (c->refcount[phys] == 1 && c->pin[phys] > 0) {    /* last reference of a block a queued copy names */
        c->deferred[c->deferred_n++] = phys;
        return;
    }
    if (--c->refcount[phys] <= 0) orc_cm_free_block(c, phys);
}

static void lru_remove(orc_cm *c, int b, int l)
{
    int w = 0;                                           /* std::remove, cache_manager.cpp:125-127 */
    for (int i = 0; i < c->lru_n; i++)
        if (!(c->lru_b[i] == b && c->lru_l[i] == l)) { c->lru_b[w] = c->lru_b[i]; c->lru_l[w] = c->lru_l[i]; w++; }
    c->lru_n = w;
}
static void lru_push(orc_cm *c, int b, int l)
{
    c->lru_b[c->lru_n] = b; c->lru_l[c->lru_n] = l; c->lru_n++;
}

#define CELL(c, b, l) ((size_t)(b) * (c)->max_logical + (l))

/* cache_manager.cpp:185-205.  Builder-specified filters: an entry whose physical block is
 * referenced by more than one table is pinned, and so is a block a queued copy names.  Cells of
 * the current step (held) are passed over; only when nothing else is left (second pass) may a
 * branch's allocation take that branch's own held cells, and an explicit request (for_branch < 0)
 * any held cell. */
static int pick_victim(orc_cm *c, int *vb, int *vl, int for_branch)
{
    for (int pass = 0; pass < 2; pass++) {
        int best = -1;
        for (int i = 0; i < c->lru_n; i++) {
            int b = c->lru_b[i], l = c->lru_l[i];
            int phys = c->table[CELL(c, b, l)];
            if (c->loc[CELL(c, b, l)] != 0 || phys < 0 || c->refcount[phys] != 1 || c->pin[phys] > 0) continue;
            if ((c->held[CELL(c, b, l)] != 0) != (pass == 1)) continue;
            if (pass == 1 && for_branch >= 0 && b != for_branch) continue;
            if (!c->scores) { best = i; break; }              /* lru_order_.front() */
            int cell = CELL(c, b, l), cbest = best < 0 ? 0 : CELL(c, c->lru_b[best], c->lru_l[best]);
            float s = cell < c->nscores ? c->scores[cell] : 0.0f;
            float sb = best < 0 ? 0.0f : (cbest < c->nscores ? c->scores[cbest] : 0.0f);
            if (best < 0 || s < sb) best = i;                 /* first minimum */
        }
        if (best >= 0) {
            *vb = c->lru_b[best]; *vl = c->lru_l[best];
            return 1;
        }
    }
    return 0;
}

/* cache_manager.cpp:118-156 without a swapper: discard */
static int evict_for(orc_cm *c, int n, int for_branch)
{
    int evicted = 0;
    while (evicted < n && c->lru_n > 0) {
        int b, l;
        if (!pick_victim(c, &b, &l, for_branch)) break;
        lru_remove(c, b, l);
        int phys = c->table[CELL(c, b, l)];
        drop_ref(c, phys);
        c->table[CELL(c, b, l)] = -1;
        c->loc[CELL(c, b, l)] = -1;
        evicted++;
    }
    return evicted;
}
int orc_cm_evict_blocks(orc_cm *c, int n) { return evict_for(c, n, -1); }

/* cache_manager.cpp:158-164 */
static int ensure_free_for(orc_cm *c, int n_free, int for_branch)
{
    while (c->free_n < n_free) {
        if (c->lru_n == 0) return 0;
        if (evict_for(c, 1, for_branch) == 0) return 0;
    }
    return 1;
}
int orc_cm_ensure_free_blocks(orc_cm *c, int n_free) { return ensure_free_for(c, n_free, -1); }

static int alloc_phys(orc_cm *c, int for_branch)         /* cache_manager.cpp:306-319 */
{
    int phys = orc_cm_alloc_block(c);
    if (phys < 0) {
        if (!ensure_free_for(c, 1, for_branch)) return -1;
        phys = orc_cm_alloc_block(c);
    }
    return phys;
}

/* cache_manager.cpp:73-95 + 306-326.  Builder-specified: a resident block that
 * other tables also reference is copied before the write (copy-on-write): a new
 * block is allocated, the (src,dst) copy is queued, the old reference dropped;
 * the entry keeps its place in the LRU order. */
int orc_cm_ensure(orc_cm *c, int b, int pos)
{
    int l = pos / c->bs;
    if (b < 0 || b >= c->max_branches || !c->alive[b] || pos < 0) return 0;
    if (l >= c->max_logical) return 0;
    size_t cell = CELL(c, b, l);
    if (c->loc[cell] == 0) {
        int phys = c->table[cell];
        c->held[cell] = 1;                                /* before the allocation below looks for a victim */
        if (c->refcount[phys] > 1) {
            int np = alloc_phys(c, b);
            if (np < 0) return 0;
            if (c->cp_n == c->cp_cap) {
                c->cp_cap *= 2;
                c->cp_src = (int32_t *)realloc(c->cp_src, sizeof(int32_t) * c->cp_cap);
                c->cp_dst = (int32_t *)realloc(c->cp_dst, sizeof(int32_t) * c->cp_cap);
            }
            c->cp_src[c->cp_n] = phys; c->cp_dst[c->cp_n] = np; c->cp_n++;
            c->pin[phys]++; c->pin[np]++;
            c->refcount[phys]--;
            c->table[cell] = np;
        }
        return 1;
    }
    int phys = alloc_phys(c, b);
    if (phys < 0) return 0;
    c->table[cell] = phys;                                /* cache_manager.cpp:321-323 */
    c->loc[cell] = 0;
    c->held[cell] = 1;
    lru_push(c, b, l);
    return 1;
}

/* cache_manager.cpp:97-106 */
int orc_cm_ensure_range(orc_cm *c, int b, int pos_start, int M)
{
    int first = pos_start / c->bs, last = (pos_start + M - 1) / c->bs;
    for (int blk = first; blk <= last; blk++)
        if (!orc_cm_ensure(c, b, blk * c->bs)) return 0;
    return 1;
}

/* Builder-specified: the child shares every resident block that holds tokens
 * [0, pos) of the parent; each gains a reference and an LRU entry at the back
 * in ascending logical order.  Lowest free branch id is used. */
int orc_cm_fork(orc_cm *c, int parent, int pos)
{
    if (parent < 0 || parent >= c->max_branches || !c->alive[parent] || pos < 0) return -1;
    int id = -1;
    for (int i = 0; i < c->max_branches; i++) if (!c->alive[i]) { id = i; break; }
    if (id < 0) return -1;
    int nshared = (pos + c->bs - 1) / c->bs;
    if (nshared > c->max_logical) return -1;
    c->alive[id] = 1; c->seq_len[id] = pos;
    for (int l = 0; l < nshared; l++) {
        size_t pc = CELL(c, parent, l), cc = CELL(c, id, l);
        if (c->loc[pc] != 0) continue;
        c->table[cc] = c->table[pc]; c->loc[cc] = 0;
        c->refcount[c->table[pc]]++;
        lru_push(c, id, l);
    }
    return id;
}

/* Builder-specified: drop every reference of the branch, ascending logical. */
void orc_cm_release(orc_cm *c, int b)
{
    if (b < 0 || b >= c->max_branches || !c->alive[b]) return;
    for (int l = 0; l < c->max_logical; l++) {
        size_t cell = CELL(c, b, l);
        if (c->loc[cell] != 0) continue;
        lru_remove(c, b, l);
        drop_ref(c, c->table[cell]);
        c->table[cell] = -1; c->loc[cell] = -1;
    }
    c->seq_len[b] = 0;
    if (b != 0) c->alive[b] = 0;
}

/* Builder-specified recency update: move the entry to the back. */
void orc_cm_touch(orc_cm *c, int b, int l)
{
    if (b < 0 || b >= c->max_branches || l < 0 || l >= c->max_logical) return;
    if (c->loc[CELL(c, b, l)] != 0) return;
    lru_remove(c, b, l);
    lru_push(c, b, l);
}

void orc_cm_set_scores(orc_cm *c, const float *scores, int n)
{
    free(c->scores); c->scores = NULL; c->nscores = 0;
    if (!scores) return;
    c->scores = (float *)malloc(sizeof(float) * n);
    memcpy(c->scores, scores, sizeof(float) * n);
    c->nscores = n;
}

int orc_cm_max_logical(const orc_cm *c) { return c->max_logical; }
int orc_cm_gpu_blocks_used(const orc_cm *c) { return c->NB - c->free_n; }  /* cache_manager.cpp:294-296 */
const int32_t *orc_cm_table(const orc_cm *c, int b) { return c->table + CELL(c, b, 0); }
const int8_t *orc_cm_location(const orc_cm *c, int b) { return c->loc + CELL(c, b, 0); }
int orc_cm_seq_len(const orc_cm *c, int b) { return c->seq_len[b]; }
void orc_cm_set_seq_len(orc_cm *c, int b, int len) { c->seq_len[b] = len; }
int orc_cm_lru(const orc_cm *c, int32_t *bo, int32_t *lo, int cap)
{
    int n = c->lru_n < cap ? c->lru_n : cap;
    memcpy(bo, c->lru_b, sizeof(int32_t) * n);
    memcpy(lo, c->lru_l, sizeof(int32_t) * n);
    return c->lru_n;
}
int orc_cm_drain_copies(orc_cm *c, int32_t *so, int32_t *dn, int cap)
{
    int n = c->cp_n < cap ? c->cp_n : cap;
    memcpy(so, c->cp_src, sizeof(int32_t) * n);
    memcpy(dn, c->cp_dst, sizeof(int32_t) * n);
    int total = c->cp_n;
    /* the copies count as issued: pins, deferred frees (in the order they were deferred) and holds end */
    for (int i = 0; i < c->cp_n; i++) { c->pin[c->cp_src[i]]--; c->pin[c->cp_dst[i]]--; }
    c->cp_n = 0;
    for (int i = 0; i < c->deferred_n; i++) drop_ref(c, c->deferred[i]);
    c->deferred_n = 0;
    memset(c->held, 0, (size_t)c->max_branches * c->max_logical);
    return total;
}
