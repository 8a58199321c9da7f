// drk_pages.hip -- data movement between token-major buffers and pages:
// append (with int8 / fp8 quantisation on the way in), extract, inject,
// copy-on-write block copies, importance-score update.
//
// All of it is HBM-bound byte work.  Every thread moves 16-byte chunks; the
// chunk index inside a workgroup enumerates [token][head][chunk], which is the
// order of the token-major side, so that side is read or written as one
// contiguous run per workgroup and the paged side as whole head rows.
#include "drk_common.hpp"
#include "drk_codec.hpp"

namespace drk {

constexpr int kThreads = 256;
// Tokens one workgroup moves per (layer, K|V) = chunk target / chunks per token, at most 16.
// Plain copies run best in many short workgroups -- measured on 2 048 tokens x 36 layers, 8 x 128
// bf16: append 5.14 / 5.39 / 5.57 TB/s at 2 048 / 512 / 256 chunks per workgroup, extract 5.78 /
// 5.94 / 5.80, inject 5.06 / 5.35 / 5.42 -- the quantising modes with four rounds of loads in
// flight once per workgroup (1 024 chunks: int8 4.3 TB/s, fp8 5.0; 4.15 and 4.7 at 2 048).
int g_copy_chunks = 256, g_flat_chunks = 512, g_quant_chunks = 1024;
int g_quant_pairs = 1;                      // quantising append: 32 source bytes per thread (0: 16, the one-chunk kernel)
static int tokens_per_group(unsigned chunks_per_token, int target_chunks)
{
    const unsigned target = (unsigned)target_chunks;
    unsigned t = target / (chunks_per_token ? chunks_per_token : 1u);
    return (int)(t < 1u ? 1u : (t > 16u ? 16u : t));
}

// ------------------------------------------------------------------------
// extract / inject
// grid = (token groups, num_layers*2); flat side [layer][K|V][token][head][dim]
// ------------------------------------------------------------------------
template <bool EXTRACT>
__global__ __launch_bounds__(kThreads) void flat_copy_kernel(
    Lay a, uint8_t *__restrict__ pool, uint8_t *__restrict__ flat, uint8_t *__restrict__ flat_scales,
    const int32_t *__restrict__ table, int start_token, int num_tokens, int tpg, Div tok_div, Div row_div,
    Div bs_div)
{
    const int tg = blockIdx.x;
    const int layer = blockIdx.y >> 1, kv = blockIdx.y & 1;
    const int t0 = tg * tpg;
    const int ntok = min(tpg, num_tokens - t0);
    const unsigned rc = row_div.d;                       // 16-byte chunks per row
    const unsigned items = (unsigned)ntok * tok_div.d;   // tok_div.d = KVH*rc
    uint8_t *fbase = flat + ((size_t)(layer * 2 + kv) * num_tokens + t0) * a.KVH * a.row_bytes;

    constexpr int U = 4;
    for (unsigned base = threadIdx.x; base < items; base += kThreads * U) {
        uint4 val[U];
        size_t poff[U];
        bool live[U], hole[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            unsigned ci = base + u * kThreads;
            live[u] = ci < items;
            hole[u] = true;
            poff[u] = 0;
            val[u] = make_uint4(0, 0, 0, 0);
            if (live[u]) {
                unsigned t = dv(ci, tok_div), r = ci - t * tok_div.d;
                unsigned h = dv(r, row_div), c = r - h * rc;
                unsigned gt = (unsigned)(start_token + t0) + t;
                unsigned lb = dv(gt, bs_div);
                int blk = table[lb];
                if (blk >= 0 && blk < a.NB) {
                    hole[u] = false;
                    poff[u] = row_off(a, layer, blk, kv, h, gt - lb * bs_div.d) + (size_t)c * 16;
                }
                if (EXTRACT) { if (!hole[u]) val[u] = ld_stream128(pool + poff[u]); }
                else val[u] = ld_stream128(fbase + (size_t)ci * 16);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            unsigned ci = base + u * kThreads;
            if (!live[u]) continue;
            if (EXTRACT) st_stream128(fbase + (size_t)ci * 16, val[u]);         // hole => zeros
            else if (!hole[u]) st_stream128(pool + poff[u], val[u]);            // hole => skip
        }
    }

    if (a.dtype == DRK_INT8 && flat_scales) {
        uint8_t *sbase = flat_scales + ((size_t)(layer * 2 + kv) * num_tokens + t0) * a.KVH * 2;
        for (unsigned i = threadIdx.x; i < (unsigned)ntok * a.KVH; i += kThreads) {
            unsigned t = i / a.KVH, h = i - t * a.KVH;
            unsigned gt = (unsigned)(start_token + t0) + t;
            unsigned lb = dv(gt, bs_div);
            int blk = table[lb];
            bool ok = blk >= 0 && blk < a.NB;
            size_t so = ok ? scale_off(a, layer, blk, kv, h, gt - lb * bs_div.d) : 0;
            if (EXTRACT) *(uint16_t *)(sbase + (size_t)i * 2) = ok ? *(const uint16_t *)(pool + so) : (uint16_t)0;
            else if (ok) *(uint16_t *)(pool + so) = *(const uint16_t *)(sbase + (size_t)i * 2);
        }
    }
}

// ------------------------------------------------------------------------
// append
// grid = (token groups, layer_count, 2); source [layer][token][head][dim] of
// 16-bit elements, one 16-byte chunk (8 elements) per thread.
// "token" i is position pos_start+i of one table (batch mode, d_pos == NULL) or
// the single new token of branch i at d_pos[i] + pos_start with table row i (branch mode; pos_start is 0 there,
// or -1 when the array holds lengths that already count the token).
// QMODE 0: copy.  1: int8 codes + fp16 scale per row.  2: fp8 e4m3 codes.
// ------------------------------------------------------------------------
template <int QMODE>
__global__ __launch_bounds__(kThreads) void append_kernel(
    Lay a, uint8_t *__restrict__ pool, const int32_t *__restrict__ tables, int table_stride,
    const int32_t *__restrict__ d_pos, int pos_start, int ntokens, int layer0,
    const uint8_t *__restrict__ src_k, const uint8_t *__restrict__ src_v, int src_dtype, int tpg, Div tok_div,
    Div row_div, Div bs_div)
{
    const int tg = blockIdx.x, li = blockIdx.y, kv = blockIdx.z;
    const int layer = layer0 + li;
    const int t0 = tg * tpg;
    const int ntok = min(tpg, ntokens - t0);
    const unsigned rc = row_div.d;                       // D/8 chunks per source row
    const unsigned items = (unsigned)ntok * tok_div.d;   // tok_div.d = KVH*rc
    const size_t src_row = (size_t)a.D * 2;
    const uint8_t *sbase = (kv ? src_v : src_k) + ((size_t)li * ntokens + t0) * a.KVH * src_row;
    const unsigned rounds = (items + kThreads - 1) / kThreads;

    // U rounds at a time: all their source loads are issued before the first is consumed
    constexpr int U = QMODE == 0 ? 2 : 4;
    for (unsigned rnd0 = 0; rnd0 < rounds; rnd0 += U) {
        uint4 val[U];
        size_t poff[U], soff[U];
        unsigned cc[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const unsigned ci = (rnd0 + u) * kThreads + threadIdx.x;
            val[u] = make_uint4(0, 0, 0, 0);
            poff[u] = soff[u] = 0;
            cc[u] = 0;
            ok[u] = false;
            if (ci < items) {
                unsigned t = dv(ci, tok_div), r = ci - t * tok_div.d;
                unsigned h = dv(r, row_div);
                cc[u] = r - h * rc;
                int ti = t0 + (int)t;
                int pos = d_pos ? d_pos[ti] + pos_start : pos_start + ti;
                const int32_t *tab = tables + (size_t)(d_pos ? ti : 0) * table_stride;
                if (pos >= 0) {
                    unsigned lb = dv((unsigned)pos, bs_div);
                    int blk = tab[lb];
                    if (blk >= 0 && blk < a.NB) {
                        ok[u] = true;
                        int p = pos - lb * bs_div.d;
                        poff[u] = row_off(a, layer, blk, kv, h, p);
                        if (QMODE == 1) soff[u] = scale_off(a, layer, blk, kv, h, p);
                    }
                }
                val[u] = ld_stream128(sbase + (size_t)ci * 16);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            store_page_chunk<QMODE>(pool, poff[u], soff[u], cc[u], rc, val[u], src_dtype, ok[u]);
        }
    }
}

// The quantising append for rows of at least two chunks: one thread takes 32 source bytes (16 elements) and stores
// their 16 codes with one 16-byte store -- half the index arithmetic, scale arithmetic and lane exchanges per byte
// of the one-chunk form above, which is bound by instruction issue and not by memory.  Same grid and arguments;
// row_div divides by the row's 32-byte items (head_dim / 16), tok_div by KVH times that.
template <int QMODE>
__global__ __launch_bounds__(kThreads) void append_quant_kernel(
    Lay a, uint8_t *__restrict__ pool, const int32_t *__restrict__ tables, int table_stride,
    const int32_t *__restrict__ d_pos, int pos_start, int ntokens, int layer0,
    const uint8_t *__restrict__ src_k, const uint8_t *__restrict__ src_v, int src_dtype, int tpg, Div tok_div,
    Div row_div, Div bs_div)
{
    static_assert(QMODE == 1 || QMODE == 2, "int8 or fp8");
    const int tg = blockIdx.x, li = blockIdx.y, kv = blockIdx.z;
    const int layer = layer0 + li;
    const int t0 = tg * tpg;
    const int ntok = min(tpg, ntokens - t0);
    const unsigned rc2 = row_div.d;                      // 32-byte items per source row
    const unsigned items = (unsigned)ntok * tok_div.d;
    const uint8_t *sbase = (kv ? src_v : src_k) + ((size_t)li * ntokens + t0) * a.KVH * ((size_t)a.D * 2);
    const unsigned rounds = (items + kThreads - 1) / kThreads;

    constexpr int U = 2;                                 // four 16-byte loads in flight per thread
    for (unsigned rnd0 = 0; rnd0 < rounds; rnd0 += U) {
        uint4 va[U], vb[U];
        size_t poff[U], soff[U];
        bool ok[U], first[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const unsigned ci = (rnd0 + u) * kThreads + threadIdx.x;
            va[u] = vb[u] = make_uint4(0, 0, 0, 0);
            poff[u] = soff[u] = 0;
            ok[u] = first[u] = false;
            if (ci < items) {
                const unsigned t = dv(ci, tok_div), r = ci - t * tok_div.d;
                const unsigned h = dv(r, row_div), c2 = r - h * rc2;
                const int ti = t0 + (int)t;
                const int pos = d_pos ? d_pos[ti] + pos_start : pos_start + ti;
                const int32_t *tab = tables + (size_t)(d_pos ? ti : 0) * table_stride;
                if (pos >= 0) {
                    const unsigned lb = dv((unsigned)pos, bs_div);
                    const int blk = tab[lb];
                    if (blk >= 0 && blk < a.NB) {
                        ok[u] = true;
                        first[u] = c2 == 0;
                        const int p = pos - lb * bs_div.d;
                        poff[u] = row_off(a, layer, blk, kv, h, p) + (size_t)c2 * 16;
                        if (QMODE == 1) soff[u] = scale_off(a, layer, blk, kv, h, p);
                    }
                }
                const uint8_t *s = sbase + (size_t)ci * 32;
                va[u] = ld_stream128(s);
                vb[u] = ld_stream128(s + 16);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            float x[16];
            unpack8(va[u], src_dtype, x);
            unpack8(vb[u], src_dtype, x + 8);
            uint4 codes;
            if (QMODE == 1) {
                float amax = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; i++) amax = fmaxf(amax, fabsf(x[i]));
                if (rc2 == 8) {                               // head_dim 128: a row is half a DPP row
                    amax = fmaxf(amax, codec_dpp<0xB1>(amax));
                    amax = fmaxf(amax, codec_dpp<0x4E>(amax));
                    amax = fmaxf(amax, codec_dpp<0x141>(amax));
                } else {
                    for (unsigned off = rc2 >> 1; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, (int)off));
                }
                uint16_t sh;
                float rcp;
                int8_row_scale<false>(amax, sh, rcp);
                int8_codes8(x, rcp, codes.x, codes.y);
                int8_codes8(x + 8, rcp, codes.z, codes.w);
                if (first[u]) *(uint16_t *)(pool + soff[u]) = sh;
            } else {
                fp8_codes8(x, codes.x, codes.y);
                fp8_codes8(x + 8, codes.z, codes.w);
            }
            if (ok[u]) st_stream128(pool + poff[u], codes);
        }
    }
}

// Every input the int8 scale arithmetic can meet, through both of its forms (see int8_row_scale): thread i takes
// the 16-bit pattern i as a bf16 and as an fp16 magnitude (scale bits must agree) and as an fp16 scale
// (reciprocal bits must agree).  *mismatches counts the disagreements.
__global__ void int8_scale_math_check_kernel(unsigned *__restrict__ mismatches)
{
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= 65536u) return;
    unsigned bad = 0;
    for (int fmt = 0; fmt < 2; fmt++) {
        const float x = fabsf(elem16_to_f((uint16_t)i, fmt == 0 ? DRK_BF16 : DRK_F16));
        if (x != x) continue;                                 // a row maximum is never NaN (fmaxf drops it)
        uint16_t s0, s1;
        float r0, r1;
        int8_row_scale<true>(x, s0, r0);
        int8_row_scale<false>(x, s1, r1);
        bad += (s0 != s1) || (__float_as_uint(r0) != __float_as_uint(r1));
    }
    if (bad) atomicAdd(mismatches, bad);
}

// ------------------------------------------------------------------------
// copy-on-write: every layer of block src -> block dst
// grid = (chunk groups, L, pairs)
// ------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void copy_blocks_kernel(Lay a, uint8_t *__restrict__ pool,
                                                               const int32_t *__restrict__ pairs)
{
    const int layer = blockIdx.y;
    const int src = pairs[2 * blockIdx.z], dst = pairs[2 * blockIdx.z + 1];
    if (src < 0 || dst < 0 || src >= a.NB || dst >= a.NB || src == dst) return;
    const uint4 *s = (const uint4 *)(pool + lay_block_base(a, layer, src));
    uint4 *d = (uint4 *)(pool + lay_block_base(a, layer, dst));
    const unsigned n = a.block_stride / 16;
    constexpr int U = 4;
    for (unsigned base = blockIdx.x * kThreads * U + threadIdx.x; base < n; base += gridDim.x * kThreads * U) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            unsigned i = base + u * kThreads;
            if (i < n) v[u] = s[i];
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            unsigned i = base + u * kThreads;
            if (i < n) d[i] = v[u];
        }
    }
}

// importance_update_kernel, importance_scorer.cu:27-36: score*decay + new.  The
// reference is built by nvcc, which contracts that expression into one fused
// multiply-add; the fused form is written out here so the rounding is fixed.
__global__ void importance_update_kernel(float *__restrict__ scores, const float *__restrict__ new_scores,
                                         int n, float decay)
{
    int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < n) scores[b] = __builtin_fmaf(scores[b], decay, new_scores[b]);
}

// The same fold for a range whose new scores are spent with it: they are cleared in the same pass
// (a fill kernel of its own would be one more launch; a memset node may not be recorded into a graph).
__global__ void importance_fold_clear_kernel(float *__restrict__ scores, float *__restrict__ new_scores, int n, float decay)
{
    int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < n) {
        scores[b] = __builtin_fmaf(scores[b], decay, new_scores[b]);
        new_scores[b] = 0.0f;
    }
}

static int check_src_dtype(int d)
{
    if (d != DRK_F16 && d != DRK_BF16) return fail(DRK_ERR_INVALID, "src_dtype must be F16 or BF16");
    return DRK_OK;
}

int launch_append(const drk_kv_layout *g, void *pool, const int32_t *tables, int table_stride,
                  const int32_t *d_pos, int pos_start, int ntokens, int layer, int layer_count,
                  const void *src_k, const void *src_v, int src_dtype, void *stream)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    if ((rc = check_src_dtype(src_dtype))) return rc;
    if (!pool || !tables || !src_k || !src_v) return fail(DRK_ERR_INVALID, "append: NULL pointer");
    if (layer < 0 || layer_count < 1 || layer + layer_count > a.L)
        return fail(DRK_ERR_INVALID, "append: layers [%d,%d) outside [0,%d)", layer, layer + layer_count, a.L);
    if (layer_count > 65535) return fail(DRK_ERR_INVALID, "append: layer_count > 65535");
    if (ntokens < 0 || (pos_start < 0 && !(d_pos && pos_start == -1)))
        return fail(DRK_ERR_INVALID, "append: negative token count or position");
    if (ntokens == 0) return DRK_OK;
    if ((a.dtype == DRK_F16 || a.dtype == DRK_BF16) && src_dtype != a.dtype)
        return fail(DRK_ERR_INVALID, "append: src_dtype %d differs from the pool's %d", src_dtype, a.dtype);
    unsigned rowc = a.D / 8;
    if (a.dtype == DRK_INT8 || a.dtype == DRK_FP8_E4M3) {
        if (ilog2_exact(rowc) < 0 || rowc > 64)
            return fail(DRK_ERR_UNSUPPORTED, "append: quantising pools need head_dim in {8..512} power of two, got %d", a.D);
    }
    Div tok_div = mk_div((unsigned)a.KVH * rowc), row_div = mk_div(rowc), bs_div = mk_div((unsigned)a.bs);
    const bool quant = a.dtype == DRK_INT8 || a.dtype == DRK_FP8_E4M3;
    const int tpg = tokens_per_group((unsigned)a.KVH * rowc, quant ? g_quant_chunks : g_copy_chunks);
    dim3 grid((ntokens + tpg - 1) / tpg, layer_count, 2);
    hipStream_t s = (hipStream_t)stream;
    if (quant && rowc >= 2 && g_quant_pairs) {           // 32 source bytes per thread
        const Div tok2 = mk_div((unsigned)a.KVH * (rowc / 2)), row2 = mk_div(rowc / 2);
#define GO2(Q)                                                                                          \
    hipLaunchKernelGGL(append_quant_kernel<Q>, grid, dim3(kThreads), 0, s, a, (uint8_t *)pool, tables,  \
                       table_stride, d_pos, pos_start, ntokens, layer, (const uint8_t *)src_k,          \
                       (const uint8_t *)src_v, src_dtype, tpg, tok2, row2, bs_div)
        if (a.dtype == DRK_INT8) GO2(1);
        else GO2(2);
#undef GO2
        DRK_LAUNCH_CHECK("append_quant_kernel");
        return DRK_OK;
    }
#define GO(Q)                                                                                       \
    hipLaunchKernelGGL(append_kernel<Q>, grid, dim3(kThreads), 0, s, a, (uint8_t *)pool, tables,    \
                       table_stride, d_pos, pos_start, ntokens, layer, (const uint8_t *)src_k,      \
                       (const uint8_t *)src_v, src_dtype, tpg, tok_div, row_div, bs_div)
    if (a.dtype == DRK_INT8) GO(1);
    else if (a.dtype == DRK_FP8_E4M3) GO(2);
    else GO(0);
#undef GO
    DRK_LAUNCH_CHECK("append_kernel");
    return DRK_OK;
}

static int launch_flat(bool extract, const drk_kv_layout *g, void *pool, void *flat, void *flat_scales,
                       const int32_t *table, int start_token, int num_tokens, int num_layers, void *stream)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    if (!pool || !flat || !table) return fail(DRK_ERR_INVALID, "extract/inject: NULL pointer");
    if (num_layers < 0 || num_layers > a.L) return fail(DRK_ERR_INVALID, "extract/inject: num_layers %d outside [0,%d]", num_layers, a.L);
    if (start_token < 0 || num_tokens < 0) return fail(DRK_ERR_INVALID, "extract/inject: negative token range");
    if (num_tokens == 0 || num_layers == 0) return DRK_OK;
    if (a.row_bytes % 16) return fail(DRK_ERR_UNSUPPORTED, "extract/inject: row of %u bytes is not a multiple of 16", a.row_bytes);
    if (num_layers * 2 > 65535) return fail(DRK_ERR_INVALID, "extract/inject: too many layers");
    unsigned rowc = a.row_bytes / 16;
    Div tok_div = mk_div((unsigned)a.KVH * rowc), row_div = mk_div(rowc), bs_div = mk_div((unsigned)a.bs);
    const int tpg = tokens_per_group((unsigned)a.KVH * rowc, g_flat_chunks);
    dim3 grid((num_tokens + tpg - 1) / tpg, num_layers * 2);
    hipStream_t s = (hipStream_t)stream;
    if (extract)
        hipLaunchKernelGGL(flat_copy_kernel<true>, grid, dim3(kThreads), 0, s, a, (uint8_t *)pool, (uint8_t *)flat,
                           (uint8_t *)flat_scales, table, start_token, num_tokens, tpg, tok_div, row_div, bs_div);
    else
        hipLaunchKernelGGL(flat_copy_kernel<false>, grid, dim3(kThreads), 0, s, a, (uint8_t *)pool, (uint8_t *)flat,
                           (uint8_t *)flat_scales, table, start_token, num_tokens, tpg, tok_div, row_div, bs_div);
    DRK_LAUNCH_CHECK("flat_copy_kernel");
    return DRK_OK;
}

} // namespace drk

using namespace drk;

extern "C" {

int drk_debug_check_int8_scale_math(unsigned *d_mismatches, void *stream)
{
    if (!d_mismatches) return fail(DRK_ERR_INVALID, "check_int8_scale_math: NULL counter");
    hipLaunchKernelGGL(int8_scale_math_check_kernel, dim3(256), dim3(256), 0, (hipStream_t)stream, d_mismatches);
    DRK_LAUNCH_CHECK("int8_scale_math_check_kernel");
    return DRK_OK;
}

void drk_debug_set_quant_append_pairs(int on) { g_quant_pairs = on ? 1 : 0; }

void drk_debug_set_append_chunks(int copy_chunks, int flat_chunks, int quant_chunks)
{
    g_copy_chunks = copy_chunks > 0 ? copy_chunks : 256;
    g_flat_chunks = flat_chunks > 0 ? flat_chunks : 512;
    g_quant_chunks = quant_chunks > 0 ? quant_chunks : 1024;
}

int drk_kv_append_token(const drk_kv_layout *g, void *pool, const int32_t *d_block_table, int layer,
                        const int32_t *d_pos, const void *src_k, const void *src_v, int src_dtype,
                        void *stream)
{
    if (!d_pos) return fail(DRK_ERR_INVALID, "append_token: d_pos is NULL");
    return launch_append(g, pool, d_block_table, 0, d_pos, 0, 1, layer, 1, src_k, src_v, src_dtype, stream);
}

int drk_kv_append_batch(const drk_kv_layout *g, void *pool, const int32_t *d_block_table, int layer,
                        int layer_count, int pos_start, int M, const void *src_k, const void *src_v,
                        int src_dtype, void *stream)
{
    return launch_append(g, pool, d_block_table, 0, nullptr, pos_start, M, layer, layer_count, src_k, src_v,
                         src_dtype, stream);
}

int drk_kv_append_branches(const drk_kv_layout *g, void *pool, const int32_t *d_tables, int table_stride,
                           const int32_t *d_pos, int B, int layer, int layer_count, const void *src_k,
                           const void *src_v, int src_dtype, void *stream)
{
    if (!d_pos) return fail(DRK_ERR_INVALID, "append_branches: d_pos is NULL");
    if (table_stride < 0) return fail(DRK_ERR_INVALID, "append_branches: negative table_stride");
    return launch_append(g, pool, d_tables, table_stride, d_pos, 0, B, layer, layer_count, src_k, src_v,
                         src_dtype, stream);
}

int drk_kv_extract(const drk_kv_layout *g, void *d_dst, void *d_dst_scales, const void *pool,
                   const int32_t *d_block_table, int start_token, int num_tokens, int num_layers,
                   void *stream)
{
    return launch_flat(true, g, (void *)pool, d_dst, d_dst_scales, d_block_table, start_token, num_tokens,
                       num_layers, stream);
}

int drk_kv_inject(const drk_kv_layout *g, void *pool, const void *d_src, const void *d_src_scales,
                  const int32_t *d_block_table, int start_token, int num_tokens, int num_layers,
                  void *stream)
{
    return launch_flat(false, g, pool, (void *)d_src, (void *)d_src_scales, d_block_table, start_token,
                       num_tokens, num_layers, stream);
}

int drk_kv_copy_blocks(const drk_kv_layout *g, void *pool, const int32_t *d_pairs, int n, void *stream)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    if (!pool || (!d_pairs && n > 0)) return fail(DRK_ERR_INVALID, "copy_blocks: NULL pointer");
    if (n < 0) return fail(DRK_ERR_INVALID, "copy_blocks: negative pair count");
    if (a.block_stride % 16) return fail(DRK_ERR_UNSUPPORTED, "copy_blocks: block of %u bytes is not a multiple of 16", a.block_stride);
    if (a.L > 65535) return fail(DRK_ERR_INVALID, "copy_blocks: too many layers");
    unsigned chunks = a.block_stride / 16;
    unsigned gx = (chunks + kThreads * 4 - 1) / (kThreads * 4);
    for (int done = 0; done < n; done += 65535) {
        int cnt = n - done < 65535 ? n - done : 65535;
        hipLaunchKernelGGL(copy_blocks_kernel, dim3(gx, a.L, cnt), dim3(kThreads), 0, (hipStream_t)stream, a,
                           (uint8_t *)pool, d_pairs + 2 * (size_t)done);
        DRK_LAUNCH_CHECK("copy_blocks_kernel");
    }
    return DRK_OK;
}

int drk_importance_update(float *d_scores, const float *d_new_scores, int n, float decay, void *stream)
{
    if (n <= 0) return DRK_OK;
    if (!d_scores || !d_new_scores) return fail(DRK_ERR_INVALID, "importance_update: NULL pointer");
    hipLaunchKernelGGL(importance_update_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       d_scores, d_new_scores, n, decay);
    DRK_LAUNCH_CHECK("importance_update_kernel");
    return DRK_OK;
}

int drk_importance_fold_clear(float *d_scores, float *d_new_scores, int n, float decay, void *stream)
{
    if (n <= 0) return DRK_OK;
    if (!d_scores || !d_new_scores) return fail(DRK_ERR_INVALID, "importance_fold_clear: NULL pointer");
    hipLaunchKernelGGL(importance_fold_clear_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       d_scores, d_new_scores, n, decay);
    DRK_LAUNCH_CHECK("importance_fold_clear_kernel");
    return DRK_OK;
}

} // extern "C"
