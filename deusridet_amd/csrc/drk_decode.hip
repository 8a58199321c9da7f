// drk_decode.hip -- paged GQA decode attention for gfx950, split-K over the
// context with an (o, m, l) merge.
//
// Work decomposition: one workgroup per (split, kv head, branch); the query
// heads that share the kv head are handled by the same workgroup so every K/V
// byte is fetched from HBM once (the reference launches one block per query head
// and re-reads the kv head's pages QH/KVH times, paged_attention.cu:179-282).
//
// The production kernel is decode_stream_kernel (drk_decode_stream.hip: head_dim 128 or
// 256, up to 16 query heads per kv head, every storage type).  Two more kernels produce
// partials here, for everything else and as cross-checks:
//   decode_tiled_kernel    head_dim 128, 16-bit K/V, 4 query heads per kv head:
//                          64-token K tiles staged in LDS (row-padded so that
//                          lane = token reads are bank-conflict free), Q held in
//                          SGPRs, QK^T by v_dot2 with no cross-lane reduction,
//                          tile softmax by wave reductions, P broadcast through
//                          LDS, V consumed straight from 128-bit global loads.
//   decode_portable_kernel any head_dim multiple of 64 (<= 512), any group size
//                          <= 16, any storage type (dequantises int8 / fp8);
//                          token-at-a-time, one wave per query head.
// decode_merge_kernel folds the partials (max-rescaled, as the reference's only
// split-K precedent does: asr_ops_attn.cu:84-108).
//
// Scores are kept in the log2 domain: s = (q.k) * scale * log2(e), weights are
// exp2(s - m).  The result depends on the logical token order only, never on
// which physical block holds a page.
#include "drk_common.hpp"

#include <math.h>

#include <mutex>

// Scratch of drk_paged_decode_attention_branches_static: the split-K partials of the one
// entry point that takes no workspace.  Every GPU the library runs on holds its own copy
// until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels are given the address that call returned, never the name.
static __device__ __align__(256) unsigned char scratch[DRK_STATIC_SCRATCH_BYTES];

namespace drk {

int g_force_portable = 0;                    // diagnostic, shared with the prefill unit
static int g_decode_kernel = 0;               // diagnostic: 0 auto, 2 fixed-split tiled kernel, 3 stream kernel
int g_skip_merge = 0;                         // measurement aid: leave the partials unmerged (drk_debug_set_skip_merge)
static int g_lds_pad = 0;                     // diagnostic: extra dynamic LDS per workgroup (caps occupancy)

constexpr int kTile = 64;            // tokens per tile
constexpr int kKRow = 272;           // LDS bytes per staged K row: 256 + 16 pad
constexpr float kLog2e = 1.4426950408889634f;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

template <int DT>
__device__ __forceinline__ float dot2acc(uint32_t k, uint32_t q, float acc)
{
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (DT == DRK_BF16)
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, k), __builtin_bit_cast(bf16x2_t, q), acc, false);
    else
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, k), __builtin_bit_cast(f16x2_t, q), acc, false);
#else
    (void)k; (void)q;
    return acc;
#endif
}

template <int DT>
__device__ __forceinline__ void unpack2(uint32_t w, float &lo, float &hi)
{
    if constexpr (DT == DRK_BF16) {
        lo = bf16_lo(w);
        hi = bf16_hi(w);
    } else {
        lo = f16_bits_to_f((uint16_t)(w & 0xffffu));
        hi = f16_bits_to_f((uint16_t)(w >> 16));
    }
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
    return v;
}
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

__device__ __forceinline__ float fast_exp2(float x)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_exp2f(x);
#else
    return exp2f(x);
#endif
}

// ------------------------------------------------------------------------
// tiled kernel: D = 128, 16-bit storage, 4 query heads per kv head
// block = 256 threads = 4 waves; wave w owns query head kvh*4 + w in the QK^T /
// softmax phase and the 16-token group w of every tile in the load / PV phase.
// ------------------------------------------------------------------------
struct Group4 {          // one wave's 16-token group: 4 x (64 lanes x 16 B) = 4 KiB
    uint4 r0, r1, r2, r3;
};

__device__ __forceinline__ Group4 load_group(const uint8_t *__restrict__ base, bool valid, size_t off, int lane)
{
    Group4 g;
    g.r0 = g.r1 = g.r2 = g.r3 = make_uint4(0, 0, 0, 0);
    if (valid) {
        const uint8_t *p = base + off + (size_t)lane * 16;
        g.r0 = ld_stream128(p);
        g.r1 = ld_stream128(p + 1024);
        g.r2 = ld_stream128(p + 2048);
        g.r3 = ld_stream128(p + 3072);
    }
    return g;
}

struct TiledArgs {
    const uint8_t *pool_layer;     // pool + layer * layer_stride
    const int32_t *tables;
    const int32_t *seq_lens;
    const uint8_t *q;
    float *part_o, *part_m, *part_l;
    int table_stride, seq_len_host, causal_base;
    int split_tokens, S, QH, NB, bs, bs_shift;
    unsigned head_stride, kv_plane, block_stride;
    float scale_log2e;
};

template <int DT>
__device__ __forceinline__ void pv_rows(float (&o)[4][8], const uint4 vv, const float4 pp)
{
    float x[8];
    unpack2<DT>(vv.x, x[0], x[1]);
    unpack2<DT>(vv.y, x[2], x[3]);
    unpack2<DT>(vv.z, x[4], x[5]);
    unpack2<DT>(vv.w, x[6], x[7]);
#pragma unroll
    for (int e = 0; e < 8; e++) {
        o[0][e] = fmaf(pp.x, x[e], o[0][e]);
        o[1][e] = fmaf(pp.y, x[e], o[1][e]);
        o[2][e] = fmaf(pp.z, x[e], o[2][e]);
        o[3][e] = fmaf(pp.w, x[e], o[3][e]);
    }
}

template <int DT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void decode_tiled_kernel(TiledArgs A)
{
    __shared__ __align__(16) uint8_t k_lds[2][kTile * kKRow];
    __shared__ __align__(16) float p_lds[2][kTile * 4];
    __shared__ __align__(16) float alpha_lds[2][4];
    __shared__ int valid_lds[2][4];

    const int s = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const int seq_len = A.seq_lens ? A.seq_lens[b] : (A.causal_base >= 0 ? A.causal_base + b + 1 : A.seq_len_host);
    const int t0 = s * A.split_tokens;
    if (t0 >= seq_len) return;
    const int t1 = min(t0 + A.split_tokens, seq_len);
    const int ntiles = (t1 - t0 + kTile - 1) / kTile;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int lrow = lane >> 4, lchunk = lane & 15;
    const int32_t *tab = A.tables + (size_t)b * A.table_stride;
    const int h = kvh * 4 + w;

    // the wave's query head, 64 packed pairs, uniform -> scalar registers
    const uint32_t *qp = (const uint32_t *)(A.q + ((size_t)b * A.QH + h) * 256);
    uint32_t qs[64];
#pragma unroll
    for (int i = 0; i < 64; i++) qs[i] = qp[i];

    const uint8_t *kbase = A.pool_layer + (size_t)kvh * A.head_stride;

    // this wave's 16-token group of a tile: valid flag + byte offset of its K rows
    auto lookup = [&](int tile, bool &valid) -> size_t {
        int tg = t0 + tile * kTile + w * 16;
        valid = false;
        if (tg >= t1) return 0;
        int lb = A.bs_shift >= 0 ? (tg >> A.bs_shift) : (tg / A.bs);
        int blk = tab[lb];
        if (blk < 0 || blk >= A.NB) return 0;
        valid = true;
        return (size_t)blk * A.block_stride + (size_t)(tg - lb * A.bs) * 256;
    };

    float o[4][8];
#pragma unroll
    for (int hh = 0; hh < 4; hh++)
#pragma unroll
        for (int e = 0; e < 8; e++) o[hh][e] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    bool cur_valid, nxt_valid = false;
    size_t cur_off = lookup(0, cur_valid), nxt_off = 0;
    Group4 kreg = load_group(kbase, cur_valid, cur_off, lane);
    Group4 vreg = load_group(kbase + A.kv_plane, cur_valid, cur_off, lane);
    if (ntiles > 1) nxt_off = lookup(1, nxt_valid);

    for (int i = 0; i < ntiles; i++) {
        const int buf = i & 1;
        // ---- A: stage this tile's K rows, start the next tile's K loads ----
        {
            uint8_t *dst = &k_lds[buf][(w * 16 + lrow) * kKRow + lchunk * 16];
            *(uint4 *)(dst) = kreg.r0;
            *(uint4 *)(dst + 4 * kKRow) = kreg.r1;
            *(uint4 *)(dst + 8 * kKRow) = kreg.r2;
            *(uint4 *)(dst + 12 * kKRow) = kreg.r3;
            if (lane == 0) valid_lds[buf][w] = cur_valid ? 1 : 0;
        }
        if (i + 1 < ntiles) kreg = load_group(kbase, nxt_valid, nxt_off, lane);
        __syncthreads();

        // ---- B: scores of head w for the tile's 64 tokens, tile softmax ----
        {
            const uint8_t *krow = &k_lds[buf][lane * kKRow];
            // 16 chunks of 8 dims, read four at a time with the next four in
            // flight while the current four are multiplied
            float acc = 0.0f;
            uint4 ka[4], kb[4];
#pragma unroll
            for (int c = 0; c < 4; c++) ka[c] = *(const uint4 *)(krow + c * 16);
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                if (g4 < 3) {
#pragma unroll
                    for (int c = 0; c < 4; c++) kb[c] = *(const uint4 *)(krow + ((g4 + 1) * 4 + c) * 16);
                }
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const int qi = (g4 * 4 + c) * 4;
                    acc = dot2acc<DT>(ka[c].x, qs[qi + 0], acc);
                    acc = dot2acc<DT>(ka[c].y, qs[qi + 1], acc);
                    acc = dot2acc<DT>(ka[c].z, qs[qi + 2], acc);
                    acc = dot2acc<DT>(ka[c].w, qs[qi + 3], acc);
                }
                asm volatile("" : "+v"(acc) :: "memory");   // keep at most two groups of LDS reads in flight
#pragma unroll
                for (int c = 0; c < 4; c++) ka[c] = kb[c];
            }
            const int tok = t0 + i * kTile + lane;
            const bool live = tok < t1 && valid_lds[buf][lane >> 4] != 0;
            const float sc = live ? acc * A.scale_log2e : -INFINITY;
            const float m_new = fmaxf(m_run, wave_max(sc));
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float p = fast_exp2(sc - m_use);
            const float alpha = fast_exp2(m_run - m_use);
            l_run = l_run * alpha + wave_sum(p);
            m_run = m_new;
            p_lds[buf][lane * 4 + w] = p;
            if (lane == 0) alpha_lds[buf][w] = alpha;
        }
        __syncthreads();

        // ---- C: o += P V over this wave's 16 tokens, all 4 heads ----
        {
            const float4 al = *(const float4 *)&alpha_lds[buf][0];
            if (al.x != 1.0f || al.y != 1.0f || al.z != 1.0f || al.w != 1.0f) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    o[0][e] *= al.x; o[1][e] *= al.y; o[2][e] *= al.z; o[3][e] *= al.w;
                }
            }
            const int r0 = w * 16 + lrow;                 // tile row of vreg.r0; r1..r3 are +4, +8, +12
            if ((t0 + (i + 1) * kTile) > t1) {            // rows past the end may hold anything
                const int lim = t1 - t0 - i * kTile;
                const uint4 z = make_uint4(0, 0, 0, 0);
                if (r0 >= lim) vreg.r0 = z;
                if (r0 + 4 >= lim) vreg.r1 = z;
                if (r0 + 8 >= lim) vreg.r2 = z;
                if (r0 + 12 >= lim) vreg.r3 = z;
            }
            const float *pl = &p_lds[buf][r0 * 4];
            pv_rows<DT>(o, vreg.r0, *(const float4 *)(pl));
            pv_rows<DT>(o, vreg.r1, *(const float4 *)(pl + 16));
            pv_rows<DT>(o, vreg.r2, *(const float4 *)(pl + 32));
            pv_rows<DT>(o, vreg.r3, *(const float4 *)(pl + 48));
        }
        if (i + 1 < ntiles) {
            vreg = load_group(kbase + A.kv_plane, nxt_valid, nxt_off, lane);
            cur_valid = nxt_valid;
            if (i + 2 < ntiles) nxt_off = lookup(i + 2, nxt_valid);
        }
    }

    // ---- epilogue: sum the 16 partial accumulators (4 lane rows x 4 waves) ----
#pragma unroll
    for (int hh = 0; hh < 4; hh++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float v = o[hh][e];
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            o[hh][e] = v;
        }
    __syncthreads();                               // everyone is done with k_lds / p_lds
    float *o_lds = (float *)&k_lds[0][0];          // [wave][head][128] = 8 KiB
    if (lrow == 0) {
#pragma unroll
        for (int hh = 0; hh < 4; hh++) {
            float *dst = o_lds + (w * 4 + hh) * 128 + lchunk * 8;
            *(float4 *)dst = make_float4(o[hh][0], o[hh][1], o[hh][2], o[hh][3]);
            *(float4 *)(dst + 4) = make_float4(o[hh][4], o[hh][5], o[hh][6], o[hh][7]);
        }
    }
    __syncthreads();
    {
        const int d = lane * 2;
        float2 acc = make_float2(0.0f, 0.0f);
#pragma unroll
        for (int ww = 0; ww < 4; ww++) {
            float2 v = *(const float2 *)(o_lds + (ww * 4 + w) * 128 + d);
            acc.x += v.x;
            acc.y += v.y;
        }
        const size_t pi = ((size_t)b * A.QH + h) * A.S + s;
        *(float2 *)(A.part_o + pi * 128 + d) = acc;
        if (lane == 0) {
            A.part_m[pi] = m_run;
            A.part_l[pi] = l_run;
        }
    }
}

// ------------------------------------------------------------------------
// portable kernel: block = G waves (one per query head of the group); lane owns
// EPL = D/64 consecutive dims; token at a time with a wave all-reduce per dot.
// ------------------------------------------------------------------------
template <int DT, int EPL>
__device__ __forceinline__ void load_elems(const uint8_t *p, float scale, float *x)
{
    if constexpr (DT == DRK_F16 || DT == DRK_BF16) {
        uint16_t raw[EPL];
        if constexpr (EPL == 1) raw[0] = *(const uint16_t *)p;
        else if constexpr (EPL == 2) { uint32_t v = *(const uint32_t *)p; raw[0] = v & 0xffff; raw[1] = v >> 16; }
        else if constexpr (EPL == 4) { uint2 v = *(const uint2 *)p; raw[0] = v.x & 0xffff; raw[1] = v.x >> 16; raw[2] = v.y & 0xffff; raw[3] = v.y >> 16; }
        else { uint4 v = *(const uint4 *)p; const uint32_t wv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
               for (int i = 0; i < 4; i++) { raw[2 * i] = wv[i] & 0xffff; raw[2 * i + 1] = wv[i] >> 16; } }
#pragma unroll
        for (int e = 0; e < EPL; e++) x[e] = elem16_to_f(raw[e], DT);
    } else {
        uint8_t raw[EPL];
        if constexpr (EPL == 1) raw[0] = *p;
        else if constexpr (EPL == 2) { uint16_t v = *(const uint16_t *)p; raw[0] = v & 0xff; raw[1] = v >> 8; }
        else if constexpr (EPL == 4) { uint32_t v = *(const uint32_t *)p;
#pragma unroll
               for (int i = 0; i < 4; i++) raw[i] = (v >> (8 * i)) & 0xff; }
        else { uint2 v = *(const uint2 *)p;
#pragma unroll
               for (int i = 0; i < 4; i++) { raw[i] = (v.x >> (8 * i)) & 0xff; raw[4 + i] = (v.y >> (8 * i)) & 0xff; } }
#pragma unroll
        for (int e = 0; e < EPL; e++) {
            if constexpr (DT == DRK_INT8) x[e] = (float)(int8_t)raw[e] * scale;
            else {
#if defined(__HIP_DEVICE_COMPILE__)
                x[e] = __builtin_amdgcn_cvt_f32_fp8((int)raw[e], 0);
#else
                x[e] = 0.0f;
#endif
            }
        }
    }
}

template <int DT, int EPL>
__global__ void decode_portable_kernel(
    Lay a, const uint8_t *__restrict__ pool, const int32_t *__restrict__ tables, int table_stride,
    const int32_t *__restrict__ seq_lens, int seq_len_host, int causal_base, const uint8_t *__restrict__ q, int io_dtype,
    float scale_log2e, int split_tokens, int S, float *__restrict__ part_o, float *__restrict__ part_m,
    float *__restrict__ part_l, int layer)
{
    const int s = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const int seq_len = seq_lens ? seq_lens[b] : (causal_base >= 0 ? causal_base + b + 1 : seq_len_host);
    const int t0 = s * split_tokens;
    if (t0 >= seq_len) return;
    const int t1 = min(t0 + split_tokens, seq_len);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int G = a.QH / a.KVH;
    const int h = kvh * G + wave;
    const int d0 = lane * EPL;
    const int32_t *tab = tables + (size_t)b * table_stride;

    float qv[EPL], o[EPL];
    const uint16_t *qh = (const uint16_t *)q + ((size_t)b * a.QH + h) * a.D + d0;
#pragma unroll
    for (int e = 0; e < EPL; e++) { qv[e] = elem16_to_f(qh[e], io_dtype); o[e] = 0.0f; }
    float m_run = -INFINITY, l_run = 0.0f;

    for (int t = t0; t < t1; t++) {
        const int lb = t / a.bs, p = t - lb * a.bs;
        const int blk = tab[lb];
        if (blk < 0 || blk >= a.NB) continue;                    // hole: skipped
        const size_t base = lay_block_base(a, layer, blk);
        const size_t roff = base + (size_t)kvh * a.head_stride + (size_t)p * a.row_bytes + (size_t)d0 * a.E;
        float ks = 1.0f, vs = 1.0f;
        if constexpr (DT == DRK_INT8) {
            const size_t so = base + 2 * (size_t)a.kv_plane + ((size_t)kvh * a.bs + p) * 2;
            ks = f16_bits_to_f(*(const uint16_t *)(pool + so));
            vs = f16_bits_to_f(*(const uint16_t *)(pool + so + a.scale_plane));
        }
        float x[EPL];
        load_elems<DT, EPL>(pool + roff, ks, x);
        float dot = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; e++) dot = fmaf(qv[e], x[e], dot);
        dot = wave_sum(dot);
        const float sc = dot * scale_log2e;
        const float m_new = fmaxf(m_run, sc);
        const float alpha = fast_exp2(m_run - m_new);
        const float pw = fast_exp2(sc - m_new);
        load_elems<DT, EPL>(pool + roff + a.kv_plane, vs, x);
#pragma unroll
        for (int e = 0; e < EPL; e++) o[e] = fmaf(o[e], alpha, x[e] * pw);
        l_run = l_run * alpha + pw;
        m_run = m_new;
    }
    const size_t pi = ((size_t)b * a.QH + h) * S + s;
#pragma unroll
    for (int e = 0; e < EPL; e++) part_o[pi * a.D + d0 + e] = o[e];
    if (lane == 0) { part_m[pi] = m_run; part_l[pi] = l_run; }
}

// ------------------------------------------------------------------------
// merge: grid (QH, B), block = D threads
// out is written only when some token took part (the reference leaves `out`
// untouched when l == 0, paged_attention.cu:266).
// ------------------------------------------------------------------------
__global__ void decode_merge_kernel(const float *__restrict__ part_o, const float *__restrict__ part_m,
                                    const float *__restrict__ part_l, uint16_t *__restrict__ out,
                                    const int32_t *__restrict__ seq_lens, int seq_len_host, int causal_base,
                                    int split_tokens, int S, int D, int QH, int io_dtype)
{
    const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
    const int seq_len = seq_lens ? seq_lens[b] : (causal_base >= 0 ? causal_base + b + 1 : seq_len_host);
    const int ns = min((seq_len + split_tokens - 1) / split_tokens, S);
    const size_t base = ((size_t)b * QH + h) * S;
    float M = -INFINITY;
    for (int s = 0; s < ns; s++)
        if (part_l[base + s] > 0.0f) M = fmaxf(M, part_m[base + s]);
    float acc = 0.0f, L = 0.0f;
    for (int s = 0; s < ns; s++) {
        const float pl = part_l[base + s];
        if (!(pl > 0.0f)) continue;
        const float wgt = fast_exp2(part_m[base + s] - M);
        acc = fmaf(part_o[(base + s) * D + d], wgt, acc);
        L = fmaf(pl, wgt, L);
    }
    if (L > 0.0f) out[((size_t)b * QH + h) * D + d] = f_to_elem16(acc / L, io_dtype);
}

// ------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------
static int choose_split(const Lay &a, int B, int max_seq_len)
{
    // Longest run (a multiple of the tile, at most 4096 tokens) that still yields
    // two workgroups per CU of a 256-CU part: measured on MI355X, long runs win
    // because the per-workgroup prologue (table -> first K/V tile) and epilogue are
    // paid once, and a grid that is resident in a single round has no tail.
    const long want = 512;
    int split = 4096;
    while (split > kTile) {
        long wgs = (long)B * a.KVH * ((max_seq_len + split - 1) / split);
        if (wgs >= want) break;
        split >>= 1;
    }
    return split;
}

static size_t workspace_need(const Lay &a, int B, int max_seq_len, int split)
{
    size_t S = (size_t)(max_seq_len + split - 1) / split;
    if (S == 0) S = 1;
    return (size_t)B * a.QH * S * (a.D + 2) * sizeof(float);
}

int launch_decode(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *tables,
                         int table_stride, const int32_t *d_seq_lens, int seq_len_host, int causal_base,
                         int B, int max_seq_len, void *out, int layer, float scale, int io_dtype, int split_tokens,
                         void *workspace, size_t workspace_bytes, void *stream, const void *gate, size_t gate_stride,
                         DecodePlan plan)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    const bool plan_only = plan.ptr && plan.mode == 1;              // builds the unit descriptors: reads tables and lengths only
    if (!tables || (!plan_only && (!q || !pool || !out))) return fail(DRK_ERR_INVALID, "decode: NULL pointer");
    if (gate && (gate_stride < (size_t)a.D || (gate_stride % 8) || ((uintptr_t)gate % 16)))
        return fail(DRK_ERR_INVALID, "decode: gate rows must be 16-byte aligned and at least head_dim apart");
    if (io_dtype != DRK_F16 && io_dtype != DRK_BF16) return fail(DRK_ERR_INVALID, "decode: io_dtype must be F16 or BF16");
    if ((a.dtype == DRK_F16 || a.dtype == DRK_BF16) && io_dtype != a.dtype)
        return fail(DRK_ERR_INVALID, "decode: io_dtype %d differs from the pool's %d", io_dtype, a.dtype);
    if (layer < 0 || layer >= a.L) return fail(DRK_ERR_INVALID, "decode: layer %d outside [0,%d)", layer, a.L);
    if (B < 0 || max_seq_len < 0 || table_stride < 0) return fail(DRK_ERR_INVALID, "decode: negative size");
    if (B == 0 || max_seq_len == 0) return DRK_OK;
    if (B > 65535 || a.KVH > 65535) return fail(DRK_ERR_INVALID, "decode: more than 65535 branches or kv heads");
    const int G = a.QH / a.KVH;
    if (a.D % 64 || a.D > 512) return fail(DRK_ERR_UNSUPPORTED, "decode: head_dim %d (need a multiple of 64, <= 512)", a.D);
    if (G > 16) return fail(DRK_ERR_UNSUPPORTED, "decode: %d query heads per kv head (max 16)", G);
    if (split_tokens < 0 || (split_tokens % kTile)) return fail(DRK_ERR_INVALID, "decode: split_tokens must be a multiple of %d", kTile);
    // more branches than one launch of the tiled kernel takes: 64 at a time, one after the other
    // through the same workspace (the launches are ordered by the stream)
    if (B > 64 && d_seq_lens && !g_force_portable && g_decode_kernel != 2 && causal_base < 0 && stream_decode_supported(a, 64)) {
        if (plan.ptr) return fail(DRK_ERR_UNSUPPORTED, "decode: a plan covers at most 64 branches");
        const size_t row = (size_t)a.QH * a.D * 2;
        for (int b0 = 0; b0 < B; b0 += 64) {
            const int nb = B - b0 < 64 ? B - b0 : 64;
            rc = launch_decode(g, (const uint8_t *)q + b0 * row, pool, tables + (size_t)b0 * table_stride, table_stride,
                               d_seq_lens + b0, 0, -1, nb, max_seq_len, (uint8_t *)out + b0 * row, layer, scale, io_dtype,
                               split_tokens, workspace, workspace_bytes, stream,
                               gate ? (const uint8_t *)gate + (size_t)b0 * a.QH * gate_stride * 2 : nullptr, gate_stride);
            if (rc) return rc;
        }
        return DRK_OK;
    }
    const int split = split_tokens ? split_tokens : choose_split(a, B, max_seq_len);
    const int S = (max_seq_len + split - 1) / split;
    const bool use_stream = !g_force_portable && g_decode_kernel != 2 && causal_base < 0 && stream_decode_supported(a, B);
    // the persistent kernel keeps one descriptor per tile of a workgroup's run in LDS
    if (use_stream && split_tokens > kStreamMaxSplitTokens)
        return fail(DRK_ERR_INVALID, "decode: split_tokens %d exceeds %d (the tiled kernel's run length)", split_tokens,
                    kStreamMaxSplitTokens);
    if (plan.ptr && (!use_stream || split_tokens))
        return fail(DRK_ERR_UNSUPPORTED, "decode: plans are for the tiled kernel with its own split");
    const size_t need = use_stream ? stream_workspace_need(a, B, max_seq_len, split_tokens) : workspace_need(a, B, max_seq_len, split);
    if (plan_only)
        return launch_decode_stream(a, q, pool, tables, table_stride, d_seq_lens, seq_len_host, B, max_seq_len, out, layer,
                                    scale, io_dtype, split_tokens, workspace, false, (hipStream_t)stream, 0, nullptr, nullptr,
                                    nullptr, 0, nullptr, 0, nullptr, nullptr, 0, plan);
    if (!workspace || workspace_bytes < need)
        return fail(DRK_ERR_WORKSPACE, "decode: workspace of %zu bytes, need %zu", workspace_bytes, need);
    if (((uintptr_t)workspace) % 16) return fail(DRK_ERR_INVALID, "decode: workspace must be 16-byte aligned");

    float *part_o = (float *)workspace;
    float *part_m = part_o + (size_t)B * a.QH * S * a.D;
    float *part_l = part_m + (size_t)B * a.QH * S;
    const float sl2 = scale * kLog2e;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(S, a.KVH, B);

    const bool tiled = !g_force_portable && a.D == 128 && a.E == 2 && G == 4 && (a.bs % 16) == 0;
    if (use_stream) {
        rc = launch_decode_stream(a, q, pool, tables, table_stride, d_seq_lens, seq_len_host, B, max_seq_len, out, layer,
                                  scale, io_dtype, split_tokens, workspace, false, st, 0, nullptr, nullptr, nullptr, 0, nullptr,
                                  0, nullptr, nullptr, 0, plan);
        if (rc) return rc;
    } else if (tiled) {
        TiledArgs A;
        A.pool_layer = (const uint8_t *)pool + (size_t)layer * a.layer_stride;
        A.tables = tables; A.seq_lens = d_seq_lens; A.q = (const uint8_t *)q;
        A.part_o = part_o; A.part_m = part_m; A.part_l = part_l;
        A.table_stride = table_stride; A.seq_len_host = seq_len_host; A.causal_base = causal_base;
        A.split_tokens = split; A.S = S; A.QH = a.QH; A.NB = a.NB; A.bs = a.bs;
        A.bs_shift = ilog2_exact((unsigned)a.bs);
        A.head_stride = a.head_stride; A.kv_plane = a.kv_plane; A.block_stride = a.block_stride;
        A.scale_log2e = sl2;
        if (a.dtype == DRK_BF16) hipLaunchKernelGGL(decode_tiled_kernel<DRK_BF16>, grid, dim3(256), g_lds_pad, st, A);
        else hipLaunchKernelGGL(decode_tiled_kernel<DRK_F16>, grid, dim3(256), g_lds_pad, st, A);
        DRK_LAUNCH_CHECK("decode_tiled_kernel");
    } else {
        if ((a.dtype == DRK_INT8 || a.dtype == DRK_FP8_E4M3) && a.D / 64 > 8)
            return fail(DRK_ERR_UNSUPPORTED, "decode: head_dim %d", a.D);
        dim3 block(G * 64);
#define GO(DTV, EPLV)                                                                                         \
    hipLaunchKernelGGL((decode_portable_kernel<DTV, EPLV>), grid, block, 0, st, a, (const uint8_t *)pool, tables, \
                       table_stride, d_seq_lens, seq_len_host, causal_base, (const uint8_t *)q, io_dtype, sl2, split, S, \
                       part_o, part_m, part_l, layer)
#define GO_EPL(DTV)                                                                                           \
    switch (a.D / 64) {                                                                                       \
    case 1: GO(DTV, 1); break;                                                                                \
    case 2: GO(DTV, 2); break;                                                                                \
    case 4: GO(DTV, 4); break;                                                                                \
    case 8: GO(DTV, 8); break;                                                                                \
    default: return fail(DRK_ERR_UNSUPPORTED, "decode: head_dim %d (need 64, 128, 256 or 512)", a.D);         \
    }
        switch (a.dtype) {
        case DRK_F16: GO_EPL(DRK_F16); break;
        case DRK_BF16: GO_EPL(DRK_BF16); break;
        case DRK_INT8: GO_EPL(DRK_INT8); break;
        default: GO_EPL(DRK_FP8_E4M3); break;
        }
#undef GO_EPL
#undef GO
        DRK_LAUNCH_CHECK("decode_portable_kernel");
    }
    if (g_skip_merge) return DRK_OK;
    if (use_stream)
        return launch_decode_stream(a, q, pool, tables, table_stride, d_seq_lens, seq_len_host, B, max_seq_len, out, layer,
                                    scale, io_dtype, split_tokens, workspace, true, st, 0, nullptr, nullptr, nullptr, 0,
                                    gate, gate_stride);
    hipLaunchKernelGGL(decode_merge_kernel, dim3(a.QH, B), dim3(a.D), 0, st, part_o, part_m, part_l, (uint16_t *)out,
                       d_seq_lens, seq_len_host, causal_base, split, S, a.D, a.QH, io_dtype);
    DRK_LAUNCH_CHECK("decode_merge_kernel");
    if (gate) return launch_sigmoid_gate(out, gate, out, (size_t)B * a.QH, a.D, gate_stride, io_dtype, st);
    return DRK_OK;
}

// Shared-prefix decode: tokens [0, shared) live in the same physical pages for all
// B branches, so their K/V are streamed once for all B*QH query rows (matrix-core
// pass), the private tails go through the stream kernel, one merge folds both.
// exact: what a launch with this very prefix length uses (short tails keep few pieces); otherwise
// an upper bound for any prefix up to `shared`, which is what callers size their workspace by
static size_t shared_need(const Lay &a, int B, int max_seq_len, int shared, size_t *stream_part, bool exact)
{
    int ct, ns;
    shared_prefix_shape(a, B, shared, &ct, &ns);
    if (!exact && ns < g_shared_splits) ns = g_shared_splits;
    size_t sp = stream_workspace_need(a, B, max_seq_len, 0, exact ? shared / kTile : 0);
    sp = (sp + 255) & ~(size_t)255;
    if (stream_part) *stream_part = sp;
    return sp + (size_t)B * a.QH * ns * (a.D + 2) * sizeof(float);
}

static bool shared_path_ok(const Lay &a, int B, int shared)
{
    // the prefix pass is the MFMA prefill kernel in its shared mode (every shape the stream kernel takes)
    return !g_force_portable && stream_decode_supported(a, B) && shared >= kTile;   // the caller checks scale > 0
}

int launch_decode_shared(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *tables,
                         int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len, int shared_tokens,
                         void *out, int layer, float scale, int io_dtype, void *workspace, size_t workspace_bytes,
                         void *stream, const void *gate, size_t gate_stride)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    const int shared = shared_tokens > 0 ? (shared_tokens / kTile) * kTile : 0;
    if (!shared_path_ok(a, B, shared) || shared > max_seq_len || !(scale > 0.0f))
        return launch_decode(g, q, pool, tables, table_stride, d_seq_lens, 0, -1, B, max_seq_len, out, layer, scale,
                             io_dtype, 0, workspace, workspace_bytes, stream, gate, gate_stride);
    if (!q || !pool || !tables || !out || !d_seq_lens) return fail(DRK_ERR_INVALID, "decode: NULL pointer");
    if (io_dtype != DRK_F16 && io_dtype != DRK_BF16) return fail(DRK_ERR_INVALID, "decode: io_dtype must be F16 or BF16");
    if ((a.dtype == DRK_F16 || a.dtype == DRK_BF16) && io_dtype != a.dtype)
        return fail(DRK_ERR_INVALID, "decode: io_dtype %d differs from the pool's %d", io_dtype, a.dtype);
    if (layer < 0 || layer >= a.L) return fail(DRK_ERR_INVALID, "decode: layer %d outside [0,%d)", layer, a.L);
    // one prefix for all branches is the simplest tree: shared and private tiles in one launch
    // (16-bit pages; 8-bit pages are faster on the prefix pass + tail kernel pair below)
    if (grouped_decode_supported(a, B) && a.E == 2 && B * (a.QH / a.KVH) <= 64) {
        const drk_prefix_group all = {0, B, 0, shared};
        return launch_decode_grouped(g, q, pool, tables, table_stride, d_seq_lens, B, max_seq_len, &all, 1, out, layer, scale,
                                     io_dtype, workspace, workspace_bytes, stream, gate, gate_stride);
    }
    size_t sp;
    const size_t need = shared_need(a, B, max_seq_len, shared, &sp, true);
    if (!workspace || workspace_bytes < need)
        return fail(DRK_ERR_WORKSPACE, "decode: workspace of %zu bytes, need %zu", workspace_bytes, need);
    if (((uintptr_t)workspace) % 16) return fail(DRK_ERR_INVALID, "decode: workspace must be 16-byte aligned");
    int ct, ns;
    shared_prefix_shape(a, B, shared, &ct, &ns);
    float *pre_o = (float *)((uint8_t *)workspace + sp);
    float *pre_m = pre_o + (size_t)B * a.QH * ns * a.D;
    float *pre_l = pre_m + (size_t)B * a.QH * ns;
    hipStream_t st = (hipStream_t)stream;
    // branch 0's table addresses the shared pages (identical in every row by the caller's promise)
    if ((rc = launch_shared_prefix(a, q, pool, tables, d_seq_lens, B, shared, layer, scale, io_dtype, pre_o, pre_m, pre_l, st))) return rc;
    if ((rc = launch_decode_stream(a, q, pool, tables, table_stride, d_seq_lens, 0, B, max_seq_len, out, layer, scale,
                                   io_dtype, 0, workspace, false, st, shared / kTile))) return rc;
    if (g_skip_merge) return DRK_OK;
    return launch_decode_stream(a, q, pool, tables, table_stride, d_seq_lens, 0, B, max_seq_len, out, layer, scale,
                                io_dtype, 0, workspace, true, st, shared / kTile, pre_o, pre_m, pre_l, ns, gate, gate_stride);
}

size_t decode_plan_need(const Lay &a, int B, int max_seq_len, const drk_prefix_group *groups, int n_groups)
{
    if (g_force_portable || g_decode_kernel == 2 || B < 1 || B > 64 || max_seq_len < 1 || !stream_decode_supported(a, B)) return 0;
    size_t need = stream_plan_need(a, B, max_seq_len);
    if (n_groups > 0 && grouped_decode_supported(a, B)) {
        const size_t g2 = grouped_plan_need(a, B, max_seq_len, groups, n_groups);
        if (g2 > need) need = g2;
    }
    return need;
}

} // namespace drk

using namespace drk;

extern "C" {

size_t drk_decode_plan_bytes(const drk_kv_layout *g, int B, int max_seq_len, int n_groups)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK) return 0;
    return decode_plan_need(a, B, max_seq_len, nullptr, n_groups);
}

int drk_decode_plan_build(const drk_kv_layout *g, const int32_t *d_tables, int table_stride, const int32_t *d_seq_lens, int B,
                          int max_seq_len, const drk_prefix_group *groups, int n_groups, void *d_plan, size_t plan_bytes,
                          void *stream)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    if (!d_tables || !d_seq_lens || !d_plan) return fail(DRK_ERR_INVALID, "decode_plan: NULL pointer");
    if (((uintptr_t)d_plan) % 16) return fail(DRK_ERR_INVALID, "decode_plan: the plan must be 16-byte aligned");
    const size_t need = decode_plan_need(a, B, max_seq_len, groups, n_groups);
    if (need == 0) return fail(DRK_ERR_UNSUPPORTED, "decode_plan: this geometry or number of branches takes no plan");
    if (plan_bytes < need) return fail(DRK_ERR_WORKSPACE, "decode_plan: plan of %zu bytes, need %zu", plan_bytes, need);
    DecodePlan plan;
    plan.ptr = (uint8_t *)d_plan;
    plan.mode = 1;
    const int io = a.dtype == DRK_F16 ? DRK_F16 : DRK_BF16;
    if (n_groups > 0 && grouped_decode_supported(a, B))
        return launch_decode_grouped(g, nullptr, nullptr, d_tables, table_stride, d_seq_lens, B, max_seq_len, groups, n_groups,
                                     nullptr, 0, 1.0f, io, nullptr, 0, stream, nullptr, 0, plan);
    return launch_decode(g, nullptr, nullptr, d_tables, table_stride, d_seq_lens, 0, -1, B, max_seq_len, nullptr, 0, 1.0f, io, 0,
                         nullptr, 0, stream, nullptr, 0, plan);
}

int drk_paged_decode_attention_planned(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *d_tables,
                                       int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len,
                                       const drk_prefix_group *groups, int n_groups, const void *d_plan, void *out, int layer,
                                       float scale, int io_dtype, const void *gate, size_t gate_stride, void *workspace,
                                       size_t workspace_bytes, void *stream)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    if (!d_plan) return fail(DRK_ERR_INVALID, "decode_planned: d_plan is NULL");
    if (decode_plan_need(a, B, max_seq_len, groups, n_groups) == 0)
        return fail(DRK_ERR_UNSUPPORTED, "decode_planned: this geometry or number of branches takes no plan");
    DecodePlan plan;
    plan.ptr = (uint8_t *)const_cast<void *>(d_plan);
    plan.mode = 2;
    if (n_groups > 0 && grouped_decode_supported(a, B))
        return launch_decode_grouped(g, q, pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, groups, n_groups, out, layer,
                                     scale, io_dtype, workspace, workspace_bytes, stream, gate, gate_stride, plan);
    return launch_decode(g, q, pool, d_tables, table_stride, d_seq_lens, 0, -1, B, max_seq_len, out, layer, scale, io_dtype, 0,
                         workspace, workspace_bytes, stream, gate, gate_stride, plan);
}

int drk_kv_append_decode_planned(const drk_kv_layout *g, void *pool, const int32_t *d_tables, int table_stride,
                                 const int32_t *d_seq_lens, int B, int max_seq_len, const drk_prefix_group *groups,
                                 int n_groups, const void *d_plan, const void *new_k, const void *new_v, int src_dtype,
                                 const void *q, void *out, int layer, float scale, int io_dtype, const void *gate,
                                 size_t gate_stride, void *workspace, size_t workspace_bytes, void *stream)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    if (!d_plan || !new_k || !new_v || !d_seq_lens || !pool) return fail(DRK_ERR_INVALID, "append_decode: NULL pointer");
    if (decode_plan_need(a, B, max_seq_len, groups, n_groups) == 0)
        return fail(DRK_ERR_UNSUPPORTED, "append_decode: this geometry or number of branches takes no plan");
    DecodePlan plan;
    plan.ptr = (uint8_t *)const_cast<void *>(d_plan);
    plan.mode = 2;
    const bool grouped = n_groups > 0 && grouped_decode_supported(a, B);
    // the tiled kernels (plain and grouped) write the new rows themselves when they are in the pages' own 16-bit type;
    // otherwise the append is a launch of its own, at position length - 1
    const bool fused = a.E == 2 && src_dtype == a.dtype && (((uintptr_t)new_k | (uintptr_t)new_v) % 16) == 0 &&
                       (!grouped || grouped_decode_writes_new_rows(a));
    if (fused) {
        plan.new_k = (const uint8_t *)new_k;
        plan.new_v = (const uint8_t *)new_v;
    } else if ((rc = launch_append(g, pool, d_tables, table_stride, d_seq_lens, -1, B, layer, 1, new_k, new_v, src_dtype, stream))) {
        return rc;
    }
    if (grouped)
        return launch_decode_grouped(g, q, pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, groups, n_groups, out, layer,
                                     scale, io_dtype, workspace, workspace_bytes, stream, gate, gate_stride, plan);
    return launch_decode(g, q, pool, d_tables, table_stride, d_seq_lens, 0, -1, B, max_seq_len, out, layer, scale, io_dtype, 0,
                         workspace, workspace_bytes, stream, gate, gate_stride, plan);
}

size_t drk_decode_workspace_bytes(const drk_kv_layout *g, int B, int max_seq_len)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK || B <= 0 || max_seq_len <= 0) return 0;
    size_t need = workspace_need(a, B, max_seq_len, choose_split(a, B, max_seq_len));
    const int bs = B < 64 ? B : 64;                      // the tiled kernel takes 64 branches per launch
    if (stream_decode_supported(a, bs)) {
        size_t s2 = stream_workspace_need(a, bs, max_seq_len, 0);
        if (s2 > need) need = s2;
    }
    return need;
}

size_t drk_decode_workspace_bytes_for_split(const drk_kv_layout *g, int B, int max_seq_len, int split_tokens)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK || B <= 0 || max_seq_len <= 0 || split_tokens <= 0) return 0;
    size_t need = workspace_need(a, B, max_seq_len, split_tokens);
    const int bs = B < 64 ? B : 64;
    if (stream_decode_supported(a, bs)) {
        size_t s2 = stream_workspace_need(a, bs, max_seq_len, split_tokens);
        if (s2 > need) need = s2;
    }
    return need;
}

int drk_decode_default_split(const drk_kv_layout *g, int B, int max_seq_len)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK || B <= 0 || max_seq_len <= 0) return 0;
    return choose_split(a, B, max_seq_len);
}

void drk_debug_force_portable_decode(int on) { g_force_portable = on ? 1 : 0; }
void drk_debug_set_decode_kernel(int which) { g_decode_kernel = which; }
void drk_debug_set_stream_workgroups(int n) { g_stream_wgs = n > 0 ? n : 0; }
void drk_debug_set_stream_descriptors_only(int on) { g_stream_stop_after_descriptors = on ? 1 : 0; }
void drk_debug_set_shared_splits(int n) { g_shared_splits = n > 0 ? (n < 256 ? n : 256) : 64; }
void drk_debug_set_prefix_stream(int on) { g_prefix_stream = on ? 1 : 0; }

void drk_debug_set_skip_merge(int on) { g_skip_merge = on ? 1 : 0; }
void drk_debug_set_decode_lds_pad(int bytes) { g_lds_pad = bytes > 0 ? bytes : 0; }

int drk_paged_decode_attention(const drk_kv_layout *g, const void *q, const void *pool,
                               const int32_t *d_block_table, void *out, int layer, int seq_len, float scale,
                               int io_dtype, void *workspace, size_t workspace_bytes, void *stream)
{
    if (seq_len < 0) return fail(DRK_ERR_INVALID, "decode: negative seq_len");
    return launch_decode(g, q, pool, d_block_table, 0, nullptr, seq_len, -1, 1, seq_len, out, layer, scale, io_dtype,
                         0, workspace, workspace_bytes, stream);
}

size_t drk_decode_shared_workspace_bytes(const drk_kv_layout *g, int B, int max_seq_len, int shared_tokens)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK || B <= 0 || max_seq_len <= 0) return 0;
    size_t need = drk_decode_workspace_bytes(g, B, max_seq_len);
    const int shared = shared_tokens > 0 ? (shared_tokens / kTile) * kTile : 0;
    if (stream_decode_supported(a, B) && shared >= kTile) {
        size_t s2 = shared_need(a, B, max_seq_len, shared, nullptr, false);
        if (s2 > need) need = s2;
        if (a.D == 128 && B * (a.QH / a.KVH) <= 64) {        // the grouped kernel may take the call
            s2 = grouped_workspace_need_max(a, B, max_seq_len, 1);
            if (s2 > need) need = s2;
        }
    }
    return need;
}

int drk_paged_decode_attention_shared(const drk_kv_layout *g, const void *q, const void *pool,
                                      const int32_t *d_tables, int table_stride, const int32_t *d_seq_lens, int B,
                                      int max_seq_len, int shared_tokens, void *out, int layer, float scale,
                                      int io_dtype, void *workspace, size_t workspace_bytes, void *stream)
{
    if (!d_seq_lens) return fail(DRK_ERR_INVALID, "decode: d_seq_lens is NULL");
    if (B < 0 || max_seq_len < 0 || table_stride < 0 || shared_tokens < 0) return fail(DRK_ERR_INVALID, "decode: negative size");
    if (B == 0 || max_seq_len == 0) return DRK_OK;
    return launch_decode_shared(g, q, pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, shared_tokens, out,
                                layer, scale, io_dtype, workspace, workspace_bytes, stream);
}

int drk_paged_decode_attention_branches(const drk_kv_layout *g, const void *q, const void *pool,
                                        const int32_t *d_tables, int table_stride, const int32_t *d_seq_lens,
                                        int B, int max_seq_len, void *out, int layer, float scale,
                                        int io_dtype, int split_tokens, void *workspace,
                                        size_t workspace_bytes, void *stream)
{
    if (!d_seq_lens) return fail(DRK_ERR_INVALID, "decode: d_seq_lens is NULL");
    return launch_decode(g, q, pool, d_tables, table_stride, d_seq_lens, 0, -1, B, max_seq_len, out, layer, scale,
                         io_dtype, split_tokens, workspace, workspace_bytes, stream);
}

// ---- attention mass per block (importance scoring) -----------------------------------
static size_t mass_extra(const Lay &a, int B, int max_seq_len, int *lse_stride)
{
    const int ls = 4 * ((max_seq_len + kTile - 1) / kTile);
    if (lse_stride) *lse_stride = ls;
    return ((size_t)B * a.QH * ls + (size_t)B * a.QH) * sizeof(float);
}

size_t drk_decode_mass_workspace_bytes(const drk_kv_layout *g, int B, int max_seq_len)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK || B <= 0 || max_seq_len <= 0 || !stream_decode_supported(a, B)) return 0;
    size_t sp = stream_workspace_need(a, B, max_seq_len, 0);
    sp = (sp + 255) & ~(size_t)255;
    return sp + mass_extra(a, B, max_seq_len, nullptr);
}

// Decode attention that also reports, per (branch, logical block), the attention mass the
// block received: sum over its tokens and all query heads of the softmax probability --
// the "new importance values from attention" ImportanceScorer::update takes
// (importance_scorer.h:37-41; docs/en/architecture/02-memoria.md:40-44).
static int decode_mass_impl(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *d_tables,
                            int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len, const void *d_plan, void *out,
                            int layer, float scale, int io_dtype, const void *gate, size_t gate_stride, float *d_block_mass,
                            int mass_stride, int accumulate, void *workspace, size_t workspace_bytes, void *stream)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    if (gate && (gate_stride < (size_t)a.D || (gate_stride % 8) || ((uintptr_t)gate % 16)))
        return fail(DRK_ERR_INVALID, "decode_mass: gate rows must be 16-byte aligned and at least head_dim apart");
    DecodePlan plan;
    if (d_plan) {
        if (decode_plan_need(a, B, max_seq_len, nullptr, 0) == 0)
            return fail(DRK_ERR_UNSUPPORTED, "decode_mass: this geometry or number of branches takes no plan");
        plan.ptr = (uint8_t *)const_cast<void *>(d_plan);
        plan.mode = 2;
    }
    if (!q || !pool || !d_tables || !out || !d_seq_lens || !d_block_mass) return fail(DRK_ERR_INVALID, "decode_mass: NULL pointer");
    if (io_dtype != DRK_F16 && io_dtype != DRK_BF16) return fail(DRK_ERR_INVALID, "decode_mass: io_dtype must be F16 or BF16");
    if ((a.dtype == DRK_F16 || a.dtype == DRK_BF16) && io_dtype != a.dtype)
        return fail(DRK_ERR_INVALID, "decode_mass: io_dtype %d differs from the pool's %d", io_dtype, a.dtype);
    if (layer < 0 || layer >= a.L) return fail(DRK_ERR_INVALID, "decode_mass: layer %d outside [0,%d)", layer, a.L);
    if (B < 0 || max_seq_len < 0 || table_stride < 0 || mass_stride < 0) return fail(DRK_ERR_INVALID, "decode_mass: negative size");
    if (B == 0 || max_seq_len == 0) return DRK_OK;
    if (B > 65535) return fail(DRK_ERR_INVALID, "decode_mass: more than 65535 branches");
    if (g_force_portable || !stream_decode_supported(a, B))
        return fail(DRK_ERR_UNSUPPORTED, "decode_mass: needs head_dim 128 or 256, at most 16 query heads per kv head, block_size %% 16 == 0, at most 64 branches");
    if (mass_stride < (max_seq_len + a.bs - 1) / a.bs)
        return fail(DRK_ERR_INVALID, "decode_mass: mass_stride %d is less than the %d blocks of max_seq_len", mass_stride,
                    (max_seq_len + a.bs - 1) / a.bs);
    int ls;
    size_t sp = stream_workspace_need(a, B, max_seq_len, 0);
    sp = (sp + 255) & ~(size_t)255;
    const size_t need = sp + mass_extra(a, B, max_seq_len, &ls);
    if (!workspace || workspace_bytes < need)
        return fail(DRK_ERR_WORKSPACE, "decode_mass: workspace of %zu bytes, need %zu", workspace_bytes, need);
    if (((uintptr_t)workspace) % 16) return fail(DRK_ERR_INVALID, "decode_mass: workspace must be 16-byte aligned");
    float *lse_groups = (float *)((uint8_t *)workspace + sp);
    float *lse_rows = lse_groups + (size_t)B * a.QH * ls;
    hipStream_t st = (hipStream_t)stream;
    if ((rc = launch_decode_stream(a, q, pool, d_tables, table_stride, d_seq_lens, 0, B, max_seq_len, out, layer, scale,
                                   io_dtype, 0, workspace, false, st, 0, nullptr, nullptr, nullptr, 0, nullptr, 0,
                                   lse_groups, lse_rows, ls, plan)))
        return rc;
    if ((rc = launch_decode_stream(a, q, pool, d_tables, table_stride, d_seq_lens, 0, B, max_seq_len, out, layer, scale,
                                   io_dtype, 0, workspace, true, st, 0, nullptr, nullptr, nullptr, 0, gate, gate_stride,
                                   lse_groups, lse_rows, ls)))
        return rc;
    return launch_block_mass(lse_groups, lse_rows, d_seq_lens, B, a.QH, ls, a.bs, d_block_mass, mass_stride, accumulate, st);
}

int drk_paged_decode_attention_mass(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *d_tables,
                                    int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len, void *out,
                                    int layer, float scale, int io_dtype, float *d_block_mass, int mass_stride,
                                    int accumulate, void *workspace, size_t workspace_bytes, void *stream)
{
    return decode_mass_impl(g, q, pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, nullptr, out, layer, scale, io_dtype,
                            nullptr, 0, d_block_mass, mass_stride, accumulate, workspace, workspace_bytes, stream);
}

int drk_paged_decode_attention_mass_gated(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *d_tables,
                                          int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len,
                                          const void *d_plan, void *out, int layer, float scale, int io_dtype, const void *gate,
                                          size_t gate_stride, float *d_block_mass, int mass_stride, int accumulate,
                                          void *workspace, size_t workspace_bytes, void *stream)
{
    return decode_mass_impl(g, q, pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, d_plan, out, layer, scale, io_dtype,
                            gate, gate_stride, d_block_mass, mass_stride, accumulate, workspace, workspace_bytes, stream);
}

// ---- decode that allocates nothing and takes no workspace ------------------------------
constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];        // device address of `scratch` on device i, once looked up
static std::mutex g_scratch_mu;

// The address of this device's copy of `scratch` (each GPU maps the array at an address of
// its own), looked up once per device with that device current.
static int static_scratch(void **ptr)
{
    int dev = -1;
    DRK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(DRK_ERR_INVALID, "decode_static: device %d outside [0,%d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        DRK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(DRK_ERR_HIP, "decode_static: the scratch array has no address on device %d", dev);
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return DRK_OK;
}

int drk_paged_decode_attention_branches_static(const drk_kv_layout *g, const void *q, const void *pool,
                                               const int32_t *d_tables, int table_stride,
                                               const int32_t *d_seq_lens, int B, int max_seq_len, void *out,
                                               int layer, float scale, int io_dtype, void *stream)
{
    if (!d_seq_lens) return fail(DRK_ERR_INVALID, "decode_static: d_seq_lens is NULL");
    if (B < 0 || max_seq_len < 0) return fail(DRK_ERR_INVALID, "decode_static: negative size");
    if (B == 0 || max_seq_len == 0) return DRK_OK;
    const size_t need = drk_decode_workspace_bytes(g, B, max_seq_len);
    if (need == 0) return fail(DRK_ERR_INVALID, "decode_static: bad layout");
    if (need > (size_t)DRK_STATIC_SCRATCH_BYTES)
        return fail(DRK_ERR_WORKSPACE,
                    "decode_static: %d branches of up to %d tokens need %zu bytes of partials, the static scratch holds %zu; "
                    "use drk_paged_decode_attention_branches with a workspace",
                    B, max_seq_len, need, (size_t)DRK_STATIC_SCRATCH_BYTES);
    void *ptr = nullptr;
    int rc = static_scratch(&ptr);
    if (rc) return rc;
    // nothing in the scratch has to start at zero: the partial kernel writes every slot the merge reads
    return launch_decode(g, q, pool, d_tables, table_stride, d_seq_lens, 0, -1, B, max_seq_len, out, layer, scale,
                         io_dtype, 0, ptr, (size_t)DRK_STATIC_SCRATCH_BYTES, stream);
}

// steps 6 + 7 of full_attention_forward_paged (paged_attention.cu:362-370) in one call:
// out = attention * sigmoid(gate); gate rows [B * num_q_heads] are gate_stride elements apart
int drk_paged_decode_attention_gated(const drk_kv_layout *g, const void *q, const void *pool,
                                     const int32_t *d_tables, int table_stride, const int32_t *d_seq_lens,
                                     int B, int max_seq_len, void *out, int layer, float scale, int io_dtype,
                                     const void *gate, size_t gate_stride, void *workspace,
                                     size_t workspace_bytes, void *stream)
{
    if (!d_seq_lens) return fail(DRK_ERR_INVALID, "decode: d_seq_lens is NULL");
    if (!gate) return fail(DRK_ERR_INVALID, "decode: gate is NULL");
    return launch_decode(g, q, pool, d_tables, table_stride, d_seq_lens, 0, -1, B, max_seq_len, out, layer, scale,
                         io_dtype, 0, workspace, workspace_bytes, stream, gate, gate_stride);
}

} // extern "C"
