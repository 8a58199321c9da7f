// drk_decode_stream.hip -- the production paged GQA decode kernel: persistent,
// stream-K style, for head_dim 128 with 4 query heads per KV head and fp16, bf16,
// int8 (+fp16 scale per token and head) or fp8-e4m3 pages.
//
// The unit of work is one 64-token tile of one (branch, kv head).  Units are
// numbered branch-major, then kv head, then tile; workgroup g owns the run
// [g*U, (g+1)*U).  Every workgroup therefore streams the same number of tiles
// whatever the branch lengths are, the whole grid is resident in one round, and a
// run that crosses from one (branch, kv head) to the next keeps its load pipeline
// full: the next unit's K/V (and the next segment's Q) are already in flight when
// the current segment's partial result is written.  A (branch, kv head) is cut
// into at most ceil(tiles/U)+1 pieces; each piece leaves (o[128], m, l) per query
// head in the workspace and stream_merge_kernel folds them.
//
// Per tile (the same three phases as decode_tiled_kernel in drk_decode.hip):
//   A  each wave stores the 16-token page row run it loaded one tile earlier into
//      LDS (K only; 272-byte pitch), converting int8 / fp8 codes to fp16 on the
//      way, and issues the 128-bit loads of the next unit's K;
//   B  wave w = query head w: lane = token, Q in 64 SGPRs, v_dot2 over the row in
//      LDS, no cross-lane reduction for the dot; tile softmax by wave reductions;
//      p (times the V scale for int8) to LDS;
//   C  wave w multiplies its own 16 tokens of V, straight from the global loads,
//      into 4 heads x 8 dims of fp32 per lane; then issues the next unit's V loads.
#include "drk_common.hpp"

#include <math.h>

namespace drk {

// Workgroups of the persistent grid on a 256-CU part; 0 = by storage type: 2 per CU
// for 16-bit pages (bandwidth-bound: fewer, longer runs stream best), 3 per CU for
// 8-bit pages (the dequantising waves need the extra latency hiding).
int g_stream_wgs = 0;
static inline int stream_wgs(const Lay &a) { return g_stream_wgs > 0 ? g_stream_wgs : (a.E == 1 ? 768 : 512); }

constexpr int kSTile = 64;
constexpr int kSRow = 272;
constexpr float kSLog2e = 1.4426950408889634f;

typedef __bf16 s_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 s_f16x2 __attribute__((ext_vector_type(2)));

template <int DT> struct KvTraits;
template <> struct KvTraits<DRK_F16>      { static constexpr bool q8 = false; static constexpr int dot = DRK_F16; };
template <> struct KvTraits<DRK_BF16>     { static constexpr bool q8 = false; static constexpr int dot = DRK_BF16; };
template <> struct KvTraits<DRK_INT8>     { static constexpr bool q8 = true;  static constexpr int dot = DRK_F16; };
template <> struct KvTraits<DRK_FP8_E4M3> { static constexpr bool q8 = true;  static constexpr int dot = DRK_F16; };

template <int DOT>
__device__ __forceinline__ float s_dot2(uint32_t k, uint32_t q, float acc)
{
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (DOT == DRK_BF16)
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(s_bf16x2, k), __builtin_bit_cast(s_bf16x2, q), acc, false);
    else
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(s_f16x2, k), __builtin_bit_cast(s_f16x2, q), acc, false);
#else
    (void)k; (void)q;
    return acc;
#endif
}

__device__ __forceinline__ float s_exp2(float x)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_exp2f(x);
#else
    return exp2f(x);
#endif
}

// Wave-wide reductions: four DPP steps reduce inside each row of 16 lanes
// (quad swaps, then half-row and row mirrors), four v_readlane fold the rows.
template <int CTRL>
__device__ __forceinline__ float s_dpp(float v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
#else
    return v;
#endif
}
__device__ __forceinline__ float s_lane(float v, int l)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
#else
    (void)l;
    return v;
#endif
}
__device__ __forceinline__ float s_wave_max(float v)
{
    v = fmaxf(v, s_dpp<0xB1>(v));      // quad_perm [1,0,3,2]
    v = fmaxf(v, s_dpp<0x4E>(v));      // quad_perm [2,3,0,1]
    v = fmaxf(v, s_dpp<0x141>(v));     // row_half_mirror
    v = fmaxf(v, s_dpp<0x140>(v));     // row_mirror
    return fmaxf(fmaxf(s_lane(v, 0), s_lane(v, 16)), fmaxf(s_lane(v, 32), s_lane(v, 48)));
}
__device__ __forceinline__ float s_wave_sum(float v)
{
    v += s_dpp<0xB1>(v);
    v += s_dpp<0x4E>(v);
    v += s_dpp<0x141>(v);
    v += s_dpp<0x140>(v);
    return (s_lane(v, 0) + s_lane(v, 16)) + (s_lane(v, 32) + s_lane(v, 48));
}

__device__ __forceinline__ uint32_t s_perm(uint32_t hi, uint32_t lo, uint32_t sel)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_amdgcn_perm(hi, lo, sel);      // result byte i = byte sel[i] of {lo: 0-3, hi: 4-7}
#else
    (void)hi; (void)sel;
    return lo;
#endif
}

// int8 codes travel as fp16 1152 + code: byte (code ^ 0x80) under the exponent byte 0x64
// is exactly that number, so a code costs one byte permute and the constant is taken
// out once per dot product (1152 * sum of the other operand) instead of once per value.
constexpr float kI8Bias = 1152.0f;
constexpr uint32_t kF16Ones = 0x3C003C00u;

// four int8 codes -> two dwords of packed fp16 (1152 + code)
__device__ __forceinline__ void int8x4_to_f16x4(uint32_t w, uint32_t &lo, uint32_t &hi)
{
    const uint32_t x = w ^ 0x80808080u;
    lo = s_perm(0x64646464u, x, 0x04010400u);   // bytes x0,64,x1,64
    hi = s_perm(0x64646464u, x, 0x04030402u);   // bytes x2,64,x3,64
}

// two fp8-e4m3 codes (the low or the high half of w) -> packed fp16 (exact: e4m3 fits in fp16)
template <bool HIGH>
__device__ __forceinline__ uint32_t fp8x2_to_f16x2(uint32_t w)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, HIGH));
#else
    return w;
#endif
}
__device__ __forceinline__ void fp8x4_to_f16x4(uint32_t w, uint32_t &lo, uint32_t &hi)
{
    lo = fp8x2_to_f16x2<false>(w);
    hi = fp8x2_to_f16x2<true>(w);
}

struct StreamArgs {
    const uint8_t *pool_layer;      // pool + layer * layer_stride
    const int32_t *tables;
    const int32_t *seq_lens;        // [B] on the device, or NULL: one sequence of seq_len_host
    const uint8_t *q;
    float *part_o, *part_m, *part_l;
    int table_stride, seq_len_host, B, KVH, QH, NB, bs, bs_shift, io_dtype;
    int unit_tiles;                 // tiles per workgroup, or 0: ceil(total / gridDim.x)
    int Pmax;                       // partial slots per (branch, q head)
    int start_tile;                 // tiles [0, start_tile) of every branch are handled elsewhere (shared prefix)
    unsigned head_stride, kv_plane, block_stride, scale_plane, row_bytes;
    float scale_log2e;
    // optional: log2-sum-exp of every 16-token group's scaled scores, [B*QH][lse_stride]
    // (what the attention-mass pass needs; -inf for a group without a visible token)
    float *lse_groups;
    int lse_stride;
};

constexpr int kMaxUnits = 256;       // units one workgroup may own (descriptor table in LDS)

struct UnitDesc {                    // one 64-token tile of one (branch, kv head)
    int tile_lim;                    // tokens of the tile that exist: seq_len - tile*64 (may exceed 64)
    int flags;                       // bit 0: first tile of a segment of this workgroup, bit 1: last; bits 2..: tile index
    int bq;                          // branch*QH + kvh*4: first query row of the group (Q, partial slots)
    int piece;                       // partial slot of the segment inside its (branch, q head)
};

// one wave's 16-token group of a tile, as loaded from the pool
template <int DT> struct KRegs { uint4 r0, r1, r2, r3; };
template <> struct KRegs<DRK_INT8> { uint4 r0, r1; };
template <> struct KRegs<DRK_FP8_E4M3> { uint4 r0, r1; };
template <int DT> struct VRegs { uint4 r0, r1, r2, r3; };
template <> struct VRegs<DRK_INT8> { uint2 r0, r1, r2, r3; };
template <> struct VRegs<DRK_FP8_E4M3> { uint2 r0, r1, r2, r3; };

// The 16-token run of one kv head at offset `off` of the layer, in units of 16 bytes (kNone:
// the run has no page).  A missing run is loaded from offset 0 -- always mapped -- instead of being
// predicated off: its K only feeds scores that are masked anyway, and its V is cleared
// by the consumer where a stale bit pattern could matter.
template <int DT>
__device__ __forceinline__ KRegs<DT> load_k(const uint8_t *__restrict__ layer, uint32_t off, int lane)
{
    KRegs<DT> k;
    const uint8_t *p = layer + ((size_t)(off == 0xffffffffu ? 0u : off) << 4) + (size_t)lane * 16;
    if constexpr (KvTraits<DT>::q8) {
        k.r0 = ld_stream128(p);
        k.r1 = ld_stream128(p + 1024);
    } else {
        k.r0 = ld_stream128(p);
        k.r1 = ld_stream128(p + 1024);
        k.r2 = ld_stream128(p + 2048);
        k.r3 = ld_stream128(p + 3072);
    }
    return k;
}

template <int DT>
__device__ __forceinline__ VRegs<DT> load_v(const uint8_t *__restrict__ layer, uint32_t off, uint32_t kv_plane, int lane)
{
    VRegs<DT> v;
    const uint8_t *p = layer + ((size_t)(off == 0xffffffffu ? 0u : off) << 4) + kv_plane;
    if constexpr (KvTraits<DT>::q8) {
        p += (size_t)lane * 8;
        v.r0 = ld_stream64(p);
        v.r1 = ld_stream64(p + 512);
        v.r2 = ld_stream64(p + 1024);
        v.r3 = ld_stream64(p + 1536);
    } else {
        p += (size_t)lane * 16;
        v.r0 = ld_stream128(p);
        v.r1 = ld_stream128(p + 1024);
        v.r2 = ld_stream128(p + 2048);
        v.r3 = ld_stream128(p + 3072);
    }
    return v;
}

// stage the wave's 16 K rows as 16-bit values: rows w*16 .. w*16+15 of the tile
template <int DT>
__device__ __forceinline__ void stage_k(uint8_t *tile_lds, const KRegs<DT> &k, int w, int lane)
{
    if constexpr (KvTraits<DT>::q8) {
        // a loaded register holds 16 codes of row (lane>>3) + 8*j, dims (lane&7)*16 ..
        uint8_t *dst = tile_lds + (w * 16 + (lane >> 3)) * kSRow + (lane & 7) * 32;
        const uint4 regs[2] = {k.r0, k.r1};
#pragma unroll
        for (int j = 0; j < 2; j++) {
            uint32_t h[8];
            if constexpr (DT == DRK_INT8) {
                int8x4_to_f16x4(regs[j].x, h[0], h[1]);
                int8x4_to_f16x4(regs[j].y, h[2], h[3]);
                int8x4_to_f16x4(regs[j].z, h[4], h[5]);
                int8x4_to_f16x4(regs[j].w, h[6], h[7]);
            } else {
                fp8x4_to_f16x4(regs[j].x, h[0], h[1]);
                fp8x4_to_f16x4(regs[j].y, h[2], h[3]);
                fp8x4_to_f16x4(regs[j].z, h[4], h[5]);
                fp8x4_to_f16x4(regs[j].w, h[6], h[7]);
            }
            *(uint4 *)(dst + j * 8 * kSRow) = make_uint4(h[0], h[1], h[2], h[3]);
            *(uint4 *)(dst + j * 8 * kSRow + 16) = make_uint4(h[4], h[5], h[6], h[7]);
        }
    } else {
        uint8_t *dst = tile_lds + (w * 16 + (lane >> 4)) * kSRow + (lane & 15) * 16;
        *(uint4 *)(dst) = k.r0;
        *(uint4 *)(dst + 4 * kSRow) = k.r1;
        *(uint4 *)(dst + 8 * kSRow) = k.r2;
        *(uint4 *)(dst + 12 * kSRow) = k.r3;
    }
}

// o[h][e] += p[a][h] * V[a][e] + p[b][h] * V[b][e] for two token rows a, b and the 8 dims of
// this lane: one v_dot2 per (head, dim) over the token pair.  pp holds, per head, the packed
// 16-bit weights (p[a], p[b]); the rows' values are paired up by byte permutes.
template <int DT, typename VR>
__device__ __forceinline__ void pv_pair(float (&o)[4][8], float (&psum)[4], const VR &va, const VR &vb, const uint4 pp)
{
    constexpr int DOT = KvTraits<DT>::dot;
    uint32_t pr[8];
    if constexpr (KvTraits<DT>::q8) {
        const uint32_t i0 = s_perm(vb.x, va.x, 0x05010400u), i1 = s_perm(vb.x, va.x, 0x07030602u);   // a0 b0 a1 b1 | a2 b2 a3 b3
        const uint32_t i2 = s_perm(vb.y, va.y, 0x05010400u), i3 = s_perm(vb.y, va.y, 0x07030602u);
        if constexpr (DT == DRK_INT8) {
            int8x4_to_f16x4(i0, pr[0], pr[1]);
            int8x4_to_f16x4(i1, pr[2], pr[3]);
            int8x4_to_f16x4(i2, pr[4], pr[5]);
            int8x4_to_f16x4(i3, pr[6], pr[7]);
            psum[0] = s_dot2<DOT>(pp.x, kF16Ones, psum[0]);          // the +1152 is taken out at the end
            psum[1] = s_dot2<DOT>(pp.y, kF16Ones, psum[1]);
            psum[2] = s_dot2<DOT>(pp.z, kF16Ones, psum[2]);
            psum[3] = s_dot2<DOT>(pp.w, kF16Ones, psum[3]);
        } else {
            fp8x4_to_f16x4(i0, pr[0], pr[1]);
            fp8x4_to_f16x4(i1, pr[2], pr[3]);
            fp8x4_to_f16x4(i2, pr[4], pr[5]);
            fp8x4_to_f16x4(i3, pr[6], pr[7]);
        }
    } else {
        const uint32_t wa[4] = {va.x, va.y, va.z, va.w}, wb[4] = {vb.x, vb.y, vb.z, vb.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            pr[2 * i] = s_perm(wb[i], wa[i], 0x05040100u);
            pr[2 * i + 1] = s_perm(wb[i], wa[i], 0x07060302u);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
        o[0][e] = s_dot2<DOT>(pr[e], pp.x, o[0][e]);
        o[1][e] = s_dot2<DOT>(pr[e], pp.y, o[1][e]);
        o[2][e] = s_dot2<DOT>(pr[e], pp.z, o[2][e]);
        o[3][e] = s_dot2<DOT>(pr[e], pp.w, o[3][e]);
    }
}

template <int DT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void decode_stream_kernel(StreamArgs A)
{
    constexpr bool Q8 = KvTraits<DT>::q8;
    constexpr int DOT = KvTraits<DT>::dot;
    constexpr uint32_t kNone = 0xffffffffu;
    __shared__ __align__(16) uint8_t k_lds[2][kSTile * kSRow];
    __shared__ __align__(16) uint16_t p_lds[2][kSTile * 4];   // [pair of rows][head][row of the pair], 16-bit weights
    __shared__ __align__(16) float alpha_lds[2][4];
    __shared__ __align__(16) float kscale_lds[2][kSTile];
    __shared__ __align__(16) float vscale_lds[2][kSTile];
    __shared__ __align__(16) UnitDesc udesc[kMaxUnits];
    __shared__ __align__(16) uint2 gdesc[kMaxUnits][4];       // per 16-token group: K offset (kNone: skip), scale offset; 16-byte units
    __shared__ int s_incl[64], s_len[64];

    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int lrow = lane >> 4, lchunk = lane & 15;

    // ---- the workgroup's run of units and one descriptor per unit ---------------------
    const int len_i = lane < A.B ? (A.seq_lens ? A.seq_lens[lane] : A.seq_len_host) : 0;
    const int nt_i = len_i > 0 ? max((len_i + kSTile - 1) / kSTile - A.start_tile, 0) : 0;
    int incl = nt_i;                                           // inclusive prefix of tiles over branches
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int t = __shfl_up(incl, off);
        if (lane >= off) incl += t;
    }
    const int T = __builtin_amdgcn_readlane(incl, 63) * A.KVH;
    if (T == 0) return;
    const int U = A.unit_tiles > 0 ? A.unit_tiles : (T + (int)gridDim.x - 1) / (int)gridDim.x;
    const int u0 = (int)blockIdx.x * U;
    if (u0 >= T) return;
    const int nunits = min(U, T - u0);
    if (w == 0) { s_incl[lane] = incl; s_len[lane] = len_i; }
    __syncthreads();
    for (int i = threadIdx.x; i < nunits * 4; i += 256) {
        const int ui = i >> 2, grp = i & 3, u = u0 + ui;
        int lo = 0, hi = A.B - 1;                              // first branch whose cumulative units exceed u
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (A.KVH * s_incl[mid] > u) hi = mid; else lo = mid + 1;
        }
        const int b = lo;
        const int excl = b ? s_incl[b - 1] : 0, nt = s_incl[b] - excl, len = s_len[b];
        const int rem = u - A.KVH * excl, kvh = rem / nt, trel = rem - kvh * nt;
        const int tile = trel + A.start_tile;                  // absolute tile of the branch
        const int tg = tile * kSTile + grp * 16;
        uint2 gd = make_uint2(kNone, 0u);
        if (tg < len) {
            const int lb = A.bs_shift >= 0 ? (tg >> A.bs_shift) : (tg / A.bs);
            const int blk = A.tables[(size_t)b * A.table_stride + lb];
            if (blk >= 0 && blk < A.NB) {
                // every term is a multiple of 16 bytes (pp is a multiple of 16, plane sizes of 16 * 16)
                const unsigned pp = (unsigned)(tg - lb * A.bs);
                const size_t base = (size_t)blk * A.block_stride;
                gd.x = (unsigned)((base + (size_t)kvh * A.head_stride + (size_t)pp * A.row_bytes) >> 4);
                gd.y = (unsigned)((base + 2 * (size_t)A.kv_plane + ((size_t)kvh * A.bs + pp) * 2) >> 4);
            }
        }
        gdesc[ui][grp] = gd;
        if (grp == 0) {
            UnitDesc d;
            d.tile_lim = len - tile * kSTile;
            d.flags = ((ui == 0 || trel == 0) ? 1 : 0) | ((ui == nunits - 1 || trel + 1 == nt) ? 2 : 0) | (tile << 2);
            d.bq = b * A.QH + kvh * 4;
            d.piece = (int)blockIdx.x - (A.KVH * excl + kvh * nt) / U;
            udesc[ui] = d;
        }
    }
    __syncthreads();

    auto load_scales = [&](uint2 gd) -> uint32_t {
        // lanes 0-15: K scale of token lane, lanes 16-31: V scale of token lane-16
        if (DT != DRK_INT8 || gd.x == kNone || lane >= 32) return 0u;
        return *(const uint16_t *)(A.pool_layer + ((size_t)gd.y << 4) + (lane & 15) * 2 + (lane >= 16 ? A.scale_plane : 0u));
    };
    auto load_q = [&](int bq) -> uint32_t {
        // one packed pair of query head (bq + w) per lane; quantised pages multiply in fp16
        uint32_t v = ((const uint32_t *)(A.q + (size_t)(bq + w) * 256))[lane];
#if defined(__HIP_DEVICE_COMPILE__)
        if (Q8 && A.io_dtype == DRK_BF16)
            v = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v), bf16_hi(v)));
#endif
        return v;
    };

    float o[4][8], psum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int hh = 0; hh < 4; hh++)
#pragma unroll
        for (int e = 0; e < 8; e++) o[hh][e] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f, qbias = 0.0f;
    uint32_t qs[64];

    // Loads run PF tiles ahead of their use: one for 16-bit pages; two for 8-bit pages, whose
    // tiles are half the bytes, so that as much is in flight per workgroup.
    constexpr int PF = Q8 ? 2 : 1;
    uint2 gd0 = gdesc[0][w];
    KRegs<DT> kreg0 = load_k<DT>(A.pool_layer, gd0.x, lane);
    VRegs<DT> vreg0 = load_v<DT>(A.pool_layer, gd0.x, A.kv_plane, lane);
    bool vhole0 = gd0.x == kNone;                             // the run vreg was loaded for has no page
    uint32_t sreg0 = load_scales(gd0);
    uint2 gd1 = make_uint2(kNone, 0u);
    KRegs<DT> kreg1 = {};
    VRegs<DT> vreg1 = {};
    bool vhole1 = true;
    uint32_t sreg1 = 0u;
    if (PF == 2 && nunits > 1) {
        gd1 = gdesc[1][w];
        kreg1 = load_k<DT>(A.pool_layer, gd1.x, lane);
        vreg1 = load_v<DT>(A.pool_layer, gd1.x, A.kv_plane, lane);
        vhole1 = gd1.x == kNone;
        sreg1 = load_scales(gd1);
    }
    uint32_t qv = load_q(udesc[0].bq);

    auto tile_step = [&](const int it, KRegs<DT> &kreg, VRegs<DT> &vreg, uint32_t &sreg, bool &vhole, uint2 &gd) {
        const int buf = it & 1;
        const UnitDesc ud = udesc[it];
        const int flags = __builtin_amdgcn_readfirstlane(ud.flags);
        const int tile_lim = __builtin_amdgcn_readfirstlane(ud.tile_lim);
        const bool has_next = it + PF < nunits;
        if (flags & 1) {                          // Q of the segment's head into scalar registers
#pragma unroll
            for (int i = 0; i < 64; i++) qs[i] = __builtin_amdgcn_readlane(qv, i);
            if (DT == DRK_INT8) {                 // sum of the head's (fp16) query values, for the code offset
                float sq = 0.0f;
#pragma unroll
                for (int i = 0; i < 64; i++) sq = s_dot2<DOT>(qs[i], kF16Ones, sq);
                qbias = kI8Bias * sq;
            }
        }

        // ---- A: stage K (and scales), start the next unit's K loads -------------------
        stage_k<DT>(&k_lds[buf][0], kreg, w, lane);
        if (DT == DRK_INT8 && lane < 32) {
            const float sc = f16_bits_to_f((uint16_t)sreg);
            if (lane < 16) kscale_lds[buf][w * 16 + lane] = sc;
            else vscale_lds[buf][w * 16 + lane - 16] = sc;
        }
        if (has_next) {
            gd = gdesc[it + PF][w];
            kreg = load_k<DT>(A.pool_layer, gd.x, lane);
            sreg = load_scales(gd);
        }
        if ((flags & 2) && it + 1 < nunits) qv = load_q(udesc[it + 1].bq);
        __syncthreads();

        // ---- B: scores of head w for the tile's 64 tokens, tile softmax -----------------
        {
            const uint8_t *krow = &k_lds[buf][lane * kSRow];
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
                    acc = s_dot2<DOT>(ka[c].x, qs[qi + 0], acc);
                    acc = s_dot2<DOT>(ka[c].y, qs[qi + 1], acc);
                    acc = s_dot2<DOT>(ka[c].z, qs[qi + 2], acc);
                    acc = s_dot2<DOT>(ka[c].w, qs[qi + 3], acc);
                }
                asm volatile("" : "+v"(acc) :: "memory");   // at most two groups of LDS reads in flight
#pragma unroll
                for (int c = 0; c < 4; c++) ka[c] = kb[c];
            }
            const bool live = lane < tile_lim && gdesc[it][lane >> 4].x != kNone;
            if (DT == DRK_INT8) acc = (acc - qbias) * kscale_lds[buf][lane];
            float sc = acc * A.scale_log2e;
            sc = live ? sc : -INFINITY;
            const float m_new = fmaxf(m_run, s_wave_max(sc));
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float p = s_exp2(sc - m_use);
            const float alpha = s_exp2(m_run - m_use);
            // sum of p: the DPP steps leave each row of 16 lanes (= one 16-token group) with its own sum
            float rs = p;
            rs += s_dpp<0xB1>(rs);
            rs += s_dpp<0x4E>(rs);
            rs += s_dpp<0x141>(rs);
            rs += s_dpp<0x140>(rs);
            l_run = l_run * alpha + ((s_lane(rs, 0) + s_lane(rs, 16)) + (s_lane(rs, 32) + s_lane(rs, 48)));
            if (A.lse_groups && (lane & 15) == 0) {
                const int gi = (flags >> 2) * 4 + (lane >> 4);
                if (gi < A.lse_stride)
                    A.lse_groups[(size_t)(ud.bq + w) * A.lse_stride + gi] = rs > 0.0f ? m_use + __builtin_log2f(rs) : -INFINITY;
            }
            m_run = m_new;
            float pw = p;
            if (DT == DRK_INT8) pw = live ? p * vscale_lds[buf][lane] : 0.0f;   // a stale scale may be anything
            {
                // rows r, r+4 of a wave's 16 form a pair, and so do r+8, r+12: phase C holds exactly these
                uint16_t pb;
                if constexpr (DOT == DRK_BF16) pb = __builtin_bit_cast(uint16_t, (__bf16)pw);
                else pb = __builtin_bit_cast(uint16_t, (_Float16)pw);
                const int r = lane & 15, pidx = ((lane >> 4) * 4 + (r & 3)) * 2 + (r >> 3);
                p_lds[buf][(pidx * 4 + w) * 2 + ((r >> 2) & 1)] = pb;
            }
            if (lane == 0) alpha_lds[buf][w] = alpha;
        }
        __syncthreads();

        // ---- C: o += P V over this wave's 16 tokens, all 4 heads ----------------------
        {
            const float4 al = *(const float4 *)&alpha_lds[buf][0];
            if (al.x != 1.0f || al.y != 1.0f || al.z != 1.0f || al.w != 1.0f) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    o[0][e] *= al.x; o[1][e] *= al.y; o[2][e] *= al.z; o[3][e] *= al.w;
                }
                psum[0] *= al.x; psum[1] *= al.y; psum[2] *= al.z; psum[3] *= al.w;
            }
            const int r0 = w * 16 + lrow;
            if (DT != DRK_INT8 && (tile_lim < kSTile || vhole)) {   // rows without a token may hold anything (NaN)
                if (vhole || r0 >= tile_lim) vreg.r0 = {};
                if (vhole || r0 + 4 >= tile_lim) vreg.r1 = {};
                if (vhole || r0 + 8 >= tile_lim) vreg.r2 = {};
                if (vhole || r0 + 12 >= tile_lim) vreg.r3 = {};
            }
            const uint4 *pl = (const uint4 *)&p_lds[buf][(w * 4 + lrow) * 16];
            pv_pair<DT>(o, psum, vreg.r0, vreg.r1, pl[0]);
            pv_pair<DT>(o, psum, vreg.r2, vreg.r3, pl[1]);
        }
        if (has_next) {
            vreg = load_v<DT>(A.pool_layer, gd.x, A.kv_plane, lane);
            vhole = gd.x == kNone;
        }

        // ---- the segment's last tile: leave (o, m, l) for the merge ----------------------
        if (flags & 2) {
#pragma unroll
            for (int hh = 0; hh < 4; hh++)
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    float v = o[hh][e];
                    if (DT == DRK_INT8) v -= kI8Bias * psum[hh];
                    v += __shfl_xor(v, 16);
                    v += __shfl_xor(v, 32);
                    o[hh][e] = v;
                }
            float *o_lds = (float *)&k_lds[0][0];        // [wave][head][128] fp32 = 8 KiB; K reads are done
            __syncthreads();
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
                    const float2 v = *(const float2 *)(o_lds + (ww * 4 + w) * 128 + d);
                    acc.x += v.x;
                    acc.y += v.y;
                }
                const size_t pi = (size_t)(ud.bq + w) * A.Pmax + ud.piece;
                *(float2 *)(A.part_o + pi * 128 + d) = acc;
                if (lane == 0) {
                    A.part_m[pi] = m_run;
                    A.part_l[pi] = l_run;
                }
            }
            __syncthreads();                             // o_lds is free again before the next tile is staged
#pragma unroll
            for (int hh = 0; hh < 4; hh++) {
                psum[hh] = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) o[hh][e] = 0.0f;
            }
            m_run = -INFINITY;
            l_run = 0.0f;
        }
    };

    if constexpr (PF == 1) {
        for (int it = 0; it < nunits; it++) tile_step(it, kreg0, vreg0, sreg0, vhole0, gd0);
    } else {
        for (int it = 0; it < nunits; it += 2) {
            tile_step(it, kreg0, vreg0, sreg0, vhole0, gd0);
            if (it + 1 < nunits) tile_step(it + 1, kreg1, vreg1, sreg1, vhole1, gd1);
        }
    }
}

// grid (QH, B), block 256: fold the pieces of (branch, q head) -- the stream kernel's
// and, in shared-prefix mode, the prefix pass's; out is written only when some
// token took part (paged_attention.cu:266).  Lane s of every wave owns the (m, l) of
// piece s (+64, ...), so they arrive in one round of loads; wave w then folds the o
// rows of pieces w, w+4, ... for two dims per lane, eight rows in flight, and the four
// waves' sums meet in LDS.
__global__ __launch_bounds__(256) void stream_merge_kernel(const float *__restrict__ part_o, const float *__restrict__ part_m,
                                                           const float *__restrict__ part_l, uint16_t *__restrict__ out,
                                                           const int32_t *__restrict__ seq_lens, int seq_len_host, int B,
                                                           int KVH, int QH, int unit_tiles, int grid_wgs, int Pmax,
                                                           int io_dtype, int start_tile, const float *__restrict__ pre_o,
                                                           const float *__restrict__ pre_m, const float *__restrict__ pre_l,
                                                           int pre_splits, const uint16_t *__restrict__ gate,
                                                           size_t gate_stride, float *__restrict__ lse_rows)
{
    __shared__ float2 red[4][64];
    const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x & 63, wv = threadIdx.x >> 6, d = lane * 2;
    int excl = 0, total = 0, nt_b = 0;
    for (int i = 0; i < B; i++) {
        const int len = seq_lens ? seq_lens[i] : seq_len_host;
        const int nt = len > 0 ? max((len + kSTile - 1) / kSTile - start_tile, 0) : 0;
        if (i < b) excl += nt;
        if (i == b) nt_b = nt;
        total += nt;
    }
    int npieces = 0;
    if (nt_b > 0) {
        const int T = total * KVH;
        const int U = unit_tiles > 0 ? unit_tiles : (T + grid_wgs - 1) / grid_wgs;
        const int kvh = h / (QH / KVH);
        const int first = KVH * excl + kvh * nt_b, last = first + nt_b - 1;
        npieces = last / U - first / U + 1;
    }
    const size_t base = ((size_t)b * QH + h) * Pmax;
    const size_t pbase = ((size_t)b * QH + h) * pre_splits;
    const int n_all = npieces + pre_splits;                  // pieces 0..npieces-1: stream kernel; then the prefix pass
    float M = -INFINITY;
    for (int s = lane; s < n_all; s += 64) {
        const float pl = s < npieces ? part_l[base + s] : pre_l[pbase + (s - npieces)];
        const float pm = s < npieces ? part_m[base + s] : pre_m[pbase + (s - npieces)];
        if (pl > 0.0f) M = fmaxf(M, pm);
    }
    M = s_wave_max(M);
    float2 acc = make_float2(0.0f, 0.0f);
    float L = 0.0f;
    for (int c0 = 0; c0 < n_all; c0 += 64) {
        const int s = c0 + lane, cnt = min(64, n_all - c0);
        float w = 0.0f;
        if (s < n_all) {
            const float pl = s < npieces ? part_l[base + s] : pre_l[pbase + (s - npieces)];
            const float pm = s < npieces ? part_m[base + s] : pre_m[pbase + (s - npieces)];
            if (pl > 0.0f) { w = s_exp2(pm - M); L = fmaf(pl, w, L); }
        }
        for (int j = wv; j < cnt; j += 32) {
            float2 o[8];
            float wj[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int jj = min(j + 4 * u, cnt - 1), sj = c0 + jj;
                wj[u] = j + 4 * u < cnt ? s_lane(w, jj) : 0.0f;
                o[u] = *(const float2 *)(sj < npieces ? part_o + (base + sj) * 128 + d : pre_o + (pbase + (sj - npieces)) * 128 + d);
            }
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (wj[u] != 0.0f) { acc.x = fmaf(o[u].x, wj[u], acc.x); acc.y = fmaf(o[u].y, wj[u], acc.y); }   // a piece without tokens may hold anything
        }
    }
    L = s_wave_sum(L);
    if (lse_rows && threadIdx.x == 0) lse_rows[(size_t)b * QH + h] = L > 0.0f ? M + __builtin_log2f(L) : -INFINITY;
    red[wv][lane] = acc;
    __syncthreads();
    if (wv == 0) {
        // with a gate the row is always rewritten: the reference gates whatever the attention
        // kernel left in out, also when no token took part (paged_attention.cu:266, 368-370)
        uint32_t *dst = (uint32_t *)(out + ((size_t)b * QH + h) * 128 + d);
        uint32_t packed;
        if (L > 0.0f) {
            const float2 a1 = red[1][lane], a2 = red[2][lane], a3 = red[3][lane];
            const float x = ((acc.x + a1.x) + (a2.x + a3.x)) / L, y = ((acc.y + a1.y) + (a2.y + a3.y)) / L;
            packed = (uint32_t)f_to_elem16(x, io_dtype) | ((uint32_t)f_to_elem16(y, io_dtype) << 16);
        } else {
            if (!gate) return;
            packed = *dst;
        }
        if (gate) {
            const uint32_t g2 = *(const uint32_t *)(gate + ((size_t)b * QH + h) * gate_stride + d);
            packed = (uint32_t)gated_elem16((uint16_t)(packed & 0xffffu), (uint16_t)(g2 & 0xffffu), io_dtype) |
                     ((uint32_t)gated_elem16((uint16_t)(packed >> 16), (uint16_t)(g2 >> 16), io_dtype) << 16);
        }
        *dst = packed;
    }
}

// Attention mass per (branch, logical block): sum over the block's tokens and all query heads of
// the softmax probability, from the per-group and per-row log-sum-exps the two kernels above
// left.  One thread per (branch, block); consecutive threads read consecutive groups.
__global__ __launch_bounds__(256) void block_mass_kernel(const float *__restrict__ lse_groups, const float *__restrict__ lse_rows,
                                                         const int32_t *__restrict__ seq_lens, int B, int QH, int lse_stride,
                                                         int bs, float *__restrict__ mass, int mass_stride, int accumulate)
{
    const int lb = (int)(blockIdx.x * 256 + threadIdx.x), b = blockIdx.y;
    if (lb >= mass_stride) return;
    const int len = seq_lens[b];
    const int nblk = len > 0 ? (len + bs - 1) / bs : 0;
    float *dst = mass + (size_t)b * mass_stride + lb;
    if (lb >= nblk) {
        if (!accumulate) *dst = 0.0f;
        return;
    }
    const int g0 = lb * (bs / 16), g1 = min(g0 + bs / 16, lse_stride);
    float m = 0.0f;
    for (int h = 0; h < QH; h++) {
        const float row = lse_rows[(size_t)b * QH + h];
        const float *grp = lse_groups + ((size_t)b * QH + h) * lse_stride;
        for (int gi = g0; gi < g1; gi++) {
            const float v = grp[gi];
            if (v > -INFINITY && row > -INFINITY) m += s_exp2(v - row);
        }
    }
    *dst = accumulate ? *dst + m : m;
}

int launch_block_mass(const float *lse_groups, const float *lse_rows, const int32_t *d_seq_lens, int B, int QH,
                      int lse_stride, int bs, float *mass, int mass_stride, int accumulate, hipStream_t st)
{
    hipLaunchKernelGGL(block_mass_kernel, dim3((mass_stride + 255) / 256, B), dim3(256), 0, st, lse_groups, lse_rows,
                       d_seq_lens, B, QH, lse_stride, bs, mass, mass_stride, accumulate);
    DRK_LAUNCH_CHECK("block_mass_kernel");
    return DRK_OK;
}

bool stream_decode_supported(const Lay &a, int B)
{
    // offsets inside a layer are kept in 32 bits, in units of 16 bytes, by the unit descriptors:
    // a layer of the pool may hold up to 64 GiB
    return a.D == 128 && a.QH / a.KVH == 4 && (a.bs % 16) == 0 && B >= 1 && B <= 64 &&
           a.layer_stride <= (0xffff0000ull << 4);
}

static void stream_shape(const Lay &a, int B, int max_seq_len, int split_tokens, int *grid, int *unit_tiles, int *Pmax)
{
    const long t_upper = (long)a.KVH * B * ((max_seq_len + kSTile - 1) / kSTile);
    if (split_tokens > 0) {
        const int U = split_tokens / kSTile;
        *unit_tiles = U;
        *grid = (int)((t_upper + U - 1) / U);
        *Pmax = ((max_seq_len + kSTile - 1) / kSTile + U - 1) / U + 2;
    } else {
        long G = t_upper < stream_wgs(a) ? t_upper : stream_wgs(a);
        if ((t_upper + G - 1) / G > kMaxUnits) G = (t_upper + kMaxUnits - 1) / kMaxUnits;   // descriptor table size
        *unit_tiles = 0;
        *grid = (int)G;
        *Pmax = (int)((G + a.KVH - 1) / a.KVH) + 2;
    }
}

size_t stream_workspace_need(const Lay &a, int B, int max_seq_len, int split_tokens)
{
    int grid, U, Pmax;
    stream_shape(a, B, max_seq_len, split_tokens, &grid, &U, &Pmax);
    return (size_t)B * a.QH * Pmax * (a.D + 2) * sizeof(float);
}

// launches the partial kernel; *merge_fn_args are filled for the caller to launch the merge
int launch_decode_stream(const Lay &a, const void *q, const void *pool, const int32_t *tables, int table_stride,
                         const int32_t *d_seq_lens, int seq_len_host, int B, int max_seq_len, void *out, int layer,
                         float scale, int io_dtype, int split_tokens, void *workspace, bool merge_only, hipStream_t st,
                         int start_tile, const float *pre_o, const float *pre_m, const float *pre_l, int pre_splits,
                         const void *gate, size_t gate_stride, float *lse_groups, float *lse_rows, int lse_stride)
{
    int grid, U, Pmax;
    stream_shape(a, B, max_seq_len, split_tokens, &grid, &U, &Pmax);
    float *part_o = (float *)workspace;
    float *part_m = part_o + (size_t)B * a.QH * Pmax * a.D;
    float *part_l = part_m + (size_t)B * a.QH * Pmax;
    if (!merge_only) {
        StreamArgs A;
        A.pool_layer = (const uint8_t *)pool + (size_t)layer * a.layer_stride;
        A.tables = tables; A.seq_lens = d_seq_lens; A.q = (const uint8_t *)q;
        A.part_o = part_o; A.part_m = part_m; A.part_l = part_l;
        A.table_stride = table_stride; A.seq_len_host = seq_len_host; A.B = B; A.KVH = a.KVH; A.QH = a.QH;
        A.NB = a.NB; A.bs = a.bs; A.bs_shift = ilog2_exact((unsigned)a.bs); A.io_dtype = io_dtype;
        A.unit_tiles = U; A.Pmax = Pmax; A.start_tile = start_tile;
        A.head_stride = a.head_stride; A.kv_plane = a.kv_plane; A.block_stride = a.block_stride;
        A.scale_plane = a.scale_plane; A.row_bytes = a.row_bytes;
        A.scale_log2e = scale * kSLog2e;
        A.lse_groups = lse_groups; A.lse_stride = lse_stride;
        switch (a.dtype) {
        case DRK_F16: hipLaunchKernelGGL(decode_stream_kernel<DRK_F16>, dim3(grid), dim3(256), 0, st, A); break;
        case DRK_BF16: hipLaunchKernelGGL(decode_stream_kernel<DRK_BF16>, dim3(grid), dim3(256), 0, st, A); break;
        case DRK_INT8: hipLaunchKernelGGL(decode_stream_kernel<DRK_INT8>, dim3(grid), dim3(256), 0, st, A); break;
        default: hipLaunchKernelGGL(decode_stream_kernel<DRK_FP8_E4M3>, dim3(grid), dim3(256), 0, st, A); break;
        }
        DRK_LAUNCH_CHECK("decode_stream_kernel");
    } else {
        hipLaunchKernelGGL(stream_merge_kernel, dim3(a.QH, B), dim3(256), 0, st, part_o, part_m, part_l, (uint16_t *)out,
                           d_seq_lens, seq_len_host, B, a.KVH, a.QH, U, grid, Pmax, io_dtype, start_tile, pre_o, pre_m,
                           pre_l, pre_splits, (const uint16_t *)gate, gate_stride, lse_rows);
        DRK_LAUNCH_CHECK("stream_merge_kernel");
    }
    return DRK_OK;
}

} // namespace drk
