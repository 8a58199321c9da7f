// drk_decode_stream.hip -- the production paged GQA decode kernel: persistent,
// stream-K style, for head_dim 128 or 256 with 1..16 query heads per KV head and fp16,
// bf16, int8 (+fp16 scale per token and head) or fp8-e4m3 pages.
//
// The unit of work is one 64-token tile of one (branch, kv head).  Units are
// numbered branch-major, then kv head, then tile; workgroup g owns the run
// [g*U, (g+1)*U).  Every workgroup therefore streams the same number of tiles
// whatever the branch lengths are, the whole grid is resident in one round, and a
// run that crosses from one (branch, kv head) to the next keeps its load pipeline
// full: the next unit's K/V (and the next segment's Q) are already in flight when
// the current segment's partial result is written.  A (branch, kv head) is cut
// into at most ceil(tiles/U)+1 pieces; each piece leaves (o[D], m, l) per query
// head in the workspace and stream_merge_kernel folds them.
//
// Inside the tile loop a wave never waits for another.  Wave w owns tokens [16w, 16w+16)
// of every tile with a softmax state of its own (running maximum and sum per query head,
// heads x head_dim of output), and both products run on the matrix cores with the query
// heads of the group padded to a 16-wide operand (for head_dim D):
//   S[token][head] = K[16 tokens x D dims] Q^T                  D/32 x v_mfma_f32_16x16x32
//   O[head][dim]  += P[heads x 16 tokens] V[16 tokens x D dims]   D/16 x v_mfma_f32_16x16x16
// The accumulator layout of the first product (lane = head + 16 g, registers = tokens
// 4g..4g+3) is exactly the A-operand layout of the second, so the probabilities never
// leave their lane.  K goes through a wave-private LDS region (pitch 2 D + 16 bytes) only to
// change lanes -- 16-byte chunks as loaded become one token row per lane -- and int8 /
// fp8 codes become fp16 on the way; V is loaded with tokens 4g..4g+3 of 8 dims in each
// lane and paired up by byte permutes (which is also where its codes become fp16).  The
// padding costs nothing that matters: the matrix cores are idle otherwise, and the vector
// ALU work per tile is a third of what the same products cost as v_dot2.  The four waves'
// states meet once per segment, through LDS, in the usual (o, m, l) algebra.
#include "drk_stream_tile.hpp"

namespace drk {

// Workgroups of the persistent grid on a 256-CU part; 0 = by storage type: 2 per CU
// for 16-bit pages (bandwidth-bound: fewer, longer runs stream best) and for head_dim
// 256 (all that fit), 4 per CU for 8-bit pages of head_dim 128, whose tiles are half the bytes.
int g_stream_wgs = 0;
int g_stream_stop_after_descriptors = 0;   // measurement aid (drk_debug_set_stream_descriptors_only)
static inline int stream_wgs(const Lay &a) { return g_stream_wgs > 0 ? g_stream_wgs : (a.E == 1 && a.D == 128 ? 1024 : 512); }

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
    int stop_after_descriptors;     // measurement aid: leave once the workgroup's unit descriptors are built
    uint8_t *plan;                  // the descriptors of every workgroup in global memory, see DecodePlan
    int plan_mode;                  // 0: build and use; 1: build, store, leave; 2: read
    const uint8_t *new_k, *new_v;   // or NULL: one new token per branch, [B][KVH][D] of the pages' 16-bit type, to be
                                    // written at position seq_len - 1 before the tile that holds it is read
    uint8_t *pool_layer_w;          // the layer's pages, writable (with new_k)
};

constexpr int kMaxUnits = kStreamMaxUnits;    // units one workgroup may own (descriptor table in LDS)

struct UnitDesc {                    // one 64-token tile of one (branch, kv head)
    int tile_lim;                    // tokens of the tile that exist: seq_len - tile*64 (may exceed 64)
    int flags;                       // bit 0: first tile of a segment of this workgroup, bit 1: last; bits 2..: tile index
    int bq;                          // branch*QH + kvh*(QH/KVH): first query row of the group (Q, partial slots)
    int piece;                       // partial slot of the segment inside its (branch, q head)
};

// G4: at most 4 query heads per kv head -- they all live in lane group 0 of the accumulators, so
// per-head factors are wave-uniform (v_readlane) and a segment ends in one round.
template <int DT, int D, bool G4>
__global__ __launch_bounds__(256, D == 128 ? 4 : 2) void decode_stream_kernel(StreamArgs A)
{
    using Geo = StreamGeo<DT, D>;
    [[maybe_unused]] constexpr bool Q8 = Geo::q8;
    constexpr int DOT = KvTraits<DT>::dot;
    constexpr uint32_t kNone = 0xffffffffu;
    __shared__ __align__(16) uint8_t k_lds[4][16 * Geo::PITCH];
    __shared__ __align__(16) float o_lds[4][4][D];            // [wave][head of the round][dim], segment ends only
    __shared__ float mw_lds[4][16], lw_lds[4][16];
    __shared__ __align__(16) UnitDesc udesc[kMaxUnits];
    __shared__ __align__(16) uint2 gdesc[kMaxUnits][4];
    __shared__ int s_incl[64], s_len[64];

    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4, c = lane & 15;
    const int GQ = A.QH / A.KVH;                               // query heads per kv head, 1..16
    // ---- the workgroup's run of units and one descriptor per unit ---------------------
    int nunits = 0;
    if (A.plan_mode == 2) {
        nunits = plan_load<UnitDesc, kMaxUnits>(A.plan, udesc, gdesc);
    } else {
        const int len_i = lane < A.B ? (A.seq_lens ? A.seq_lens[lane] : A.seq_len_host) : 0;
        const int nt_i = len_i > 0 ? max((len_i + kSTile - 1) / kSTile - A.start_tile, 0) : 0;
        int incl = nt_i;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        const int T = __builtin_amdgcn_readlane(incl, 63) * A.KVH;
        const int U = A.unit_tiles > 0 ? A.unit_tiles : (T + (int)gridDim.x - 1) / (int)gridDim.x;
        const int u0 = (int)blockIdx.x * U;
        // the host sizes U from max_seq_len; a length on the device beyond that bound must not overrun the
        // descriptor table (the tiles past it are then left out: the caller broke its promise)
        nunits = (T == 0 || u0 >= T) ? 0 : min(min(U, T - u0), kMaxUnits);
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
                d.bq = b * A.QH + kvh * GQ;
                d.piece = (int)blockIdx.x - (A.KVH * excl + kvh * nt) / U;
                udesc[ui] = d;
            }
        }
        __syncthreads();
        if (A.plan_mode == 1) {
            plan_store<UnitDesc, kMaxUnits>(A.plan, nunits, udesc, gdesc);
            return;
        }
    }
    if (nunits == 0) return;
    if (A.new_k) {
        // The step's append, folded in: the unit that is a (branch, kv head)'s last tile holds the new token's
        // position, and only this workgroup reads that tile -- so it writes the row itself, K and V, 16 bytes per
        // thread, before its first request.  The barrier below orders the stores before the loads of every wave of
        // the workgroup (one CU, one vector cache in front of the L2 the stores went to).  A missing page is
        // skipped, as the append kernel skips it.
        if constexpr (!KvTraits<DT>::q8) {
            constexpr int CH = D * 2 / 16;                       // 16-byte chunks per row
            for (int i = threadIdx.x; i < nunits * 2 * CH; i += 256) {
                const int ui = i / (2 * CH), rest = i - ui * (2 * CH), kv = rest / CH, ch = rest - kv * CH;
                const UnitDesc ud = udesc[ui];
                if (ud.tile_lim < 1 || ud.tile_lim > kSTile) continue;           // not the last tile of its run
                const int r = ud.tile_lim - 1;
                const uint32_t gx = gdesc[ui][r >> 4].x;
                if (gx == kNone) continue;
                const int b = ud.bq / A.QH, kvh = (ud.bq - b * A.QH) / GQ;
                const uint8_t *src = (kv ? A.new_v : A.new_k) + ((size_t)(b * A.KVH + kvh) * D * 2) + ch * 16;
                uint8_t *dst = A.pool_layer_w + ((size_t)gx << 4) + (size_t)(r & 15) * A.row_bytes + (kv ? A.kv_plane : 0) + ch * 16;
                *(uint4 *)dst = *(const uint4 *)src;
            }
        }
        __syncthreads();
    }
    if (A.stop_after_descriptors) return;

    uint8_t *const klds = &k_lds[w][0];
    // the 4 K scales and the 4 V scales of tokens 4g..4g+3 (int8 pages)
    auto load_scales = [&](uint2 gd, uint2 &ks, uint2 &vs) {
        if (DT != DRK_INT8) return;
        const uint8_t *p = A.pool_layer + ((size_t)(gd.x == kNone ? 0u : gd.y) << 4) + g * 8;
        ks = *(const uint2 *)p;
        vs = *(const uint2 *)(p + A.scale_plane);
    };

    w_f32x4 o[Geo::NPV];
#pragma unroll
    for (int e = 0; e < Geo::NPV; e++) o[e] = w_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY, l_lane = 0.0f, ps_lane = 0.0f, qbias = 0.0f;
    uint4 qop[Geo::NQK];

    uint2 gd = gdesc[0][w], ksr = {}, vsr = {};
    KRegs<DT, D> kreg = load_k<DT, D>(A.pool_layer, gd.x, lane);
    VRegs<DT, D> vreg = load_v<DT, D>(A.pool_layer, gd.x, A.kv_plane, lane);
    load_scales(gd, ksr, vsr);

    for (int it = 0; it < nunits; it++) {
        const UnitDesc ud = udesc[it];
        const int flags = __builtin_amdgcn_readfirstlane(ud.flags);
        const int tile_lim = __builtin_amdgcn_readfirstlane(ud.tile_lim);
        const bool hole = __builtin_amdgcn_readfirstlane((int)gd.x) == (int)kNone;   // the group the registers were loaded for
        const int lim = hole ? 0 : tile_lim;                    // tokens of the tile this wave may look at
        const bool has_next = it + 1 < nunits;
        if (flags & 1) {
            // Q^T as the B operand: lane (head c, dims 32 kk + 8 g ..) -- heads GQ..15 are padding
            float sq = 0.0f;
#pragma unroll
            for (int kk = 0; kk < Geo::NQK; kk++) {
                uint4 v = make_uint4(0u, 0u, 0u, 0u);
                if (c < GQ) v = *(const uint4 *)(A.q + (size_t)(ud.bq + c) * (D * 2) + kk * 64 + g * 16);
#if defined(__HIP_DEVICE_COMPILE__)
                if (Q8 && A.io_dtype == DRK_BF16) {          // quantised pages multiply in fp16
                    v.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.x), bf16_hi(v.x)));
                    v.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.y), bf16_hi(v.y)));
                    v.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.z), bf16_hi(v.z)));
                    v.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.w), bf16_hi(v.w)));
                }
#endif
                qop[kk] = v;
                if (DT == DRK_INT8) {
                    sq = s_dot2<DOT>(v.x, kF16Ones, sq);
                    sq = s_dot2<DOT>(v.y, kF16Ones, sq);
                    sq = s_dot2<DOT>(v.z, kF16Ones, sq);
                    sq = s_dot2<DOT>(v.w, kF16Ones, sq);
                }
            }
            if (DT == DRK_INT8) {                            // sum of the head's query values, for the code offset
                sq += __shfl_xor(sq, 16);
                sq += __shfl_xor(sq, 32);
                qbias = kI8Bias * sq;
            }
        }

        // ---- K: registers -> the wave's LDS rows -> one token row per lane; next K loads ----
        stage_k<DT, D>(klds, kreg, lane);
        float ks[4] = {1.0f, 1.0f, 1.0f, 1.0f}, vs[4] = {1.0f, 1.0f, 1.0f, 1.0f};
        if (DT == DRK_INT8) {
            ks[0] = f16_bits_to_f((uint16_t)(ksr.x & 0xffffu)); ks[1] = f16_bits_to_f((uint16_t)(ksr.x >> 16));
            ks[2] = f16_bits_to_f((uint16_t)(ksr.y & 0xffffu)); ks[3] = f16_bits_to_f((uint16_t)(ksr.y >> 16));
            vs[0] = f16_bits_to_f((uint16_t)(vsr.x & 0xffffu)); vs[1] = f16_bits_to_f((uint16_t)(vsr.x >> 16));
            vs[2] = f16_bits_to_f((uint16_t)(vsr.y & 0xffffu)); vs[3] = f16_bits_to_f((uint16_t)(vsr.y >> 16));
        }
        if (has_next) {
            gd = gdesc[it + 1][w];
            kreg = load_k<DT, D>(A.pool_layer, gd.x, lane);
            load_scales(gd, ksr, vsr);
        }
        w_f32x4 sacc = {0.0f, 0.0f, 0.0f, 0.0f};
        {
            const uint8_t *arow = klds + c * Geo::PITCH + g * 16;
#pragma unroll
            for (int k0 = 0; k0 < Geo::NQK; k0 += 4) {
                uint4 ka[4];
#pragma unroll
                for (int kk = 0; kk < 4; kk++) ka[kk] = *(const uint4 *)(arow + (k0 + kk) * 64);
#pragma unroll
                for (int kk = 0; kk < 4; kk++) sacc = w_mfma_qk<DOT>(ka[kk], qop[k0 + kk], sacc);
            }
        }

        // ---- softmax of head c over this wave's tokens 4g..4g+3 (+ the other three lane groups) ----
        const int t0 = w * 16 + g * 4;
        float sc[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float x = sacc[j];
            if (DT == DRK_INT8) x = (x - qbias) * ks[j];
            x *= A.scale_log2e;
            sc[j] = t0 + j < lim ? x : -INFINITY;
        }
        float mloc = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 16));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
        const float m_new = fmaxf(m_run, mloc);
        const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha = s_exp2(m_run - m_use);
        m_run = m_new;
        float p[4];
#pragma unroll
        for (int j = 0; j < 4; j++) p[j] = s_exp2(sc[j] - m_use);
        uint2 pa;                                             // A operand of the second product: P[head c][tokens 4g..4g+3]
        {
            float pw[4];
#pragma unroll
            for (int j = 0; j < 4; j++) pw[j] = (DT == DRK_INT8) ? (t0 + j < lim ? p[j] * vs[j] : 0.0f) : p[j];
            if constexpr (DOT == DRK_BF16) {
                pa.x = (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)pw[0]) | ((uint32_t)__builtin_bit_cast(uint16_t, (__bf16)pw[1]) << 16);
                pa.y = (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)pw[2]) | ((uint32_t)__builtin_bit_cast(uint16_t, (__bf16)pw[3]) << 16);
            } else {
                pa.x = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)pw[0]) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)pw[1]) << 16);
                pa.y = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)pw[2]) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)pw[3]) << 16);
            }
            if (DT == DRK_INT8) {                             // sum of the weights as the product sees them, for the code offset
                float t = s_dot2<DOT>(pa.x, kF16Ones, 0.0f);
                t = s_dot2<DOT>(pa.y, kF16Ones, t);
                ps_lane = fmaf(ps_lane, alpha, t);
            }
        }
        // The row's denominator is the sum of the weights the second product multiplies -- the rounded
        // ones, as in the prefill kernel -- so that numerator and denominator carry the same rounding.
        // (int8: the product multiplies p times the V scale, rounded; its sum of plain p stays exact.)
        float rs;
        if (DT == DRK_INT8) rs = (p[0] + p[1]) + (p[2] + p[3]);
        else rs = s_dot2<DOT>(pa.y, DOT == DRK_BF16 ? kBf16Ones : kF16Ones, s_dot2<DOT>(pa.x, DOT == DRK_BF16 ? kBf16Ones : kF16Ones, 0.0f));
        l_lane = fmaf(l_lane, alpha, rs);
        if (A.lse_groups) {
            float rt = rs;
            rt += __shfl_xor(rt, 16);
            rt += __shfl_xor(rt, 32);
            const int gi = (flags >> 2) * 4 + w;
            if (lane < GQ && gi < A.lse_stride)
                A.lse_groups[(size_t)(ud.bq + lane) * A.lse_stride + gi] = rt > 0.0f ? m_use + __builtin_log2f(rt) : -INFINITY;
        }

        // ---- O: rescale (register j of lane group g holds head 4g + j), then P V ----------------
        {
            if constexpr (G4) {
                const float a0 = s_lane(alpha, 0), a1 = s_lane(alpha, 1), a2 = s_lane(alpha, 2), a3 = s_lane(alpha, 3);
                if (a0 != 1.0f || a1 != 1.0f || a2 != 1.0f || a3 != 1.0f) {
#pragma unroll
                    for (int e = 0; e < Geo::NPV; e++) { o[e][0] *= a0; o[e][1] *= a1; o[e][2] *= a2; o[e][3] *= a3; }
                }
            } else if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
                const float a0 = __shfl(alpha, 4 * g), a1 = __shfl(alpha, 4 * g + 1);
                const float a2 = __shfl(alpha, 4 * g + 2), a3 = __shfl(alpha, 4 * g + 3);
#pragma unroll
                for (int e = 0; e < Geo::NPV; e++) { o[e][0] *= a0; o[e][1] *= a1; o[e][2] *= a2; o[e][3] *= a3; }
            }
            if (DT != DRK_INT8 && w * 16 + 16 > lim) {               // rows without a token may hold anything (NaN)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (t0 + j >= lim) {
#pragma unroll
                        for (int ch = 0; ch < Geo::NCH; ch++) vreg.r[j][ch] = {};
                    }
            }
#pragma unroll
            for (int ch = 0; ch < Geo::NCH; ch++) {
                uint2 vb[8];
                v_operands<DT>(vreg.r[0][ch], vreg.r[1][ch], vreg.r[2][ch], vreg.r[3][ch], vb);
#pragma unroll
                for (int e = 0; e < 8; e++) o[ch * 8 + e] = w_mfma_pv<DOT>(pa, vb[e], o[ch * 8 + e]);
            }
        }
        if (has_next) vreg = load_v<DT, D>(A.pool_layer, gd.x, A.kv_plane, lane);

        // ---- the segment's last tile: fold the four waves, leave (o, m, l) for the merge ----
        if (flags & 2) {
            float lw = l_lane, pw = ps_lane;
            lw += __shfl_xor(lw, 16);
            lw += __shfl_xor(lw, 32);
            if (DT == DRK_INT8) {
                pw += __shfl_xor(pw, 16);
                pw += __shfl_xor(pw, 32);
            }
            if (lane < 16) { mw_lds[w][lane] = m_run; lw_lds[w][lane] = lw; }   // padded heads too: defined values
            __syncthreads();
            float f_own[4], bias[4];                                 // this wave's weight / code offset for head 4g + j
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int h = G4 ? j : 4 * g + j;
                const float M = fmaxf(fmaxf(mw_lds[0][h], mw_lds[1][h]), fmaxf(mw_lds[2][h], mw_lds[3][h]));
                const float mo = mw_lds[w][h];
                f_own[j] = mo == -INFINITY ? 0.0f : s_exp2(mo - M);
                if constexpr (G4) bias[j] = DT == DRK_INT8 ? kI8Bias * s_lane(pw, j) : 0.0f;
                else bias[j] = DT == DRK_INT8 ? kI8Bias * __shfl(pw, h) : 0.0f;
            }
            const int rounds = G4 ? 1 : (GQ + 3) >> 2;               // 4 heads per round: head 4r + w is stored by wave w
            for (int r = 0; r < rounds; r++) {
                if (r > 0) __syncthreads();                          // the previous round's sums have been read
                if (g == r) {
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int ch = 0; ch < Geo::NCH; ch++) {
                            float *dst = &o_lds[w][j][ch * 128 + c * 8];
                            const w_f32x4 *oc = &o[ch * 8];
                            *(float4 *)dst = make_float4((oc[0][j] - bias[j]) * f_own[j], (oc[1][j] - bias[j]) * f_own[j],
                                                         (oc[2][j] - bias[j]) * f_own[j], (oc[3][j] - bias[j]) * f_own[j]);
                            *(float4 *)(dst + 4) = make_float4((oc[4][j] - bias[j]) * f_own[j], (oc[5][j] - bias[j]) * f_own[j],
                                                               (oc[6][j] - bias[j]) * f_own[j], (oc[7][j] - bias[j]) * f_own[j]);
                        }
                }
                // (m, l) of head 4r + w over the four waves; read here, before the barrier, because a wave
                // that is through with this segment may overwrite its slots for the next one
                const int h = 4 * r + w;
                const float M = fmaxf(fmaxf(mw_lds[0][h], mw_lds[1][h]), fmaxf(mw_lds[2][h], mw_lds[3][h]));
                float L = 0.0f;
#pragma unroll
                for (int ww = 0; ww < 4; ww++) {
                    const float mm = mw_lds[ww][h];
                    if (mm != -INFINITY) L = fmaf(lw_lds[ww][h], s_exp2(mm - M), L);
                }
                __syncthreads();
                if (h < GQ) {
                    constexpr int VEC = D / 64;
                    const int d = lane * VEC;
                    float acc[VEC];
#pragma unroll
                    for (int x = 0; x < VEC; x++) acc[x] = 0.0f;
#pragma unroll
                    for (int ww = 0; ww < 4; ww++)
#pragma unroll
                        for (int x = 0; x < VEC; x++) acc[x] += o_lds[ww][w][d + x];
                    const size_t pi = (size_t)(ud.bq + h) * A.Pmax + ud.piece;
#pragma unroll
                    for (int x = 0; x < VEC; x++) A.part_o[pi * D + d + x] = acc[x];
                    if (lane == 0) {
                        A.part_m[pi] = M;
                        A.part_l[pi] = L;
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < Geo::NPV; e++) o[e] = w_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            m_run = -INFINITY;
            l_lane = 0.0f;
            ps_lane = 0.0f;
        }
    }
}

// grid (QH, B), block 256: fold the pieces of (branch, q head) -- the stream kernel's
// and, in shared-prefix mode, the prefix pass's; out is written only when some
// token took part (paged_attention.cu:266).  Lane s of every wave owns the (m, l) of
// piece s (+64, ...), so they arrive in one round of loads; wave w then folds the o
// rows of pieces w, w+4, ... for two dims per lane, eight rows in flight, and the four
// waves' sums meet in LDS.
template <int D>
__global__ __launch_bounds__(256) void stream_merge_kernel(const float *__restrict__ part_o, const float *__restrict__ part_m,
                                                           const float *__restrict__ part_l, uint16_t *__restrict__ out,
                                                           const int32_t *__restrict__ seq_lens, int seq_len_host, int B,
                                                           int KVH, int QH, int unit_tiles, int grid_wgs, int Pmax,
                                                           int io_dtype, int start_tile, const float *__restrict__ pre_o,
                                                           const float *__restrict__ pre_m, const float *__restrict__ pre_l,
                                                           int pre_splits, const uint16_t *__restrict__ gate,
                                                           size_t gate_stride, float *__restrict__ lse_rows)
{
    constexpr int VEC = D / 64;                                  // dims per lane: 2 or 4
    typedef float fvec __attribute__((ext_vector_type(VEC)));
    __shared__ fvec red[4][64];
    const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x & 63, wv = threadIdx.x >> 6, d = lane * VEC;
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
    fvec acc = {};
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
            fvec o[8];
            float wj[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int jj = min(j + 4 * u, cnt - 1), sj = c0 + jj;
                wj[u] = j + 4 * u < cnt ? s_lane(w, jj) : 0.0f;
                o[u] = *(const fvec *)(sj < npieces ? part_o + (base + sj) * D + d : pre_o + (pbase + (sj - npieces)) * D + d);
            }
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (wj[u] != 0.0f) {                                  // a piece without tokens may hold anything
#pragma unroll
                    for (int x = 0; x < VEC; x++) acc[x] = fmaf(o[u][x], wj[u], acc[x]);
                }
        }
    }
    L = s_wave_sum(L);
    if (lse_rows && threadIdx.x == 0) lse_rows[(size_t)b * QH + h] = L > 0.0f ? M + __builtin_log2f(L) : -INFINITY;
    red[wv][lane] = acc;
    __syncthreads();
    if (wv == 0) {
        // with a gate the row is always rewritten: the reference gates whatever the attention
        // kernel left in out, also when no token took part (paged_attention.cu:266, 368-370)
        uint16_t *dst = out + ((size_t)b * QH + h) * D + d;
        uint16_t vals[VEC];
        if (L > 0.0f) {
            const fvec a1 = red[1][lane], a2 = red[2][lane], a3 = red[3][lane];
#pragma unroll
            for (int x = 0; x < VEC; x++) vals[x] = f_to_elem16(((acc[x] + a1[x]) + (a2[x] + a3[x])) / L, io_dtype);
        } else {
            if (!gate) return;
#pragma unroll
            for (int x = 0; x < VEC; x++) vals[x] = dst[x];
        }
        if (gate) {
            const uint16_t *gp = gate + ((size_t)b * QH + h) * gate_stride + d;
#pragma unroll
            for (int x = 0; x < VEC; x++) vals[x] = gated_elem16(vals[x], gp[x], io_dtype);
        }
        if constexpr (VEC == 2) {
            *(uint32_t *)dst = (uint32_t)vals[0] | ((uint32_t)vals[1] << 16);
        } else {
            *(uint2 *)dst = make_uint2((uint32_t)vals[0] | ((uint32_t)vals[1] << 16), (uint32_t)vals[2] | ((uint32_t)vals[3] << 16));
        }
    }
}

// Attention mass per (branch, logical block): sum over the block's tokens and all query heads of
// the softmax probability, from the per-group and per-row log-sum-exps the two kernels above
// left.  A workgroup takes 64 blocks of one branch; wave w sums the heads w, w+4, ... (consecutive
// lanes read consecutive groups), the four sums meet in LDS.
__global__ __launch_bounds__(256) void block_mass_kernel(const float *__restrict__ lse_groups, const float *__restrict__ lse_rows,
                                                         const int32_t *__restrict__ seq_lens, int B, int QH, int lse_stride,
                                                         int bs, float *__restrict__ mass, int mass_stride, int accumulate)
{
    __shared__ float part[4][64];
    const int x = threadIdx.x & 63, hq = threadIdx.x >> 6;
    const int lb = (int)blockIdx.x * 64 + x, b = blockIdx.y;
    const int len = seq_lens[b];
    const int nblk = len > 0 ? (len + bs - 1) / bs : 0;
    float m = 0.0f;
    if (lb < nblk) {
        // only the groups of tiles that exist were written by this launch (a block may span several tiles)
        const int g0 = lb * (bs / 16), g1 = min(min(g0 + bs / 16, lse_stride), ((len + kSTile - 1) / kSTile) * 4);
        for (int h = hq; h < QH; h += 4) {
            const float row = lse_rows[(size_t)b * QH + h];
            const float *grp = lse_groups + ((size_t)b * QH + h) * lse_stride;
            for (int gi = g0; gi < g1; gi++) {
                const float v = grp[gi];
                if (v > -INFINITY && row > -INFINITY) m += s_exp2(v - row);
            }
        }
    }
    part[hq][x] = m;
    __syncthreads();
    if (hq != 0 || lb >= mass_stride) return;
    float *dst = mass + (size_t)b * mass_stride + lb;
    if (lb >= nblk) {
        if (!accumulate) *dst = 0.0f;
        return;
    }
    m = (part[0][x] + part[1][x]) + (part[2][x] + part[3][x]);
    *dst = accumulate ? *dst + m : m;
}

int launch_block_mass(const float *lse_groups, const float *lse_rows, const int32_t *d_seq_lens, int B, int QH,
                      int lse_stride, int bs, float *mass, int mass_stride, int accumulate, hipStream_t st)
{
    hipLaunchKernelGGL(block_mass_kernel, dim3((mass_stride + 63) / 64, B), dim3(256), 0, st, lse_groups, lse_rows,
                       d_seq_lens, B, QH, lse_stride, bs, mass, mass_stride, accumulate);
    DRK_LAUNCH_CHECK("block_mass_kernel");
    return DRK_OK;
}

bool stream_decode_supported(const Lay &a, int B)
{
    // offsets inside a layer are kept in 32 bits, in units of 16 bytes, by the unit descriptors:
    // a layer of the pool may hold up to 64 GiB
    return (a.D == 128 || a.D == 256) && a.KVH > 0 && a.QH % a.KVH == 0 && a.QH / a.KVH <= 16 && (a.bs % 16) == 0 &&
           B >= 1 && B <= 64 && a.layer_stride <= (0xffff0000ull << 4);
}

static void stream_shape(const Lay &a, int B, int max_seq_len, int split_tokens, int start_tile, int *grid, int *unit_tiles,
                         int *Pmax)
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
        // a branch's run of n tiles meets at most n + 1 workgroups: short private tails behind a long
        // shared prefix (start_tile > 0) need far fewer pieces than the grid could give one branch
        const int tail_tiles = (max_seq_len + kSTile - 1) / kSTile - start_tile;
        if (start_tile > 0 && tail_tiles + 2 < *Pmax) *Pmax = (tail_tiles > 0 ? tail_tiles : 0) + 2;
    }
}

size_t stream_plan_need(const Lay &a, int B, int max_seq_len)
{
    int grid, U, Pmax;
    stream_shape(a, B, max_seq_len, 0, 0, &grid, &U, &Pmax);
    return (size_t)grid * plan_record_bytes(kMaxUnits);
}

size_t stream_workspace_need(const Lay &a, int B, int max_seq_len, int split_tokens, int start_tile)
{
    int grid, U, Pmax;
    stream_shape(a, B, max_seq_len, split_tokens, start_tile, &grid, &U, &Pmax);
    return (size_t)B * a.QH * Pmax * (a.D + 2) * sizeof(float);
}

// launches the partial kernel; *merge_fn_args are filled for the caller to launch the merge
int launch_decode_stream(const Lay &a, const void *q, const void *pool, const int32_t *tables, int table_stride,
                         const int32_t *d_seq_lens, int seq_len_host, int B, int max_seq_len, void *out, int layer,
                         float scale, int io_dtype, int split_tokens, void *workspace, bool merge_only, hipStream_t st,
                         int start_tile, const float *pre_o, const float *pre_m, const float *pre_l, int pre_splits,
                         const void *gate, size_t gate_stride, float *lse_groups, float *lse_rows, int lse_stride,
                         DecodePlan plan)
{
    int grid, U, Pmax;
    stream_shape(a, B, max_seq_len, split_tokens, start_tile, &grid, &U, &Pmax);
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
        A.stop_after_descriptors = g_stream_stop_after_descriptors;
        A.plan = plan.ptr; A.plan_mode = plan.ptr ? plan.mode : 0;
        const bool fused_append = plan.new_k && plan.new_v && a.E == 2 && start_tile == 0 && plan.mode != 1;
        A.new_k = fused_append ? plan.new_k : nullptr;
        A.new_v = fused_append ? plan.new_v : nullptr;
        A.pool_layer_w = (uint8_t *)const_cast<void *>(pool) + (size_t)layer * a.layer_stride;
#define DRK_STREAM_LAUNCH(DT)                                                                                           \
    do {                                                                                                                \
        const bool g4 = a.QH / a.KVH <= 4;                                                                              \
        if (a.D == 128 && g4) hipLaunchKernelGGL((decode_stream_kernel<DT, 128, true>), dim3(grid), dim3(256), 0, st, A);   \
        else if (a.D == 128) hipLaunchKernelGGL((decode_stream_kernel<DT, 128, false>), dim3(grid), dim3(256), 0, st, A);   \
        else if (g4) hipLaunchKernelGGL((decode_stream_kernel<DT, 256, true>), dim3(grid), dim3(256), 0, st, A);            \
        else hipLaunchKernelGGL((decode_stream_kernel<DT, 256, false>), dim3(grid), dim3(256), 0, st, A);                   \
    } while (0)
        switch (a.dtype) {
        case DRK_F16: DRK_STREAM_LAUNCH(DRK_F16); break;
        case DRK_BF16: DRK_STREAM_LAUNCH(DRK_BF16); break;
        case DRK_INT8: DRK_STREAM_LAUNCH(DRK_INT8); break;
        default: DRK_STREAM_LAUNCH(DRK_FP8_E4M3); break;
        }
#undef DRK_STREAM_LAUNCH
        DRK_LAUNCH_CHECK("decode_stream_kernel");
    } else {
        if (a.D == 128)
            hipLaunchKernelGGL(stream_merge_kernel<128>, dim3(a.QH, B), dim3(256), 0, st, part_o, part_m, part_l, (uint16_t *)out,
                               d_seq_lens, seq_len_host, B, a.KVH, a.QH, U, grid, Pmax, io_dtype, start_tile, pre_o, pre_m,
                               pre_l, pre_splits, (const uint16_t *)gate, gate_stride, lse_rows);
        else
            hipLaunchKernelGGL(stream_merge_kernel<256>, dim3(a.QH, B), dim3(256), 0, st, part_o, part_m, part_l, (uint16_t *)out,
                               d_seq_lens, seq_len_host, B, a.KVH, a.QH, U, grid, Pmax, io_dtype, start_tile, pre_o, pre_m,
                               pre_l, pre_splits, (const uint16_t *)gate, gate_stride, lse_rows);
        DRK_LAUNCH_CHECK("stream_merge_kernel");
    }
    return DRK_OK;
}

} // namespace drk
