// drk_decode_group.hip -- paged GQA decode for branches that share pages: one persistent,
// stream-K style launch over shared and private tiles alike.
//
// Decode branches forked copy-on-write from one context hold the same physical pages for
// the tokens before their fork points: a tree of shared ranges ("groups": branches
// [first, first + count) hold tokens [begin, end) in the same pages) with a private tail
// per branch behind it.  A shared range is streamed from HBM once for all its branches:
// the unit of work is, as in decode_stream_kernel, one 64-token tile of one kv head, and
// a tile of a shared range serves up to 64 query rows (branches x query heads of the kv
// head, in row groups of 16 = one matrix-core operand each) where a private tile serves
// the one branch's heads.  Units are numbered groups first (kv head, then tile), then the
// tails (branch, kv head, tile); workgroup g owns the run [g*U, (g+1)*U), so every
// workgroup streams the same number of bytes whatever the shape of the tree is, the grid is
// resident in one round, and shared and private tiles are in flight side by side.
//
// Per wave and tile (the wave owns 16 of the tile's 64 tokens, as in the stream kernel):
//   K rows through the wave's LDS region into the A operand, once for all row groups;
//   per row group: S = K Q^T (Q from LDS, loaded once per segment), softmax state of its
//   own, P packed in place; V operands by byte permutes, once; per row group O += P V.
// A segment (the run's tiles of one kv head of one group or tail) ends with the four waves'
// states folded through LDS, 16 rows per round, and (o, m, l) per query row left in the
// workspace slot of this piece; group_merge_kernel folds a row's pieces -- those of every
// group the branch belongs to and those of its tail.
#include "drk_stream_tile.hpp"

#include <type_traits>

namespace drk {

int g_grouped_mode = 0;                        // diagnostic: 0 auto, 1 never (the prefix pass + tail kernel pair), see drk_debug.h

constexpr int kGMaxGroups = DRK_MAX_PREFIX_GROUPS;
constexpr int kGMaxUnits = 128;                // 64-token tiles one workgroup may own (descriptor table in LDS)
constexpr int kGMaxPieces = 2048;              // pieces the merge folds for one query row
constexpr int kGWgs = 512;                     // two workgroups per CU of a 256-CU part: all that fit

struct GSeg {                                  // one shared range, in tiles
    int first, count;                          // branches [first, first + count)
    int tile0, ntile;                          // tiles [tile0, tile0 + ntile)
    int slot;                                  // first workspace slot of its pieces in each of its rows
    int unit0;                                 // its first unit: kv head h's tiles are units [unit0 + h*ntile, +ntile)
};

struct GroupedArgs {
    const uint8_t *pool_layer;                 // pool + layer * layer_stride
    const int32_t *tables;
    const int32_t *seq_lens;                   // [B], on the device
    const uint8_t *q;
    float *part_o, *part_m, *part_l;
    int table_stride, B, KVH, QH, NB, bs, bs_shift, io_dtype;
    int Ptot;                                  // workspace slots per (branch, q head)
    int ngroups, group_units;                  // units of all groups together
    unsigned head_stride, kv_plane, block_stride, scale_plane, row_bytes;
    float scale_log2e;
    GSeg seg[kGMaxGroups];
    int b_start[64];                           // first tile of each branch's private tail
    int b_slot[64];                            // first workspace slot of the tail's pieces
    uint8_t *plan;                             // the descriptors of every workgroup in global memory, see DecodePlan
    int plan_mode;                             // 0: build and use; 1: build, store, leave (build_units returns 0); 2: read
    int max_units;                             // the descriptor table of the kernel that takes the call: no workgroup's run is longer
    // or NULL: one new token per branch, [B][KVH][D] of the pages' 16-bit type, written by the workgroup that owns the
    // last tile of the branch's tail before it reads that tile (decode_group16_kernel only)
    const uint8_t *new_k, *new_v;
    uint8_t *pool_layer_w;                     // the layer's pages, writable (with new_k)
};

struct GUnit {                                 // one 64-token tile of one kv head of a group or a tail
    int tile_lim;                              // tokens of the tile that exist for every row (may exceed 64)
    int flags;                                 // bit 0: first tile of a segment of this workgroup, bit 1: last; bits 8..15: query rows
    int row0;                                  // first_branch*QH + kvh*(QH/KVH): query row R is row0 + (R / GQ)*QH + R % GQ
    int slot;                                  // workspace slot of the segment's piece in each of its rows
};

// Reductions over the four lane groups (lanes c, c + 16, c + 32, c + 48) with the row swaps of gfx950:
// no trip through LDS.
__device__ __forceinline__ float max_lane_groups(float x)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
#endif
    return x;
}
__device__ __forceinline__ float sum_lane_groups(float x)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(a[0]) + __uint_as_float(a[1]);
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(b[0]) + __uint_as_float(b[1]);
#endif
    return x;
}

// Maximum of the four scores a lane holds, read straight out of the matrix cores' result registers.  Assembly
// spares the canonicalising copy the compiler puts in front of every fmaxf of a value it has not produced with
// a vector instruction -- but the compiler does not look into assembly for the wait states a read of a matrix
// result needs behind the product that writes it (it pads its own reads with s_nop), and it is free to place
// that product right in front of this statement, so the wait states are here: without them the maximum is
// taken of what the registers held before the product.
__device__ __forceinline__ float max4_asm(float a, float b, float c, float d)
{
#if defined(__HIP_DEVICE_COMPILE__)
    float r;
    asm volatile("s_nop 7\n\ts_nop 7\n\tv_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %4" : "=&v"(r) : "v"(a), "v"(b), "v"(c), "v"(d));
    return r;
#else
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
#endif
}
// two fp32 -> one dword of the 16-bit type the products run in, round to nearest even, one instruction
typedef float g_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 g_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 g_f16x2 __attribute__((ext_vector_type(2)));
template <int DOT>
__device__ __forceinline__ uint32_t pack16(float a, float b)
{
    const g_f32x2 v = {a, b};
    if constexpr (DOT == DRK_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, g_bf16x2));
    else return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, g_f16x2));
}

// how far (in bits of the exponent) a row's maximum may run ahead of the reference its weights are taken to
constexpr float kLazy = 5.0f;

// The grid is dealt to the two kinds of units by what they cost: a tile of a shared range (its waves meet at two
// barriers) takes about 13 parts of time where a tile of a private tail takes 12 -- and every tail (one kv head of one
// branch: its own query rows, its first tile's latency, its own partial results) 16 more, which is what counts right
// after a fork, when 128 tails of one tile each wait behind a long prefix (dealt by tiles alone they went to 7 of 512
// workgroups, 19 each, and the launch took 77 us instead of 50; with 4 / 8 / 16 / 24 more per tail a step of 36 such
// layers takes 2.79 / 2.63 / 2.50 / 2.51 ms).  Workgroups [0, Gs) take runs of Us units of the
// shared ranges, the others runs of Ut units of the tails; neither run is longer than the kernel's descriptor table
// (`cap`).  Kernel and merge compute it alike.
struct RegionSplit { int Gs, Us, Ut; };
__host__ __device__ inline RegionSplit region_split(int group_units, int tail_units, int tail_runs, int grid, int cap)
{
    RegionSplit r;
    const long long cs = 13LL * group_units, ct = 12LL * tail_units + 16LL * tail_runs;
    if (group_units <= 0) r.Gs = 0;
    else if (tail_units <= 0 || grid < 2) r.Gs = grid;
    else {
        long long gs = (cs * grid + (cs + ct) / 2) / (cs + ct);
        r.Gs = (int)(gs < 1 ? 1 : (gs > grid - 1 ? grid - 1 : gs));
        const int lo = (group_units + cap - 1) / cap, hi = grid - (tail_units + cap - 1) / cap;
        if (lo <= hi) r.Gs = r.Gs < lo ? lo : (r.Gs > hi ? hi : r.Gs);
    }
    r.Us = r.Gs > 0 ? (group_units + r.Gs - 1) / r.Gs : 1;
    r.Ut = grid - r.Gs > 0 ? (tail_units + (grid - r.Gs) - 1) / (grid - r.Gs) : 1;
    if (r.Us < 1) r.Us = 1;
    if (r.Ut < 1) r.Ut = 1;
    return r;
}

// The workgroup's run of units and one descriptor per unit, in LDS: returns how many (0: nothing to do).
// Every thread of the workgroup must call it (it holds barriers).
template <int MAXU>
__device__ __forceinline__ int build_units(const GroupedArgs &A, GUnit *udesc, uint2 (*gdesc)[4], int *s_incl, int *s_len, int *s_gmin)
{
    constexpr uint32_t kNone = 0xffffffffu;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int GQ = A.QH / A.KVH;
    if (A.plan_mode == 2) return plan_load<GUnit, MAXU>(A.plan, udesc, gdesc);
    // ---- the workgroup's run of units and one descriptor per unit ---------------------
    const int len_i = lane < A.B ? A.seq_lens[lane] : 0;
    const int nt_i = len_i > 0 ? max((len_i + kSTile - 1) / kSTile - A.b_start[lane], 0) : 0;
    int incl = nt_i;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int t = __shfl_up(incl, off);
        if (lane >= off) incl += t;
    }
    const int tail_units = __builtin_amdgcn_readlane(incl, 63) * A.KVH;
    const int tail_runs = __popcll(__builtin_amdgcn_ballot_w64(nt_i > 0)) * A.KVH;
    const RegionSplit rs = region_split(A.group_units, tail_units, tail_runs, (int)gridDim.x, A.max_units);
    const bool tail_wg = (int)blockIdx.x >= rs.Gs;
    const int U = tail_wg ? rs.Ut : rs.Us;
    const int wg_rel = tail_wg ? (int)blockIdx.x - rs.Gs : (int)blockIdx.x;      // the workgroup's place among those of its kind
    const int region_units = tail_wg ? tail_units : A.group_units;
    const int u0 = wg_rel * U;                                   // its first unit, counted within its kind
    // the host sizes the grid from max_seq_len; lengths on the device beyond that bound must not overrun
    // the descriptor table (the tiles past it are then left out: the caller broke its promise)
    const int nunits = u0 >= region_units ? 0 : min(min(U, region_units - u0), MAXU);
    if (w == 0) { s_incl[lane] = incl; s_len[lane] = len_i; }
    __syncthreads();
    if ((int)threadIdx.x < A.ngroups) {
        // a shared tile is visible to all its rows: no further than the shortest member reaches
        const GSeg sg = A.seg[threadIdx.x];
        int mn = 0x7fffffff;
        for (int i = 0; i < sg.count; i++) mn = min(mn, s_len[sg.first + i]);
        s_gmin[threadIdx.x] = max(mn, 0);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nunits * 4; i += 256) {
        const int ui = i >> 2, grp = i & 3, u = u0 + ui;
        int b, kvh, trel, nt, tile, len, nrows, slot0, run0;     // run0: first unit of the run (one kv head of a range or tail), within its kind
        if (!tail_wg) {
            int gi = 0;
            while (gi + 1 < A.ngroups && A.seg[gi + 1].unit0 <= u) gi++;
            const GSeg sg = A.seg[gi];
            const int rem = u - sg.unit0;
            nt = sg.ntile; kvh = rem / nt; trel = rem - kvh * nt;
            tile = sg.tile0 + trel; b = sg.first; len = s_gmin[gi]; nrows = sg.count * GQ;
            slot0 = sg.slot; run0 = sg.unit0 + kvh * nt;
        } else {
            const int v = u;
            int lo = 0, hi = A.B - 1;                              // first branch whose cumulative units exceed v
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (A.KVH * s_incl[mid] > v) hi = mid; else lo = mid + 1;
            }
            b = lo;
            const int excl = b ? s_incl[b - 1] : 0;
            nt = s_incl[b] - excl; len = s_len[b];
            const int rem = v - A.KVH * excl;
            kvh = rem / nt; trel = rem - kvh * nt;
            tile = trel + A.b_start[b]; nrows = GQ;
            slot0 = A.b_slot[b]; run0 = A.KVH * excl + kvh * nt;
        }
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
            GUnit d;
            d.tile_lim = len - tile * kSTile;
            d.flags = ((ui == 0 || trel == 0) ? 1 : 0) | ((ui == nunits - 1 || trel + 1 == nt) ? 2 : 0) | (nrows << 8);
            d.row0 = b * A.QH + kvh * GQ;
            d.slot = slot0 + (wg_rel - run0 / U);
            udesc[ui] = d;
        }
    }
    __syncthreads();
    if (A.plan_mode == 1) {
        plan_store<GUnit, MAXU>(A.plan, nunits, udesc, gdesc);
        return 0;
    }
    return nunits;
}

// ---- 16-bit pages: the tile in LDS, rows dealt to the waves -------------------------------------------
// decode_group_kernel below gives every wave 16 of a tile's tokens and ALL of a unit's query rows: 64 rows are
// 128 accumulator registers per lane, K and V wait in registers besides, and the compiler spills.  For 16-bit
// pages a tile needs no registers on its way: each wave requests its 16-token slice of K and of V straight
// into LDS (global_load_lds_dwordx4, two buffers, the next unit's slices travel while this one is computed),
// and a unit of a shared range with more than 16 rows is then split by ROWS: wave w multiplies row group w
// (16 rows: 32 accumulator registers) against all four slices -- S = K Q^T with Q in registers for the whole
// segment, O += P V as v_mfma_f32_16x16x32 over token pairs of slices with V read transposed from LDS
// (ds_read_b64_tr_b16), half the matrix instructions of the token split and no byte permutes.  A wave then
// holds complete rows: a segment ends without a fold.  The price is one workgroup barrier per tile (every wave
// reads every slice).  Units of one row group (private tails, small groups) keep the token split -- wave w
// multiplies its own slice, the four waves fold at the segment's end -- and need no barrier.
// LDS rows are unpadded 256 bytes; K: 16-byte chunk x of row r at position x ^ r (whole-row reads by 16 rows);
// V: 32-byte slot y of row r at position y ^ (r & 7) (transposed reads touch 4 rows x 32 bytes per 16 lanes) --
// applied on the global side by the lane that fills the position.
constexpr int kG16MaxUnits = 64;

__device__ __forceinline__ uint2 lds_read_tr16_b64(const uint8_t *p)
{
#if defined(__HIP_DEVICE_COMPILE__)
    typedef short tr_v4s __attribute__((ext_vector_type(4)));
    const tr_v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_v4s __attribute__((address_space(3))) *)p);
    return __builtin_bit_cast(uint2, r);
#else
    (void)p;
    return make_uint2(0u, 0u);
#endif
}

template <int DT>
__global__ __launch_bounds__(256, 2) void decode_group16_kernel(GroupedArgs A)
{
    constexpr int D = 128;
    constexpr int DOT = DT;
    constexpr uint32_t kNone = 0xffffffffu;
    constexpr uint32_t kOnes = DT == DRK_BF16 ? kBf16Ones : kF16Ones;
    __shared__ __align__(256) uint8_t ring[2][2][4][4096];       // [buffer][K | V][slice = wave that requests it][16 rows x 256 B]
    __shared__ __align__(16) float o_lds[4][4][D];               // token split: [wave][row of the round][dim], segment ends only
    __shared__ float mw_lds[4][16], lw_lds[4][16];
    __shared__ __align__(16) GUnit udesc[kG16MaxUnits];
    __shared__ __align__(16) uint2 gdesc[kG16MaxUnits][4];
    __shared__ int s_incl[64], s_len[64], s_gmin[kGMaxGroups];

    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4, c = lane & 15;
    const int GQ = A.QH / A.KVH;
    const int nunits = build_units<kG16MaxUnits>(A, udesc, gdesc, s_incl, s_len, s_gmin);
    if (nunits == 0) return;
    if (A.new_k) {
        // The step's append, folded in as in decode_stream_kernel: the unit that is the last tile of a branch's tail
        // (a tail unit has the rows of one kv head, a shared one those of two branches or more) holds the new token's
        // position, the page is the branch's own, and only this workgroup reads the tile -- so it writes the row
        // itself, K and V, 16 bytes per thread, and the barrier orders the stores before every wave's requests.
        constexpr int CH = D * 2 / 16;
        for (int i = threadIdx.x; i < nunits * 2 * CH; i += 256) {
            const int ui = i / (2 * CH), rest = i - ui * (2 * CH), kv = rest / CH, ch = rest - kv * CH;
            const GUnit ud = udesc[ui];
            if (((ud.flags >> 8) & 0xff) != GQ || ud.tile_lim < 1 || ud.tile_lim > kSTile) continue;
            const int r = ud.tile_lim - 1;
            const uint32_t gx = gdesc[ui][r >> 4].x;
            if (gx == kNone) continue;
            const int b = ud.row0 / A.QH, kvh = (ud.row0 - b * A.QH) / GQ;
            const uint8_t *src = (kv ? A.new_v : A.new_k) + ((size_t)(b * A.KVH + kvh) * D * 2) + ch * 16;
            uint8_t *dst = A.pool_layer_w + ((size_t)gx << 4) + (size_t)(r & 15) * A.row_bytes + (kv ? A.kv_plane : 0) + ch * 16;
            *(uint4 *)dst = *(const uint4 *)src;
        }
        __syncthreads();
    }

    // ---- requests: lane l of load j fills position l % 16 of row 4j + l / 16 of the wave's slice ----
    const uint32_t dma_row = (uint32_t)((lane >> 4) * 256);
    const uint32_t kdma_x = (uint32_t)(((lane & 15) ^ (lane >> 4)) << 4);            // K: chunk (l % 16) ^ row, row = 4j | l / 16
    const uint32_t vdma_x = (uint32_t)(((lane & 15) ^ ((lane >> 4) << 1)) << 4);     // V: slot (l % 16 / 2) ^ (row & 7), row & 7 = 4 (j & 1) | l / 16
    auto request = [&](int un) {
        const uint32_t off = (uint32_t)__builtin_amdgcn_readfirstlane((int)gdesc[un][w].x);
        const uint8_t *base = A.pool_layer + ((size_t)(off == kNone ? 0u : off) << 4);   // no page: any mapped bytes (the rows are masked)
        const uint32_t lk = lds_addr32(&ring[un & 1][0][w][0]), lv = lds_addr32(&ring[un & 1][1][w][0]);
        uint32_t kx = kdma_x, vx = vdma_x;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("" : "+v"(kx), "+v"(vx));               // computed here, each time: offsets held across the loop would cost registers
#endif
#pragma unroll
        for (int j = 0; j < 4; j++) lds_dma16(base, (kx ^ (uint32_t)(j << 6)) + dma_row + 1024u * j, lk + 1024 * j);
        const uint8_t *vbase = base + A.kv_plane;
#pragma unroll
        for (int j = 0; j < 4; j++) lds_dma16(vbase, (vx ^ (uint32_t)((j & 1) << 7)) + dma_row + 1024u * j, lv + 1024 * j);
    };

    // ---- Q^T of the segment as the B operand, in registers: lane (row c, dims 32 kk + 8 g ..), times scale * log2 e
    // (rounded to the 16-bit type once: a product then arrives as its exponent) ----
    uint4 qop[4];
    auto scaled16 = [&](uint32_t v) -> uint32_t {
        float lo, hi;
        if constexpr (DT == DRK_BF16) { lo = bf16_lo(v); hi = bf16_hi(v); }
        else { lo = f16_bits_to_f((uint16_t)(v & 0xffffu)); hi = f16_bits_to_f((uint16_t)(v >> 16)); }
        return pack16<DOT>(lo * A.scale_log2e, hi * A.scale_log2e);
    };
    // The next segment's rows are fetched while the last unit of this one is computed and folded (a tail of one tile
    // is a segment of its own: waiting for its rows at its head was half of what such a unit took) and scaled when
    // the segment begins.
    uint4 qraw[4];
    auto fetch_q = [&](const GUnit &d) {
        const int nrows = (d.flags >> 8) & 0xff;
        const int R = nrows > 16 ? 16 * w + c : c;           // row split: the wave's row group; token split: the one group
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (R < nrows) {
                const int bl = R / GQ, hd = R - bl * GQ;
                v = *(const uint4 *)(A.q + (size_t)(d.row0 + bl * A.QH + hd) * (D * 2) + kk * 64 + g * 16);
            }
            qraw[kk] = v;
        }
    };
    auto take_q = [&]() {                                    // (a row that does not exist was fetched as zeros and stays zero)
#pragma unroll
        for (int kk = 0; kk < 4; kk++)
            qop[kk] = make_uint4(scaled16(qraw[kk].x), scaled16(qraw[kk].y), scaled16(qraw[kk].z), scaled16(qraw[kk].w));
    };

    // where this lane finds its operands in a slice
    const uint32_t k_lane = (uint32_t)(c * 256 + (((g ^ c) & 15) << 4));             // row c, chunk g ^ c: k-step 0 (k-step kk: ^ kk << 6)
    const int vrow = 4 * g + (c >> 2);                                               // transposed read: row 4g + c / 4, dims 16 e + 4 (c % 4) ..
    const uint32_t v_lane = (uint32_t)(vrow * 256 + 8 * (c & 3)), v_x = (uint32_t)((vrow & 7) << 5);

    w_f32x4 o[8];                                            // O[row 4g + j][dim 16 e + c] = o[e][j]
#pragma unroll
    for (int e = 0; e < 8; e++) o[e] = w_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    // row c: minus the reference of the exponentials (0 until the row has one), what a score must exceed for the
    // reference to move (-inf until the row has one), this lane's share of the sum of the weights
    float negm = 0.0f, thr = -INFINITY, l_lane = 0.0f;

    // The reference moves only when a score exceeds it by more than kLazy (weights stay below 2^kLazy), or for the
    // row's first tokens; the output rows and the sum are rescaled on those occasions only -- rare enough that the
    // common path does not even fold the maximum across lanes.  Returns what to take off the scores.
    auto move_reference = [&](float lmax) -> float {
        const float mrel = max_lane_groups(lmax);            // row c's maximum over the wave's tokens of this tile
        const bool move = mrel > thr;
        const float delta = move ? mrel : 0.0f;
        const float alpha = thr == -INFINITY ? 1.0f : s_exp2(-delta);     // nothing summed yet: nothing to rescale
        negm -= delta;
        thr = move ? kLazy : thr;
        l_lane *= alpha;
        // register j of lane group g holds row 4g + j
        const float a0 = __shfl(alpha, 4 * g), a1 = __shfl(alpha, 4 * g + 1);
        const float a2 = __shfl(alpha, 4 * g + 2), a3 = __shfl(alpha, 4 * g + 3);
#pragma unroll
        for (int e = 0; e < 8; e++) { o[e][0] *= a0; o[e][1] *= a1; o[e][2] *= a2; o[e][3] *= a3; }
        return delta;
    };

    request(0);
    fetch_q(udesc[0]);
    take_q();
    for (int it = 0; it < nunits; it++) {
        const GUnit ud = udesc[it];
        const int flags = __builtin_amdgcn_readfirstlane(ud.flags);
        const int tile_lim = __builtin_amdgcn_readfirstlane(ud.tile_lim);
        const int nrows = (flags >> 8) & 0xff;
        const bool split_rows = nrows > 16;
        const bool has_next = it + 1 < nunits;
        // tokens of slice tg that exist (a slice without a page has none)
        int limt[4];
#pragma unroll
        for (int tg = 0; tg < 4; tg++)
            limt[tg] = __builtin_amdgcn_readfirstlane((int)gdesc[it][tg].x) == (int)kNone ? 0 : tile_lim - 16 * tg;

        vm_wait_all();                                       // the wave's slices of this unit have landed
        uint8_t *const kbuf = &ring[it & 1][0][0][0];
        uint8_t *const vbuf = &ring[it & 1][1][0][0];
        if (limt[w] < 16) {
            // rows without a token may hold anything (NaN): their weights are exact zeros, their V rows are cleared
            // (by the wave that owns the slice, before anyone multiplies)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int row = 4 * j + (lane >> 4);
                if (row >= limt[w]) *(uint4 *)(vbuf + w * 4096 + row * 256 + (lane & 15) * 16) = make_uint4(0u, 0u, 0u, 0u);
            }
        }
        // The next unit's slices are requested the moment this unit's have landed, so that a request is on its way
        // at all times.  They overwrite the buffer the unit before was read from -- by every wave, if it was split
        // by rows: such a unit ends with a barrier (below).  Row split: every wave reads every slice.
        if (has_next) request(it + 1);
        if (has_next && (flags & 2)) fetch_q(udesc[it + 1]);
        if (split_rows) __syncthreads();

        if (split_rows) {
            // ---- wave w: rows 16 w .. 16 w + 15 against the tile's 64 tokens --------------------------
            w_f32x4 s[4];                                     // s[tg][j]: row c, token 16 tg + 4 g + j, minus the reference
#pragma unroll
            for (int tg = 0; tg < 4; tg++) s[tg] = w_f32x4{negm, negm, negm, negm};
#pragma unroll
            for (int kk = 0; kk < 4; kk++)
#pragma unroll
                for (int tg = 0; tg < 4; tg++)
                    s[tg] = w_mfma_qk<DOT>(*(const uint4 *)(kbuf + tg * 4096 + (k_lane ^ (uint32_t)(kk << 6))), qop[kk], s[tg]);
            if (limt[0] < 16 || limt[1] < 16 || limt[2] < 16 || limt[3] < 16) {
#pragma unroll
                for (int tg = 0; tg < 4; tg++)
#pragma unroll
                    for (int j = 0; j < 4; j++) s[tg][j] = 4 * g + j < limt[tg] ? s[tg][j] : -INFINITY;
            }
            const float lmax = fmaxf(fmaxf(max4_asm(s[0][0], s[0][1], s[0][2], s[0][3]), max4_asm(s[1][0], s[1][1], s[1][2], s[1][3])),
                                     fmaxf(max4_asm(s[2][0], s[2][1], s[2][2], s[2][3]), max4_asm(s[3][0], s[3][1], s[3][2], s[3][3])));
            if (__builtin_amdgcn_ballot_w64(lmax > thr) != 0) {
                const float delta = move_reference(lmax);
#pragma unroll
                for (int tg = 0; tg < 4; tg++)
#pragma unroll
                    for (int j = 0; j < 4; j++) s[tg][j] -= delta;
            }
            uint2 pk[4];
#pragma unroll
            for (int tg = 0; tg < 4; tg++) {
                pk[tg] = make_uint2(pack16<DOT>(s_exp2(s[tg][0]), s_exp2(s[tg][1])), pack16<DOT>(s_exp2(s[tg][2]), s_exp2(s[tg][3])));
                // the row's denominator is the sum of the weights the second product multiplies -- the rounded ones
                l_lane = s_dot2<DOT>(pk[tg].y, kOnes, s_dot2<DOT>(pk[tg].x, kOnes, l_lane));
            }
            // O += P V over token pairs of slices: k-index 8 g + j is token 4 g + j of the pair's first slice (j < 4) or second
#pragma unroll
            for (int pr = 0; pr < 2; pr++) {
                const uint4 pa = make_uint4(pk[2 * pr].x, pk[2 * pr].y, pk[2 * pr + 1].x, pk[2 * pr + 1].y);
                const uint8_t *va = vbuf + (2 * pr) * 4096 + v_lane;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const uint2 b0 = lds_read_tr16_b64(va + (v_x ^ (uint32_t)(e << 5)));
                    const uint2 b1 = lds_read_tr16_b64(va + 4096 + (v_x ^ (uint32_t)(e << 5)));
                    o[e] = w_mfma_qk<DOT>(pa, make_uint4(b0.x, b0.y, b1.x, b1.y), o[e]);
                }
            }
            __syncthreads();                                 // every wave is done with this buffer
        } else {
            // ---- wave w: its own 16 tokens against the unit's one row group ----------------------------
            w_f32x4 s = {negm, negm, negm, negm};
#pragma unroll
            for (int kk = 0; kk < 4; kk++)
                s = w_mfma_qk<DOT>(*(const uint4 *)(kbuf + w * 4096 + (k_lane ^ (uint32_t)(kk << 6))), qop[kk], s);
            if (limt[w] < 16) {
#pragma unroll
                for (int j = 0; j < 4; j++) s[j] = 4 * g + j < limt[w] ? s[j] : -INFINITY;
            }
            const float lmax = max4_asm(s[0], s[1], s[2], s[3]);
            if (__builtin_amdgcn_ballot_w64(lmax > thr) != 0) {
                const float delta = move_reference(lmax);
#pragma unroll
                for (int j = 0; j < 4; j++) s[j] -= delta;
            }
            const uint2 pk = make_uint2(pack16<DOT>(s_exp2(s[0]), s_exp2(s[1])), pack16<DOT>(s_exp2(s[2]), s_exp2(s[3])));
            l_lane = s_dot2<DOT>(pk.y, kOnes, s_dot2<DOT>(pk.x, kOnes, l_lane));
            const uint8_t *va = vbuf + w * 4096 + v_lane;
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] = w_mfma_pv<DOT>(pk, lds_read_tr16_b64(va + (v_x ^ (uint32_t)(e << 5))), o[e]);
        }

        // ---- the segment's last tile: leave (o, m, l) per query row for the merge ----------------------
        if (flags & 2) {
            const float lw = sum_lane_groups(l_lane);
            const float mw = thr == -INFINITY ? -INFINITY : -negm;
            if (split_rows) {
                // the wave has seen every token of the segment for its rows: no fold
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int R = 16 * w + 4 * g + j;
                    const float mj = __shfl(mw, 4 * g + j), lj = __shfl(lw, 4 * g + j);
                    if (R < nrows) {
                        const int bl = R / GQ, hd = R - bl * GQ;
                        const size_t pi = (size_t)(ud.row0 + bl * A.QH + hd) * A.Ptot + ud.slot;
#pragma unroll
                        for (int e = 0; e < 8; e++) A.part_o[pi * D + 16 * e + c] = o[e][j];
                        if (c == 0) {
                            A.part_m[pi] = mj;
                            A.part_l[pi] = lj;
                        }
                    }
                }
            } else {
                // fold the four waves, four rows a round: row 4 r + w is stored by wave w
                if (lane < 16) { mw_lds[w][lane] = mw; lw_lds[w][lane] = lw; }       // padded rows too: defined values
                __syncthreads();
                const int rounds = (nrows + 3) >> 2;
                for (int r = 0; r < rounds; r++) {
                    if (r > 0) __syncthreads();                  // the previous round's sums have been read
                    if (g == r) {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const int h = 4 * g + j;
                            const float M = fmaxf(fmaxf(mw_lds[0][h], mw_lds[1][h]), fmaxf(mw_lds[2][h], mw_lds[3][h]));
                            const float mo = mw_lds[w][h];
                            const float f_own = mo == -INFINITY ? 0.0f : s_exp2(mo - M);
#pragma unroll
                            for (int e = 0; e < 8; e++) o_lds[w][j][16 * e + c] = o[e][j] * f_own;
                        }
                    }
                    // (m, l) of row 4 r + w over the four waves; read here, before the barrier, because a wave
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
                    if (h < nrows) {
                        const int d = lane * 2;
                        float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
                        for (int ww = 0; ww < 4; ww++) { acc0 += o_lds[ww][w][d]; acc1 += o_lds[ww][w][d + 1]; }
                        const int bl = h / GQ, hd = h - bl * GQ;
                        const size_t pi = (size_t)(ud.row0 + bl * A.QH + hd) * A.Ptot + ud.slot;
                        *(float2 *)(A.part_o + pi * D + d) = make_float2(acc0, acc1);
                        if (lane == 0) {
                            A.part_m[pi] = M;
                            A.part_l[pi] = L;
                        }
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] = w_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            negm = 0.0f; thr = -INFINITY; l_lane = 0.0f;
            if (has_next) take_q();
        }
    }
}

template <int DT, int D, int NG>
__global__ __launch_bounds__(256, 2) void decode_group_kernel(GroupedArgs A)
{
    using Geo = StreamGeo<DT, D>;
    [[maybe_unused]] constexpr bool Q8 = Geo::q8;
    constexpr int DOT = KvTraits<DT>::dot;
    constexpr uint32_t kNone = 0xffffffffu;
    constexpr int QP = D * 2 + 16;                               // LDS pitch of a query row (16-bit values)
    constexpr int NR = NG * 16;                                  // query rows a unit may serve
    constexpr int CPR = D * 2 / 16;                              // 16-byte chunks per query row
    constexpr int RPP = 256 / CPR;                               // rows the workgroup moves per pass
    constexpr int QPASS = NR / RPP;
    __shared__ __align__(16) uint8_t k_lds[4][16 * Geo::PITCH];  // a wave's 16 K rows as 16-bit values, padded rows
    __shared__ __align__(16) uint8_t q_lds[NR * QP];
    __shared__ __align__(16) float o_lds[4][8][D];               // [wave][row of the round][dim], segment ends only
    __shared__ float mw_lds[4][NR], lw_lds[4][NR];
    __shared__ __align__(16) GUnit udesc[kGMaxUnits];
    __shared__ __align__(16) uint2 gdesc[kGMaxUnits][4];
    __shared__ int s_incl[64], s_len[64], s_gmin[kGMaxGroups];

    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4, c = lane & 15;
    const int GQ = A.QH / A.KVH;
    const int nunits = build_units<kGMaxUnits>(A, udesc, gdesc, s_incl, s_len, s_gmin);
    if (nunits == 0) return;

    // the 4 K scales and the 4 V scales of tokens 4g..4g+3 (int8 pages)
    auto load_scales = [&](uint2 gd, uint2 &ks, uint2 &vs) {
        if (DT != DRK_INT8) return;
        const uint8_t *p = A.pool_layer + ((size_t)(gd.x == kNone ? 0u : gd.y) << 4) + g * 8;
        ks = *(const uint2 *)p;
        vs = *(const uint2 *)(p + A.scale_plane);
    };
    // A segment's query rows: requested into registers (the segment before is still being folded),
    // then stored to LDS as the 16-bit type the products run in; rows past the segment's are zeros.
    const int qr = (int)threadIdx.x / CPR, qc = (int)threadIdx.x % CPR;
    auto q_issue = [&](const GUnit &d, uint4 (&qn)[QPASS]) {
        const int nrows = (d.flags >> 8) & 0xff;
#pragma unroll
        for (int i = 0; i < QPASS; i++) {
            const int R = i * RPP + qr;
            qn[i] = make_uint4(0u, 0u, 0u, 0u);
            if (R < nrows) {
                const int bl = R / GQ, hd = R - bl * GQ;
                qn[i] = *(const uint4 *)(A.q + (size_t)(d.row0 + bl * A.QH + hd) * (D * 2) + qc * 16);
            }
        }
    };
    // (times scale * log2 e, rounded to the 16-bit type once: a product then arrives as its exponent)
    auto scaled16 = [&](uint32_t v) -> uint32_t {
        float lo, hi;
        if (A.io_dtype == DRK_BF16) { lo = bf16_lo(v); hi = bf16_hi(v); }
        else { lo = f16_bits_to_f((uint16_t)(v & 0xffffu)); hi = f16_bits_to_f((uint16_t)(v >> 16)); }
        lo *= A.scale_log2e; hi *= A.scale_log2e;
        if constexpr (DOT == DRK_BF16) return (uint32_t)f_to_bf16_bits(lo) | ((uint32_t)f_to_bf16_bits(hi) << 16);
        else return (uint32_t)__half_as_ushort(__float2half_rn(lo)) | ((uint32_t)__half_as_ushort(__float2half_rn(hi)) << 16);
    };
    auto q_store = [&](uint4 (&qn)[QPASS]) {
#pragma unroll
        for (int i = 0; i < QPASS; i++) {
            uint4 v = qn[i];
            v.x = scaled16(v.x); v.y = scaled16(v.y); v.z = scaled16(v.z); v.w = scaled16(v.w);
            *(uint4 *)(q_lds + (i * RPP + qr) * QP + qc * 16) = v;
        }
    };
    // Q^T as the B operand of row group rg: lane (row c of the group, dims 32 kk + 8 g ..)
    auto q_operand = [&](int rg, int kk) -> uint4 { return *(const uint4 *)(q_lds + (rg * 16 + c) * QP + kk * 64 + g * 16); };

    w_f32x4 o[NG][Geo::NPV];
    // per row group and row c: minus the reference of the exponentials (0 until the row has one), what a score
    // must exceed for the reference to move (-inf until the row has one), the sum of the weights
    float negm[NG], thr[NG], l_lane[NG], ps_lane[NG], qbias[NG];
#pragma unroll
    for (int rg = 0; rg < NG; rg++) {
#pragma unroll
        for (int e = 0; e < Geo::NPV; e++) o[rg][e] = w_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        negm[rg] = 0.0f; thr[rg] = -INFINITY; l_lane[rg] = 0.0f; ps_lane[rg] = 0.0f; qbias[rg] = 0.0f;
    }
    // int8 pages: the sum of every row's query values, for the code offset
    auto q_bias = [&]() {
        if (DT != DRK_INT8) return;
#pragma unroll
        for (int rg = 0; rg < NG; rg++) {
            float sq = 0.0f;
#pragma unroll
            for (int kk = 0; kk < Geo::NQK; kk++) {
                const uint4 v = q_operand(rg, kk);
                sq = s_dot2<DOT>(v.x, kF16Ones, sq);
                sq = s_dot2<DOT>(v.y, kF16Ones, sq);
                sq = s_dot2<DOT>(v.z, kF16Ones, sq);
                sq = s_dot2<DOT>(v.w, kF16Ones, sq);
            }
            qbias[rg] = kI8Bias * sum_lane_groups(sq);
        }
    };

    // V of a unit: the run's address is the same for the whole wave (scalar registers), the lane adds 32 bits
    const uint32_t v_lane_off = (uint32_t)((lane >> 4) * (4 * Geo::RB) + (lane & 15) * (Q8 ? 8 : 16));
    auto load_v_uniform = [&](uint32_t off) -> VRegs<DT, D> {
        VRegs<DT, D> v;
        const uint8_t *base = A.pool_layer + ((size_t)(off == kNone ? 0u : off) << 4) + A.kv_plane;
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int ch = 0; ch < Geo::NCH; ch++) {
                if constexpr (Q8) v.r[j][ch] = ld_stream64(base + (v_lane_off + (uint32_t)(j * Geo::RB + ch * 128)));
                else v.r[j][ch] = ld_stream128(base + (v_lane_off + (uint32_t)(j * Geo::RB + ch * 256)));
            }
        return v;
    };
    uint2 gd = gdesc[0][w], ksr = {}, vsr = {};
    KRegs<DT, D> kreg = load_k<DT, D>(A.pool_layer, gd.x, lane);
    VRegs<DT, D> vreg = load_v_uniform(__builtin_amdgcn_readfirstlane(gd.x));
    load_scales(gd, ksr, vsr);
    {
        uint4 qn[QPASS];
        q_issue(udesc[0], qn);
        q_store(qn);
        __syncthreads();
        q_bias();
    }

    for (int it = 0; it < nunits; it++) {
        const GUnit ud = udesc[it];
        const int flags = __builtin_amdgcn_readfirstlane(ud.flags);
        const int tile_lim = __builtin_amdgcn_readfirstlane(ud.tile_lim);
        const int nrows = (flags >> 8) & 0xff;
        const int nga = (nrows + 15) >> 4;                      // row groups of this unit
        const bool hole = __builtin_amdgcn_readfirstlane((int)gd.x) == (int)kNone;   // the group the registers were loaded for
        const int lim = hole ? 0 : tile_lim;                    // tokens of the tile this wave may look at
        const bool has_next = it + 1 < nunits;
        const bool partial = w * 16 + 16 > lim;                 // some of the wave's 16 tokens do not exist

        // ---- K: registers -> the wave's LDS rows -> one token row per lane; V: registers -> B operands;
        // then the loads of the next unit's K and V, so that they travel during all of this unit's arithmetic
        stage_k<DT, D>(&k_lds[w][0], kreg, lane);
        float ks[4] = {1.0f, 1.0f, 1.0f, 1.0f}, vs[4] = {1.0f, 1.0f, 1.0f, 1.0f};
        if (DT == DRK_INT8) {
            ks[0] = f16_bits_to_f((uint16_t)(ksr.x & 0xffffu)); ks[1] = f16_bits_to_f((uint16_t)(ksr.x >> 16));
            ks[2] = f16_bits_to_f((uint16_t)(ksr.y & 0xffffu)); ks[3] = f16_bits_to_f((uint16_t)(ksr.y >> 16));
            vs[0] = f16_bits_to_f((uint16_t)(vsr.x & 0xffffu)); vs[1] = f16_bits_to_f((uint16_t)(vsr.x >> 16));
            vs[2] = f16_bits_to_f((uint16_t)(vsr.y & 0xffffu)); vs[3] = f16_bits_to_f((uint16_t)(vsr.y >> 16));
        }
        const int t0 = w * 16 + g * 4;
        if (DT != DRK_INT8 && partial) {                        // rows without a token may hold anything (NaN)
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (t0 + j >= lim) {
#pragma unroll
                    for (int ch = 0; ch < Geo::NCH; ch++) vreg.r[j][ch] = {};
                }
        }
        uint2 vb[Geo::NCH][8];
#pragma unroll
        for (int ch = 0; ch < Geo::NCH; ch++) v_operands<DT>(vreg.r[0][ch], vreg.r[1][ch], vreg.r[2][ch], vreg.r[3][ch], vb[ch]);
        if (has_next) {
            gd = gdesc[it + 1][w];
            vreg = load_v_uniform(__builtin_amdgcn_readfirstlane(gd.x));
            kreg = load_k<DT, D>(A.pool_layer, gd.x, lane);
            load_scales(gd, ksr, vsr);
        }
        // the A operand: dims 32 kk + 8 g .. of token row c of the wave's 16
        const uint8_t *const krows = &k_lds[w][0];
        auto k_operand = [&](int kk) -> uint4 { return *(const uint4 *)(krows + c * Geo::PITCH + g * 16 + kk * 64); };

        // ---- scores, softmax, O += P V: for the unit's row groups (one, or all NG: a group of padding rows
        // multiplies zeros and its state is never stored) ----------------------------------------------
        auto tile_body = [&](auto NC) {
            constexpr int N = decltype(NC)::value;
            // S = K Q^T - m: the reference of row c's exponentials is the products' C operand, so a score arrives
            // as the exponent of its weight; N independent chains, so that a product never waits for the one before
            w_f32x4 s[N];
#pragma unroll
            for (int rg = 0; rg < N; rg++) {
                const float nm = DT == DRK_INT8 ? 0.0f : negm[rg];
                s[rg] = w_f32x4{nm, nm, nm, nm};
            }
#pragma unroll
            for (int kk = 0; kk < Geo::NQK; kk++) {
                const uint4 ka = k_operand(kk);
#pragma unroll
                for (int rg = 0; rg < N; rg++) s[rg] = w_mfma_qk<DOT>(ka, q_operand(rg, kk), s[rg]);
            }
            uint2 pa[N];                                      // A operands of the second product: P[row c][tokens 4g..4g+3]
#pragma unroll
            for (int rg = 0; rg < N; rg++) {
                if (DT == DRK_INT8) {                           // codes carry an offset and the token's scale
#pragma unroll
                    for (int j = 0; j < 4; j++) s[rg][j] = fmaf(s[rg][j] - qbias[rg], ks[j], negm[rg]);
                }
                if (partial) {
#pragma unroll
                    for (int j = 0; j < 4; j++) s[rg][j] = t0 + j < lim ? s[rg][j] : -INFINITY;
                }
                // The reference moves only when a score exceeds it by more than kLazy (weights stay below 2^kLazy), or
                // for the row's first tokens (thr = -inf until then); the output rows and sums are rescaled on those
                // occasions only -- rare enough that the common path does not even fold the maximum across lanes.
                const float lmax = max4_asm(s[rg][0], s[rg][1], s[rg][2], s[rg][3]);
                if (__builtin_amdgcn_ballot_w64(lmax > thr[rg]) != 0) {
                    const float mrel = max_lane_groups(lmax);       // row c's maximum over this wave's 16 tokens
                    const bool move = mrel > thr[rg];
                    const bool first = thr[rg] == -INFINITY;
                    const float delta = move ? mrel : 0.0f;
                    const float alpha = first ? 1.0f : s_exp2(-delta);    // nothing summed yet: nothing to rescale
                    negm[rg] -= delta;
                    thr[rg] = move ? kLazy : thr[rg];
#pragma unroll
                    for (int j = 0; j < 4; j++) s[rg][j] -= delta;
                    l_lane[rg] *= alpha;
                    if constexpr (DT == DRK_INT8) ps_lane[rg] *= alpha;
                    // register j of lane group g holds row 4g + j of the group
                    const float a0 = __shfl(alpha, 4 * g), a1 = __shfl(alpha, 4 * g + 1);
                    const float a2 = __shfl(alpha, 4 * g + 2), a3 = __shfl(alpha, 4 * g + 3);
#pragma unroll
                    for (int e = 0; e < Geo::NPV; e++) { o[rg][e][0] *= a0; o[rg][e][1] *= a1; o[rg][e][2] *= a2; o[rg][e][3] *= a3; }
                }
                float p[4], pw[4];
#pragma unroll
                for (int j = 0; j < 4; j++) p[j] = s_exp2(s[rg][j]);
#pragma unroll
                for (int j = 0; j < 4; j++) pw[j] = (DT == DRK_INT8) ? (t0 + j < lim ? p[j] * vs[j] : 0.0f) : p[j];
                const uint2 pk = make_uint2(pack16<DOT>(pw[0], pw[1]), pack16<DOT>(pw[2], pw[3]));
                pa[rg] = pk;
                // The row's denominator is the sum of the weights the second product multiplies -- the rounded
                // ones -- so that numerator and denominator carry the same rounding.  (int8: the product
                // multiplies p times the V scale, rounded; its sum of plain p stays exact, and the sum of the
                // rounded weights is kept for the code offset.)
                if (DT == DRK_INT8) {
                    float t = s_dot2<DOT>(pk.x, kF16Ones, 0.0f);
                    ps_lane[rg] += s_dot2<DOT>(pk.y, kF16Ones, t);
                    l_lane[rg] += (p[0] + p[1]) + (p[2] + p[3]);
                } else {
                    l_lane[rg] = s_dot2<DOT>(pk.y, DOT == DRK_BF16 ? kBf16Ones : kF16Ones, s_dot2<DOT>(pk.x, DOT == DRK_BF16 ? kBf16Ones : kF16Ones, l_lane[rg]));
                }
            }
            // O += P V; the V operands serve all row groups
#pragma unroll
            for (int ch = 0; ch < Geo::NCH; ch++)
#pragma unroll
                for (int e = 0; e < 8; e++)
#pragma unroll
                    for (int rg = 0; rg < N; rg++) o[rg][ch * 8 + e] = w_mfma_pv<DOT>(pa[rg], vb[ch][e], o[rg][ch * 8 + e]);
        };
        if (nga > 1) tile_body(std::integral_constant<int, NG>{});
        else tile_body(std::integral_constant<int, 1>{});
        // ---- the segment's last tile: fold the four waves, leave (o, m, l) for the merge ----
        if (flags & 2) {
            uint4 qn[QPASS];
            if (has_next) q_issue(udesc[it + 1], qn);          // the next segment's query rows travel during the fold
            float pwv[NG];
#pragma unroll
            for (int rg = 0; rg < NG; rg++) {
                pwv[rg] = 0.0f;
                if (rg < nga) {
                    const float lw = sum_lane_groups(l_lane[rg]);
                    if (DT == DRK_INT8) pwv[rg] = sum_lane_groups(ps_lane[rg]);
                    if (lane < 16) { mw_lds[w][rg * 16 + lane] = thr[rg] == -INFINITY ? -INFINITY : -negm[rg]; lw_lds[w][rg * 16 + lane] = lw; }   // padded rows too: defined values
                }
            }
            __syncthreads();
#pragma unroll
            for (int rg = 0; rg < NG; rg++) {
                if (rg < nga) {
                    float bias[4];                                   // code offset of row 4g + j (read from its lane while every lane is on)
#pragma unroll
                    for (int j = 0; j < 4; j++) bias[j] = DT == DRK_INT8 ? kI8Bias * __shfl(pwv[rg], 4 * g + j) : 0.0f;
#pragma unroll
                    for (int t = 0; t < 2; t++) {                    // rows 8t .. 8t + 7 of the group
                        // this wave's rows 4g + j of the group, weighted for the fold and freed of the code offset
                        if ((g >> 1) == t) {
#pragma unroll
                            for (int j = 0; j < 4; j++) {
                                const int h = rg * 16 + 4 * g + j;
                                const float M = fmaxf(fmaxf(mw_lds[0][h], mw_lds[1][h]), fmaxf(mw_lds[2][h], mw_lds[3][h]));
                                const float mo = mw_lds[w][h];
                                const float f_own = mo == -INFINITY ? 0.0f : s_exp2(mo - M);
#pragma unroll
                                for (int ch = 0; ch < Geo::NCH; ch++) {
                                    float *dst = &o_lds[w][4 * (g & 1) + j][ch * 128 + c * 8];
                                    const w_f32x4 *oc = &o[rg][ch * 8];
                                    *(float4 *)dst = make_float4((oc[0][j] - bias[j]) * f_own, (oc[1][j] - bias[j]) * f_own,
                                                                 (oc[2][j] - bias[j]) * f_own, (oc[3][j] - bias[j]) * f_own);
                                    *(float4 *)(dst + 4) = make_float4((oc[4][j] - bias[j]) * f_own, (oc[5][j] - bias[j]) * f_own,
                                                                       (oc[6][j] - bias[j]) * f_own, (oc[7][j] - bias[j]) * f_own);
                                }
                            }
                        }
                        __syncthreads();
                        // wave w sums rows 8t + w and 8t + w + 4 of the group over the four waves
#pragma unroll
                        for (int i = 0; i < 2; i++) {
                            const int hl = w + 4 * i, R = rg * 16 + 8 * t + hl;
                            if (R < nrows) {
                                const float M = fmaxf(fmaxf(mw_lds[0][R], mw_lds[1][R]), fmaxf(mw_lds[2][R], mw_lds[3][R]));
                                float L = 0.0f;
#pragma unroll
                                for (int ww = 0; ww < 4; ww++) {
                                    const float mm = mw_lds[ww][R];
                                    if (mm != -INFINITY) L = fmaf(lw_lds[ww][R], s_exp2(mm - M), L);
                                }
                                constexpr int VEC = D / 64;
                                const int d = lane * VEC;
                                float acc[VEC];
#pragma unroll
                                for (int x = 0; x < VEC; x++) acc[x] = 0.0f;
#pragma unroll
                                for (int ww = 0; ww < 4; ww++)
#pragma unroll
                                    for (int x = 0; x < VEC; x++) acc[x] += o_lds[ww][hl][d + x];
                                const int bl = R / GQ, hd = R - bl * GQ;
                                const size_t pi = (size_t)(ud.row0 + bl * A.QH + hd) * A.Ptot + ud.slot;
#pragma unroll
                                for (int x = 0; x < VEC; x++) A.part_o[pi * D + d + x] = acc[x];
                                if (lane == 0) {
                                    A.part_m[pi] = M;
                                    A.part_l[pi] = L;
                                }
                            }
                        }
                        __syncthreads();
                    }
                }
            }
#pragma unroll
            for (int rg = 0; rg < NG; rg++) {
#pragma unroll
                for (int e = 0; e < Geo::NPV; e++) o[rg][e] = w_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                negm[rg] = 0.0f; thr[rg] = -INFINITY; l_lane[rg] = 0.0f; ps_lane[rg] = 0.0f;
            }
            if (has_next) {
                q_store(qn);
                __syncthreads();
                q_bias();
            }
        }
    }
}

// grid (QH, B), block 256: fold the pieces of (branch, q head): those of every group the branch
// belongs to and those of its tail; out is written only when some token took part
// (paged_attention.cu:266).  The piece list is put together first (which slots hold pieces follows
// from the lengths, exactly as the kernel above cut its runs); then lane s of every wave owns the
// (m, l) of piece s (+64, ...), wave w folds the o rows of pieces w, w+4, ... eight at a time, and
// the four waves' sums meet in LDS.
template <int D>
__global__ __launch_bounds__(256) void group_merge_kernel(GroupedArgs A, uint16_t *__restrict__ out, int grid_wgs,
                                                          const uint16_t *__restrict__ gate, size_t gate_stride)
{
    constexpr int VEC = D / 64;                                  // dims per lane: 2 or 4
    typedef float fvec __attribute__((ext_vector_type(VEC)));
    __shared__ fvec red[4][64];
    __shared__ int seg_base[kGMaxGroups + 1], seg_cnt[kGMaxGroups + 1], seg_off[kGMaxGroups + 2], nseg_s;
    __shared__ short slot_of[kGMaxPieces];
    const int h = blockIdx.x, b = blockIdx.y, lane = threadIdx.x & 63, wv = threadIdx.x >> 6, d = lane * VEC;
    // The pieces of this row: those of every shared range the branch is a member of, in the order of the ranges, then
    // those of its tail.  One lane per branch scans the tail tiles (one round of loads), then one lane per range (and
    // one for the tail) works out how many workgroups its run of units was dealt to; a scan gives the offsets.
    if (wv == 0) {
        const int len = lane < A.B ? A.seq_lens[lane] : 0;
        const int nt = len > 0 ? max((len + kSTile - 1) / kSTile - A.b_start[lane], 0) : 0;
        int incl = nt;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int t = __shfl_up(incl, off);
            if (lane >= off) incl += t;
        }
        const int total = __builtin_amdgcn_readlane(incl, 63);
        const int nt_b = __shfl(nt, b), excl = __shfl(incl, b) - nt_b;
        int cnt = 0, slot0 = 0;
        if (A.group_units + total * A.KVH > 0) {
            const RegionSplit rs = region_split(A.group_units, total * A.KVH, __popcll(__builtin_amdgcn_ballot_w64(nt > 0)) * A.KVH,
                                                grid_wgs, A.max_units);
            const int kvh = h / (A.QH / A.KVH);
            if (lane < A.ngroups) {
                const GSeg sg = A.seg[lane];
                if (b >= sg.first && b < sg.first + sg.count) {
                    const int first = sg.unit0 + kvh * sg.ntile, last = first + sg.ntile - 1;
                    slot0 = sg.slot; cnt = last / rs.Us - first / rs.Us + 1;
                }
            } else if (lane == A.ngroups && nt_b > 0) {
                const int first = A.KVH * excl + kvh * nt_b, last = first + nt_b - 1;
                slot0 = A.b_slot[b]; cnt = last / rs.Ut - first / rs.Ut + 1;
            }
        }
        int cincl = cnt;
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) {                 // at most kGMaxGroups + 1 entries
            const int t = __shfl_up(cincl, off);
            if (lane >= off) cincl += t;
        }
        if (lane <= A.ngroups) { seg_base[lane] = slot0; seg_cnt[lane] = cnt; seg_off[lane] = cincl - cnt; }
        if (lane == A.ngroups) { seg_off[lane + 1] = min(cincl, kGMaxPieces); nseg_s = lane + 1; }
    }
    __syncthreads();
    const int nseg = nseg_s, n_all = seg_off[nseg];
    for (int k = 0; k < nseg; k++)
        for (int i = threadIdx.x; i < seg_cnt[k] && seg_off[k] + i < kGMaxPieces; i += 256) slot_of[seg_off[k] + i] = (short)(seg_base[k] + i);
    __syncthreads();
    const size_t base = ((size_t)b * A.QH + h) * A.Ptot;
    // the first 64 pieces' sums and maxima stay in registers for the second pass (a row rarely has more)
    float M = -INFINITY, pl0 = 0.0f, pm0 = 0.0f;
    if (lane < n_all) {
        const size_t pi = base + slot_of[lane];
        pl0 = A.part_l[pi];
        pm0 = A.part_m[pi];
        if (pl0 > 0.0f) M = pm0;
    }
    for (int s = lane + 64; s < n_all; s += 64) {
        const size_t pi = base + slot_of[s];
        if (A.part_l[pi] > 0.0f) M = fmaxf(M, A.part_m[pi]);
    }
    M = s_wave_max(M);
    fvec acc = {};
    float L = 0.0f;
    for (int c0 = 0; c0 < n_all; c0 += 64) {
        const int s = c0 + lane, cnt = min(64, n_all - c0);
        float wt = 0.0f;
        if (s < n_all) {
            const size_t pi = base + slot_of[s];
            const float pl = c0 == 0 ? pl0 : A.part_l[pi];
            if (pl > 0.0f) { wt = s_exp2((c0 == 0 ? pm0 : A.part_m[pi]) - M); L = fmaf(pl, wt, L); }
        }
        for (int j = wv; j < cnt; j += 32) {
            fvec o[8];
            float wj[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int jj = min(j + 4 * u, cnt - 1);
                wj[u] = j + 4 * u < cnt ? s_lane(wt, jj) : 0.0f;
                o[u] = *(const fvec *)(A.part_o + (base + slot_of[c0 + jj]) * D + d);
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
    red[wv][lane] = acc;
    __syncthreads();
    if (wv == 0) {
        // with a gate the row is always rewritten: the reference gates whatever the attention
        // kernel left in out, also when no token took part (paged_attention.cu:266, 368-370)
        uint16_t *dst = out + ((size_t)b * A.QH + h) * D + d;
        uint16_t vals[VEC];
        if (L > 0.0f) {
            const fvec a1 = red[1][lane], a2 = red[2][lane], a3 = red[3][lane];
#pragma unroll
            for (int x = 0; x < VEC; x++) vals[x] = f_to_elem16(((acc[x] + a1[x]) + (a2[x] + a3[x])) / L, A.io_dtype);
        } else {
            if (!gate) return;
#pragma unroll
            for (int x = 0; x < VEC; x++) vals[x] = dst[x];
        }
        if (gate) {
            const uint16_t *gp = gate + ((size_t)b * A.QH + h) * gate_stride + d;
#pragma unroll
            for (int x = 0; x < VEC; x++) vals[x] = gated_elem16(vals[x], gp[x], A.io_dtype);
        }
        if constexpr (VEC == 2) {
            *(uint32_t *)dst = (uint32_t)vals[0] | ((uint32_t)vals[1] << 16);
        } else {
            *(uint2 *)dst = make_uint2((uint32_t)vals[0] | ((uint32_t)vals[1] << 16), (uint32_t)vals[2] | ((uint32_t)vals[3] << 16));
        }
    }
}

// ---- host side ------------------------------------------------------------------------------
bool grouped_decode_supported(const Lay &a, int B)
{
    return !g_force_portable && g_grouped_mode != 1 && a.D == 128 && stream_decode_supported(a, B);
}

struct GroupPlan {
    int ngroups, group_units, grid, Ptot;
    GSeg seg[kGMaxGroups];
    int b_start[64], b_slot[64];
};

// Shared ranges in tokens -> tiles, checked: for every branch the ranges it belongs to must follow
// one another from token 0 without gap or overlap (then every token of a branch is read exactly once:
// by one range or by the branch's tail).  Ranges are cut down to whole 64-token tiles; what a range
// loses at its end, the range or tail behind it reads.
// units one workgroup may own: the descriptor table of the kernel that takes the call
// (times 12 / 13: the workgroups of the tails take runs up to 13 / 12 of the even share, see region_split)
// workgroups for t_upper units at most: all that fit on the chip, or as many as keep a workgroup's run within max_units
static long grouped_grid(long t_upper, int max_units)
{
    long G = t_upper < kGWgs ? t_upper : kGWgs;
    if (G < 1) G = 1;
    if ((t_upper + G - 1) / G > max_units) G = (t_upper + max_units - 1) / max_units;   // descriptor table size
    return G;
}
static int group_max_units(const Lay &a) { return (a.E == 2 && g_grouped_mode != 2 ? kG16MaxUnits : kGMaxUnits) * 12 / 13; }

static int plan_groups(const Lay &a, int B, int max_seq_len, const drk_prefix_group *groups, int n_in, GroupPlan *P)
{
    const int max_units = group_max_units(a);
    if (n_in < 0 || n_in > kGMaxGroups) return fail(DRK_ERR_INVALID, "decode_grouped: %d groups (0..%d)", n_in, kGMaxGroups);
    if (n_in > 0 && !groups) return fail(DRK_ERR_INVALID, "decode_grouped: groups is NULL");
    const int GQ = a.QH / a.KVH;
    const int max_tiles = (max_seq_len + kSTile - 1) / kSTile;
    int n = 0;
    for (int i = 0; i < n_in; i++) {
        const drk_prefix_group &gr = groups[i];
        if (gr.first_branch < 0 || gr.n_branches < 1 || gr.first_branch + gr.n_branches > B || gr.tok_begin < 0 ||
            gr.tok_end < gr.tok_begin || gr.tok_end > max_seq_len)
            return fail(DRK_ERR_INVALID, "decode_grouped: group %d = branches [%d, +%d) tokens [%d, %d) does not fit %d branches of up to %d tokens",
                        i, gr.first_branch, gr.n_branches, gr.tok_begin, gr.tok_end, B, max_seq_len);
        const int t0 = gr.tok_begin / kSTile, t1 = gr.tok_end / kSTile;
        if (t1 <= t0) continue;
        if (gr.n_branches * GQ > 64)
            return fail(DRK_ERR_UNSUPPORTED, "decode_grouped: group %d has %d branches x %d query heads per kv head (at most 64 rows: split it)",
                        i, gr.n_branches, GQ);
        GSeg s;
        s.first = gr.first_branch; s.count = gr.n_branches; s.tile0 = t0; s.ntile = t1 - t0; s.slot = -1; s.unit0 = 0;
        int k = n++;
        while (k > 0 && P->seg[k - 1].tile0 > s.tile0) { P->seg[k] = P->seg[k - 1]; k--; }   // ordered by first tile
        P->seg[k] = s;
    }
    P->ngroups = n;
    int units = 0;
    for (int k = 0; k < n; k++) { P->seg[k].unit0 = units; units += a.KVH * P->seg[k].ntile; }
    P->group_units = units;
    long t_upper = units;
    for (int b = 0; b < B; b++) {
        int start = 0;
        for (int k = 0; k < n; k++) {
            const GSeg &s = P->seg[k];
            if (b < s.first || b >= s.first + s.count) continue;
            if (s.tile0 != start)
                return fail(DRK_ERR_INVALID, "decode_grouped: the ranges of branch %d do not follow one another from token 0 (tile %d after tile %d)",
                            b, s.tile0, start);
            start = s.tile0 + s.ntile;
        }
        P->b_start[b] = start;
        t_upper += (long)a.KVH * (max_tiles > start ? max_tiles - start : 0);
    }
    for (int b = B; b < 64; b++) P->b_start[b] = P->b_slot[b] = 0;
    const long G = grouped_grid(t_upper, max_units);
    P->grid = (int)G;
    // a run of n tiles of one kv head meets at most min(n, G / KVH + 2) workgroups
    const int cap = (int)(G / a.KVH) + 2;
    auto pub = [&](int tiles) { return tiles <= 0 ? 0 : (tiles < cap ? tiles : cap); };
    int Ptot = 1;
    for (int b = 0; b < B; b++) {
        int slot = 0;
        for (int k = 0; k < n; k++) {
            GSeg &s = P->seg[k];
            if (b < s.first || b >= s.first + s.count) continue;
            if (s.slot < 0) s.slot = slot;
            else if (s.slot != slot)
                return fail(DRK_ERR_INVALID, "decode_grouped: the branches of a group must belong to the same groups before it (branch %d)", b);
            slot += pub(s.ntile);
        }
        P->b_slot[b] = slot;
        slot += pub(max_tiles - P->b_start[b]);
        if (slot > Ptot) Ptot = slot;
    }
    if (Ptot > kGMaxPieces)
        return fail(DRK_ERR_UNSUPPORTED, "decode_grouped: %d pieces per query row (at most %d)", Ptot, kGMaxPieces);
    P->Ptot = Ptot;
    return DRK_OK;
}

size_t grouped_workspace_need(const Lay &a, int B, int max_seq_len, const drk_prefix_group *groups, int n_groups)
{
    GroupPlan P;
    if (B < 1 || B > 64 || plan_groups(a, B, max_seq_len, groups, n_groups, &P) != DRK_OK) return 0;
    return (size_t)B * a.QH * P.Ptot * (a.D + 2) * sizeof(float);
}

// every plan with ranges nested at most max_depth deep fits: each level and the tail take at most kGWgs / KVH + 2 slots
size_t grouped_workspace_need_max(const Lay &a, int B, int max_seq_len, int max_depth)
{
    const int max_tiles = (max_seq_len + kSTile - 1) / kSTile;
    long G = kGWgs;
    const long t_upper = (long)a.KVH * B * max_tiles;
    const int max_units = kG16MaxUnits * 12 / 13;                // the smaller table gives the larger grid, and so the larger bound
    if ((t_upper + G - 1) / G > max_units) G = (t_upper + max_units - 1) / max_units;
    long cap = G / a.KVH + 2;
    if (cap > max_tiles) cap = max_tiles;
    long P = (long)(max_depth + 1) * cap;
    if (P > max_tiles + 2L * (max_depth + 1)) P = max_tiles + 2L * (max_depth + 1);
    if (P < 1) P = 1;
    return (size_t)B * a.QH * (size_t)P * (a.D + 2) * sizeof(float);
}

bool grouped_decode_writes_new_rows(const Lay &a) { return a.E == 2 && g_grouped_mode != 2; }

int launch_decode_grouped(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *tables, int table_stride,
                          const int32_t *d_seq_lens, int B, int max_seq_len, const drk_prefix_group *groups, int n_groups,
                          void *out, int layer, float scale, int io_dtype, void *workspace, size_t workspace_bytes,
                          void *stream, const void *gate, size_t gate_stride, DecodePlan plan)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    const bool plan_only = plan.ptr && plan.mode == 1;              // builds the unit descriptors: reads tables and lengths only
    if (!tables || !d_seq_lens || (!plan_only && (!q || !pool || !out))) return fail(DRK_ERR_INVALID, "decode_grouped: NULL pointer");
    if (gate && (gate_stride < (size_t)a.D || (gate_stride % 8) || ((uintptr_t)gate % 16)))
        return fail(DRK_ERR_INVALID, "decode_grouped: gate rows must be 16-byte aligned and at least head_dim apart");
    if (io_dtype != DRK_F16 && io_dtype != DRK_BF16) return fail(DRK_ERR_INVALID, "decode_grouped: io_dtype must be F16 or BF16");
    if ((a.dtype == DRK_F16 || a.dtype == DRK_BF16) && io_dtype != a.dtype)
        return fail(DRK_ERR_INVALID, "decode_grouped: io_dtype %d differs from the pool's %d", io_dtype, a.dtype);
    if (layer < 0 || layer >= a.L) return fail(DRK_ERR_INVALID, "decode_grouped: layer %d outside [0,%d)", layer, a.L);
    if (B < 0 || max_seq_len < 0 || table_stride < 0) return fail(DRK_ERR_INVALID, "decode_grouped: negative size");
    if (B == 0 || max_seq_len == 0) return DRK_OK;
    if (!grouped_decode_supported(a, B) || !(scale > 0.0f))
        return fail(DRK_ERR_UNSUPPORTED, "decode_grouped: needs head_dim 128, at most 16 query heads per kv head, block_size %% 16 == 0, at most 64 branches, scale > 0");
    GroupPlan P;
    if ((rc = plan_groups(a, B, max_seq_len, groups, n_groups, &P))) return rc;
    if (P.ngroups == 0)                                            // nothing shared (after rounding to tiles): the plain kernel
        return launch_decode(g, q, pool, tables, table_stride, d_seq_lens, 0, -1, B, max_seq_len, out, layer, scale, io_dtype,
                             0, workspace, workspace_bytes, stream, gate, gate_stride, plan);
    const size_t need = (size_t)B * a.QH * P.Ptot * (a.D + 2) * sizeof(float);
    if (!plan_only && (!workspace || workspace_bytes < need))
        return fail(DRK_ERR_WORKSPACE, "decode_grouped: workspace of %zu bytes, need %zu", workspace_bytes, need);
    if (((uintptr_t)workspace) % 16) return fail(DRK_ERR_INVALID, "decode_grouped: workspace must be 16-byte aligned");

    GroupedArgs A;
    A.pool_layer = (const uint8_t *)pool + (size_t)layer * a.layer_stride;
    A.tables = tables; A.seq_lens = d_seq_lens; A.q = (const uint8_t *)q;
    A.part_o = (float *)workspace;
    A.part_m = A.part_o + (size_t)B * a.QH * P.Ptot * a.D;
    A.part_l = A.part_m + (size_t)B * a.QH * P.Ptot;
    A.table_stride = table_stride; A.B = B; A.KVH = a.KVH; A.QH = a.QH; A.NB = a.NB; A.bs = a.bs;
    A.bs_shift = ilog2_exact((unsigned)a.bs); A.io_dtype = io_dtype; A.Ptot = P.Ptot;
    A.ngroups = P.ngroups; A.group_units = P.group_units;
    A.head_stride = a.head_stride; A.kv_plane = a.kv_plane; A.block_stride = a.block_stride;
    A.scale_plane = a.scale_plane; A.row_bytes = a.row_bytes;
    A.scale_log2e = scale * kSLog2e;
    for (int k = 0; k < kGMaxGroups; k++) A.seg[k] = k < P.ngroups ? P.seg[k] : GSeg{0, 0, 0, 0, 0, 0x7fffffff};
    for (int b = 0; b < 64; b++) { A.b_start[b] = P.b_start[b]; A.b_slot[b] = P.b_slot[b]; }
    A.plan = plan.ptr; A.plan_mode = plan.ptr ? plan.mode : 0;
    hipStream_t st = (hipStream_t)stream;
    // 16-bit pages: the tile in LDS, rows dealt to the waves; 8-bit pages (and, as a cross-check, 16-bit pages in
    // diagnostic mode 2): tokens dealt to the waves, K and V through registers
    const bool tile16 = a.E == 2 && g_grouped_mode != 2;
    A.max_units = tile16 ? kG16MaxUnits : kGMaxUnits;
    const bool fused_append = plan.new_k && plan.new_v && plan.mode != 1;
    if (fused_append && !tile16) return fail(DRK_ERR_INVALID, "decode_grouped: only the 16-bit tile kernel writes the new rows itself");
    A.new_k = fused_append ? plan.new_k : nullptr;
    A.new_v = fused_append ? plan.new_v : nullptr;
    A.pool_layer_w = (uint8_t *)const_cast<void *>(pool) + (size_t)layer * a.layer_stride;
    switch (a.dtype) {
    case DRK_F16:
        if (tile16) hipLaunchKernelGGL((decode_group16_kernel<DRK_F16>), dim3(P.grid), dim3(256), 0, st, A);
        else hipLaunchKernelGGL((decode_group_kernel<DRK_F16, 128, 4>), dim3(P.grid), dim3(256), 0, st, A);
        break;
    case DRK_BF16:
        if (tile16) hipLaunchKernelGGL((decode_group16_kernel<DRK_BF16>), dim3(P.grid), dim3(256), 0, st, A);
        else hipLaunchKernelGGL((decode_group_kernel<DRK_BF16, 128, 4>), dim3(P.grid), dim3(256), 0, st, A);
        break;
    case DRK_INT8: hipLaunchKernelGGL((decode_group_kernel<DRK_INT8, 128, 4>), dim3(P.grid), dim3(256), 0, st, A); break;
    default: hipLaunchKernelGGL((decode_group_kernel<DRK_FP8_E4M3, 128, 4>), dim3(P.grid), dim3(256), 0, st, A); break;
    }
    DRK_LAUNCH_CHECK("decode_group_kernel");
    if (g_skip_merge || plan_only) return DRK_OK;
    hipLaunchKernelGGL(group_merge_kernel<128>, dim3(a.QH, B), dim3(256), 0, st, A, (uint16_t *)out, P.grid,
                       (const uint16_t *)gate, gate_stride);
    DRK_LAUNCH_CHECK("group_merge_kernel");
    return DRK_OK;
}

size_t grouped_plan_need(const Lay &a, int B, int max_seq_len, const drk_prefix_group *groups, int n_groups)
{
    (void)a; (void)B; (void)max_seq_len; (void)groups; (void)n_groups;
    return (size_t)kGWgs * plan_record_bytes(kGMaxUnits);          // either kernel's records fit
}

} // namespace drk

using namespace drk;

extern "C" {

void drk_debug_set_grouped_decode(int mode) { g_grouped_mode = (mode == 1 || mode == 2) ? mode : 0; }

int drk_debug_grouped_grid(int kvh, int group_units, int tail_units_upper, int descriptor_table)
{
    (void)kvh;
    return (int)grouped_grid((long)group_units + tail_units_upper, descriptor_table * 12 / 13);
}

void drk_debug_grouped_region_split(int group_units, int tail_units, int tail_runs, int grid, int descriptor_table, int out[3])
{
    const RegionSplit r = region_split(group_units, tail_units, tail_runs, grid, descriptor_table);
    out[0] = r.Gs; out[1] = r.Us; out[2] = r.Ut;
}

size_t drk_decode_grouped_workspace_bytes(const drk_kv_layout *g, int B, int max_seq_len, const drk_prefix_group *groups,
                                          int n_groups)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK || B <= 0 || max_seq_len <= 0) return 0;
    size_t need = drk_decode_workspace_bytes(g, B, max_seq_len);      // no group left after rounding: the plain kernel
    if (a.D == 128 && stream_decode_supported(a, B)) {
        const size_t s2 = grouped_workspace_need(a, B, max_seq_len, groups, n_groups);
        if (s2 == 0) return 0;
        if (s2 > need) need = s2;
    }
    return need;
}

size_t drk_decode_grouped_workspace_bytes_max(const drk_kv_layout *g, int B, int max_seq_len, int max_depth)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK || B <= 0 || max_seq_len <= 0 || max_depth < 0) return 0;
    size_t need = drk_decode_workspace_bytes(g, B, max_seq_len);
    if (a.D == 128 && stream_decode_supported(a, B)) {
        const size_t s2 = grouped_workspace_need_max(a, B, max_seq_len, max_depth);
        if (s2 > need) need = s2;
    }
    return need;
}

int drk_paged_decode_attention_grouped(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *d_tables,
                                       int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len,
                                       const drk_prefix_group *groups, int n_groups, void *out, int layer, float scale,
                                       int io_dtype, const void *gate, size_t gate_stride, void *workspace,
                                       size_t workspace_bytes, void *stream)
{
    return launch_decode_grouped(g, q, pool, d_tables, table_stride, d_seq_lens, B, max_seq_len, groups, n_groups, out, layer,
                                 scale, io_dtype, workspace, workspace_bytes, stream, gate, gate_stride);
}

} // extern "C"
