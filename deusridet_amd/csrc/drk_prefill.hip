// drk_prefill.hip -- paged causal prefill attention on the gfx950 matrix cores.
//
// Replaces paged_prefill_attention_kernel (paged_attention.cu:465-554), which runs
// the token-at-a-time decode loop once per (query head, query token): O(M*L)
// serial dot products, no tensor cores.  Here the one dense contraction of the
// path, QK^T and PV of a chunk against all pages before it, runs on
// v_mfma_f32_32x32x16_{bf16,f16}.
//
// Formulation: everything is kept transposed so that one lane owns one query row.
//   S^T[token][row] = K[token][:] . Q[row][:]      A = K tile (LDS), B = Q (registers)
//   O^T[d][row]    += V^T[d][token] . P^T[token][row]   A = V tile read transposed
//                                                       (ds_read_b64_tr_b16), B = P
// The C layout of the first product (lane l: column l%32 = query row, 16 tokens)
// is, after exp2 and packing to 16 bit, exactly the B layout of the second, so P
// never moves between lanes, and the online-softmax rescale of O^T is a per-lane
// scalar multiply.  "Row" = (query token, query head of the group): the 4 query
// heads that share a KV head are stacked into the row dimension, so K/V tiles are
// read once for all of them.
//
// Workgroup = 4 waves = 128 rows = 32 query tokens x 4 heads of one KV head; it
// walks the KV tiles (64 tokens) from token 0 to its causal limit.  K/V tiles are
// gathered from 16-token page row runs with 128-bit loads (next tile in flight
// while the current one is multiplied) and staged in LDS with a 272-byte pitch.
#include "drk_common.hpp"

#include <math.h>

namespace drk {

constexpr int kPfBN = 64;         // KV tokens per tile
// LDS bytes per staged row.  The LDS has 32 four-byte banks.  K rows are read whole-row
// (lane = token, 16 bytes per lane, 8 lanes per clock): consecutive rows must start 4 banks
// apart -> 256 + 16.  V rows are read transposed (16 lanes per clock touch 4 consecutive
// rows, 4 x 8 bytes each): consecutive rows must start 8 banks apart -> 256 + 32; with the
// K pitch every other row pair collides (measured: half of the LDS-active cycles were
// bank-conflict cycles).  For head_dim D: 2 D + 16 and 2 D + 32.
constexpr float kLog2eP = 1.4426950408889634f;

typedef __bf16 pf_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 pf_f16x8 __attribute__((ext_vector_type(8)));
typedef float pf_f32x16 __attribute__((ext_vector_type(16)));
typedef short pf_v4s __attribute__((ext_vector_type(4)));

template <int DT>
__device__ __forceinline__ pf_f32x16 mfma32(const uint4 &a, const uint4 &b, pf_f32x16 c)
{
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (DT == DRK_BF16)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(pf_bf16x8, a), __builtin_bit_cast(pf_bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(pf_f16x8, a), __builtin_bit_cast(pf_f16x8, b), c, 0, 0, 0);
#else
    (void)a; (void)b;
    return c;
#endif
}

// two fp32 -> one dword of two 16-bit values, round to nearest even
template <int DT>
__device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
    if constexpr (DT == DRK_BF16) {
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        b2 v = {(__bf16)lo, (__bf16)hi};
        return __builtin_bit_cast(uint32_t, v);
    } else {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 v = {(_Float16)lo, (_Float16)hi};
        return __builtin_bit_cast(uint32_t, v);
    }
}

// acc + the eight 16-bit values packed in v
template <int DT>
__device__ __forceinline__ float pf_sum2(const uint4 &v, float acc)
{
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (DT == DRK_BF16) {
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        const b2 one = {(__bf16)1.0f, (__bf16)1.0f};
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, v.x), one, acc, false);
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, v.y), one, acc, false);
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, v.z), one, acc, false);
        acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, v.w), one, acc, false);
    } else {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 one = {(_Float16)1.0f, (_Float16)1.0f};
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, v.x), one, acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, v.y), one, acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, v.z), one, acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, v.w), one, acc, false);
    }
#else
    (void)v;
#endif
    return acc;
}

// LDS transpose read: the 16 lanes of a group pass 16 addresses of 4 consecutive
// 16-bit elements; lane i receives, for k = 0..3, element (i % 4) at the address
// given by lane (i / 4 + 4 * k) of its group.
__device__ __forceinline__ uint2 lds_read_tr16(const uint8_t *p)
{
#if defined(__HIP_DEVICE_COMPILE__)
    pf_v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pf_v4s __attribute__((address_space(3))) *)p);
    return __builtin_bit_cast(uint2, r);
#else
    (void)p;
    return make_uint2(0, 0);
#endif
}

// 32-bit LDS addresses, for code that does its own address arithmetic (xor swizzles)
typedef uint32_t pf_u32x4 __attribute__((ext_vector_type(4)));
typedef const pf_u32x4 __attribute__((address_space(3))) *pf_lds_u4_t;
typedef pf_v4s __attribute__((address_space(3))) *pf_lds_v4s_t;
__device__ __forceinline__ uint32_t pf_lds_addr(const void *p)
{
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}
__device__ __forceinline__ uint4 pf_lds_read128(uint32_t addr, int offset)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const pf_u32x4 v = *(pf_lds_u4_t)(uintptr_t)(addr + (uint32_t)offset);
    return make_uint4(v.x, v.y, v.z, v.w);
#else
    (void)addr; (void)offset;
    return make_uint4(0, 0, 0, 0);
#endif
}
__device__ __forceinline__ uint2 pf_lds_read_tr16(uint32_t addr, int offset)
{
#if defined(__HIP_DEVICE_COMPILE__)
    pf_v4s r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((pf_lds_v4s_t)(uintptr_t)(addr + (uint32_t)offset));
    return __builtin_bit_cast(uint2, r);
#else
    (void)addr; (void)offset;
    return make_uint2(0, 0);
#endif
}

// Workgroup barrier for kernels whose LDS is filled by direct loads from global memory: LDS reads and writes
// of the wave are complete, its outstanding global loads are NOT waited for (__syncthreads would drain them,
// the fence it carries covers every store into LDS) -- the caller counts those itself.
// The same, with the wait written so that the compiler knows of it: a scalar load issued before the barrier counts as
// arrived behind it (otherwise its first use drains the LDS reads issued since).
__device__ __forceinline__ void pf_barrier_lgkm()
{
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xc07f);                      // lgkmcnt(0)
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
#endif
}
__device__ __forceinline__ void pf_barrier_lds()
{
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_sched_barrier(0);                       // nor may the scheduler move work from one side to the other
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
#endif
}
// 16 bytes per lane from global memory straight into LDS: lane i's land at lds_addr + 16 i (lds_addr is the same
// for the whole wave).  Written as assembly so that the compiler does not know of the store into LDS: it would
// wait for every outstanding load ahead of the next LDS read.  The caller counts the loads (s_waitcnt vmcnt).
// The LDS address travels in M0, which the compiler reserves for instructions of its own that need it (indirect
// register indexing, its own direct loads) and loads right before each of them; the kernels that call this have
// none of those -- their arrays are indexed by constants after unrolling -- so nothing else reads M0, and the
// compiler's remark about the clobber is switched off here.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void pf_load_to_lds16(const void *base, uint32_t lane_offset, uint32_t lds_addr)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane_offset), "s"(base), "s"(lds_addr) : "memory", "m0");
#else
    (void)base; (void)lane_offset; (void)lds_addr;
#endif
}
#pragma clang diagnostic pop

struct PrefillArgs {
    const uint8_t *pool_layer;    // pool + layer * layer_stride
    const int32_t *table;
    const uint8_t *q;
    uint8_t *out;
    int pos_start, M, QH, KVH, NB, bs, bs_shift;
    int tpw;                      // query tokens per workgroup: 128 / (QH / KVH)
    unsigned head_stride, kv_plane, block_stride, scale_plane;
    float scale_log2e;
    // shared-prefix mode: row "token" = branch; every row sees tokens [0, min(len, shared))
    const int32_t *seq_lens;      // [M] on the device
    int shared, chunk_tiles, nsplits;
    float *part_o, *part_m, *part_l;
    // optional epilogue: out *= sigmoid(gate), gate rows gate_stride elements apart
    const uint16_t *gate;
    size_t gate_stride;
    // optional: the row's log2-sum-exp of its scaled scores, [M][QH] (+inf for a row that saw no token).  Written
    // by the chunk kernels where a row's walk ends; read by the mass kernel, which then walks the keys once.
    float *lse_rows;
    // prefill_d256_kernel only: a workgroup's 128 rows are 128 / gh query tokens x gh query heads (gh divides the
    // heads per kv head); nqt row blocks of tokens; workgroups [0, n_full) take whole walks, the others one of
    // kparts pieces of a walk each (tile ranges) and leave (o, m, l) per row and piece in part_o / part_m / part_l
    int gh, nqt, n_full, kparts;
};

// scheduling hints: order instruction groups inside one basic block
template <int MASK, int N>
__device__ __forceinline__ void pf_sched_group()
{
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_sched_group_barrier(MASK, N, 0);
#endif
}
__device__ __forceinline__ void pf_sched_barrier()
{
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_sched_barrier(0);
#endif
}

// one wave's group of ROWS consecutive tokens of a tile: ROWS rows of RB bytes = NL 128-bit loads per lane
template <int RB, int ROWS = 16>
struct PfGroup {
    static constexpr int NL = RB * ROWS / 1024;
    uint4 r[NL];
};

template <bool ONCE, int RB, int ROWS = 16>
__device__ __forceinline__ PfGroup<RB, ROWS> pf_load_group(const uint8_t *__restrict__ base, bool valid, size_t off, int lane)
{
    PfGroup<RB, ROWS> g;
#pragma unroll
    for (int j = 0; j < PfGroup<RB, ROWS>::NL; j++) g.r[j] = make_uint4(0, 0, 0, 0);
    if (valid) {
        const uint8_t *p = base + off + (size_t)lane * 16;
#pragma unroll
        for (int j = 0; j < PfGroup<RB, ROWS>::NL; j++) {
            if constexpr (ONCE) g.r[j] = ld_stream128(p + 1024 * j);   // every page is read by one workgroup only: stream it
            else g.r[j] = *(const uint4 *)(p + 1024 * j);              // the row tiles of a chunk share each page through the L2
        }
    }
    return g;
}

// 16-bit pages: the 16-byte chunk j of a lane belongs to row (lane * 16 + 1024 j) / RB of the group.
// Rows at or past `lim` may hold anything and are stored as zeros.
template <int PITCH, int RB, int ROWS = 16>
__device__ __forceinline__ void pf_store_group(uint8_t *lds, const PfGroup<RB, ROWS> &g, int w, int lane, int lim)
{
    const int bp0 = lane * 16, row0 = bp0 / RB;
    uint8_t *dst = lds + (w * ROWS + row0) * PITCH + bp0 % RB;
    constexpr int RSTEP = 1024 / RB;                          // rows between a lane's consecutive chunks
    if (lim >= ROWS) {                                        // the common case, wave-uniform
#pragma unroll
        for (int j = 0; j < PfGroup<RB, ROWS>::NL; j++) *(uint4 *)(dst + j * RSTEP * PITCH) = g.r[j];
    } else {
#pragma unroll
        for (int j = 0; j < PfGroup<RB, ROWS>::NL; j++)
            *(uint4 *)(dst + j * RSTEP * PITCH) = row0 + j * RSTEP < lim ? g.r[j] : make_uint4(0, 0, 0, 0);
    }
}

// 8-bit pages: chunk j of a lane holds 16 codes of row (lane * 16 + 1024 j) / RB; they are stored as
// the fp16 values code * scale (int8; sc[j] = the row's fp16 scale) or as the fp8 values themselves.
// Rows at or past `lim` may hold anything -- codes and scales -- and are stored as zeros.
template <int PITCH, int KV, int RB, int ROWS = 16>
__device__ __forceinline__ void pf_store_group_q8(uint8_t *lds, const PfGroup<RB, ROWS> &g, int w, int lane,
                                                  const uint16_t (&sc)[PfGroup<RB, ROWS>::NL], int lim)
{
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int j = 0; j < PfGroup<RB, ROWS>::NL; j++) {
        const int bp = lane * 16 + 1024 * j, row = bp / RB, col = bp % RB;
        uint32_t h[8];
        if constexpr (KV == DRK_INT8) {
            int8x4_to_f16x4(g.r[j].x, h[0], h[1]);
            int8x4_to_f16x4(g.r[j].y, h[2], h[3]);
            int8x4_to_f16x4(g.r[j].z, h[4], h[5]);
            int8x4_to_f16x4(g.r[j].w, h[6], h[7]);
            const uint32_t s16 = sc[j];
            const h2 scale = __builtin_bit_cast(h2, s16 | (s16 << 16));
            const h2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
#pragma unroll
            for (int i = 0; i < 8; i++) {                     // (1152 + code) - 1152 is exact; one rounding in the product
                const h2 v = (__builtin_bit_cast(h2, h[i]) - bias) * scale;
                h[i] = __builtin_bit_cast(uint32_t, v);
            }
        } else {
            fp8x4_to_f16x4(g.r[j].x, h[0], h[1]);
            fp8x4_to_f16x4(g.r[j].y, h[2], h[3]);
            fp8x4_to_f16x4(g.r[j].z, h[4], h[5]);
            fp8x4_to_f16x4(g.r[j].w, h[6], h[7]);
        }
        if (row >= lim) {
#pragma unroll
            for (int i = 0; i < 8; i++) h[i] = 0u;
        }
        uint8_t *dst = lds + (w * ROWS + row) * PITCH + col * 2;
        *(uint4 *)(dst) = make_uint4(h[0], h[1], h[2], h[3]);
        *(uint4 *)(dst + 16) = make_uint4(h[4], h[5], h[6], h[7]);
    }
}

// grid = (ceil(M/TPW) * KVH, 1[, splits]), TPW = 128 / (QH/KVH) query tokens per workgroup; block = 256.
// SHARED = false: causal prefill of a chunk, normalised output.
// SHARED = true:  the M rows are decode branches that share the pages of tokens
//                 [0, shared); workgroup z handles tokens [z, z+1) * chunk_tiles * 64 of
//                 them, no causal mask, and leaves (o, m, l) per (branch, q head, z).
// DT: the type the matrix cores multiply in; KV: the pages' storage type (DT, or int8 / fp8 with
// DT = fp16: the codes are dequantised on their way into LDS); IO: the type of q and out.
// D: head_dim, 128 (two workgroups per CU) or 256 (one: twice the LDS and the accumulators).
template <int DT, bool SHARED, int KV = DT, int IO = DT, int D = 128>
__global__ __launch_bounds__(256, D == 128 ? 2 : 1) void prefill_mfma_kernel(PrefillArgs A)
{
    constexpr bool Q8 = KV == DRK_INT8 || KV == DRK_FP8_E4M3;
    constexpr int RB = D * (Q8 ? 1 : 2);                    // bytes of one token row of one kv head
    constexpr int kPitchK = D * 2 + 16, kPitchV = D * 2 + 32;   // LDS row pitches: conflict-free for the two read patterns
    constexpr int NKS = D / 16;                             // k-steps of the first product
    constexpr int NDT = D / 32;                             // 32-dim tiles of the second
    // Two buffers per operand.  The loop is software-pipelined by one tile: while the softmax of
    // tile i runs on the vector ALU, the matrix cores already compute the scores of tile i+1, so
    // K is staged one tile further ahead than V.  One barrier per tile.
    __shared__ __align__(16) uint8_t k_lds2[2][kPfBN * kPitchK];
    __shared__ __align__(16) uint8_t v_lds2[2][kPfBN * kPitchV];
    __shared__ int valid_lds4[4][4];                       // page present, per (tile & 3, 16-token group)

    // Workgroups are dealt to the 8 XCDs round-robin by linear id; kv head = id % KVH
    // keeps one kv head's pages in one XCD's L2 (8 kv heads on 8 XCDs).
    const int kvh = (int)blockIdx.x % A.KVH;
    int qt = (int)blockIdx.x / A.KVH;
    if (!SHARED) {
        // causal chunks: row tile q walks pos_start + 32 (q + 1) tokens.  The second half of the grid is
        // taken in reverse, so that the two workgroups a CU holds when the grid is one resident round
        // (dispatch order: all first slots, then all second slots) are a short walk and a long one
        const int nqt = (int)gridDim.x / A.KVH, half = (nqt + 1) / 2;
        if (qt >= half) qt = nqt - 1 - (qt - half);
    }
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int n = lane & 31, g = lane >> 5;

    // this lane's query row: row r of the workgroup's 128 = token r / G of its TPW = 128 / G query
    // tokens, head r % G of the kv head's G query heads (the last 128 - TPW * G rows are idle)
    const int G = A.QH / A.KVH, TPW = A.tpw;
    const int r = w * 32 + n, rt = r / G;
    const int tq = qt * TPW + rt;
    const int head = kvh * G + (r - rt * G);
    const bool row_live = rt < TPW && tq < A.M;
    // shared mode with few branches: a wave whose 32 rows are all idle only helps to stage the
    // tiles; its first row decides, the rows of a wave being consecutive
    const bool wave_live = (w * 32) / G < TPW && qt * TPW + (w * 32) / G < A.M;
    int vis, lim_wg, t_begin = 0, first_masked_tile = 0;
    if (SHARED) {
        // a row's length: the branch's, or -- the rows being the tokens of a chunk -- pos_start + t + 1
        const int len = row_live ? (A.seq_lens ? A.seq_lens[tq] : A.pos_start + tq + 1) : 0;
        vis = min(len, A.shared);                               // tokens [0, vis) are visible to the row
        t_begin = (int)blockIdx.z * A.chunk_tiles;
        lim_wg = min(A.shared, (t_begin + A.chunk_tiles) * kPfBN);
    } else {
        vis = A.pos_start + tq + 1;
        lim_wg = A.pos_start + min((qt + 1) * TPW, A.M);        // exclusive limit over the workgroup
        first_masked_tile = (A.pos_start + qt * TPW + 1) / kPfBN;  // tiles below are fully visible
    }
    const int ntiles = (lim_wg + kPfBN - 1) / kPfBN;

    // Q as the B operand of S^T: NKS k-steps of 16 dims; lane holds dims ks*16 + g*8 .. +8
    uint4 qf[NKS];
    {
        const uint8_t *qrow = A.q + ((size_t)tq * A.QH + head) * (D * 2) + g * 16;
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            uint4 v = row_live ? *(const uint4 *)(qrow + ks * 32) : make_uint4(0, 0, 0, 0);
#if defined(__HIP_DEVICE_COMPILE__)
            if constexpr (IO == DRK_BF16 && DT == DRK_F16) {      // 8-bit pages multiply in fp16
                v.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.x), bf16_hi(v.x)));
                v.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.y), bf16_hi(v.y)));
                v.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.z), bf16_hi(v.z)));
                v.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.w), bf16_hi(v.w)));
            }
#endif
            qf[ks] = v;
        }
    }

    const uint8_t *kbase = A.pool_layer + (size_t)kvh * A.head_stride;
    // byte offset of the wave's 16-token row run of `tile` (soff: of its 16 fp16 K scales, int8 pages)
    auto lookup = [&](int tile, bool &valid, size_t &soff) -> size_t {
        int tg = tile * kPfBN + w * 16;
        valid = false;
        soff = 0;
        if (tg >= lim_wg) return 0;
        int lb = A.bs_shift >= 0 ? (tg >> A.bs_shift) : (tg / A.bs);
        int blk = A.table[lb];
        if (blk < 0 || blk >= A.NB) return 0;
        valid = true;
        const size_t base = (size_t)blk * A.block_stride;
        soff = base + 2 * (size_t)A.kv_plane + ((size_t)kvh * A.bs + (tg - lb * A.bs)) * 2;
        return base + (size_t)(tg - lb * A.bs) * RB;
    };

    pf_f32x16 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    // registers -> LDS; rows at or past the workgroup's limit may hold anything and are cleared
    bool kreg_valid = false;
    PfGroup<RB> kreg, vreg;
    constexpr int NL = PfGroup<RB>::NL;
    uint16_t ksc[NL], vsc[NL];                 // int8 pages: the fp16 scales of the rows of this lane's chunks
#pragma unroll
    for (int j = 0; j < NL; j++) ksc[j] = vsc[j] = 0;
    auto load_scales = [&](bool valid, size_t soff, uint16_t (&sc)[NL]) {
#pragma unroll
        for (int j = 0; j < NL; j++) {
            const int row = (lane * 16 + 1024 * j) / RB;
            sc[j] = (KV == DRK_INT8 && valid) ? *(const uint16_t *)(A.pool_layer + soff + row * 2) : (uint16_t)0;   // no page: zero codes times zero
        }
    };
    auto fetch_k = [&](int tile) {
        size_t soff;
        const size_t off = lookup(tile, kreg_valid, soff);
        kreg = pf_load_group<SHARED, RB>(kbase, kreg_valid, off, lane);
        load_scales(kreg_valid, soff, ksc);
    };
    auto fetch_v = [&](int tile) {
        bool ok;
        size_t soff;
        const size_t off = lookup(tile, ok, soff);
        vreg = pf_load_group<SHARED, RB>(kbase + A.kv_plane, ok, off, lane);
        load_scales(ok, soff + A.scale_plane, vsc);
    };
    auto stage_k = [&](int tile) {
        const int lim = lim_wg - tile * kPfBN - w * 16;        // rows of this wave's group that exist
        if constexpr (Q8) pf_store_group_q8<kPitchK, KV, RB>(&k_lds2[(tile - t_begin) & 1][0], kreg, w, lane, ksc, lim);
        else pf_store_group<kPitchK, RB>(&k_lds2[(tile - t_begin) & 1][0], kreg, w, lane, lim);
        if (lane == 0) valid_lds4[tile & 3][w] = kreg_valid ? 1 : 0;
    };
    auto stage_v = [&](int tile) {
        const int lim = lim_wg - tile * kPfBN - w * 16;
        if constexpr (Q8) pf_store_group_q8<kPitchV, KV, RB>(&v_lds2[(tile - t_begin) & 1][0], vreg, w, lane, vsc, lim);
        else pf_store_group<kPitchV, RB>(&v_lds2[(tile - t_begin) & 1][0], vreg, w, lane, lim);
    };
    // S^T = K Q^T : two 32-token tiles x 32 rows, NKS k-steps of 16 dims
    auto qk = [&](int tile, pf_f32x16 (&s)[2]) {
        const uint8_t *ka = &k_lds2[(tile - t_begin) & 1][0] + n * kPitchK + g * 16;
        const pf_f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};     // constant C operand of the first k-step
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            const uint4 a0 = *(const uint4 *)(ka + ks * 32);
            const uint4 a1 = *(const uint4 *)(ka + 32 * kPitchK + ks * 32);
            s[0] = mfma32<DT>(a0, qf[ks], ks == 0 ? zero : s[0]);
            s[1] = mfma32<DT>(a1, qf[ks], ks == 0 ? zero : s[1]);
        }
    };

    pf_f32x16 s_even[2], s_odd[2];          // scores of the tiles at even / odd distance from t_begin
    pf_f32x16 (&s)[2] = s_even;
    if (t_begin < ntiles) {
        fetch_k(t_begin);
        fetch_v(t_begin);
        stage_k(t_begin);
        stage_v(t_begin);
        if (t_begin + 1 < ntiles) {
            fetch_k(t_begin + 1);
            fetch_v(t_begin + 1);
        }
    }
    __syncthreads();
    if (t_begin < ntiles) {
        if (!SHARED || wave_live) qk(t_begin, s);
        if (t_begin + 1 < ntiles) {
            stage_k(t_begin + 1);
            if (t_begin + 2 < ntiles) fetch_k(t_begin + 2);
        }
    }
    __syncthreads();

    auto tile_step = [&](int it, pf_f32x16 (&s)[2], pf_f32x16 (&s_next)[2]) {
        // here: s = scores of tile it; K(it+1) and V(it) are in LDS; kreg holds K(it+2), vreg V(it+1)
        const int tile_t = it * kPfBN;
        const uint8_t *v_lds = &v_lds2[(it - t_begin) & 1][0];
        const int *valid_lds = &valid_lds4[it & 3][0];
        if (it + 2 < ntiles) {
            stage_k(it + 2);                       // into the buffer K(it) was read from one iteration ago
            if (it + 3 < ntiles) fetch_k(it + 3);
        }
        if (it + 1 < ntiles) {
            stage_v(it + 1);                       // into the buffer V(it-1) was read from
            if (it + 2 < ntiles) fetch_v(it + 2);
        }
        if (!SHARED || wave_live) {                           // (a chunk's rows are all live but for its last workgroup)
            // ---- tile softmax for this lane's row; register i of tile tt is token
            //      tile_t + tt*32 + 8*(i/4) + 4*g + i%4 ----
            const bool all_groups_valid = (valid_lds[0] & valid_lds[1] & valid_lds[2] & valid_lds[3]) != 0;
            const bool need_mask = !all_groups_valid ||
                                   (SHARED ? (__any(tile_t + kPfBN > vis) != 0) : (it >= first_masked_tile));
            // raw scores stay in s; the scale (> 0) is folded into the exponent's fma
            if (need_mask) {                                         // one uniform branch around all 32 selects
    #pragma unroll
                for (int tt = 0; tt < 2; tt++)
    #pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int tl = tt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
                        const bool ok = (tile_t + tl) < vis && valid_lds[tl >> 4] != 0;
                        s[tt][i] = ok ? s[tt][i] : -INFINITY;
                    }
            }
            float tmax = -INFINITY;
    #pragma unroll
            for (int tt = 0; tt < 2; tt++)
    #pragma unroll
                for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[tt][i]);
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32));               // the row's other 32 tokens
            const float m_new = fmaxf(m_run, tmax * A.scale_log2e);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
            float psum = 0.0f;
            uint4 pb[2][2];                                          // [token tile][k-half]: B operand of PV
    #pragma unroll
            for (int tt = 0; tt < 2; tt++) {
                float p[16];
    #pragma unroll
                for (int i = 0; i < 16; i++) p[i] = __builtin_amdgcn_exp2f(fmaf(s[tt][i], A.scale_log2e, -m_use));
                pb[tt][0] = make_uint4(pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7]));
                pb[tt][1] = make_uint4(pack2<DT>(p[8], p[9]), pack2<DT>(p[10], p[11]), pack2<DT>(p[12], p[13]), pack2<DT>(p[14], p[15]));
                // the row sum is taken over the rounded weights, the ones PV multiplies: one dot2 per pair
                psum = pf_sum2<DT>(pb[tt][0], psum);
                psum = pf_sum2<DT>(pb[tt][1], psum);
            }
            l_run = l_run * alpha + psum;
            m_run = m_new;
            if (!__all(alpha == 1.0f)) {
    #pragma unroll
                for (int dt = 0; dt < NDT; dt++)
    #pragma unroll
                    for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
            }

            // The next tile's scores, in the same basic block as the exponentials and the PV product so
            // that matrix and vector instructions alternate.  Unconditional: past the last tile it
            // multiplies whatever the other K buffer holds and the result is dropped.
            qk(it + 1, s_next);

            // ---- O^T += V^T P^T : k-slot j of MFMA (tt, mh) is token tt*32 + 16*mh + 8*(j/4) + 4*g + j%4 ----
            {
                const int j16 = lane & 15;
                const int dsub = 16 * ((lane >> 4) & 1) + 4 * (j16 & 3);           // d offset inside a 32-d tile
                const uint8_t *vb = v_lds + (4 * g + (j16 >> 2)) * kPitchV + dsub * 2;
    #pragma unroll
                for (int tt = 0; tt < 2; tt++)
    #pragma unroll
                    for (int mh = 0; mh < 2; mh++) {
                        const uint8_t *vt = vb + (tt * 32 + 16 * mh) * kPitchV;
    #pragma unroll
                        for (int dt = 0; dt < NDT; dt++) {
                            const uint2 lo = lds_read_tr16(vt + dt * 64);
                            const uint2 hi = lds_read_tr16(vt + 8 * kPitchV + dt * 64);
                            o[dt] = mfma32<DT>(make_uint4(lo.x, lo.y, hi.x, hi.y), pb[tt][mh], o[dt]);
                        }
                    }
            }
        }
        __syncthreads();
    };
    // two tiles per trip, the two score register sets swapping roles (no copies)
    for (int it = t_begin; it < ntiles; it += 2) {
        tile_step(it, s_even, s_odd);
        if (it + 1 < ntiles) tile_step(it + 1, s_odd, s_even);
    }

    // ---- register i of tile dt is d = dt*32 + 8*(i/4) + 4*g + i%4 ----
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (!SHARED && A.lse_rows && row_live && g == 0)
        A.lse_rows[(size_t)tq * A.QH + head] = l_tot > 0.0f ? m_run + __builtin_log2f(l_tot) : INFINITY;
    if (SHARED) {
        if (row_live) {                      // unnormalised partial; an empty range leaves (0, -inf, 0)
            const size_t pi = ((size_t)tq * A.QH + head) * A.nsplits + blockIdx.z;
            float *orow = A.part_o + pi * D;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int b4 = 0; b4 < 4; b4++)
                    *(float4 *)(orow + dt * 32 + 8 * b4 + 4 * g) =
                        make_float4(o[dt][4 * b4], o[dt][4 * b4 + 1], o[dt][4 * b4 + 2], o[dt][4 * b4 + 3]);
            if (g == 0) {
                A.part_m[pi] = m_run;
                A.part_l[pi] = l_tot;
            }
        }
    } else if (row_live && (l_tot > 0.0f || A.gate)) {
        // with a gate the row is always rewritten: the reference gates whatever the attention
        // kernel left in out, also when no token took part (paged_attention.cu:551, 633-634)
        const bool have = l_tot > 0.0f;
        const float inv = have ? 1.0f / l_tot : 0.0f;
        uint8_t *orow = A.out + ((size_t)tq * A.QH + head) * (D * 2);
        const uint16_t *grow = A.gate ? A.gate + ((size_t)tq * A.QH + head) * A.gate_stride : nullptr;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int b4 = 0; b4 < 4; b4++) {
                const int d0 = dt * 32 + 8 * b4 + 4 * g;
                uint2 v = have ? make_uint2(pack2<IO>(o[dt][4 * b4] * inv, o[dt][4 * b4 + 1] * inv),
                                            pack2<IO>(o[dt][4 * b4 + 2] * inv, o[dt][4 * b4 + 3] * inv))
                               : *(const uint2 *)(orow + d0 * 2);
                if (grow) {
                    const uint2 gv = *(const uint2 *)(grow + d0);
                    v.x = (uint32_t)gated_elem16((uint16_t)(v.x & 0xffffu), (uint16_t)(gv.x & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.x >> 16), (uint16_t)(gv.x >> 16), IO) << 16);
                    v.y = (uint32_t)gated_elem16((uint16_t)(v.y & 0xffffu), (uint16_t)(gv.y & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.y >> 16), (uint16_t)(gv.y >> 16), IO) << 16);
                }
                *(uint2 *)(orow + d0 * 2) = v;
            }
    }
}

// As pf_store_group, without a branch: every chunk is a select between the loaded bytes and zeros.
template <int PITCH, int RB, int ROWS>
__device__ __forceinline__ void pf_store_group_sel(uint8_t *lds, const PfGroup<RB, ROWS> &g, int w, int lane, int lim)
{
    const int bp0 = lane * 16, row0 = bp0 / RB;
    uint8_t *dst = lds + (w * ROWS + row0) * PITCH + bp0 % RB;
    constexpr int RSTEP = 1024 / RB;
#pragma unroll
    for (int j = 0; j < PfGroup<RB, ROWS>::NL; j++) {
        const bool ok = row0 + j * RSTEP < lim;
        const uint4 v = g.r[j];
        *(uint4 *)(dst + j * RSTEP * PITCH) = make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
    }
}

// max(x of lane n, x of lane n ^ 32) without a trip through LDS
__device__ __forceinline__ float pf_max_halves(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

// ---- the chunk kernel in two phases ("ping-pong") ---------------------------------------------
// In the kernel above the matrix cores and the vector ALU mostly take turns: the two waves that
// share a SIMD (from two independent workgroups) drift into the same phase and then wait for the
// same unit.  Here ONE workgroup of eight waves holds 256 rows (wave w: rows 32 w .. 32 w + 31),
// waves w and w + 4 share a SIMD, and the two halves of the workgroup are kept half a tile apart
// by the workgroup barrier itself: between two barriers waves 0-3 run the softmax of tile t on the
// vector ALU while waves 4-7 run their matrix products (PV of tile t-1, QK^T of tile t); after the
// next barrier the roles swap.  The matrix pipe of every SIMD always has one wave to take work from.
//
//   even phase 2t    A (waves 0-3): its share of K(t+1), V(t) -> LDS; softmax(t)
//                    B (waves 4-7): PV(t-1), QK^T(t)
//   odd phase 2t+1   A: PV(t), QK^T(t+1)
//                    B: softmax(t); its share of K(t+2), V(t+1) -> LDS
//
// The memory side of a tile rides in the wave's vector phase (registers -> LDS, then the global loads
// of the next tile into the same registers); it is straight-line code -- a taken branch costs a wave
// tens of cycles, and a staging step with a dozen of them cost more than the softmax.  A buffer is
// rewritten between its last reader's barrier and its next reader's: K(x) in phase 2x-3 or 2x-2,
// V(x) in phase 2x-1 or 2x.  One set of score registers per wave is enough: the scores of a tile are
// dead once its weights are packed.
// grid = ceil(M / TPW) * KVH with TPW = 256 / (QH/KVH) query tokens per workgroup, longest walk
// first; block = 512; one workgroup per CU.  head_dim 128; causal chunks only.
template <int DT, int KV = DT, int IO = DT>
__global__ __launch_bounds__(512, 1) void prefill_pp_kernel(PrefillArgs A)
{
    constexpr int D = 128;
    constexpr bool Q8 = KV == DRK_INT8 || KV == DRK_FP8_E4M3;
    constexpr int RB = D * (Q8 ? 1 : 2);
    constexpr int kPitchK = D * 2 + 16, kPitchV = D * 2 + 32;
    constexpr int NKS = D / 16, NDT = D / 32;
    constexpr int ROWS = 8;                                 // tokens of a tile one wave stages
    __shared__ __align__(16) uint8_t k_lds2[2][kPfBN * kPitchK];
    __shared__ __align__(16) uint8_t v_lds2[2][kPfBN * kPitchV];

    // workgroup = (walk, part), as in prefill_ppd_kernel: with A.kparts > 1 a part is one of A.kparts ranges of the
    // walk's tiles and leaves (o, m, l) per row for prefill_merge_kernel
    const int kp = A.kparts;
    const int walk = (int)blockIdx.x / kp, part = (int)blockIdx.x - walk * kp;
    const int kvh = walk % A.KVH;
    const int nqt = (int)gridDim.x / (A.KVH * kp);
    const int qt = nqt - 1 - walk / A.KVH;                   // the longest walks are dispatched first
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int n = lane & 31, g = lane >> 5;
    const bool grpA = w < 4;

    const int G = A.QH / A.KVH, TPW = A.tpw;
    const int r = w * 32 + n, rt = r / G;
    const int tq = qt * TPW + rt;
    const int head = kvh * G + (r - rt * G);
    const bool row_live = rt < TPW && tq < A.M;
    const int vis = A.pos_start + tq + 1;
    const int lim_wg = A.pos_start + min((qt + 1) * TPW, A.M);
    const int first_masked_tile = (A.pos_start + qt * TPW + 1) / kPfBN;
    const int nt_walk = (lim_wg + kPfBN - 1) / kPfBN;
    const int t_begin = __builtin_amdgcn_readfirstlane((int)((long)part * nt_walk / kp));
    const int ntiles = __builtin_amdgcn_readfirstlane((int)((long)(part + 1) * nt_walk / kp));   // the part's tiles: [t_begin, ntiles)
    const int lim_part = min(lim_wg, ntiles * kPfBN);        // rows past the part's end are stored as zeros
    if (t_begin >= ntiles) {                                 // more parts than tiles: an empty piece
        if (row_live && g == 0) A.part_l[((size_t)tq * A.QH + head) * kp + part] = 0.0f;
        return;
    }

    // Q as the B operand, multiplied by scale * log2(e) on the way in (rounded once more to the 16-bit
    // type): the products then are the exponents themselves and the softmax needs no multiply per score.
    uint4 qf[NKS];
    {
        const uint8_t *qrow = A.q + ((size_t)tq * A.QH + head) * (D * 2) + g * 16;
        const float c = A.scale_log2e;
        auto scaled = [&](uint32_t w2) -> uint32_t {
            return pack2<DT>(elem16_to_f((uint16_t)(w2 & 0xffffu), IO) * c, elem16_to_f((uint16_t)(w2 >> 16), IO) * c);
        };
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            const uint4 v = row_live ? *(const uint4 *)(qrow + ks * 32) : make_uint4(0, 0, 0, 0);
            qf[ks] = make_uint4(scaled(v.x), scaled(v.y), scaled(v.z), scaled(v.w));
        }
    }

    const uint8_t *kbase = A.pool_layer + (size_t)kvh * A.head_stride;
    // ---- pages -------------------------------------------------------------------------------------
    // The block size is a power of two >= 16 (the host dispatches other sizes to the kernel above), so the
    // 8 tokens a wave stages lie in one block, a 16-token run has one page, and a tile's blocks never
    // straddle a multiple of 64.  Table entries come in windows of 64, one per lane, by a vector load (a
    // scalar load would be waited for at every barrier, whose LDS wait counts on the same counter); two
    // windows are held, so an entry is in a register long before its tile is reached.  Everything here is
    // wave-uniform, straight-line code: the only branch is the change of window, every 64 blocks.
    const int sh = A.bs_shift;
    const int tgw = w * ROWS;                                 // the wave's first token within a tile
    const int nblk_needed = (lim_wg + A.bs - 1) >> sh;
    auto load_window = [&](int lb0) -> int {
        const int i = lb0 + lane;
        return i < nblk_needed ? A.table[i] : -1;             // entries past the chunk's last block are never read
    };
    auto pages_of = [&](int win) -> unsigned long long { return __builtin_amdgcn_ballot_w64(win >= 0 && win < A.NB); };
    int win_lb0 = (((t_begin * kPfBN) >> sh) >> 6) << 6;
    int win_a = load_window(win_lb0), win_b = load_window(win_lb0 + 64);
    unsigned long long present_a = pages_of(win_a);           // bit i: block win_lb0 + i has a page
    // the wave's page in `tile` (-1: a hole, or past the end) and the tile's four page flags, one per 16-token run
    auto lookup = [&](int tile, int &blk, int &flags) {
        const int lb0 = (tile * kPfBN) >> sh;
        if (__builtin_expect(lb0 >= win_lb0 + 64, 0)) {       // tiles are asked for in ascending order
            win_lb0 += 64;
            win_a = win_b;
            win_b = load_window(win_lb0 + 64);
            present_a = pages_of(win_a);
        }
        const uint32_t m = (uint32_t)(present_a >> (lb0 - win_lb0));
        flags = (int)((m & 1u) | (((m >> (16 >> sh)) & 1u) << 1) | (((m >> (32 >> sh)) & 1u) << 2) | (((m >> (48 >> sh)) & 1u) << 3));
        const int tg = tile * kPfBN + tgw;
        const int li = (tg >> sh) - win_lb0;
        const int b = __builtin_amdgcn_readlane(win_a, li);
        blk = (((present_a >> li) & 1ull) != 0 && tg < lim_part) ? b : -1;
    };

    pf_f32x16 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.0f;
    // The softmax reference m_ref (per row): the products start from -m_ref (the C operand), so a score
    // arrives as its exponent relative to the reference.  The reference moves only when a tile's maximum
    // exceeds it by more than kLazy (or is the row's first finite one): weights stay below 2^kLazy, and O
    // and the row sum are rescaled on those rare occasions only.  out = O / l does not depend on it.
    constexpr float kLazy = 8.0f;
    float m_ref = 0.0f, l_run = 0.0f;
    bool m_init = false;
    pf_f32x16 negm;
#pragma unroll
    for (int i = 0; i < 16; i++) negm[i] = 0.0f;

    // ---- staging -----------------------------------------------------------------------------------
    // A wave moves 8 rows of K and of V per tile: global -> registers one tile ahead, registers -> LDS when
    // the buffer's last readers have passed.  No branches: a missing page is read from block 0 instead and
    // stored as zeros, like the rows past the chunk's end (which may hold anything).
    constexpr int NL = PfGroup<RB, ROWS>::NL;
    PfGroup<RB, ROWS> kreg, vreg;
    uint16_t ksc[NL], vsc[NL];
    int klim = 0, vlim = 0;                                  // rows of kreg / vreg that are real
    auto fetch = [&](PfGroup<RB, ROWS> &reg, uint16_t (&sc)[NL], int &lim, bool is_v, int tile, int blk) {
        const int tg = tile * kPfBN + tgw;
        const int tin = tg & (A.bs - 1);
        const size_t boff = (size_t)max(blk, 0) * A.block_stride;
        const uint8_t *p = kbase + (is_v ? A.kv_plane : 0) + boff + (size_t)tin * RB + (size_t)lane * 16;
#pragma unroll
        for (int j = 0; j < NL; j++) reg.r[j] = *(const uint4 *)(p + 1024 * j);   // the row tiles of a chunk share each page through the L2
#pragma unroll
        for (int j = 0; j < NL; j++) {
            if constexpr (KV == DRK_INT8) {
                const int row = (lane * 16 + 1024 * j) / RB;
                const size_t soff = boff + 2 * (size_t)A.kv_plane + (is_v ? A.scale_plane : 0) + ((size_t)kvh * A.bs + tin + row) * 2;
                sc[j] = *(const uint16_t *)(A.pool_layer + soff);
            } else {
                sc[j] = 0;
            }
        }
        lim = blk >= 0 ? lim_part - tg : 0;
    };
    auto stage_k = [&](int tile) {
        if constexpr (Q8) pf_store_group_q8<kPitchK, KV, RB, ROWS>(&k_lds2[tile & 1][0], kreg, w, lane, ksc, klim);
        else pf_store_group_sel<kPitchK, RB, ROWS>(&k_lds2[tile & 1][0], kreg, w, lane, klim);
    };
    auto stage_v = [&](int tile) {
        if constexpr (Q8) pf_store_group_q8<kPitchV, KV, RB, ROWS>(&v_lds2[tile & 1][0], vreg, w, lane, vsc, vlim);
        else pf_store_group_sel<kPitchV, RB, ROWS>(&v_lds2[tile & 1][0], vreg, w, lane, vlim);
    };

    pf_f32x16 s[2];                 // scores of the tile in flight: [32-token half][16 per lane]
    uint4 pb[2][2];                 // its weights, packed: [token half][k-half], the B operand of PV

    // S^T = K Q^T.  The operand reads run two k-steps ahead of the products that use them; scheduling
    // barriers pin that order, so that at most six operands are in registers at a time.
    auto qk = [&](int tile) {
        const uint8_t *ka = &k_lds2[tile & 1][0] + n * kPitchK + g * 16;
        uint4 a[NKS][2];
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            a[ks][0] = *(const uint4 *)(ka + ks * 32);
            a[ks][1] = *(const uint4 *)(ka + 32 * kPitchK + ks * 32);
        }
        pf_sched_barrier();
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            if (ks + 2 < NKS) {
                a[ks + 2][0] = *(const uint4 *)(ka + (ks + 2) * 32);
                a[ks + 2][1] = *(const uint4 *)(ka + 32 * kPitchK + (ks + 2) * 32);
            }
            if (ks == 0) {                                   // the products start from minus the row's reference
                s[0] = mfma32<DT>(a[ks][0], qf[ks], negm);
                s[1] = mfma32<DT>(a[ks][1], qf[ks], negm);
            } else {
                s[0] = mfma32<DT>(a[ks][0], qf[ks], s[0]);
                s[1] = mfma32<DT>(a[ks][1], qf[ks], s[1]);
            }
            pf_sched_barrier();
        }
    };
    // O^T += V^T P^T: 16 products, two transposed 8-byte reads each, the reads four products ahead
    auto pv = [&](int tile) {
        const uint8_t *v_lds = &v_lds2[tile & 1][0];
        const int j16 = lane & 15;
        const int dsub = 16 * ((lane >> 4) & 1) + 4 * (j16 & 3);
        const uint8_t *vb = v_lds + (4 * g + (j16 >> 2)) * kPitchV + dsub * 2;
        uint2 lo[16], hi[16];
        auto rd = [&](int i) {                               // product i = (tt, mh, dt) = (i / 8, (i / 4) & 1, i & 3)
            const uint8_t *vt = vb + ((i >> 3) * 32 + 16 * ((i >> 2) & 1)) * kPitchV + (i & 3) * 64;
            lo[i] = lds_read_tr16(vt);
            hi[i] = lds_read_tr16(vt + 8 * kPitchV);
        };
#pragma unroll
        for (int i = 0; i < 4; i++) rd(i);
        pf_sched_barrier();
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if (i + 4 < 16) rd(i + 4);
            o[i & 3] = mfma32<DT>(make_uint4(lo[i].x, lo[i].y, hi[i].x, hi[i].y), pb[i >> 3][(i >> 2) & 1], o[i & 3]);
            pf_sched_barrier();
        }
    };
    // scores of tile `it` (page flags `flags`) -> packed weights, running maximum and sum, rescale of O^T
    auto softmax = [&](int it, int flags) {
        const int tile_t = it * kPfBN;
        if (flags != 15 || it >= first_masked_tile) {
#pragma unroll
            for (int tt = 0; tt < 2; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int tl = tt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
                    const bool ok = (tile_t + tl) < vis && ((flags >> (tl >> 4)) & 1) != 0;
                    s[tt][i] = ok ? s[tt][i] : -INFINITY;
                }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[tt][i]);
        tmax = pf_max_halves(tmax);                          // a row's scores lie in lanes n and n + 32
        const bool move = m_init ? tmax > kLazy : tmax > -INFINITY;
        if (__any(move)) {
            const float delta = move ? tmax : 0.0f;
            m_init = m_init || move;
            m_ref += delta;
            const float alpha = __builtin_amdgcn_exp2f(-delta);
            l_run *= alpha;
#pragma unroll
            for (int tt = 0; tt < 2; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) s[tt][i] -= delta;
#pragma unroll
            for (int i = 0; i < 16; i++) negm[i] = -m_ref;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
        }
        float psum = 0.0f;
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
            float p[16];
#pragma unroll
            for (int i = 0; i < 16; i++) p[i] = __builtin_amdgcn_exp2f(s[tt][i]);
            pb[tt][0] = make_uint4(pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7]));
            pb[tt][1] = make_uint4(pack2<DT>(p[8], p[9]), pack2<DT>(p[10], p[11]), pack2<DT>(p[12], p[13]), pack2<DT>(p[14], p[15]));
            psum = pf_sum2<DT>(pb[tt][0], psum);
            psum = pf_sum2<DT>(pb[tt][1], psum);
        }
        l_run += psum;
    };

    // The memory side of tile t, this wave's share: K(t+1) and V(t) go from registers to LDS, then K(t+2)
    // and V(t+1) are requested.  fl0 / fl1 / fl2 are the page flags of tiles t, t+1, t+2 afterwards.
    int blk_next, fl0 = 15, fl1, fl2;                         // blk_next: the wave's page in tile t+1
    auto stage = [&](int t) {
        stage_k(t + 1);
        stage_v(t);
        int blk2, f;
        lookup(t + 2, blk2, f);
        fetch(kreg, ksc, klim, false, t + 2, blk2);
        fetch(vreg, vsc, vlim, true, t + 1, blk_next);
        blk_next = blk2;
        fl0 = fl1;
        fl1 = fl2;
        fl2 = f;
    };

    // ---- prologue: K(0) in LDS; K(1) and V(0) in registers (tiles counted from the part's first) ----
    {
        int blk0;
        lookup(t_begin, blk0, fl1);
        fetch(kreg, ksc, klim, false, t_begin, blk0);
        stage_k(t_begin);
        lookup(t_begin + 1, blk_next, fl2);
        fetch(kreg, ksc, klim, false, t_begin + 1, blk_next);
        fetch(vreg, vsc, vlim, true, t_begin, blk0);
    }
    __syncthreads();
    // Both halves pass the same number of barriers, 2 ntiles + 1.  The loop bodies are straight-line code
    // (the accumulators are updated in place): the product past the last tile multiplies whatever the other
    // K buffer holds and its result is never read, and the staging past the last tile stores zeros.
    // A buffer is rewritten only between its last reader's barrier and its next reader's: K(x) in phases
    // 2x-3 or 2x-2, V(x) in phases 2x-1 or 2x (phase 2t: softmax of A / products of B for tile t).
    if (grpA) {
        qk(t_begin);
#pragma unroll 1
        for (int t = t_begin; t < ntiles; t++) {
            stage(t);                                        // phase 2t: K(t+1), V(t)
            softmax(t, fl0);
            __syncthreads();
            pv(t);
            qk(t + 1);
            __syncthreads();
        }
        __syncthreads();
    } else {
        stage(t_begin);                                      // phase 0: K(1), V(0)
        qk(t_begin);
        __syncthreads();
#pragma unroll 1
        for (int t = t_begin; t < ntiles; t++) {
            softmax(t, fl0);
            stage(t + 1);                                    // phase 2t+1: K(t+2), V(t+1)
            __syncthreads();
            pv(t);
            qk(t + 1);
            __syncthreads();
        }
    }

    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (kp > 1) {                                            // a piece: the sums as they are, relative to m_ref (log2 units)
        if (row_live) {
            const size_t slot = ((size_t)tq * A.QH + head) * kp + part;
            if (g == 0) {
                A.part_m[slot] = m_ref;
                A.part_l[slot] = l_tot;
            }
            float *po = A.part_o + slot * D;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int b4 = 0; b4 < 4; b4++)
                    *(float4 *)(po + dt * 32 + 8 * b4 + 4 * g) = make_float4(o[dt][4 * b4], o[dt][4 * b4 + 1], o[dt][4 * b4 + 2], o[dt][4 * b4 + 3]);
        }
        return;
    }
    if (A.lse_rows && row_live && g == 0)      // m_ref is the reference the weights were taken against, in log2 units
        A.lse_rows[(size_t)tq * A.QH + head] = l_tot > 0.0f ? m_ref + __builtin_log2f(l_tot) : INFINITY;
    if (row_live && (l_tot > 0.0f || A.gate)) {
        const bool have = l_tot > 0.0f;
        const float inv = have ? 1.0f / l_tot : 0.0f;
        uint8_t *orow = A.out + ((size_t)tq * A.QH + head) * (D * 2);
        const uint16_t *grow = A.gate ? A.gate + ((size_t)tq * A.QH + head) * A.gate_stride : nullptr;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int b4 = 0; b4 < 4; b4++) {
                const int d0 = dt * 32 + 8 * b4 + 4 * g;
                uint2 v = have ? make_uint2(pack2<IO>(o[dt][4 * b4] * inv, o[dt][4 * b4 + 1] * inv),
                                            pack2<IO>(o[dt][4 * b4 + 2] * inv, o[dt][4 * b4 + 3] * inv))
                               : *(const uint2 *)(orow + d0 * 2);
                if (grow) {
                    const uint2 gv = *(const uint2 *)(grow + d0);
                    v.x = (uint32_t)gated_elem16((uint16_t)(v.x & 0xffffu), (uint16_t)(gv.x & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.x >> 16), (uint16_t)(gv.x >> 16), IO) << 16);
                    v.y = (uint32_t)gated_elem16((uint16_t)(v.y & 0xffffu), (uint16_t)(gv.y & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.y >> 16), (uint16_t)(gv.y >> 16), IO) << 16);
                }
                *(uint2 *)(orow + d0 * 2) = v;
            }
    }
}

// ---- the two-phase kernel for 16-bit pages: global -> LDS without registers -------------------------
// As prefill_pp_kernel, but the tiles go from global memory straight into LDS (global_load_lds_dwordx4): a wave's
// share of a tile is four memory instructions instead of four loads, four LDS writes and the selects between
// them, and holds no registers, so the requests can run two tiles ahead of their use (four buffers per operand)
// where registers allowed one.  Swizzled rows without padding instead of padded rows.  What bounds a wave's vector
// phase is its instruction count -- a wave issues one instruction in about four clocks, scalar ones included --
// so the phase is kept short: one straight path for whole pages, page addresses from scalar registers, the rare
// cases (masked tiles, a moving softmax reference, pages in part) out of line.  8-bit pages keep the kernel above
// (their codes are converted on the way).  A chunk too short to give every CU a walk (A.kparts > 1: the context-split
// path, 256 or more rows per kv head) has every walk in parts -- ranges of its tiles, a workgroup each -- that leave
// (o, m, l) per row for prefill_merge_kernel.
template <int DT, int IO = DT>
__global__ __launch_bounds__(512, 1) void prefill_ppd_kernel(PrefillArgs A)
{
    constexpr int D = 128;
    constexpr int RB = D * 2;                                // bytes of a token row of one kv head, also the LDS row
    constexpr int kTileBytes = kPfBN * RB;                   // 16 KB per operand and tile
    constexpr int NKS = D / 16, NDT = D / 32;
    constexpr int ROWS = 8;                                 // tokens of a tile one wave stages
    constexpr int kRing = 4;                                // buffers per operand
    __shared__ __align__(256) uint8_t k_lds3[kRing][kTileBytes];    // 256: the xor swizzle is applied to whole addresses
    __shared__ __align__(256) uint8_t v_lds3[kRing][kTileBytes];

    // workgroup = (walk, part): a walk is (row block, kv head); A.kparts > 1 (a chunk too short to fill the chip with its
    // walks): a part is one of A.kparts ranges of the walk's tiles and leaves (o, m, l) per row for prefill_merge_kernel
    const int kp = A.kparts;
    const int walk = (int)blockIdx.x / kp, part = (int)blockIdx.x - walk * kp;
    const int kvh = walk % A.KVH;
    const int nqt = (int)gridDim.x / (A.KVH * kp);
    const int qt = nqt - 1 - walk / A.KVH;                   // the longest walks are dispatched first
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int n = lane & 31, g = lane >> 5;
    const bool grpA = w < 4;

    const int G = A.QH / A.KVH, TPW = A.tpw;
    const int r = w * 32 + n, rt = r / G;
    const int tq = qt * TPW + rt;
    const int head = kvh * G + (r - rt * G);
    const bool row_live = rt < TPW && tq < A.M;
    const int vis = A.pos_start + tq + 1;
    const int lim_wg = A.pos_start + min((qt + 1) * TPW, A.M);
    const int first_masked_tile = (A.pos_start + qt * TPW + 1) / kPfBN;
    const int nt_walk = (lim_wg + kPfBN - 1) / kPfBN;
    const int t_begin = __builtin_amdgcn_readfirstlane((int)((long)part * nt_walk / kp));
    const int ntiles = __builtin_amdgcn_readfirstlane((int)((long)(part + 1) * nt_walk / kp));   // the part's tiles: [t_begin, ntiles)
    const int lim_part = min(lim_wg, ntiles * kPfBN);        // nothing past the part's end is requested
    if (t_begin >= ntiles) {                                 // more parts than tiles: an empty piece
        if (row_live && g == 0) A.part_l[((size_t)tq * A.QH + head) * kp + part] = 0.0f;
        return;
    }

    // Q as the B operand, multiplied by scale * log2(e) on the way in (rounded once more to the 16-bit
    // type): the products then are the exponents themselves and the softmax needs no multiply per score.
    uint4 qf[NKS];
    {
        const uint8_t *qrow = A.q + ((size_t)tq * A.QH + head) * (D * 2) + g * 16;
        const float c = A.scale_log2e;
        auto scaled = [&](uint32_t w2) -> uint32_t {
            return pack2<DT>(elem16_to_f((uint16_t)(w2 & 0xffffu), IO) * c, elem16_to_f((uint16_t)(w2 >> 16), IO) * c);
        };
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            const uint4 v = row_live ? *(const uint4 *)(qrow + ks * 32) : make_uint4(0, 0, 0, 0);
            qf[ks] = make_uint4(scaled(v.x), scaled(v.y), scaled(v.z), scaled(v.w));
        }
    }

    const uint8_t *kbase = A.pool_layer + (size_t)kvh * A.head_stride;
    // ---- pages -------------------------------------------------------------------------------------
    // The block size is a power of two >= 16 (the host dispatches other sizes to the kernel above), so the
    // 8 tokens a wave stages lie in one block, a 16-token run has one page, and a tile's blocks never
    // straddle a multiple of 64.  Table entries come in windows of 64, one per lane, by a vector load (a
    // scalar load would be waited for at every barrier, whose LDS wait counts on the same counter); two
    // windows are held, so an entry is in a register long before its tile is reached.  Everything here is
    // wave-uniform, straight-line code: the only branch is the change of window, every 64 blocks.
    const int sh = A.bs_shift;
    const int tgw = w * ROWS;                                 // the wave's first token within a tile
    const int nblk_needed = (lim_wg + A.bs - 1) >> sh;
    auto load_window = [&](int lb0) -> int {
        const int i = lb0 + lane;
        return i < nblk_needed ? A.table[i] : -1;             // entries past the chunk's last block are never read
    };
    auto pages_of = [&](int win) -> unsigned long long { return __builtin_amdgcn_ballot_w64(win >= 0 && win < A.NB); };
    int win_lb0 = (((t_begin * kPfBN) >> sh) >> 6) << 6;
    int win_a = load_window(win_lb0), win_b = load_window(win_lb0 + 64);
    unsigned long long present_a = pages_of(win_a);           // bit i: block win_lb0 + i has a page
    // the wave's page in `tile` (-1: a hole, or past the end) and the tile's four page flags, one per 16-token run
    auto lookup = [&](int tile, int &blk, int &flags) {
        const int lb0 = (tile * kPfBN) >> sh;
        if (__builtin_expect(lb0 >= win_lb0 + 64, 0)) {       // tiles are asked for in ascending order
            win_lb0 += 64;
            win_a = win_b;
            win_b = load_window(win_lb0 + 64);
            present_a = pages_of(win_a);
        }
        const uint32_t m = (uint32_t)(present_a >> (lb0 - win_lb0));
        flags = (int)((m & 1u) | (((m >> (16 >> sh)) & 1u) << 1) | (((m >> (32 >> sh)) & 1u) << 2) | (((m >> (48 >> sh)) & 1u) << 3));
        const int tg = tile * kPfBN + tgw;
        const int li = (tg >> sh) - win_lb0;
        const int b = __builtin_amdgcn_readlane(win_a, li);
        blk = (((present_a >> li) & 1ull) != 0 && tg < lim_part) ? b : -1;
    };

    pf_f32x16 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.0f;
    // The softmax reference m_ref (per row): the products start from -m_ref (the C operand), so a score
    // arrives as its exponent relative to the reference.  The reference moves only when a tile's maximum
    // exceeds it by more than kLazy (or is the row's first finite one): weights stay below 2^kLazy, and O
    // and the row sum are rescaled on those rare occasions only.  out = O / l does not depend on it.
    constexpr float kLazy = 8.0f;
    float m_ref = 0.0f, l_run = 0.0f;
    bool m_init = false;
    pf_f32x16 negm;
#pragma unroll
    for (int i = 0; i < 16; i++) negm[i] = 0.0f;

    // ---- staging -----------------------------------------------------------------------------------
    // A wave moves 8 rows of K and of V per tile straight from global memory into LDS: two loads of 1 KB per
    // operand, each landing as the wave's 64 lanes x 16 bytes in a row -- four token rows of 256 bytes.  The LDS
    // rows have no padding; instead the 16-byte chunk c of row r sits at position c ^ sK(r) (K: sK = r & 15,
    // whole-row reads by 16 consecutive rows) or c ^ sV(r) (V: sV = (r & 3) << 2, transposed reads of
    // 4 rows x 64 bytes by 32 lanes), which the loading lane applies on the global side: the lane that fills
    // position p of a row fetches chunk p ^ s(row).  Rows past the chunk's end and missing pages are not
    // loaded at all: the buffers start out as zeros and only ever receive real rows, so what such a row holds
    // is finite, and its scores are masked and its weights are exact zeros.
    uint32_t goff_k[2], goff_v[2];                           // byte offset of this lane's chunk within the wave's 8 rows
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int rr = lane >> 4, cp = lane & 15, row = tgw + 4 * j + rr;
        goff_k[j] = (uint32_t)((4 * j + rr) * RB + ((cp ^ (row & 15)) << 4));
        goff_v[j] = (uint32_t)((4 * j + rr) * RB + ((cp ^ ((row & 3) << 2)) << 4));
    }
    // one request: four of the wave's 8 rows (j = which four) from `src`, the wave's first row of the tile in its
    // page, to `lds`; `rows` of the 8 exist
    auto request = [&](const uint8_t *src, uint32_t goff, uint32_t lds, int j, int rows) {
        if (4 * j + (lane >> 4) < rows) pf_load_to_lds16(src, goff, lds);
    };
    // at most n of this wave's loads are still on their way (they land in order)
    auto wait_loads = [&](auto n) {
        constexpr int N = decltype(n)::value;
        __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0f70);
    };

    pf_f32x16 s[2];                 // scores of the tile in flight: [32-token half][16 per lane]
    uint4 pb[2][2];                 // its weights, packed: [token half][k-half], the B operand of PV

    // where this lane finds its operands in a tile (see the staging above for the two swizzles): K row n (and
    // n + 32), chunk 2 ks + g, i.e. byte ((g ^ n & 15) << 4) ^ (ks << 5) of the row -- the xor with ks is made
    // where it is used (an instruction the compiler may not hoist: eight more registers would spill); V rows
    // 4 g + j16 / 4 + R (R a multiple of 8, which the swizzle does not see), 8 bytes at dims 32 dt + 16 (lane / 16 % 2)
    // + 4 (j16 % 4).
    uint32_t voff[NDT];
    const uint32_t kx1 = (uint32_t)(n * RB + ((g ^ (n & 15)) << 4));     // row n, chunk g ^ sK(n): k-step 0
    // the address of k-step ks = that of k-step 0 with ks xor-ed into bits 5-7 (the buffers are 256-byte aligned)
    auto kaddr = [&](uint32_t base, int ks) -> uint32_t {
        uint32_t r;
        asm volatile("v_xor_b32 %0, %2, %1" : "=v"(r) : "v"(base), "s"((uint32_t)(ks << 5)));
        return r;
    };
    {
        const int j16 = lane & 15;
        const int rowl = 4 * g + (j16 >> 2);
        const int clane = 2 * ((lane >> 4) & 1) + ((j16 & 3) >> 1), half = j16 & 1;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
            voff[dt] = (uint32_t)(rowl * RB + ((((dt ^ (rowl & 3)) << 2) | clane) << 4) + (half << 3));
    }

    // S^T = K Q^T.  The operand reads run two k-steps ahead of the products that use them; scheduling
    // barriers pin that order, so that at most six operands are in registers at a time.
    auto qk = [&](int tile) {
        const uint32_t ka0 = pf_lds_addr(&k_lds3[tile & (kRing - 1)][0]) + kx1;
        uint4 a[NKS][2];
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const uint32_t ka = kaddr(ka0, ks);
            a[ks][0] = pf_lds_read128(ka, 0);
            a[ks][1] = pf_lds_read128(ka, 32 * RB);
        }
        // The registers of the last tile's scores stay taken up to here, so that the first operands cannot land in
        // them: the products below then write the new scores where the softmax expects them, instead of somewhere
        // else with sixteen moves (and a wait for the last product) at the end.
        asm volatile("" : : "v"(s[0]), "v"(s[1]));
        pf_sched_barrier();
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            if (ks + 2 < NKS) {
                const uint32_t ka = kaddr(ka0, ks + 2);
                a[ks + 2][0] = pf_lds_read128(ka, 0);
                a[ks + 2][1] = pf_lds_read128(ka, 32 * RB);
            }
            if (ks == 0) {                                   // the products start from minus the row's reference
                s[0] = mfma32<DT>(a[ks][0], qf[ks], negm);
                s[1] = mfma32<DT>(a[ks][1], qf[ks], negm);
                asm volatile("" : : "v"(negm));              // still in use: neither product may take its registers
            } else {
                s[0] = mfma32<DT>(a[ks][0], qf[ks], s[0]);
                s[1] = mfma32<DT>(a[ks][1], qf[ks], s[1]);
            }
            pf_sched_barrier();
        }
    };
    // O^T += V^T P^T: 16 products, two transposed 8-byte reads each, the reads four products ahead
    auto pv = [&](int tile) {
        const uint32_t v_lds = pf_lds_addr(&v_lds3[tile & (kRing - 1)][0]);
        uint32_t va[NDT];
#pragma unroll
        for (int dt = 0; dt < NDT; dt++) va[dt] = v_lds + voff[dt];
        uint2 lo[16], hi[16];
        auto rd = [&](int i) {                               // product i = (tt, mh, dt) = (i / 8, (i / 4) & 1, i & 3)
            const int roff = ((i >> 3) * 32 + 16 * ((i >> 2) & 1)) * RB;
            lo[i] = pf_lds_read_tr16(va[i & 3], roff);
            hi[i] = pf_lds_read_tr16(va[i & 3], roff + 8 * RB);
        };
#pragma unroll
        for (int i = 0; i < 4; i++) rd(i);
        pf_sched_barrier();
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if (i + 4 < 16) rd(i + 4);
            o[i & 3] = mfma32<DT>(make_uint4(lo[i].x, lo[i].y, hi[i].x, hi[i].y), pb[i >> 3][(i >> 2) & 1], o[i & 3]);
            pf_sched_barrier();
        }
    };
    // scores of tile `it` (page flags `flags`) -> packed weights, running maximum and sum, rescale of O^T
    auto softmax = [&](int it, int flags) {
        const int tile_t = it * kPfBN;
        if (__builtin_expect(flags != 15 || it >= first_masked_tile, 0)) {
#pragma unroll
            for (int tt = 0; tt < 2; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int tl = tt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
                    const bool ok = (tile_t + tl) < vis && ((flags >> (tl >> 4)) & 1) != 0;
                    s[tt][i] = ok ? s[tt][i] : -INFINITY;
                }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[tt][i]);
        tmax = pf_max_halves(tmax);                          // a row's scores lie in lanes n and n + 32
        const bool move = m_init ? tmax > kLazy : tmax > -INFINITY;
        if (__builtin_expect(__any(move), 0)) {
            const float delta = move ? tmax : 0.0f;
            m_init = m_init || move;
            m_ref += delta;
            const float alpha = __builtin_amdgcn_exp2f(-delta);
            l_run *= alpha;
#pragma unroll
            for (int tt = 0; tt < 2; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) s[tt][i] -= delta;
#pragma unroll
            for (int i = 0; i < 16; i++) negm[i] = -m_ref;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
        }
        float psum = 0.0f;
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {
            float p[16];
#pragma unroll
            for (int i = 0; i < 16; i++) p[i] = __builtin_amdgcn_exp2f(s[tt][i]);
            pb[tt][0] = make_uint4(pack2<DT>(p[0], p[1]), pack2<DT>(p[2], p[3]), pack2<DT>(p[4], p[5]), pack2<DT>(p[6], p[7]));
            pb[tt][1] = make_uint4(pack2<DT>(p[8], p[9]), pack2<DT>(p[10], p[11]), pack2<DT>(p[12], p[13]), pack2<DT>(p[14], p[15]));
            // the row sum over the weights before rounding: the dot-product instructions that would sum the rounded
            // pairs run on the matrix pipe and stall the products of the wave that shares the SIMD
#pragma unroll
            for (int i = 0; i < 16; i++) psum += p[i];
        }
        l_run += psum;
    };

    // The memory side: in its vector phase a wave requests its share of K(kt) and V(kt - 1) -- kt = t + 3 for the
    // first half of the workgroup (phase 2t), t + 4 for the second (phase 2t + 1).  Four buffers per operand: the
    // buffer of tile x is free once tile x's last reader has passed (K: phase 2x, V: phase 2x + 2) and is
    // requested again for tile x + 4 from phase 2x + 1 (K) and 2x + 3 (V) on.  A request is first read five phases
    // after it was made; a wave makes sure of its own requests of two vector phases ago at the end of every vector
    // phase (wait_loads(8): all but the eight of this phase and the one before), ahead of the barrier.
    const uint32_t k_ring = pf_lds_addr(&k_lds3[0][0]) + (uint32_t)(tgw * RB);   // the wave's rows in buffer 0
    const uint32_t v_ring = pf_lds_addr(&v_lds3[0][0]) + (uint32_t)(tgw * RB);
    const uint8_t *vsrc_prev = kbase;                        // where the V rows of the tile looked up last begin
    int rows_prev = 0;                                       // how many of them exist
    bool four_issued = false, four_before = false;           // the last stage() / the one before issued exactly four loads
    // where the wave's K rows of tile kt begin and how many of the 8 exist; the tile's page flags
    auto find = [&](int kt, int &f_new, const uint8_t *&ksrc, int &rows) {
        int blk;
        lookup(kt, blk, f_new);
        const int tg = kt * kPfBN + tgw;
        rows = blk >= 0 ? lim_part - tg : 0;
        ksrc = kbase + (size_t)max(blk, 0) * A.block_stride + (size_t)((tg & (A.bs - 1)) * RB);
    };
    auto stage = [&](int kt, int &f_new) {
        const uint8_t *ksrc;
        int rows;
        find(kt, f_new, ksrc, rows);
        const uint32_t lk = k_ring + ((uint32_t)(kt & (kRing - 1)) << 14);
        const uint32_t lv = v_ring + ((uint32_t)((kt - 1) & (kRing - 1)) << 14);
        const bool all = min(rows, rows_prev) >= ROWS;
        if (__builtin_expect(all, 1)) {                      // whole pages: no lane is switched off
            pf_load_to_lds16(ksrc, goff_k[0], lk);
            pf_load_to_lds16(ksrc, goff_k[1], lk + 4 * RB);
            pf_load_to_lds16(vsrc_prev, goff_v[0], lv);
            pf_load_to_lds16(vsrc_prev, goff_v[1], lv + 4 * RB);
        } else {
            request(ksrc, goff_k[0], lk, 0, rows);
            request(ksrc, goff_k[1], lk + 4 * RB, 1, rows);
            request(vsrc_prev, goff_v[0], lv, 0, rows_prev);
            request(vsrc_prev, goff_v[1], lv + 4 * RB, 1, rows_prev);
        }
        four_before = four_issued;
        four_issued = all;
        vsrc_prev = ksrc + A.kv_plane;
        rows_prev = rows;
    };
    // everything this wave requested before its last stage() has landed (a stage that issued fewer than four
    // loads -- the chunk's end, a missing page -- waits for everything)
    auto wait_earlier_loads = [&]() {
        if (four_issued && four_before) wait_loads(std::integral_constant<int, 8>{});
        else wait_loads(std::integral_constant<int, 0>{});
    };

    // ---- prologue: the buffers cleared; K(0), K(1), K(2), V(0), V(1) (second half: also K(3), V(2)) in LDS ----
    for (int i = threadIdx.x * 16; i < kRing * kTileBytes; i += 512 * 16) {
        *(uint4 *)(&k_lds3[0][0] + i) = make_uint4(0, 0, 0, 0);
        *(uint4 *)(&v_lds3[0][0] + i) = make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
    int f0, f1, f2, f3 = 15, f4 = 15;                        // page flags of the tiles ahead (see the loops)
    {
        auto both = [&](int kt, int &f_new, bool with_v) {   // K(kt) and, if asked for, V(kt)
            const uint8_t *ksrc;
            int rows;
            find(kt, f_new, ksrc, rows);
            const uint32_t lk = k_ring + ((uint32_t)(kt & (kRing - 1)) << 14), lv = v_ring + ((uint32_t)(kt & (kRing - 1)) << 14);
            request(ksrc, goff_k[0], lk, 0, rows);
            request(ksrc, goff_k[1], lk + 4 * RB, 1, rows);
            vsrc_prev = ksrc + A.kv_plane;
            rows_prev = rows;
            if (with_v) {
                request(vsrc_prev, goff_v[0], lv, 0, rows);
                request(vsrc_prev, goff_v[1], lv + 4 * RB, 1, rows);
            }
        };
        both(t_begin, f0, true);
        both(t_begin + 1, f1, true);
        both(t_begin + 2, f2, false);
        if (!grpA) stage(t_begin + 3, f3);                   // K(3), V(2) of the part
        wait_loads(std::integral_constant<int, 0>{});
        four_issued = four_before = false;
    }
    __syncthreads();
    // Both halves pass the same number of barriers.  The loop bodies are straight-line code (the accumulators are
    // updated in place): the product past the last tile multiplies whatever that K buffer holds and its result is
    // never read; requests past the last tile load nothing (no page).
    if (grpA) {
        // f0, f1, f2 = flags of tiles t, t + 1, t + 2 at the head of iteration t; stage(t + 3) adds tile t + 3's
        qk(t_begin);
#pragma unroll 1
        for (int t = t_begin; t < ntiles; t++) {
            stage(t + 3, f3);                                // phase 2t: K(t+3), V(t+2)
            softmax(t, f0);
            f0 = f1;
            f1 = f2;
            f2 = f3;
            wait_earlier_loads();
            pf_barrier_lds();
            pv(t);                                           // phase 2t+1
            qk(t + 1);
            pf_barrier_lds();
        }
        pf_barrier_lds();
    } else {
        // f0 .. f3 = flags of tiles t .. t + 3 at the head of iteration t; stage(t + 4) adds tile t + 4's
        qk(t_begin);                                         // phase 0
        pf_barrier_lds();
#pragma unroll 1
        for (int t = t_begin; t < ntiles; t++) {
            softmax(t, f0);                                  // phase 2t+1
            stage(t + 4, f4);                                // K(t+4), V(t+3)
            f0 = f1;
            f1 = f2;
            f2 = f3;
            f3 = f4;
            wait_earlier_loads();
            pf_barrier_lds();
            pv(t);                                           // phase 2t+2
            qk(t + 1);
            pf_barrier_lds();
        }
    }

    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (kp > 1) {                                            // a piece: the sums as they are, relative to m_ref (log2 units)
        if (row_live) {
            const size_t slot = ((size_t)tq * A.QH + head) * kp + part;
            if (g == 0) {
                A.part_m[slot] = m_ref;
                A.part_l[slot] = l_tot;
            }
            float *po = A.part_o + slot * D;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int b4 = 0; b4 < 4; b4++)
                    *(float4 *)(po + dt * 32 + 8 * b4 + 4 * g) = make_float4(o[dt][4 * b4], o[dt][4 * b4 + 1], o[dt][4 * b4 + 2], o[dt][4 * b4 + 3]);
        }
        return;
    }
    if (A.lse_rows && row_live && g == 0)      // m_ref is the reference the weights were taken against, in log2 units
        A.lse_rows[(size_t)tq * A.QH + head] = l_tot > 0.0f ? m_ref + __builtin_log2f(l_tot) : INFINITY;
    if (row_live && (l_tot > 0.0f || A.gate)) {
        const bool have = l_tot > 0.0f;
        const float inv = have ? 1.0f / l_tot : 0.0f;
        uint8_t *orow = A.out + ((size_t)tq * A.QH + head) * (D * 2);
        const uint16_t *grow = A.gate ? A.gate + ((size_t)tq * A.QH + head) * A.gate_stride : nullptr;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int b4 = 0; b4 < 4; b4++) {
                const int d0 = dt * 32 + 8 * b4 + 4 * g;
                uint2 v = have ? make_uint2(pack2<IO>(o[dt][4 * b4] * inv, o[dt][4 * b4 + 1] * inv),
                                            pack2<IO>(o[dt][4 * b4 + 2] * inv, o[dt][4 * b4 + 3] * inv))
                               : *(const uint2 *)(orow + d0 * 2);
                if (grow) {
                    const uint2 gv = *(const uint2 *)(grow + d0);
                    v.x = (uint32_t)gated_elem16((uint16_t)(v.x & 0xffffu), (uint16_t)(gv.x & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.x >> 16), (uint16_t)(gv.x >> 16), IO) << 16);
                    v.y = (uint32_t)gated_elem16((uint16_t)(v.y & 0xffffu), (uint16_t)(gv.y & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.y >> 16), (uint16_t)(gv.y >> 16), IO) << 16);
                }
                *(uint2 *)(orow + d0 * 2) = v;
            }
    }
}

// ---- head_dim 256, 16-bit pages: one wave per SIMD, tiles straight into LDS -------------------------
// 128 rows per workgroup as in prefill_mfma_kernel (a wave's 32 rows x 256 dims of output are 128 accumulator
// registers, so a SIMD holds one wave), but the tiles go from global memory straight into LDS as in
// prefill_ppd_kernel: no registers hold tile data (the register kind keeps 64 of them and, short of registers,
// moves them and the Q operands between the two register files all the time), rows are swizzled instead of padded,
// and with nothing else to overlap a wave's LDS latency and vector work with, the order of its instructions is
// written out: the exponentials of tile t go between the k-steps of tile t + 1's scores, two per k-step, operand reads
// run two k-steps / four products ahead, scheduling barriers pin it.  Per tile and wave 64 products (2 048 clocks).
// Requests run one tile ahead, two buffers per operand, one barrier per tile: step t first takes the maximum of tile
// t's scores (registers only), then waits for its requests of the step before and meets the other waves, then
// requests K(t + 2) and V(t + 1) -- into the buffers of K(t) and V(t - 1) -- one request per k-step of QK(t + 1)
// (between the transposed reads of PV a request holds the wave up for over a hundred clocks).
template <int DT, int IO = DT>
__global__ __launch_bounds__(256, 1) void prefill_d256_kernel(PrefillArgs A)
{
    constexpr int D = 256, RB = D * 2;                       // bytes of a token row of one kv head, also the LDS row
    constexpr int kTileBytes = kPfBN * RB;                   // 32 KB per operand and tile
    constexpr int NKS = D / 16, NDT = D / 32;
    constexpr int ROWS = 16;                                 // tokens of a tile one wave requests
    constexpr int XQ = 3, XP = 6;                            // operand reads ahead of their products: k-steps (QK), products (PV)
    __shared__ __align__(512) uint8_t k_ldsd[2][kTileBytes]; // 512: the xor swizzle is applied to whole addresses
    __shared__ __align__(512) uint8_t v_ldsd[2][kTileBytes];
    __shared__ int valid_ldsd[4][4];                         // [tile & 3][wave]: the wave's 16-token run of the tile has a page

    // walk = (row block of tokens, kv head, group of gh query heads), the longest walks first; workgroups past
    // n_full take one piece of a walk each
    int walk = (int)blockIdx.x, part = 0, nparts = 1;
    if (walk >= A.n_full) {
        const int p = walk - A.n_full;
        walk = A.n_full + p / A.kparts;
        part = p - (p / A.kparts) * A.kparts;
        nparts = A.kparts;
    }
    const int G = A.QH / A.KVH, GH = A.gh, TPW = A.tpw, NHG = G / GH;
    const int kvh = walk % A.KVH;
    const int hg = (walk / A.KVH) % NHG;
    const int qt = A.nqt - 1 - walk / (A.KVH * NHG);
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int n = lane & 31, g = lane >> 5;

    const int r = w * 32 + n, rt = r / GH;
    const int tq = qt * TPW + rt;
    const int head = kvh * G + hg * GH + (r - rt * GH);
    const bool row_live = rt < TPW && tq < A.M;
    const int vis = A.pos_start + tq + 1;
    const int lim_walk = A.pos_start + min((qt + 1) * TPW, A.M);
    const int first_masked_tile = (A.pos_start + qt * TPW + 1) / kPfBN;
    const int nt_walk = (lim_walk + kPfBN - 1) / kPfBN;
    // a piece is a range of tiles that begins at an even tile (the two score register sets and the LDS buffers
    // take turns by the tile's parity); the last piece ends where the walk ends
    // (the same value in every lane; the divisions run on the vector unit, and the LDS addresses derived from the
    // tile number must be scalars)
    const int t0 = __builtin_amdgcn_readfirstlane(part == 0 ? 0 : ((part * nt_walk / nparts) & ~1));
    const int ntiles = __builtin_amdgcn_readfirstlane(part == nparts - 1 ? nt_walk : (((part + 1) * nt_walk / nparts) & ~1));
    const int lim_wg = min(lim_walk, ntiles * kPfBN);        // nothing past the piece's end is requested
    const size_t prow = nparts > 1 ? ((size_t)(walk - A.n_full) * 128 + r) * nparts + part : 0;   // the row's slot among the pieces
    if (t0 >= ntiles) {                                      // an empty piece (a walk of fewer tiles than pieces)
        if (row_live && g == 0) A.part_l[prow] = 0.0f;
        return;
    }

    // Q as the B operand, multiplied by scale * log2(e) on the way in (rounded once more to the 16-bit
    // type): the products then are the exponents themselves and the softmax needs no multiply per score.
    uint4 qf[NKS];
    {
        const uint8_t *qrow = A.q + ((size_t)tq * A.QH + head) * (D * 2) + g * 16;
        const float c = A.scale_log2e;
        auto scaled = [&](uint32_t w2) -> uint32_t {
            return pack2<DT>(elem16_to_f((uint16_t)(w2 & 0xffffu), IO) * c, elem16_to_f((uint16_t)(w2 >> 16), IO) * c);
        };
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            const uint4 v = row_live ? *(const uint4 *)(qrow + ks * 32) : make_uint4(0, 0, 0, 0);
            qf[ks] = make_uint4(scaled(v.x), scaled(v.y), scaled(v.z), scaled(v.w));
        }
    }

    const uint8_t *kbase = A.pool_layer + (size_t)kvh * A.head_stride;
    const int sh = A.bs_shift;                               // blocks of 16 * 2^k tokens: a wave's 16 rows lie in one block
    const int tgw = w * ROWS;                                // the wave's first token within a tile

    // ---- requests ------------------------------------------------------------------------------------
    // One request is 2 token rows (1 KB): lanes 0-31 the first, 32-63 the second; a wave has 8 per operand and tile.
    // The 16-byte chunk c of row r sits at position c ^ (r & 15) (K, xor on the low four bits: whole-row reads by 16
    // consecutive rows) or c ^ ((r & 3) << 2) (V: transposed reads of 4 rows x 64 bytes), which the requesting lane
    // applies on the global side.  Rows past the chunk's end and missing pages are not requested: the buffers
    // start out as zeros and only ever receive real rows.
    uint32_t goff_k[8], goff_v[2];
    {
        const int rr = lane >> 5, cp = lane & 31;
#pragma unroll
        for (int j = 0; j < 8; j++) goff_k[j] = (uint32_t)(rr * RB + ((cp ^ ((2 * j + rr) & 15)) << 4));
#pragma unroll
        for (int j = 0; j < 2; j++) goff_v[j] = (uint32_t)(rr * RB + ((cp ^ (((2 * j + rr) & 3) << 2)) << 4));
    }
    auto wait_loads = [&]() { __builtin_amdgcn_s_waitcnt(0x0f70); };         // vmcnt(0): every request has landed
    // the wave's page in `tile`, or -1.  Read through the scalar cache (the table is not written while the kernel
    // runs): a vector load would be waited for together with the requests, which the kernel counts itself.  The
    // step makes sure the entry is there before its products begin -- scalar loads return out of order, and with
    // one outstanding the compiler could not count the LDS reads it waits for.
    typedef const int32_t __attribute__((address_space(4))) *const_table_t;
    const const_table_t table_k = (const_table_t)(uintptr_t)A.table;
    auto page_of = [&](int tile) -> int {
        const int tg = tile * kPfBN + tgw;
        return tg < lim_wg ? table_k[tg >> sh] : -1;
    };
    const uint8_t *vsrc_prev = kbase;                        // where the V rows of the tile requested last begin
    int rows_prev = 0;                                       // how many of them exist
    const uint32_t k_ring = pf_lds_addr(&k_ldsd[0][0]) + (uint32_t)(tgw * RB);
    const uint32_t v_ring = pf_lds_addr(&v_ldsd[0][0]) + (uint32_t)(tgw * RB);
    // A tile's requests in two steps.  plan(kt, page): where K(kt) comes from and where it and V(kt - 1) go (scalar
    // work).  dma_k(j) / dma_v(j): request j of 8.  A wave's next memory instruction waits until the one before has
    // passed the address unit (some 130 clocks for these), so the 16 requests of a tile are spread over the tile's
    // products, one every four, instead of being issued in a row.
    const uint8_t *p_ksrc = kbase, *p_vsrc = kbase;
    int p_rows = 0, p_vrows = 0;
    uint32_t p_lk = 0, p_lv = 0;
    auto plan = [&](int kt, int blk_raw) {
        const int blk0 = __builtin_amdgcn_readfirstlane(blk_raw);
        const int tg = kt * kPfBN + tgw;
        const bool ok = blk0 >= 0 && blk0 < A.NB && tg < lim_wg;
        p_vsrc = vsrc_prev;
        p_vrows = rows_prev;
        p_rows = ok ? lim_wg - tg : 0;
        p_ksrc = kbase + (size_t)(ok ? blk0 : 0) * A.block_stride + (size_t)((tg & (A.bs - 1)) * RB);
        p_lk = k_ring + ((uint32_t)(kt & 1) << 15);
        p_lv = v_ring + ((uint32_t)((kt - 1) & 1) << 15);
        if (lane == 0) valid_ldsd[kt & 3][w] = ok ? 1 : 0;
        vsrc_prev = p_ksrc + A.kv_plane;
        rows_prev = p_rows;
    };
    auto dma_k = [&](int j) {
        if (__builtin_expect(p_rows >= ROWS, 1)) pf_load_to_lds16(p_ksrc + 1024 * j, goff_k[j], p_lk + 1024 * j);
        else if (2 * j + (lane >> 5) < p_rows) pf_load_to_lds16(p_ksrc + 1024 * j, goff_k[j], p_lk + 1024 * j);
    };
    auto dma_v = [&](int j) {
        if (__builtin_expect(p_vrows >= ROWS, 1)) pf_load_to_lds16(p_vsrc + 1024 * j, goff_v[j & 1], p_lv + 1024 * j);
        else if (2 * j + (lane >> 5) < p_vrows) pf_load_to_lds16(p_vsrc + 1024 * j, goff_v[j & 1], p_lv + 1024 * j);
    };

    pf_f32x16 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.0f;
    // the lazy softmax reference of prefill_pp_kernel: the products start from -m_ref (the C operand)
    pf_f32x16 negm;
#pragma unroll
    for (int i = 0; i < 16; i++) negm[i] = 0.0f;
    float m_ref = 0.0f, l_run = 0.0f;
    bool m_init = false;
    constexpr float kLazy = 8.0f;

    // where this lane finds its operands: K row n (and n + 32), chunk 2 ks + g at byte ((g ^ n & 15) << 4) ^ (ks << 5)
    // of the row; V rows 4 g + j16 / 4 (+ multiples of 8), 8 bytes at dims 32 dt + 16 (lane / 16 % 2) + 4 (j16 % 4)
    const uint32_t kx1 = (uint32_t)(n * RB + ((g ^ (n & 15)) << 4));
    uint32_t vx1;
    {
        const int j16 = lane & 15;
        const int rowl = 4 * g + (j16 >> 2);
        const int clane = 2 * ((lane >> 4) & 1) + ((j16 & 3) >> 1), half = j16 & 1;
        vx1 = (uint32_t)(rowl * RB + (((rowl & 3) << 6) | (clane << 4)) + (half << 3));
    }

    // S^T = K Q^T for the tile in buffer `slot`; between(ks): the caller's vector work for that k-step
    auto qk = [&](int slot, pf_f32x16 (&s)[2], auto &&between) {
        const uint32_t ka0 = pf_lds_addr(&k_ldsd[0][0]) + ((uint32_t)slot << 15) + kx1;
        uint4 a[NKS][2];
#pragma unroll
        for (int ks = 0; ks < XQ; ks++) {
            a[ks][0] = pf_lds_read128(ka0 ^ (uint32_t)(ks << 5), 0);
            a[ks][1] = pf_lds_read128(ka0 ^ (uint32_t)(ks << 5), 32 * RB);
        }
        pf_sched_barrier();
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            if (ks + XQ < NKS) {
                a[ks + XQ][0] = pf_lds_read128(ka0 ^ (uint32_t)((ks + XQ) << 5), 0);
                a[ks + XQ][1] = pf_lds_read128(ka0 ^ (uint32_t)((ks + XQ) << 5), 32 * RB);
            }
            between(ks);
            if (ks == 0) {
                s[0] = mfma32<DT>(a[ks][0], qf[ks], negm);
                s[1] = mfma32<DT>(a[ks][1], qf[ks], negm);
            } else {
                s[0] = mfma32<DT>(a[ks][0], qf[ks], s[0]);
                s[1] = mfma32<DT>(a[ks][1], qf[ks], s[1]);
            }
            pf_sched_barrier();
        }
    };
    // O^T += V^T P^T over the tile in buffer `slot`: 32 products, two transposed 8-byte reads each, four products ahead
    auto pv = [&](int slot, const uint4 (&pb)[2][2], auto &&between) {
        const uint32_t vb = pf_lds_addr(&v_ldsd[0][0]) + ((uint32_t)slot << 15) + vx1;
        constexpr int NP = 4 * NDT;
        uint2 lo[NP], hi[NP];
        auto rd = [&](int i) {                               // product i = (tt, mh, dt) = (i / 16, (i / 8) & 1, i % 8)
            const int roff = ((i / (2 * NDT)) * 32 + 16 * ((i / NDT) & 1)) * RB;
            const uint32_t va = vb ^ (uint32_t)((i % NDT) << 6);
            lo[i] = pf_lds_read_tr16(va, roff);
            hi[i] = pf_lds_read_tr16(va, roff + 8 * RB);
        };
#pragma unroll
        for (int i = 0; i < XP; i++) rd(i);
        pf_sched_barrier();
#pragma unroll
        for (int i = 0; i < NP; i++) {
            if (i + XP < NP) rd(i + XP);
            between(i);
            o[i % NDT] = mfma32<DT>(make_uint4(lo[i].x, lo[i].y, hi[i].x, hi[i].y), pb[i / (2 * NDT)][(i / NDT) & 1], o[i % NDT]);
            pf_sched_barrier();
        }
    };

    // ---- prologue: the buffers cleared; K(0), V(0), K(1) in LDS; the scores of tile 0 ----
    for (int i = threadIdx.x * 16; i < 2 * kTileBytes; i += 256 * 16) {
        *(uint4 *)(&k_ldsd[0][0] + i) = make_uint4(0, 0, 0, 0);
        *(uint4 *)(&v_ldsd[0][0] + i) = make_uint4(0, 0, 0, 0);
    }
    int blk_ahead;                                           // the wave's page two tiles ahead of the step
    {
        const int b0 = page_of(t0), b1 = page_of(t0 + 1);
        blk_ahead = page_of(t0 + 2);
        __syncthreads();                                     // the clearing is done (and the table entries are here)
        plan(t0, b0);
#pragma unroll
        for (int j = 0; j < 8; j++) dma_k(j);
        plan(t0 + 1, b1);                                    // K(t0 + 1), V(t0)
#pragma unroll
        for (int j = 0; j < 8; j++) { dma_k(j); dma_v(j); }
        wait_loads();
    }
    __syncthreads();
    pf_f32x16 s_even[2], s_odd[2];
    qk(0, s_even, [](int) {});

    auto tile_step = [&](int it, pf_f32x16 (&s)[2], pf_f32x16 (&s_next)[2]) {
        // here: s = scores of tile it; every wave's requests of the step before are on their way or there
        plan(it + 2, blk_ahead);                             // K(it + 2), V(it + 1): requested between the products below
        blk_ahead = page_of(it + 3);
        const int tile_t = it * kPfBN;
        const int *vl = &valid_ldsd[it & 3][0];
        const int flags = vl[0] | (vl[1] << 1) | (vl[2] << 2) | (vl[3] << 3);
        if (__builtin_expect(flags != 15 || it >= first_masked_tile, 0)) {
#pragma unroll
            for (int tt = 0; tt < 2; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int tl = tt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
                    const bool ok = (tile_t + tl) < vis && ((flags >> (tl >> 4)) & 1) != 0;
                    s[tt][i] = ok ? s[tt][i] : -INFINITY;
                }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
            for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[tt][i]);
        tmax = pf_max_halves(tmax);                          // a row's scores lie in lanes n and n + 32
        const bool move = m_init ? tmax > kLazy : tmax > -INFINITY;
        if (__builtin_expect(__any(move), 0)) {
            const float delta = move ? tmax : 0.0f;
            m_init = m_init || move;
            m_ref += delta;
            const float alpha = __builtin_amdgcn_exp2f(-delta);
            l_run *= alpha;
#pragma unroll
            for (int tt = 0; tt < 2; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) s[tt][i] -= delta;
#pragma unroll
            for (int i = 0; i < 16; i++) negm[i] = -m_ref;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
        }
        // the exponentials of this tile between the k-steps of the next tile's scores, two per k-step, packed as
        // soon as eight are there; the row sum over the weights before rounding (see prefill_ppd_kernel).  The
        // products are unconditional: past the last tile they multiply whatever that buffer holds, never read.
        float psum = 0.0f, p8[8];
        uint4 pb[2][2];
        // K(it + 1) and V(it) have landed, and every wave is done with K(it) and V(it - 1), whose buffers the
        // requests below write
        wait_loads();
        pf_barrier_lds();
        asm volatile("" : : "s"(blk_ahead));                 // the table entry read at the head of the step is here
        qk((it + 1) & 1, s_next, [&](int ks) {               // all 16 requests between the k-steps: there they cost nothing
            if ((ks & 1) == 0) dma_k(ks >> 1);
            else dma_v(ks >> 1);
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int j = ks * 2 + u, tt = j >> 4, i = j & 15;
                const float e = __builtin_amdgcn_exp2f(s[tt][i]);
                p8[j & 7] = e;
                psum += e;
                if ((j & 7) == 7)
                    pb[tt][(i >> 3) & 1] = make_uint4(pack2<DT>(p8[0], p8[1]), pack2<DT>(p8[2], p8[3]), pack2<DT>(p8[4], p8[5]), pack2<DT>(p8[6], p8[7]));
            }
        });
        l_run += psum;
        pv(it & 1, pb, [](int) {});
    };
    for (int it = t0; it < ntiles; it += 2) {                // two tiles per trip, the score registers swapping roles
        tile_step(it, s_even, s_odd);
        if (it + 1 < ntiles) tile_step(it + 1, s_odd, s_even);
    }

    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (nparts > 1) {
        // a piece of a walk: the unnormalised sums (register i of tile dt is d = dt*32 + 8*(i/4) + 4*g + i%4)
        if (row_live) {
            float *orow = A.part_o + prow * D;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int b4 = 0; b4 < 4; b4++)
                    *(float4 *)(orow + dt * 32 + 8 * b4 + 4 * g) =
                        make_float4(o[dt][4 * b4], o[dt][4 * b4 + 1], o[dt][4 * b4 + 2], o[dt][4 * b4 + 3]);
            if (g == 0) {
                A.part_m[prow] = m_ref;
                A.part_l[prow] = l_tot;
            }
        }
        return;
    }
    if (A.lse_rows && row_live && g == 0)      // m_ref is the reference the weights were taken against, in log2 units
        A.lse_rows[(size_t)tq * A.QH + head] = l_tot > 0.0f ? m_ref + __builtin_log2f(l_tot) : INFINITY;
    if (row_live && (l_tot > 0.0f || A.gate)) {
        const bool have = l_tot > 0.0f;
        const float inv = have ? 1.0f / l_tot : 0.0f;
        uint8_t *orow = A.out + ((size_t)tq * A.QH + head) * (D * 2);
        const uint16_t *grow = A.gate ? A.gate + ((size_t)tq * A.QH + head) * A.gate_stride : nullptr;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int b4 = 0; b4 < 4; b4++) {
                const int d0 = dt * 32 + 8 * b4 + 4 * g;
                uint2 v = have ? make_uint2(pack2<IO>(o[dt][4 * b4] * inv, o[dt][4 * b4 + 1] * inv),
                                            pack2<IO>(o[dt][4 * b4 + 2] * inv, o[dt][4 * b4 + 3] * inv))
                               : *(const uint2 *)(orow + d0 * 2);
                if (grow) {
                    const uint2 gv = *(const uint2 *)(grow + d0);
                    v.x = (uint32_t)gated_elem16((uint16_t)(v.x & 0xffffu), (uint16_t)(gv.x & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.x >> 16), (uint16_t)(gv.x >> 16), IO) << 16);
                    v.y = (uint32_t)gated_elem16((uint16_t)(v.y & 0xffffu), (uint16_t)(gv.y & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.y >> 16), (uint16_t)(gv.y >> 16), IO) << 16);
                }
                *(uint2 *)(orow + d0 * 2) = v;
            }
    }
}

// ---- head_dim 256, 16-bit pages: two kinds of waves, two per SIMD ------------------------------------
// prefill_d256_kernel holds one wave per SIMD because a wave's 32 rows x 256 dims of output are 128 accumulator
// registers, beside its 64 of Q and 64 of scores: nothing overlaps that wave's LDS latency, its softmax and the issue
// time of its requests.  Here the two products of a row group belong to two waves of the same SIMD:
//   wave w (0-3), the SCORE wave of row group w: Q in registers, S^T = K Q^T for tile t + 1 with the exponentials of
//     tile t between the k-steps, mask, lazy maximum, row sums; it hands the tile's weights P (16 registers per lane,
//     already in the layout of the second product's B operand) and, when the reference moved, the rows' factors to
//     its partner through LDS;
//   wave w + 4, the VALUE wave of row group w: the 128 accumulators, O^T += V^T P^T.
// Neither holds more than 256 registers, so both fit a SIMD, and each one's stalls are the other's issue slots.
// The score waves request K (their 16-token run of every tile, two tiles ahead), the value waves V (one tile ahead).
// Two barriers per tile, A and B, passed by all eight waves:
//   score wave, step t:  mask / maximum of tile t;  wait for its K requests;  A_t;  scores of tile t + 1 with the
//                        exponentials of tile t and the requests for K(t + 2) between the k-steps;  write P(t);  B_t.
//   value wave, step t:  (B_t passed: P(t) and V(t) are in LDS)  read P(t);  the first products of PV(t);  A_{t+1};
//                        the other products with the requests for V(t + 1) between them;  wait for those;  B_{t+1}.
// P has one buffer: the value wave reads P(t) ahead of A_{t+1}, the score wave writes P(t + 1) behind it.  K(t + 2)
// is requested behind A_t into the buffer of K(t), which the scores of tile t read ahead of B_{t-1}; V(t + 1) behind
// B_t into the buffer of V(t - 1), which PV(t - 1) read ahead of B_t.  Same walks, pieces, gate and row log-sum-exp
// as prefill_d256_kernel, and the same arithmetic in the same order: the two give the same bits.
// What it gains is overlap, not fewer clocks of work: a tile takes 3 900 clocks against 5 100, with the matrix pipe
// busy 57 % of them; the part then runs at 1.8 GHz instead of 2.4.  Variants that take fewer clocks per tile (all
// requests from the score waves, K from the value waves and V from the score waves, requests earlier in the step)
// ran at lower clocks still and took as long or longer; without the tile requests (wrong results, a probe) the same
// schedule takes two thirds of the time.
template <int DT, int IO = DT>
__global__ __launch_bounds__(512, 1) void prefill_d256w_kernel(PrefillArgs A)
{
    constexpr int D = 256, RB = D * 2;
    constexpr int kTileBytes = kPfBN * RB;                   // 32 KB per operand and tile
    constexpr int NKS = D / 16, NDT = D / 32;
    constexpr int ROWS = 16;
    constexpr int XQ = 3, XP = 6;
    constexpr int kFirst = 4;                                // products of PV(t) ahead of barrier A
    __shared__ __align__(512) uint8_t k_ldsw[2][kTileBytes];
    __shared__ __align__(512) uint8_t v_ldsw[2][kTileBytes];
    __shared__ __align__(16) uint4 p_ldsw[4][4][64];         // [row group][register quad][lane]: the tile's weights
    __shared__ float alpha_ldsw[4][64], l_ldsw[4][64];
    __shared__ int moved_ldsw[4];
    __shared__ int valid_ldsw[4][4];                         // [tile & 3][run]: the 16-token run of the tile has a page

    int walk = (int)blockIdx.x, part = 0, nparts = 1;
    if (walk >= A.n_full) {
        const int p = walk - A.n_full;
        walk = A.n_full + p / A.kparts;
        part = p - (p / A.kparts) * A.kparts;
        nparts = A.kparts;
    }
    const int G = A.QH / A.KVH, GH = A.gh, TPW = A.tpw, NHG = G / GH;
    const int kvh = walk % A.KVH;
    const int hg = (walk / A.KVH) % NHG;
    const int qt = A.nqt - 1 - walk / (A.KVH * NHG);
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const bool value_wave = wave >= 4;
    const int w = wave & 3;                                  // row group, and the 16-token run this wave requests
    const int lane = threadIdx.x & 63;
    const int n = lane & 31, g = lane >> 5;

    const int r = w * 32 + n, rt = r / GH;
    const int tq = qt * TPW + rt;
    const int head = kvh * G + hg * GH + (r - rt * GH);
    const bool row_live = rt < TPW && tq < A.M;
    const int vis = A.pos_start + tq + 1;
    const int lim_walk = A.pos_start + min((qt + 1) * TPW, A.M);
    const int first_masked_tile = (A.pos_start + qt * TPW + 1) / kPfBN;
    const int nt_walk = (lim_walk + kPfBN - 1) / kPfBN;
    const int t0 = __builtin_amdgcn_readfirstlane(part == 0 ? 0 : ((part * nt_walk / nparts) & ~1));
    const int ntiles = __builtin_amdgcn_readfirstlane(part == nparts - 1 ? nt_walk : (((part + 1) * nt_walk / nparts) & ~1));
    const int lim_wg = min(lim_walk, ntiles * kPfBN);
    const size_t prow = nparts > 1 ? ((size_t)(walk - A.n_full) * 128 + r) * nparts + part : 0;
    if (t0 >= ntiles) {
        if (!value_wave && row_live && g == 0) A.part_l[prow] = 0.0f;
        return;
    }

    const uint8_t *kbase = A.pool_layer + (size_t)kvh * A.head_stride;
    const int sh = A.bs_shift;
    const int tgw = w * ROWS;
    auto wait_loads = [&]() { __builtin_amdgcn_s_waitcnt(0x0f70); };         // vmcnt(0)
    typedef const int32_t __attribute__((address_space(4))) *const_table_t;
    const const_table_t table_k = (const_table_t)(uintptr_t)A.table;
    auto page_of = [&](int tile) -> int {
        const int tg = tile * kPfBN + tgw;
        return tg < lim_wg ? table_k[tg >> sh] : -1;
    };
    // where the wave's run of tile kt comes from, how many of its rows exist
    const uint8_t *p_src = kbase;
    int p_rows = 0;
    uint32_t p_lds = 0;
    const uint32_t k_ring = pf_lds_addr(&k_ldsw[0][0]) + (uint32_t)(tgw * RB);
    const uint32_t v_ring = pf_lds_addr(&v_ldsw[0][0]) + (uint32_t)(tgw * RB);
    auto plan = [&](int kt, int blk_raw) {
        const int blk0 = __builtin_amdgcn_readfirstlane(blk_raw);
        const int tg = kt * kPfBN + tgw;
        const bool ok = blk0 >= 0 && blk0 < A.NB && tg < lim_wg;
        p_rows = ok ? lim_wg - tg : 0;
        p_src = kbase + (size_t)(ok ? blk0 : 0) * A.block_stride + (size_t)((tg & (A.bs - 1)) * RB) + (value_wave ? A.kv_plane : 0);
        p_lds = (value_wave ? v_ring : k_ring) + ((uint32_t)(kt & 1) << 15);
        if (!value_wave && lane == 0) valid_ldsw[kt & 3][w] = ok ? 1 : 0;
    };
    // request j of 8: two token rows (1 KB); K chunk c of row r at c ^ (r & 15), V at c ^ ((r & 3) << 2)
    uint32_t goff[8];
    {
        const int rr = lane >> 5, cp = lane & 31;
#pragma unroll
        for (int j = 0; j < 8; j++)
            goff[j] = value_wave ? (uint32_t)(rr * RB + ((cp ^ (((2 * j + rr) & 3) << 2)) << 4))
                                 : (uint32_t)(rr * RB + ((cp ^ ((2 * j + rr) & 15)) << 4));
    }
    auto dma = [&](int j) {
        if (__builtin_expect(p_rows >= ROWS, 1)) pf_load_to_lds16(p_src + 1024 * j, goff[j], p_lds + 1024 * j);
        else if (2 * j + (lane >> 5) < p_rows) pf_load_to_lds16(p_src + 1024 * j, goff[j], p_lds + 1024 * j);
    };

    // ---- prologue: the buffers cleared; K(t0), K(t0 + 1), V(t0) in LDS ----
    for (int i = threadIdx.x * 16; i < 2 * kTileBytes; i += 512 * 16) {
        *(uint4 *)(&k_ldsw[0][0] + i) = make_uint4(0, 0, 0, 0);
        *(uint4 *)(&v_ldsw[0][0] + i) = make_uint4(0, 0, 0, 0);
    }
    int blk_ahead;
    {
        const int b0 = page_of(t0), b1 = page_of(t0 + 1);
        blk_ahead = value_wave ? b1 : page_of(t0 + 2);       // the next page this wave will ask for
        __syncthreads();
        plan(t0, b0);
#pragma unroll
        for (int j = 0; j < 8; j++) dma(j);
        if (!value_wave) {
            plan(t0 + 1, b1);
#pragma unroll
            for (int j = 0; j < 8; j++) dma(j);
        }
        wait_loads();
    }
    __syncthreads();

    const float kLazy = 8.0f;
    if (!value_wave) {
        // ================================ score wave ================================
        uint4 qf[NKS];
        {
            const uint8_t *qrow = A.q + ((size_t)tq * A.QH + head) * (D * 2) + g * 16;
            const float c = A.scale_log2e;
            auto scaled = [&](uint32_t w2) -> uint32_t {
                return pack2<DT>(elem16_to_f((uint16_t)(w2 & 0xffffu), IO) * c, elem16_to_f((uint16_t)(w2 >> 16), IO) * c);
            };
#pragma unroll
            for (int ks = 0; ks < NKS; ks++) {
                const uint4 v = row_live ? *(const uint4 *)(qrow + ks * 32) : make_uint4(0, 0, 0, 0);
                qf[ks] = make_uint4(scaled(v.x), scaled(v.y), scaled(v.z), scaled(v.w));
            }
        }
        pf_f32x16 negm;
#pragma unroll
        for (int i = 0; i < 16; i++) negm[i] = 0.0f;
        float m_ref = 0.0f, l_run = 0.0f;
        bool m_init = false;
        const uint32_t kx1 = (uint32_t)(n * RB + ((g ^ (n & 15)) << 4));
        auto qk = [&](int slot, pf_f32x16 (&s)[2], auto &&between) {
            const uint32_t ka0 = pf_lds_addr(&k_ldsw[0][0]) + ((uint32_t)slot << 15) + kx1;
            uint4 a[NKS][2];
#pragma unroll
            for (int ks = 0; ks < XQ; ks++) {
                a[ks][0] = pf_lds_read128(ka0 ^ (uint32_t)(ks << 5), 0);
                a[ks][1] = pf_lds_read128(ka0 ^ (uint32_t)(ks << 5), 32 * RB);
            }
            pf_sched_barrier();
#pragma unroll
            for (int ks = 0; ks < NKS; ks++) {
                if (ks + XQ < NKS) {
                    a[ks + XQ][0] = pf_lds_read128(ka0 ^ (uint32_t)((ks + XQ) << 5), 0);
                    a[ks + XQ][1] = pf_lds_read128(ka0 ^ (uint32_t)((ks + XQ) << 5), 32 * RB);
                }
                between(ks);
                if (ks == 0) {
                    s[0] = mfma32<DT>(a[ks][0], qf[ks], negm);
                    s[1] = mfma32<DT>(a[ks][1], qf[ks], negm);
                } else {
                    s[0] = mfma32<DT>(a[ks][0], qf[ks], s[0]);
                    s[1] = mfma32<DT>(a[ks][1], qf[ks], s[1]);
                }
                pf_sched_barrier();
            }
        };
        pf_f32x16 s_even[2], s_odd[2];
        qk(t0 & 1, s_even, [](int) {});
        // bit r: run r of the tile has a page; read one tile ahead, between the products
        auto flags_of = [&](const int4 &v) -> int {
            return __builtin_amdgcn_readfirstlane(v.x | (v.y << 1) | (v.z << 2) | (v.w << 3));
        };
        int flags = flags_of(*(const int4 *)&valid_ldsw[t0 & 3][0]);

        auto step = [&](int it, pf_f32x16 (&s)[2], pf_f32x16 (&s_next)[2]) {
            plan(it + 2, blk_ahead);                             // K(it + 2): requested between the products below
            blk_ahead = page_of(it + 3);
            const int tile_t = it * kPfBN;
            if (__builtin_expect(flags != 15 || it >= first_masked_tile, 0)) {
#pragma unroll
                for (int tt = 0; tt < 2; tt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int tl = tt * 32 + 8 * (i >> 2) + 4 * g + (i & 3);
                        const bool ok = (tile_t + tl) < vis && ((flags >> (tl >> 4)) & 1) != 0;
                        s[tt][i] = ok ? s[tt][i] : -INFINITY;
                    }
            }
            float tmax = -INFINITY;
#pragma unroll
            for (int tt = 0; tt < 2; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) tmax = fmaxf(tmax, s[tt][i]);
            tmax = pf_max_halves(tmax);
            const bool move = m_init ? tmax > kLazy : tmax > -INFINITY;
            float alpha = 1.0f;
            const bool any_move = __any(move);
            if (__builtin_expect(any_move, 0)) {
                const float delta = move ? tmax : 0.0f;
                m_init = m_init || move;
                m_ref += delta;
                alpha = __builtin_amdgcn_exp2f(-delta);
                l_run *= alpha;
#pragma unroll
                for (int tt = 0; tt < 2; tt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) s[tt][i] -= delta;
#pragma unroll
                for (int i = 0; i < 16; i++) negm[i] = -m_ref;
            }
            float psum = 0.0f, p8[8];
            uint4 pb[2][2];
            int4 flags_ahead;
            wait_loads();                                        // K(it + 1) of this wave's run has landed
            pf_barrier_lds();                                    // A_it
            asm volatile("" : : "s"(blk_ahead));
            qk((it + 1) & 1, s_next, [&](int ks) {
                if (ks == 0) flags_ahead = *(const int4 *)&valid_ldsw[(it + 1) & 3][0];
                if ((ks & 1) == 0) dma(ks >> 1);
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const int j = ks * 2 + u, tt = j >> 4, i = j & 15;
                    const float e = __builtin_amdgcn_exp2f(s[tt][i]);
                    p8[j & 7] = e;
                    psum += e;
                    asm volatile("" : "+v"(psum));               // the sum stays here, in the shadow of the products
                    if ((j & 7) == 7)
                        pb[tt][(i >> 3) & 1] = make_uint4(pack2<DT>(p8[0], p8[1]), pack2<DT>(p8[2], p8[3]), pack2<DT>(p8[4], p8[5]), pack2<DT>(p8[6], p8[7]));
                }
            });
            l_run += psum;
            flags = flags_of(flags_ahead);
            // the tile's weights and, if the reference moved, the rows' factors, to the value wave
            p_ldsw[w][0][lane] = pb[0][0];
            p_ldsw[w][1][lane] = pb[0][1];
            p_ldsw[w][2][lane] = pb[1][0];
            p_ldsw[w][3][lane] = pb[1][1];
            if (any_move) alpha_ldsw[w][lane] = alpha;
            if (lane == 0) moved_ldsw[w] = any_move ? 1 : 0;
            pf_barrier_lds();                                    // B_it
        };
        for (int it = t0; it < ntiles; it += 2) {
            step(it, s_even, s_odd);
            if (it + 1 < ntiles) step(it + 1, s_odd, s_even);
        }
        l_ldsw[w][lane] = l_run;
        pf_barrier_lds();                                        // E: the value wave may read the row sums
        const float l_tot = l_run + __shfl_xor(l_run, 32);
        if (nparts > 1) {
            if (row_live && g == 0) {
                A.part_m[prow] = m_ref;
                A.part_l[prow] = l_tot;
            }
            return;
        }
        if (A.lse_rows && row_live && g == 0)
            A.lse_rows[(size_t)tq * A.QH + head] = l_tot > 0.0f ? m_ref + __builtin_log2f(l_tot) : INFINITY;
        return;
    }

    // ================================ value wave ================================
    pf_f32x16 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.0f;
    uint32_t vx1;
    {
        const int j16 = lane & 15;
        const int rowl = 4 * g + (j16 >> 2);
        const int clane = 2 * ((lane >> 4) & 1) + ((j16 & 3) >> 1), half = j16 & 1;
        vx1 = (uint32_t)(rowl * RB + (((rowl & 3) << 6) | (clane << 4)) + (half << 3));
    }
    pf_barrier_lds();                                            // A_t0 (the score waves' first scores follow it)
    pf_barrier_lds();                                            // B_t0: P(t0) is there
#pragma unroll 1
    for (int it = t0; it < ntiles; it++) {
        const bool last = it + 1 >= ntiles;
        // the tile's weights, then the first V operands (V(it) is there since B_it); the wave waits once
        uint4 pb[2][2];
        pb[0][0] = p_ldsw[w][0][lane];
        pb[0][1] = p_ldsw[w][1][lane];
        pb[1][0] = p_ldsw[w][2][lane];
        pb[1][1] = p_ldsw[w][3][lane];
        const int moved = moved_ldsw[w];
        const uint32_t vb = pf_lds_addr(&v_ldsw[0][0]) + ((uint32_t)(it & 1) << 15) + vx1;
        constexpr int NP = 4 * NDT;
        uint2 lo[NP], hi[NP];
        auto rd = [&](int i) {                                   // product i = (tt, mh, dt) = (i / 16, (i / 8) & 1, i % 8)
            const int roff = ((i / (2 * NDT)) * 32 + 16 * ((i / NDT) & 1)) * RB;
            const uint32_t va = vb ^ (uint32_t)((i % NDT) << 6);
            lo[i] = pf_lds_read_tr16(va, roff);
            hi[i] = pf_lds_read_tr16(va, roff + 8 * RB);
        };
#pragma unroll
        for (int i = 0; i < XP; i++) rd(i);
        pf_sched_barrier();
        if (__builtin_expect(moved != 0, 0)) {
            const float alpha = alpha_ldsw[w][lane];
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[dt][i] *= alpha;
        }
        plan(it + 1, blk_ahead);                                 // V(it + 1): requested between the products below
        blk_ahead = page_of(it + 2);
        asm volatile("" : : "s"(blk_ahead));
#pragma unroll
        for (int i = 0; i < NP; i++) {
            if (i + XP < NP) rd(i + XP);
            // A_{it+1}: P(it) has been read -- the products before this one used it -- and the score wave may write
            // P(it + 1); the V operands on their way are not waited for
            if (i == kFirst && !last) {
                pf_sched_barrier();
                asm volatile("s_barrier" ::: "memory");
                pf_sched_barrier();
            }
            if (i >= kFirst && (i - kFirst) % 3 == 0 && (i - kFirst) / 3 < 8 && !last) dma((i - kFirst) / 3);
            o[i % NDT] = mfma32<DT>(make_uint4(lo[i].x, lo[i].y, hi[i].x, hi[i].y), pb[i / (2 * NDT)][(i / NDT) & 1], o[i % NDT]);
            pf_sched_barrier();
        }
        if (!last) {
            wait_loads();                                        // V(it + 1) of this wave's run has landed
            pf_barrier_lds();                                    // B_{it+1}
        }
    }
    pf_barrier_lds();                                            // E
    const float l_tot = l_ldsw[w][lane] + l_ldsw[w][lane ^ 32];
    if (nparts > 1) {
        if (row_live) {
            float *orow = A.part_o + prow * D;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int b4 = 0; b4 < 4; b4++)
                    *(float4 *)(orow + dt * 32 + 8 * b4 + 4 * g) =
                        make_float4(o[dt][4 * b4], o[dt][4 * b4 + 1], o[dt][4 * b4 + 2], o[dt][4 * b4 + 3]);
        }
        return;
    }
    if (row_live && (l_tot > 0.0f || A.gate)) {
        const bool have = l_tot > 0.0f;
        const float inv = have ? 1.0f / l_tot : 0.0f;
        uint8_t *orow = A.out + ((size_t)tq * A.QH + head) * (D * 2);
        const uint16_t *grow = A.gate ? A.gate + ((size_t)tq * A.QH + head) * A.gate_stride : nullptr;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int b4 = 0; b4 < 4; b4++) {
                const int d0 = dt * 32 + 8 * b4 + 4 * g;
                uint2 v = have ? make_uint2(pack2<IO>(o[dt][4 * b4] * inv, o[dt][4 * b4 + 1] * inv),
                                            pack2<IO>(o[dt][4 * b4 + 2] * inv, o[dt][4 * b4 + 3] * inv))
                               : *(const uint2 *)(orow + d0 * 2);
                if (grow) {
                    const uint2 gv = *(const uint2 *)(grow + d0);
                    v.x = (uint32_t)gated_elem16((uint16_t)(v.x & 0xffffu), (uint16_t)(gv.x & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.x >> 16), (uint16_t)(gv.x >> 16), IO) << 16);
                    v.y = (uint32_t)gated_elem16((uint16_t)(v.y & 0xffffu), (uint16_t)(gv.y & 0xffffu), IO) |
                          ((uint32_t)gated_elem16((uint16_t)(v.y >> 16), (uint16_t)(gv.y >> 16), IO) << 16);
                }
                *(uint2 *)(orow + d0 * 2) = v;
            }
    }
}

// ---- attention mass of a chunk ------------------------------------------------------------------
// mass[lb] += sum over the chunk's rows (query tokens x query heads) and over the tokens of logical block lb of
// the row's softmax probability: what each page of the context received from a perception frame (the
// importance scorer's input, computed for decode steps by the stream kernel).  The chunk kernels cannot give
// it -- a row's normaliser is known only when its walk ends -- so this kernel walks the keys twice and never
// touches V: the first walk finds every row's log-sum-exp, the second adds exp2(score - lse) up by key.
// The products are S = Q K^T, the transpose of the chunk kernel's: a lane stands for a key (n = lane & 31
// of each 32-token half tile) and its 16 registers for rows 8 (i / 4) + 4 g + i % 4 of the wave's 32, so a
// key's sum over rows is a sum over registers plus one exchange between the lane halves, and a page's is a
// 16-lane DPP sum.  A lane keeps its own running maximum and sum per row over the keys it sees (no exchange
// per tile); the 32 lanes of a row meet once, between the walks.
// grid = ceil(M / TPW) * KVH, TPW = 128 / (QH/KVH); block = 256.  mass is added to with float atomics
// (several workgroups -- row tiles and kv heads -- meet in every page): sums differ by rounding from run to run.
__device__ __forceinline__ float pf_row16_sum(float v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    auto dpp = [](float x, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, false));
    };
    v += dpp(v, std::integral_constant<int, 0xB1>{});
    v += dpp(v, std::integral_constant<int, 0x4E>{});
    v += dpp(v, std::integral_constant<int, 0x141>{});
    v += dpp(v, std::integral_constant<int, 0x140>{});
#endif
    return v;
}

template <int DT, int KV = DT, int IO = DT, int D = 128>
__global__ __launch_bounds__(256, D == 128 ? 2 : 1) void prefill_mass_kernel(PrefillArgs A, float *__restrict__ mass, int mass_len)
{
    constexpr bool Q8 = KV == DRK_INT8 || KV == DRK_FP8_E4M3;
    constexpr int RB = D * (Q8 ? 1 : 2);
    constexpr int kPitchK = D * 2 + 16;
    constexpr int NKS = D / 16;
    __shared__ __align__(16) uint8_t k_lds2[2][kPfBN * kPitchK];
    __shared__ int valid_lds2[2][4];                        // page present, per (buffer, 16-token run)

    // workgroup = (row tile, kv head, part): with the rows' log-sum-exps given the launcher may cut every walk into
    // A.kparts ranges of tiles (a short chunk behind a long context has few walks; the parts' sums just add up)
    const int wg = (int)blockIdx.x / A.kparts, part = (int)blockIdx.x - wg * A.kparts;
    const int kvh = wg % A.KVH;
    const int qt = wg / A.KVH;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int n = lane & 31, g = lane >> 5;
    const int G = A.QH / A.KVH, TPW = A.tpw;
    const int lim_wg = A.pos_start + min((qt + 1) * TPW, A.M);
    const int nt_walk = (lim_wg + kPfBN - 1) / kPfBN;
    const int t0 = (int)((long)part * nt_walk / A.kparts), ntiles = (int)((long)(part + 1) * nt_walk / A.kparts);   // the part's tiles: [t0, ntiles)
    if (t0 >= ntiles) return;

    // Q as the A operand: this lane's fragment belongs to row w * 32 + n
    uint4 qf[NKS];
    {
        const int r = w * 32 + n, rt = r / G;
        const int tq = qt * TPW + rt;
        const int head = kvh * G + (r - rt * G);
        const bool row_live = rt < TPW && tq < A.M;
        const uint8_t *qrow = A.q + ((size_t)tq * A.QH + head) * (D * 2) + g * 16;
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            uint4 v = row_live ? *(const uint4 *)(qrow + ks * 32) : make_uint4(0, 0, 0, 0);
#if defined(__HIP_DEVICE_COMPILE__)
            if constexpr (IO == DRK_BF16 && DT == DRK_F16) {      // 8-bit pages multiply in fp16
                v.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.x), bf16_hi(v.x)));
                v.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.y), bf16_hi(v.y)));
                v.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.z), bf16_hi(v.z)));
                v.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.w), bf16_hi(v.w)));
            }
#endif
            qf[ks] = v;
        }
    }
    // the rows this lane's registers stand for: tokens [0, vis[i]) are visible to row i (0: an idle row)
    int vis[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int r = w * 32 + 8 * (i >> 2) + 4 * g + (i & 3), rt = r / G;
        const int tq = qt * TPW + rt;
        vis[i] = (rt < TPW && tq < A.M) ? A.pos_start + tq + 1 : 0;
    }

    const uint8_t *kbase = A.pool_layer + (size_t)kvh * A.head_stride;
    bool kreg_valid = false;
    int kreg_lim = 0;
    PfGroup<RB> kreg;
    constexpr int NL = PfGroup<RB>::NL;
    uint16_t ksc[NL];
    auto fetch_k = [&](int tile) {                           // the wave's 16-token run of the tile -> registers
        const int tg = tile * kPfBN + w * 16;
        kreg_valid = false;
        kreg_lim = lim_wg - tg;
        size_t off = 0, soff = 0;
        if (tg < lim_wg) {
            const int lb = A.bs_shift >= 0 ? (tg >> A.bs_shift) : (tg / A.bs);
            const int blk = A.table[lb];
            if (blk >= 0 && blk < A.NB) {
                kreg_valid = true;
                const size_t base = (size_t)blk * A.block_stride;
                soff = base + 2 * (size_t)A.kv_plane + ((size_t)kvh * A.bs + (tg - lb * A.bs)) * 2;
                off = base + (size_t)(tg - lb * A.bs) * RB;
            }
        }
        kreg = pf_load_group<false, RB>(kbase, kreg_valid, off, lane);
#pragma unroll
        for (int j = 0; j < NL; j++) {
            const int row = (lane * 16 + 1024 * j) / RB;
            ksc[j] = (KV == DRK_INT8 && kreg_valid) ? *(const uint16_t *)(A.pool_layer + soff + row * 2) : (uint16_t)0;
        }
    };
    auto stage_k = [&](int buf) {
        if constexpr (Q8) pf_store_group_q8<kPitchK, KV, RB>(&k_lds2[buf][0], kreg, w, lane, ksc, kreg_lim);
        else pf_store_group<kPitchK, RB>(&k_lds2[buf][0], kreg, w, lane, kreg_lim);
        if (lane == 0) valid_lds2[buf][w] = kreg_valid ? 1 : 0;
    };

    constexpr float kLazy = 8.0f, kNone = -1.0e30f;
    float m[16], l[16], lse[16];
#pragma unroll
    for (int i = 0; i < 16; i++) { m[i] = kNone; l[i] = 0.0f; lse[i] = INFINITY; }

    int carry_lb = 0;                                        // second walk: the block this lane is adding up, and its sum so far
    float carry = 0.0f;
    auto walk = [&](auto second) {
        constexpr bool MASS = decltype(second)::value;
        fetch_k(t0);
        stage_k(t0 & 1);
        if (t0 + 1 < ntiles) fetch_k(t0 + 1);
        __syncthreads();
#pragma unroll 1
        for (int it = t0; it < ntiles; it++) {
            if (it + 1 < ntiles) {
                stage_k((it + 1) & 1);                       // the buffer tile it - 1 was read from, a barrier ago
                if (it + 2 < ntiles) fetch_k(it + 2);
            }
            pf_f32x16 s[2];
            {
                const uint8_t *kb = &k_lds2[it & 1][0] + n * kPitchK + g * 16;
                const pf_f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int ks = 0; ks < NKS; ks++) {
                    const uint4 b0 = *(const uint4 *)(kb + ks * 32);
                    const uint4 b1 = *(const uint4 *)(kb + 32 * kPitchK + ks * 32);
                    s[0] = mfma32<DT>(qf[ks], b0, ks == 0 ? zero : s[0]);
                    s[1] = mfma32<DT>(qf[ks], b1, ks == 0 ? zero : s[1]);
                }
            }
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
                const int key = it * kPfBN + tt * 32 + n;
                const bool kvalid = valid_lds2[it & 1][tt * 2 + (n >> 4)] != 0;
                float x[16];
                bool any_move = false;
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    x[i] = (kvalid && key < vis[i]) ? s[tt][i] * A.scale_log2e : -INFINITY;
                    if (!MASS) any_move = any_move || x[i] > m[i] + kLazy;
                }
                if constexpr (!MASS) {
                    if (__any(any_move)) {
#pragma unroll
                        for (int i = 0; i < 16; i++) {
                            const float m_new = x[i] > m[i] + kLazy ? x[i] : m[i];
                            l[i] = l[i] * __builtin_amdgcn_exp2f(m[i] - m_new) + __builtin_amdgcn_exp2f(x[i] - m_new);
                            m[i] = m_new;
                        }
                    } else {
#pragma unroll
                        for (int i = 0; i < 16; i++) l[i] += __builtin_amdgcn_exp2f(x[i] - m[i]);
                    }
                } else {
                    float cs = 0.0f;
#pragma unroll
                    for (int i = 0; i < 16; i++) cs += __builtin_amdgcn_exp2f(x[i] - lse[i]);
                    cs += __shfl_xor(cs, 32);                // the key's other 16 rows
                    cs = pf_row16_sum(cs);                   // the 16 keys of a run
                    const int run0 = it * kPfBN + tt * 32 + (n & 16);
                    if (g == 0 && (n & 15) == 0 && run0 < lim_wg) {
                        // the lane keeps adding while its runs stay in one block (blocks of 32 tokens or more) and
                        // goes to memory when the block changes: every workgroup of the launch adds to the same few
                        // blocks at about the same time, and atomics to one address queue up
                        const int lb = A.bs_shift >= 0 ? (run0 >> A.bs_shift) : (run0 / A.bs);
                        if (lb != carry_lb) {
                            if (carry != 0.0f && carry_lb < mass_len) unsafeAtomicAdd(mass + carry_lb, carry);
                            carry_lb = lb;
                            carry = 0.0f;
                        }
                        carry += cs;
                    }
                }
            }
            __syncthreads();
        }
    };
    if (A.lse_rows) {
        // the chunk's attention kernel left every row's log-sum-exp: one walk
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int r = w * 32 + 8 * (i >> 2) + 4 * g + (i & 3), rt = r / G;
            const int tq = qt * TPW + rt;
            lse[i] = vis[i] > 0 ? A.lse_rows[(size_t)tq * A.QH + kvh * G + (r - rt * G)] : INFINITY;
        }
    } else {
        walk(std::false_type{});
        // a row's lanes (the 32 of its half of the wave) meet: lse = M + log2(sum l 2^(m - M)); +inf for a row that saw nothing
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float mm = m[i];
#pragma unroll
            for (int off = 1; off < 32; off <<= 1) mm = fmaxf(mm, __shfl_xor(mm, off));
            float ll = l[i] * __builtin_amdgcn_exp2f(m[i] - mm);
#pragma unroll
            for (int off = 1; off < 32; off <<= 1) ll += __shfl_xor(ll, off);
            lse[i] = ll > 0.0f ? mm + __builtin_log2f(ll) : INFINITY;
        }
    }
    walk(std::true_type{});
    if (carry != 0.0f && carry_lb < mass_len) unsafeAtomicAdd(mass + carry_lb, carry);
}

// ---- attention mass of a chunk: 256 rows per workgroup, 16-bit tiles straight into LDS ----------------------
// prefill_mass_kernel rebuilt on the chunk kernels' machinery (one walk when the rows' log-sum-exps are given; TWO:
// the workgroup first walks its keys for them, a lane keeping a lazy running maximum and sum per row over the keys
// it sees, the 32 lanes of a row meeting once between the walks): 256 rows per workgroup (eight
// waves of 32, two per SIMD), K tiles from global memory straight into a ring of four swizzled LDS buffers,
// requested two tiles ahead between the k-steps, one barrier per tile; the products start from minus the row's
// log-sum-exp (the C operand), so a score arrives as the exponent of its probability, and the exponentials of tile t
// sit between the k-steps of tile t + 1's products, the fold of tile t - 1's sums too.  A wave's instruction
// count bounds it -- 32 exponentials (8 clocks each on this chip, measured) and 32 additions per wave and tile beside
// 16 products of 32 clocks -- so the steps in the interior of a part (no masked row, every block with a page, the
// tile requested whole: all but the last three or four of a walk) run a lean form: no validity flags, no
// conditions, the request's plan behind the first operand reads, the table entry loaded where the barrier's wait
// covers it, page sums without the exchange between the wave's halves.  A wave none of whose rows exists (a short
// frame) only takes part in the barriers and the requests.  S = Q K^T as
// in prefill_mass_kernel: a lane stands for a key, its registers for 16 of the wave's rows, a key's sum over rows is
// a sum over registers.  A page's sum goes to a table in LDS (one entry per logical block of the walk) and the
// table to `mass` with one atomic per block and workgroup when the walk ends -- 256 workgroups adding to the same
// four blocks tile after tile would queue up on them.  FOLD: the softmax scale goes into Q, rounded to the 16-bit
// type, as in the chunk kernels that do so (their log-sum-exps belong to those scores); otherwise Q stays as it
// is and the exponent is scaled.
// grid = ceil(M / TPW) * KVH * parts, TPW = 256 / (QH/KVH); block = 512; block size 16 * 2^k; at most
// kMassdBlocks<D> logical blocks in a part's range of tiles (the launcher sees to it).
template <int D>
constexpr int kMassdBlocks = D == 128 ? 8192 : 6144;
template <int DT, int IO, int D, bool FOLD, bool TWO, int KV = DT>
__global__ __launch_bounds__(512, 1) void prefill_massd_kernel(PrefillArgs A, float *__restrict__ mass, int mass_len)
{
    // Q8: 8-bit pages (head_dim 128, one walk).  A tile's codes cannot go straight into LDS: a wave's 8 rows are one
    // 16-byte load per lane into registers, requested where the 16-bit kind requests, and turned into fp16 rows of the
    // same swizzled layout at the head of the next step (a step ahead of the barrier behind which they are read).
    constexpr bool Q8 = KV == DRK_INT8 || KV == DRK_FP8_E4M3;
    static_assert(!Q8 || (D == 128 && !TWO && DT == DRK_F16), "8-bit pages: head_dim 128, fp16 products, the rows' log-sum-exps given");
    constexpr int RB = D * 2;
    constexpr int SRB = Q8 ? D : RB;                         // bytes of a token row of one kv head in its page
    constexpr int kTileBytes = kPfBN * RB, kTileShift = D == 128 ? 14 : 15;
    constexpr int NKS = D / 16;
    constexpr int kRing = 4, ROWS = 8;                       // buffers; tokens of a tile one wave requests
    constexpr int LPR = RB / 16, RPQ = 64 / LPR, NREQ = ROWS / RPQ;   // lanes per token row, rows per request, requests per wave and tile
    constexpr int XQ = 2;                                    // operand reads ahead of their products, k-steps
    constexpr int EPK = 32 / NKS;                            // exponentials per k-step
    __shared__ __align__(512) uint8_t k_ldsm[kRing][kTileBytes];
    __shared__ float mass_ldsm[kMassdBlocks<D>];
    __shared__ __align__(16) int valid_ldsm[kRing][8];                     // [tile & 3][wave]: the wave's 8-token run of the tile has a page

    // workgroup = (walk, part): a walk is (row block of tokens, kv head), the longest first; a part is one of
    // A.kparts ranges of the walk's tiles (a short chunk behind a long context has few walks: with the rows'
    // log-sum-exps known the parts need no merge, their sums just add up)
    const int walk = (int)blockIdx.x / A.kparts, part = (int)blockIdx.x - walk * A.kparts;
    const int kvh = walk % A.KVH;
    const int qt = A.nqt - 1 - walk / A.KVH;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int n = lane & 31, g = lane >> 5;
    const int G = A.QH / A.KVH, TPW = A.tpw;
    const int lim_wg = A.pos_start + min((qt + 1) * TPW, A.M);
    const int first_masked_tile = (A.pos_start + qt * TPW + 1) / kPfBN;
    const int nt_walk = (lim_wg + kPfBN - 1) / kPfBN;
    const int t0 = __builtin_amdgcn_readfirstlane((int)((long)part * nt_walk / A.kparts));
    const int ntiles = __builtin_amdgcn_readfirstlane((int)((long)(part + 1) * nt_walk / A.kparts));     // the part's tiles: [t0, ntiles)
    if (t0 >= ntiles) return;                                // more parts than tiles
    const int sh = A.bs_shift;
    const int lb0 = (t0 * kPfBN) >> sh;                      // the table in LDS begins at the part's first block
    const int nblk_wg = min(((min(lim_wg, ntiles * kPfBN) + A.bs - 1) >> sh) - lb0, kMassdBlocks<D>);   // (the launcher keeps a part within the table)

    // (while clearing the table: does every block of the part have a page?  Then most steps need no validity flags)
    int no_page = 0;
    for (int i = threadIdx.x; i < nblk_wg; i += 512) {
        mass_ldsm[i] = 0.0f;
        const int e = A.table[lb0 + i];
        no_page |= (e < 0 || e >= A.NB) ? 1 : 0;
    }
    for (int i = threadIdx.x * 16; i < kRing * kTileBytes; i += 512 * 16) *(uint4 *)(&k_ldsm[0][0] + i) = make_uint4(0, 0, 0, 0);
    const bool holes = __syncthreads_or(no_page) != 0;

    // Q as the A operand: this lane's fragment belongs to row w * 32 + n
    uint4 qf[NKS];
    {
        const int r = w * 32 + n, rt = r / G;
        const int tq = qt * TPW + rt;
        const int head = kvh * G + (r - rt * G);
        const bool row_live = rt < TPW && tq < A.M;
        const uint8_t *qrow = A.q + ((size_t)tq * A.QH + head) * (D * 2) + g * 16;
        const float c = A.scale_log2e;
        auto scaled = [&](uint32_t w2) -> uint32_t {
            return pack2<DT>(elem16_to_f((uint16_t)(w2 & 0xffffu), IO) * c, elem16_to_f((uint16_t)(w2 >> 16), IO) * c);
        };
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            const uint4 v = row_live ? *(const uint4 *)(qrow + ks * 32) : make_uint4(0, 0, 0, 0);
            if constexpr (FOLD) {
                qf[ks] = make_uint4(scaled(v.x), scaled(v.y), scaled(v.z), scaled(v.w));
            } else if constexpr (IO == DRK_BF16 && DT == DRK_F16) {     // 8-bit pages multiply in fp16
#if defined(__HIP_DEVICE_COMPILE__)
                qf[ks] = make_uint4(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.x), bf16_hi(v.x))),
                                    __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.y), bf16_hi(v.y))),
                                    __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.z), bf16_hi(v.z))),
                                    __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.w), bf16_hi(v.w))));
#endif
            } else {
                qf[ks] = v;
            }
        }
    }
    // the rows this lane's registers stand for: tokens [0, vis[i]) are visible to row i (0: an idle row); the
    // products start from -lse (FOLD) or -lse / (scale log2 e), so that the scaled score comes out less the lse
    int vis[16];
    pf_f32x16 negl;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int r = w * 32 + 8 * (i >> 2) + 4 * g + (i & 3), rt = r / G;
        const int tq = qt * TPW + rt;
        const bool live = rt < TPW && tq < A.M;
        vis[i] = live ? A.pos_start + tq + 1 : 0;
        if constexpr (!TWO) {
            const float lse = live ? A.lse_rows[(size_t)tq * A.QH + kvh * G + (r - rt * G)] : INFINITY;
            negl[i] = FOLD ? -lse : -lse / A.scale_log2e;
        } else {
            negl[i] = 0.0f;                                  // the first walk's products start from zero
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");         // from here on the kernel counts its loads itself
    bool wave_live;                                          // one of the wave's 32 rows exists
    {
        const int rt = (w * 32 + n) / G;
        wave_live = __builtin_amdgcn_ballot_w64(rt < TPW && qt * TPW + rt < A.M) != 0ull;
    }

    const uint8_t *kbase = A.pool_layer + (size_t)kvh * A.head_stride;
    const int tgw = w * ROWS;
    typedef const int32_t __attribute__((address_space(4))) *const_table_t;
    const const_table_t table_k = (const_table_t)(uintptr_t)A.table;
    const int lim_part = min(lim_wg, ntiles * kPfBN);        // nothing past the part's end is requested
    auto page_of = [&](int tile) -> int {                    // through the scalar cache: not counted with the requests
        const int tg = tile * kPfBN + tgw;
        return tg < lim_part ? table_k[tg >> sh] : -1;
    };
    const uint8_t *p_src = kbase;
    const uint8_t *p_sc = kbase;                             // int8: the fp16 scales of the wave's rows
    int p_rows = 0;
    uint32_t p_lds = 0;
    const uint32_t k_ring = pf_lds_addr(&k_ldsm[0][0]) + (uint32_t)(tgw * RB);
    auto plan = [&](int kt, int blk_raw) {
        const int blk0 = __builtin_amdgcn_readfirstlane(blk_raw);
        const int tg = kt * kPfBN + tgw;
        const bool ok = blk0 >= 0 && blk0 < A.NB && tg < lim_part;
        p_rows = ok ? lim_part - tg : 0;
        p_src = kbase + (size_t)(ok ? blk0 : 0) * A.block_stride + (size_t)((tg & (A.bs - 1)) * SRB);
        if constexpr (KV == DRK_INT8)
            p_sc = A.pool_layer + (size_t)(ok ? blk0 : 0) * A.block_stride + 2 * (size_t)A.kv_plane + ((size_t)kvh * A.bs + (tg & (A.bs - 1))) * 2;
        p_lds = k_ring + ((uint32_t)(kt & (kRing - 1)) << kTileShift);
        if (lane == 0) valid_ldsm[kt & (kRing - 1)][w] = ok ? 1 : 0;
    };
    auto plan_whole = [&](int kt, int blk_raw) {             // a tile whose pages exist and whose rows are all wanted
        const int blk0 = __builtin_amdgcn_readfirstlane(blk_raw);
        const int tg = kt * kPfBN + tgw;
        p_rows = ROWS;
        p_src = kbase + (size_t)blk0 * A.block_stride + (size_t)((tg & (A.bs - 1)) * SRB);
        if constexpr (KV == DRK_INT8)
            p_sc = A.pool_layer + (size_t)blk0 * A.block_stride + 2 * (size_t)A.kv_plane + ((size_t)kvh * A.bs + (tg & (A.bs - 1))) * 2;
        p_lds = k_ring + ((uint32_t)(kt & (kRing - 1)) << kTileShift);
        if (lane == 0) valid_ldsm[kt & (kRing - 1)][w] = 1;
    };
    // request j: RPQ token rows (1 KB); the 16-byte chunk c of row r sits at position c ^ (r & 15)
    uint32_t goff[NREQ];
    {
        const int rr = lane / LPR, cp = lane % LPR;
#pragma unroll
        for (int j = 0; j < NREQ; j++) goff[j] = (uint32_t)(rr * RB + ((cp ^ ((tgw + RPQ * j + rr) & 15)) << 4));
    }
    bool whole = false;                                      // the last tile requested made all NREQ requests
    // 8-bit pages: the codes (and scale) of the tile requested last, 16 of row lane / 8 per lane; where they go, how
    // many of the wave's rows exist
    uint4 stg = make_uint4(0, 0, 0, 0);
    uint32_t stg_sc = 0, c_lds = 0;
    int c_rows = 0;
    bool stg_live = false;
    constexpr int NREQ_EFF = Q8 ? 1 : NREQ;
    auto request = [&](int j) {
        if constexpr (Q8) {
            if (j == 0) {
                const bool ok = whole || (lane >> 3) < p_rows;
                stg = ok ? *(const uint4 *)(p_src + lane * 16) : make_uint4(0, 0, 0, 0);
                if constexpr (KV == DRK_INT8) stg_sc = ok ? (uint32_t)*(const uint16_t *)(p_sc + (lane >> 3) * 2) : 0u;
                c_lds = p_lds;
                c_rows = p_rows;
                stg_live = true;
            }
        } else {
            if (__builtin_expect(whole, 1)) pf_load_to_lds16(p_src + 1024 * j, goff[j], p_lds + 1024 * j);
            else if (RPQ * j + lane / LPR < p_rows) pf_load_to_lds16(p_src + 1024 * j, goff[j], p_lds + 1024 * j);
        }
    };
    // 8-bit pages: the staged codes as fp16 values (code x scale, rounded once; fp8 exact) into the wave's rows of their
    // buffer -- 16 dims = two 16-byte chunks 2 c, 2 c + 1 of row r, at positions chunk ^ (r & 15); rows past the end as zeros
    auto commit = [&]() {
        if constexpr (Q8) {
            typedef _Float16 h2 __attribute__((ext_vector_type(2)));
            uint32_t h[8];
            if constexpr (KV == DRK_INT8) {
                int8x4_to_f16x4(stg.x, h[0], h[1]);
                int8x4_to_f16x4(stg.y, h[2], h[3]);
                int8x4_to_f16x4(stg.z, h[4], h[5]);
                int8x4_to_f16x4(stg.w, h[6], h[7]);
                const h2 scale = __builtin_bit_cast(h2, stg_sc | (stg_sc << 16));
                const h2 bias = {(_Float16)1152.0f, (_Float16)1152.0f};
#pragma unroll
                for (int i = 0; i < 8; i++) h[i] = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(h2, h[i]) - bias) * scale);
            } else {
                fp8x4_to_f16x4(stg.x, h[0], h[1]);
                fp8x4_to_f16x4(stg.y, h[2], h[3]);
                fp8x4_to_f16x4(stg.z, h[4], h[5]);
                fp8x4_to_f16x4(stg.w, h[6], h[7]);
            }
            const int row = lane >> 3, c0 = (lane & 7) * 2, sw = (tgw + row) & 15;
            if (row >= c_rows) {
#pragma unroll
                for (int i = 0; i < 8; i++) h[i] = 0u;
            }
            const uint32_t rb = c_lds - pf_lds_addr(&k_ldsm[0][0]) + (uint32_t)(row * RB);
            *(uint4 *)(&k_ldsm[0][0] + rb + ((c0 ^ sw) << 4)) = make_uint4(h[0], h[1], h[2], h[3]);
            *(uint4 *)(&k_ldsm[0][0] + rb + (((c0 + 1) ^ sw) << 4)) = make_uint4(h[4], h[5], h[6], h[7]);
        }
    };
    auto request_tile = [&]() {
        whole = p_rows >= ROWS;
#pragma unroll
        for (int j = 0; j < NREQ_EFF; j++) request(j);
        if constexpr (Q8) commit();                          // (the prologue: straight into LDS)
    };

    // where this lane finds its B operands: K row n (and n + 32), chunk 2 ks + g at byte ((g ^ n & 15) << 4) ^ (ks << 5)
    const uint32_t kx1 = (uint32_t)(n * RB + ((g ^ (n & 15)) << 4));
    auto qk = [&](int slot, pf_f32x16 (&s)[2], auto &&between) {
        const uint32_t ka0 = pf_lds_addr(&k_ldsm[0][0]) + ((uint32_t)slot << kTileShift) + kx1;
        uint4 b[NKS][2];
#pragma unroll
        for (int ks = 0; ks < XQ; ks++) {
            b[ks][0] = pf_lds_read128(ka0 ^ (uint32_t)(ks << 5), 0);
            b[ks][1] = pf_lds_read128(ka0 ^ (uint32_t)(ks << 5), 32 * RB);
        }
        pf_sched_barrier();
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            if (ks + XQ < NKS) {
                b[ks + XQ][0] = pf_lds_read128(ka0 ^ (uint32_t)((ks + XQ) << 5), 0);
                b[ks + XQ][1] = pf_lds_read128(ka0 ^ (uint32_t)((ks + XQ) << 5), 32 * RB);
            }
            between(ks);
            if (ks == 0) {
                s[0] = mfma32<DT>(qf[ks], b[ks][0], negl);
                s[1] = mfma32<DT>(qf[ks], b[ks][1], negl);
            } else {
                s[0] = mfma32<DT>(qf[ks], b[ks][0], s[0]);
                s[1] = mfma32<DT>(qf[ks], b[ks][1], s[1]);
            }
            pf_sched_barrier();
        }
    };

    // One walk over the part's tiles.  LSE: the first of two walks -- every lane keeps a running maximum and sum per
    // row over the keys it sees, in units of the exponent; the second (or only) walk adds the probabilities up by key.
    const float cexp = FOLD ? 1.0f : A.scale_log2e;
    float m_run[16], l_run[16];
    auto run_walk = [&](auto lse_mode) {
        constexpr bool LSE = decltype(lse_mode)::value;
        // ---- prologue: K(t0), K(t0 + 1), K(t0 + 2) requested and there, the scores of tile t0 ----
        int blk_ahead;
        {
            const int b0 = page_of(t0), b1 = page_of(t0 + 1), b2 = page_of(t0 + 2);
            blk_ahead = page_of(t0 + 3);
            __syncthreads();                                     // the clearing is done (and the table entries are here)
            plan(t0, b0);
            request_tile();
            plan(t0 + 1, b1);
            request_tile();
            plan(t0 + 2, b2);
            request_tile();
            __builtin_amdgcn_s_waitcnt(0x0f70);                  // vmcnt(0)
            stg_live = false;
        }
        __syncthreads();
        pf_f32x16 s_even[2], s_odd[2];
        qk(t0 & (kRing - 1), s_even, [](int) {});
        // bit r: the tile's 8-token run r has a page; read one tile ahead, between the products
        auto flags_of = [&](const int4 &a, const int4 &b) -> int {
            return __builtin_amdgcn_readfirstlane(a.x | (a.y << 1) | (a.z << 2) | (a.w << 3) | (b.x << 4) | (b.y << 5) | (b.z << 6) | (b.w << 7));
        };
        int flags = flags_of(*(const int4 *)&valid_ldsm[t0 & (kRing - 1)][0], *(const int4 *)&valid_ldsm[t0 & (kRing - 1)][4]);

        // the page sums of tile `tile_t` from the lanes' key sums: a key's other 16 rows are in the other half of the
        // wave; a block is 16 keys or more
        auto fold = [&](int tile_t, const float (&cs)[2]) {
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
                const auto r2 = __builtin_amdgcn_permlane32_swap(__float_as_uint(cs[tt]), __float_as_uint(cs[tt]), false, false);
                const float c16 = pf_row16_sum(__uint_as_float(r2[0]) + __uint_as_float(r2[1]));
                const int run0 = tile_t + tt * 32 + (n & 16);
                const int bi = (run0 >> sh) - lb0;
            if (g == 0 && (n & 15) == 0 && run0 >= t0 * kPfBN && run0 < lim_part && bi < nblk_wg && c16 != 0.0f) atomicAdd(&mass_ldsm[bi], c16);
            }
        };
        // the same in a step's fast mode: every key of the tile counts and its blocks are the part's; the two halves of
        // the wave add their 16 rows each
        auto fold_whole = [&](int tile_t, const float (&cs)[2]) {
            const int sb = __builtin_amdgcn_readfirstlane((tile_t >> sh) - lb0);
#pragma unroll
            for (int tt = 0; tt < 2; tt++) {
                const float c16 = pf_row16_sum(cs[tt]);
                if ((n & 15) == 0 && c16 != 0.0f) atomicAdd(&mass_ldsm[sb + ((tt * 32 + (n & 16)) >> sh)], c16);
            }
        };
        float cs_prev[2] = {0.0f, 0.0f};                         // the key sums of the tile before, folded a step later
        constexpr float kLazy = 8.0f;
        // FAST: a step in the part's interior -- no row of tile it is masked, every block has a page, tile it + 3 is
        // whole for every wave: no flags, no conditions, and the plan behind the first operand reads
        // a wave none of whose 32 rows exists (a short frame: 16 tokens x 4 heads fill two of the eight waves) does the
        // step's memory side only -- the barrier, its share of the next tile's request -- and leaves the SIMD to its neighbour
        auto idle_step = [&](auto fast_mode, int it) {
            constexpr bool FAST = decltype(fast_mode)::value;
            if constexpr (!Q8) {
                if (FAST || __builtin_expect(whole, 1)) __builtin_amdgcn_s_waitcnt(NREQ == 2 ? 0x0f72 : 0x0f74);   // vmcnt(NREQ)
                else __builtin_amdgcn_s_waitcnt(0x0f70);
            }
            pf_barrier_lgkm();
            if constexpr (Q8) {
                if (stg_live) commit();
            }
            if constexpr (FAST) {
                plan_whole(it + 3, blk_ahead);
                whole = true;
            } else {
                plan(it + 3, blk_ahead);
                whole = p_rows >= ROWS;
            }
            blk_ahead = page_of(it + 4);
#pragma unroll
            for (int j = 0; j < NREQ_EFF; j++) request(j);
            flags = 255;                                         // (its scores are never looked at)
        };
        auto step = [&](auto fast_mode, int it, pf_f32x16 (&s)[2], pf_f32x16 (&s_next)[2]) {
            constexpr bool FAST = decltype(fast_mode)::value;
            // here: s = exponents of tile it; K(it + 1) and K(it + 2) requested
            const int tile_t = it * kPfBN;
            if (!FAST && __builtin_expect(flags != 255 || it >= first_masked_tile, 0)) {
#pragma unroll
                for (int tt = 0; tt < 2; tt++) {
                    const int key = tile_t + tt * 32 + n;
                    const bool kvalid = ((flags >> ((tt * 32 + n) >> 3)) & 1) != 0;
#pragma unroll
                    for (int i = 0; i < 16; i++) s[tt][i] = (kvalid && key < vis[i]) ? s[tt][i] : -INFINITY;
                }
            }
            if constexpr (LSE) {
                // a lane's running maximum per row over the keys it has seen moves only when a score exceeds it by kLazy
                // (in units of the exponent): the common tile costs sixteen maxima and compares
                bool mv = false;
#pragma unroll
                for (int i = 0; i < 16; i++) mv = mv || fmaxf(s[0][i], s[1][i]) * cexp > m_run[i] + kLazy;
                if (__builtin_expect(__any(mv), 0)) {
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const float x = fmaxf(s[0][i], s[1][i]) * cexp;
                        const float m_new = x > m_run[i] + kLazy ? x : m_run[i];
                        l_run[i] *= __builtin_amdgcn_exp2f(m_run[i] - m_new);
                        m_run[i] = m_new;
                    }
                }
            }
            // K(it + 1) has landed (this wave's share; the requests of K(it + 2) came after it), then everybody's
            if constexpr (!Q8) {
                if (FAST || __builtin_expect(whole, 1)) __builtin_amdgcn_s_waitcnt(NREQ == 2 ? 0x0f72 : 0x0f74);   // vmcnt(NREQ)
                else __builtin_amdgcn_s_waitcnt(0x0f70);
            }
            pf_barrier_lgkm();
            if constexpr (Q8) {
                if (stg_live) commit();                          // K(it + 2), requested a step ago, read behind the next barrier
            }
            if constexpr (!FAST) {
                asm volatile("" : : "s"(blk_ahead));
                plan(it + 3, blk_ahead);                         // into the buffer of K(it - 1), read two steps ago
                blk_ahead = page_of(it + 4);
                whole = p_rows >= ROWS;                          // requested between the products below
            }
            float cs[2] = {0.0f, 0.0f};
            int4 fa, fb;
            qk((it + 1) & (kRing - 1), s_next, [&](int ks) {
                if constexpr (FAST) {
                    if (ks == 0) {
                        plan_whole(it + 3, blk_ahead);
                        whole = true;
                    }
                    if constexpr (Q8) {
                        if (ks == 1) request(0);
                    } else {
                        if ((ks & 1) == 1 && (ks >> 1) < NREQ) pf_load_to_lds16(p_src + 1024 * (ks >> 1), goff[ks >> 1], p_lds + 1024 * (ks >> 1));
                    }
                } else {
                    if (ks == 0) {
                        fa = *(const int4 *)&valid_ldsm[(it + 1) & (kRing - 1)][0];
                        fb = *(const int4 *)&valid_ldsm[(it + 1) & (kRing - 1)][4];
                    }
                    if ((ks & 1) == 0 && (ks >> 1) < NREQ_EFF) request(ks >> 1);
                }
                if constexpr (!LSE) {
                    if (ks == NKS / 2) {
                        if constexpr (FAST) fold_whole(tile_t - kPfBN, cs_prev);
                        else fold(tile_t - kPfBN, cs_prev);
                    }
                }
#pragma unroll
                for (int u = 0; u < EPK; u++) {
                    const int j = ks * EPK + u, tt = j >> 4, i = j & 15;
                    if constexpr (LSE) {
                        l_run[i] += __builtin_amdgcn_exp2f(s[tt][i] * cexp - m_run[i]);
                        asm volatile("" : "+v"(l_run[i]));
                    } else {
                        const float e = __builtin_amdgcn_exp2f(FOLD ? s[tt][i] : s[tt][i] * A.scale_log2e);
                        cs[tt] += e;
                        asm volatile("" : "+v"(cs[tt]));         // the sum stays here, in the shadow of the products
                    }
                }
            });
            if constexpr (FAST) {
                flags = 255;
                blk_ahead = page_of(it + 4);                     // the scalar load's wait falls into the barrier's
            } else {
                flags = flags_of(fa, fb);
            }
            cs_prev[0] = cs[0];
            cs_prev[1] = cs[1];
        };
        // steps [t0, fast_end) can run in the fast mode: tile it unmasked, tile it + 3 whole for every wave
        const int fast_end = holes ? t0 : min(first_masked_tile, lim_part / kPfBN - 3);
        int it = t0;
        if (__builtin_expect(!wave_live, 0)) {                   // the same steps, the same barriers
            for (; it < fast_end; it++) idle_step(std::true_type{}, it);
            for (; it < ntiles; it++) idle_step(std::false_type{}, it);
            return;
        }
        for (; it + 2 <= fast_end; it += 2) {
            step(std::true_type{}, it, s_even, s_odd);
            step(std::true_type{}, it + 1, s_odd, s_even);
        }
        for (; it < ntiles; it += 2) {
            step(std::false_type{}, it, s_even, s_odd);
            if (it + 1 < ntiles) step(std::false_type{}, it + 1, s_odd, s_even);
        }
        if constexpr (!LSE) fold((ntiles - 1) * kPfBN, cs_prev);
    };
    if constexpr (TWO) {
#pragma unroll
        for (int i = 0; i < 16; i++) { m_run[i] = -1.0e30f; l_run[i] = 0.0f; }
        run_walk(std::true_type{});
        // a row's lanes (the 32 of its half of the wave) meet: lse = M + log2(sum l 2^(m - M)); +inf for a row that
        // saw nothing.  The second walk's products start from -lse in units of the product.
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float mm = m_run[i];
#pragma unroll
            for (int off = 1; off < 32; off <<= 1) mm = fmaxf(mm, __shfl_xor(mm, off));
            float ll = l_run[i] * __builtin_amdgcn_exp2f(m_run[i] - mm);
#pragma unroll
            for (int off = 1; off < 32; off <<= 1) ll += __shfl_xor(ll, off);
            const float lse = (vis[i] > 0 && ll > 0.0f) ? mm + __builtin_log2f(ll) : INFINITY;
            negl[i] = -lse / cexp;
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);
    }
    run_walk(std::false_type{});
    __builtin_amdgcn_s_waitcnt(0x0f70);                      // nothing is on its way when the workgroup ends
    __syncthreads();
    for (int i = threadIdx.x; i < nblk_wg; i += 512) {
        const float v = mass_ldsm[i];
        if (v != 0.0f && lb0 + i < mass_len) unsafeAtomicAdd(mass + lb0 + i, v);
    }
}

// mass[0 .. n) = 0
__global__ void pf_zero_kernel(float *__restrict__ p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

// Global loads the compiler does not count (see prefix_stream_kernel): issue, and wait until at most N of the
// wave's loads are outstanding -- the values named become usable then, and only then.
__device__ __forceinline__ pf_u32x4 pf_async_load128(const uint8_t *p)
{
    pf_u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off nt" : "=&v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ uint32_t pf_async_load16(const uint8_t *p)
{
    uint32_t v;
    asm volatile("global_load_ushort %0, %1, off" : "=&v"(v) : "v"(p) : "memory");
    return v;
}
template <int N>
__device__ __forceinline__ void pf_async_wait(pf_u32x4 &a, pf_u32x4 &b)
{
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void pf_async_wait16(uint32_t &a, uint32_t &b)
{
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}
__device__ __forceinline__ void pf_async_drain() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ---- shared-prefix pass for few rows: producer and consumer waves ---------------------------------
// With at most 64 rows (branches x query heads of one kv head) the pass is bound by HBM, and the kernel above
// -- every wave stages one tile ahead in its own registers, next to its accumulators -- keeps only 64 KB per
// CU in flight: each trip of its loop waits out a full memory latency (16 trips of 3.3 us for 1 024 tokens).
// Here a workgroup has eight waves.  Waves 4-7 only move data: wave 4 + p owns the 16-token run p of every
// tile and keeps four tiles' worth of it in registers (64 data registers), requesting tile t + 5 the moment
// tile t + 1 has gone to LDS: 128 KB in flight per CU, loads issued four steps before their use.  (One wave
// moving whole tiles was tried first: 64 memory instructions from one wave per step took 3.4 us.)
// Waves 0-3 multiply: wave = (row half, key half) of the 64 x 64 tile, each with its own running maximum and
// sum; the two key halves of a row are folded through LDS at the end.  One barrier per tile: the tile
// written in a step is read in the next.  grid = (KVH * ceil(B / TPW), 1, splits), TPW = 64 / (QH/KVH);
// block = 512, one workgroup per CU; leaves (o, m, l) per (branch, q head, split) like the kernel above.
template <int DT, int KV = DT, int IO = DT>
__global__ __launch_bounds__(512, 1) void prefix_stream_kernel(PrefillArgs A)
{
    constexpr int D = 128;
    constexpr bool Q8 = KV == DRK_INT8 || KV == DRK_FP8_E4M3;
    constexpr int RB = D * (Q8 ? 1 : 2);
    constexpr int kPitchK = D * 2 + 16, kPitchV = D * 2 + 32;
    constexpr int NKS = D / 16, NDT = D / 32;
    __shared__ __align__(16) uint8_t k_lds2[2][kPfBN * kPitchK];
    __shared__ __align__(16) uint8_t v_lds2[2][kPfBN * kPitchV];
    __shared__ int runs_lds[2][4];                           // the 16-token run of the tile in this slot has a page

    const int kvh = (int)blockIdx.x % A.KVH;
    const int qt = (int)blockIdx.x / A.KVH;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int t_begin = (int)blockIdx.z * A.chunk_tiles;
    const int lim_wg = min(A.shared, (t_begin + A.chunk_tiles) * kPfBN);
    const int nt = max(0, (lim_wg + kPfBN - 1) / kPfBN - t_begin);     // tiles of this workgroup

    if (w >= 4) {
        // ---------------- producer: the 16-token run p of every tile, kDepth tiles ahead ----------------
        const int p = w - 4;
        constexpr int kDepth = 4;
        constexpr int NLR = PfGroup<RB, 16>::NL;             // 16-byte chunks per lane, operand and run: 4 (16-bit) or 2
        // The loads are written as inline assembly and waited for by count: the compiler's own bookkeeping gives up
        // at the loop's head (it cannot tell which of the rotating buffers a pending load belongs to) and drains
        // every load there, the three tiles meant to stay in flight included.  Loads return in order, so "all but
        // the last 3 fetches" is exactly "the buffer about to be stored".
        pf_u32x4 kx[kDepth][NLR], vx[kDepth][NLR];           // tile t waits in buffer t % kDepth
        uint32_t ksx[kDepth][NLR], vsx[kDepth][NLR];         // int8: the fp16 scales of the rows of this lane's chunks
        constexpr int kLoadsPerFetch = 2 * NLR + (KV == DRK_INT8 ? 2 * NLR : 0);
        int limq[kDepth];                                    // rows of the buffered run that are real (0: no page)
        const uint8_t *kbase = A.pool_layer + (size_t)kvh * A.head_stride;
        // Read through the scalar cache (the table is not written while the kernel runs).
        typedef const int32_t __attribute__((address_space(4))) *const_table_t;
        const const_table_t table_k = (const_table_t)(uintptr_t)A.table;
        // the run's page in local tile i: the table entry, or -1 (past the end)
        auto page_of = [&](int i) -> int {
            const int tg = (t_begin + i) * kPfBN + p * 16;
            if (i >= nt || tg >= lim_wg) return -1;
            return table_k[A.bs_shift >= 0 ? (tg >> A.bs_shift) : (tg / A.bs)];
        };
        auto fetch = [&](int d, int i, int blk) {            // local tile i into buffer d
            const int tg = (t_begin + i) * kPfBN + p * 16;
            const bool ok = blk >= 0 && blk < A.NB;
            const int lb = A.bs_shift >= 0 ? (tg >> A.bs_shift) : (tg / A.bs);
            const int tin = ok ? tg - lb * A.bs : 0;
            const size_t boff = (size_t)(ok ? blk : 0) * A.block_stride;      // no page: block 0 is read and zeros are stored
            const uint8_t *src = kbase + boff + (size_t)tin * RB + (size_t)lane * 16;
#pragma unroll
            for (int j = 0; j < NLR; j++) {
                kx[d][j] = pf_async_load128(src + 1024 * j);
                vx[d][j] = pf_async_load128(src + A.kv_plane + 1024 * j);
                if constexpr (KV == DRK_INT8) {
                    const int row = (lane * 16 + 1024 * j) / RB;
                    const uint8_t *sp = A.pool_layer + boff + 2 * (size_t)A.kv_plane + ((size_t)kvh * A.bs + tin + row) * 2;
                    ksx[d][j] = pf_async_load16(sp);
                    vsx[d][j] = pf_async_load16(sp + A.scale_plane);
                } else {
                    ksx[d][j] = vsx[d][j] = 0;
                }
            }
            limq[d] = ok ? lim_wg - tg : 0;
        };
        auto store = [&](int d, int slot) {
            // everything but the last three fetches has arrived: buffer d
#pragma unroll
            for (int j = 0; j < NLR; j++) {
                pf_async_wait<3 * kLoadsPerFetch>(kx[d][j], vx[d][j]);
                if constexpr (KV == DRK_INT8) pf_async_wait16<3 * kLoadsPerFetch>(ksx[d][j], vsx[d][j]);
            }
            PfGroup<RB, 16> kq, vq;
            uint16_t ksc[NLR], vsc[NLR];
#pragma unroll
            for (int j = 0; j < NLR; j++) {
                kq.r[j] = make_uint4(kx[d][j].x, kx[d][j].y, kx[d][j].z, kx[d][j].w);
                vq.r[j] = make_uint4(vx[d][j].x, vx[d][j].y, vx[d][j].z, vx[d][j].w);
                ksc[j] = (uint16_t)ksx[d][j];
                vsc[j] = (uint16_t)vsx[d][j];
            }
            if constexpr (Q8) {
                pf_store_group_q8<kPitchK, KV, RB, 16>(&k_lds2[slot][0], kq, p, lane, ksc, limq[d]);
                pf_store_group_q8<kPitchV, KV, RB, 16>(&v_lds2[slot][0], vq, p, lane, vsc, limq[d]);
            } else {
                pf_store_group_sel<kPitchK, RB, 16>(&k_lds2[slot][0], kq, p, lane, limq[d]);
                pf_store_group_sel<kPitchV, RB, 16>(&v_lds2[slot][0], vq, p, lane, limq[d]);
            }
            if (lane == 0) runs_lds[slot][p] = limq[d] > 0 ? 1 : 0;
        };
        int first_pages[kDepth + 2];                         // all six table reads go out before the first is waited for
#pragma unroll
        for (int d = 0; d < kDepth + 2; d++) first_pages[d] = page_of(d);
#pragma unroll
        for (int d = 0; d < kDepth; d++) fetch(d, d, first_pages[d]);
        store(0, 0);
        fetch(0, kDepth, first_pages[kDepth]);
        int blk_pf = first_pages[kDepth + 1];                // looked up one step before its loads are issued
        __syncthreads();
#pragma unroll 1
        for (int i0 = 0; i0 < nt; i0 += kDepth) {
#pragma unroll
            for (int d = 0; d < kDepth; d++) {
                const int i = i0 + d;
                if (i < nt) {
                    constexpr int kNextMask = kDepth - 1;
                    const int nx = i + 1;                    // the tile the next step reads: buffer nx % kDepth = (d + 1) % kDepth
                    store((d + 1) & kNextMask, nx & 1);
                    fetch((d + 1) & kNextMask, nx + kDepth, blk_pf);
                    blk_pf = page_of(nx + kDepth + 1);
                    __syncthreads();
                }
            }
        }
        __syncthreads();                                     // the consumers' fold
        pf_async_drain();
        return;
    }

    // ---------------- consumer: rows 32 rh .. +31, keys 32 kh .. +31 of every tile ----------------
    const int n = lane & 31, g = lane >> 5;
    const int rh = w & 1, kh = w >> 1;
    const int G = A.QH / A.KVH, TPW = A.tpw;
    const int r = rh * 32 + n, rt = r / G;
    const int tq = qt * TPW + rt;
    const int head = kvh * G + (r - rt * G);
    const bool row_live = rt < TPW && tq < A.M;
    const int len = row_live ? (A.seq_lens ? A.seq_lens[tq] : A.pos_start + tq + 1) : 0;
    const int vis = row_live ? min(len, A.shared) : 0x7fffffff;      // an idle row multiplies zeros and masks nothing

    uint4 qf[NKS];
    {
        const uint8_t *qrow = A.q + ((size_t)tq * A.QH + head) * (D * 2) + g * 16;
#pragma unroll
        for (int ks = 0; ks < NKS; ks++) {
            uint4 v = row_live ? *(const uint4 *)(qrow + ks * 32) : make_uint4(0, 0, 0, 0);
#if defined(__HIP_DEVICE_COMPILE__)
            if constexpr (IO == DRK_BF16 && DT == DRK_F16) {      // 8-bit pages multiply in fp16
                v.x = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.x), bf16_hi(v.x)));
                v.y = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.y), bf16_hi(v.y)));
                v.z = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.z), bf16_hi(v.z)));
                v.w = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(bf16_lo(v.w), bf16_hi(v.w)));
            }
#endif
            qf[ks] = v;
        }
    }
    pf_f32x16 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    __syncthreads();
#pragma unroll 1
    for (int i = 0; i < nt; i++) {
        const int slot = i & 1;
        const int tile_t = (t_begin + i) * kPfBN + kh * 32;  // first token of this wave's key half
        // Every operand of the step is requested first -- one wave per SIMD multiplies, so nothing else would
        // hide the LDS latency: 8 reads of K and 16 of V, then the products.  S^T = K Q^T in two chains of four
        // (even and odd k-steps); register i4 of a lane is token tile_t + 8 (i4 / 4) + 4 g + i4 % 4.
        uint4 ka4[NKS];
        uint2 vlo[2][NDT], vhi[2][NDT];
        {
            const uint8_t *ka = &k_lds2[slot][0] + (kh * 32 + n) * kPitchK + g * 16;
#pragma unroll
            for (int ks = 0; ks < NKS; ks++) ka4[ks] = *(const uint4 *)(ka + ks * 32);
            const int j16 = lane & 15;
            const int dsub = 16 * ((lane >> 4) & 1) + 4 * (j16 & 3);
            const uint8_t *vb = &v_lds2[slot][0] + (kh * 32 + 4 * g + (j16 >> 2)) * kPitchV + dsub * 2;
#pragma unroll
            for (int mh = 0; mh < 2; mh++)
#pragma unroll
                for (int dt = 0; dt < NDT; dt++) {
                    vlo[mh][dt] = lds_read_tr16(vb + 16 * mh * kPitchV + dt * 64);
                    vhi[mh][dt] = lds_read_tr16(vb + (16 * mh + 8) * kPitchV + dt * 64);
                }
        }
        pf_f32x16 s;
        {
            const pf_f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            pf_f32x16 s1;
            s = mfma32<DT>(ka4[0], qf[0], zero);
            s1 = mfma32<DT>(ka4[1], qf[1], zero);
#pragma unroll
            for (int ks = 2; ks < NKS; ks += 2) {
                s = mfma32<DT>(ka4[ks], qf[ks], s);
                s1 = mfma32<DT>(ka4[ks + 1], qf[ks + 1], s1);
            }
#pragma unroll
            for (int i4 = 0; i4 < 16; i4++) s[i4] += s1[i4];
        }
        const int runs = runs_lds[slot][2 * kh] | (runs_lds[slot][2 * kh + 1] << 1);   // the two runs of this key half
        if (runs != 3 || __any(tile_t + 32 > vis)) {
#pragma unroll
            for (int i4 = 0; i4 < 16; i4++) {
                const int tl = 8 * (i4 >> 2) + 4 * g + (i4 & 3);
                const bool ok = (tile_t + tl) < vis && ((runs >> (tl >> 4)) & 1) != 0;
                s[i4] = ok ? s[i4] : -INFINITY;
            }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int i4 = 0; i4 < 16; i4++) tmax = fmaxf(tmax, s[i4]);
        tmax = pf_max_halves(tmax);
        const float m_new = fmaxf(m_run, tmax * A.scale_log2e);
        const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
        float pr[16];
#pragma unroll
        for (int i4 = 0; i4 < 16; i4++) pr[i4] = __builtin_amdgcn_exp2f(fmaf(s[i4], A.scale_log2e, -m_use));
        uint4 pb[2];                                         // [16-token half]: the B operand of PV
        pb[0] = make_uint4(pack2<DT>(pr[0], pr[1]), pack2<DT>(pr[2], pr[3]), pack2<DT>(pr[4], pr[5]), pack2<DT>(pr[6], pr[7]));
        pb[1] = make_uint4(pack2<DT>(pr[8], pr[9]), pack2<DT>(pr[10], pr[11]), pack2<DT>(pr[12], pr[13]), pack2<DT>(pr[14], pr[15]));
        float psum = pf_sum2<DT>(pb[0], 0.0f);               // the row sum is taken over the rounded weights
        psum = pf_sum2<DT>(pb[1], psum);
        l_run = l_run * alpha + psum;
        m_run = m_new;
        if (!__all(alpha == 1.0f)) {
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int i4 = 0; i4 < 16; i4++) o[dt][i4] *= alpha;
        }
        // O^T += V^T P^T over this wave's 32 tokens
#pragma unroll
        for (int mh = 0; mh < 2; mh++)
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
                o[dt] = mfma32<DT>(make_uint4(vlo[mh][dt].x, vlo[mh][dt].y, vhi[mh][dt].x, vhi[mh][dt].y), pb[mh], o[dt]);
        __syncthreads();
    }

    // fold the two key halves of every row: the waves of the second half leave theirs in LDS (the tiles are done)
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    float *xo = (float *)&k_lds2[0][0];                      // [dt * 16 + i4][rh][lane]: 32 KB
    float *xm = (float *)&v_lds2[0][0];                      // [rh][lane], then l
    if (kh == 1) {
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int i4 = 0; i4 < 16; i4++) xo[((dt * 16 + i4) * 2 + rh) * 64 + lane] = o[dt][i4];
        xm[rh * 64 + lane] = m_run;
        xm[128 + rh * 64 + lane] = l_tot;
    }
    __syncthreads();
    if (kh == 0 && row_live) {
        const float m1 = xm[rh * 64 + lane], l1 = xm[128 + rh * 64 + lane];
        const float m = fmaxf(m_run, m1);
        const float m_use = (m == -INFINITY) ? 0.0f : m;
        const float a0 = __builtin_amdgcn_exp2f(m_run - m_use), a1 = __builtin_amdgcn_exp2f(m1 - m_use);
        const size_t pi = ((size_t)tq * A.QH + head) * A.nsplits + blockIdx.z;
        float *orow = A.part_o + pi * D;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int b4 = 0; b4 < 4; b4++) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; e++)
                    v[e] = o[dt][4 * b4 + e] * a0 + xo[((dt * 16 + 4 * b4 + e) * 2 + rh) * 64 + lane] * a1;
                *(float4 *)(orow + dt * 32 + 8 * b4 + 4 * g) = make_float4(v[0], v[1], v[2], v[3]);
            }
        if (g == 0) {
            A.part_m[pi] = m;
            A.part_l[pi] = l_tot * a0 + l1 * a1;
        }
    }
}

// ---- shared-prefix ("cascade") decode: host side of the prefix pass -------------------
// One launch covers tokens [0, shared) for all B branches; the private tails go
// through the stream kernel with start_tile = shared / 64.
int g_shared_splits = 64;              // context splits of the prefix pass: 8 kv heads x 64 = two workgroups per CU
int g_prefix_stream = 1;               // few rows: the producer / consumer kernel (0: the kernel every wave stages in)
int g_prefix_stream_wgs = 256;         // ... with this many workgroups in all: one per CU

// the producer / consumer pass takes head_dim 128 and at most 64 rows per kv head (branches x query heads)
static bool prefix_stream_applies(const Lay &a, int B)
{
    const int G = a.QH / a.KVH;
    return g_prefix_stream && a.D == 128 && G >= 1 && G <= 64 && B * G <= 64;
}

void shared_prefix_shape(const Lay &a, int B, int shared, int *chunk_tiles, int *nsplits)
{
    const int tiles = shared / kPfBN;
    int target = g_shared_splits;
    if (prefix_stream_applies(a, B)) {
        target = g_prefix_stream_wgs / a.KVH;
        if (target < 1) target = 1;
        if (target > g_shared_splits) target = g_shared_splits;      // workspaces are sized for at most that many pieces
    }
    int ns = tiles < target ? tiles : target;
    if (ns < 1) ns = 1;
    *chunk_tiles = (tiles + ns - 1) / ns;
    if (*chunk_tiles < 1) *chunk_tiles = 1;
    *nsplits = (tiles + *chunk_tiles - 1) / *chunk_tiles;
    if (*nsplits < 1) *nsplits = 1;
}

int launch_shared_prefix(const Lay &a, const void *q, const void *pool, const int32_t *table0,
                         const int32_t *d_seq_lens, int B, int shared, int layer, float scale, int io_dtype,
                         float *part_o, float *part_m, float *part_l, hipStream_t st, int chunk_tiles, int nsplits,
                         int causal_pos_start)
{
    PrefillArgs A;
    A.pool_layer = (const uint8_t *)pool + (size_t)layer * a.layer_stride;
    A.table = table0;
    A.q = (const uint8_t *)q;
    A.out = nullptr;
    A.pos_start = causal_pos_start; A.M = B; A.QH = a.QH; A.KVH = a.KVH; A.NB = a.NB; A.bs = a.bs; A.tpw = 128 / (a.QH / a.KVH);
    A.bs_shift = ilog2_exact((unsigned)a.bs);
    A.head_stride = a.head_stride; A.kv_plane = a.kv_plane; A.block_stride = a.block_stride; A.scale_plane = a.scale_plane;
    A.scale_log2e = scale * kLog2eP;
    A.seq_lens = d_seq_lens; A.shared = shared;
    if (nsplits > 0) { A.chunk_tiles = chunk_tiles; A.nsplits = nsplits; }      // the caller's split (shared need not be whole tiles)
    else shared_prefix_shape(a, B, shared, &A.chunk_tiles, &A.nsplits);
    A.part_o = part_o; A.part_m = part_m; A.part_l = part_l;
    A.gate = nullptr; A.gate_stride = 0;
    A.lse_rows = nullptr;
    if (nsplits <= 0 && prefix_stream_applies(a, B)) {
        A.tpw = 64 / (a.QH / a.KVH);
        dim3 grid2(((B + A.tpw - 1) / A.tpw) * a.KVH, 1, A.nsplits);
#define DRK_PS(DT, KV, IO) hipLaunchKernelGGL((prefix_stream_kernel<DT, KV, IO>), grid2, dim3(512), 0, st, A)
        if (a.dtype == DRK_BF16) DRK_PS(DRK_BF16, DRK_BF16, DRK_BF16);
        else if (a.dtype == DRK_F16) DRK_PS(DRK_F16, DRK_F16, DRK_F16);
        else if (a.dtype == DRK_INT8 && io_dtype == DRK_BF16) DRK_PS(DRK_F16, DRK_INT8, DRK_BF16);
        else if (a.dtype == DRK_INT8) DRK_PS(DRK_F16, DRK_INT8, DRK_F16);
        else if (io_dtype == DRK_BF16) DRK_PS(DRK_F16, DRK_FP8_E4M3, DRK_BF16);
        else DRK_PS(DRK_F16, DRK_FP8_E4M3, DRK_F16);
#undef DRK_PS
        DRK_LAUNCH_CHECK("prefix_stream_kernel");
        return DRK_OK;
    }
    dim3 grid(((B + A.tpw - 1) / A.tpw) * a.KVH, 1, A.nsplits);
#define DRK_PF_SHARED(DT, KV, IO)                                                                                        \
    do {                                                                                                                \
        if (a.D == 128) hipLaunchKernelGGL((prefill_mfma_kernel<DT, true, KV, IO, 128>), grid, dim3(256), 0, st, A);    \
        else hipLaunchKernelGGL((prefill_mfma_kernel<DT, true, KV, IO, 256>), grid, dim3(256), 0, st, A);               \
    } while (0)
    if (a.dtype == DRK_BF16) DRK_PF_SHARED(DRK_BF16, DRK_BF16, DRK_BF16);
    else if (a.dtype == DRK_F16) DRK_PF_SHARED(DRK_F16, DRK_F16, DRK_F16);
    else if (a.dtype == DRK_INT8 && io_dtype == DRK_BF16) DRK_PF_SHARED(DRK_F16, DRK_INT8, DRK_BF16);
    else if (a.dtype == DRK_INT8) DRK_PF_SHARED(DRK_F16, DRK_INT8, DRK_F16);
    else if (io_dtype == DRK_BF16) DRK_PF_SHARED(DRK_F16, DRK_FP8_E4M3, DRK_BF16);
    else DRK_PF_SHARED(DRK_F16, DRK_FP8_E4M3, DRK_F16);
#undef DRK_PF_SHARED
    DRK_LAUNCH_CHECK("prefill_mfma_kernel<shared>");
    return DRK_OK;
}

// ---- short chunks behind a long context ------------------------------------------------
// The chunk kernel walks the whole context in every workgroup and has ceil(M / TPW) x KVH of
// them: a chunk of a few tokens behind 32k tokens keeps 8 of 256 CUs busy for a millisecond.
// Such a chunk is the shared-prefix pass over again -- row t is a "branch" of length
// pos_start + t + 1, all rows read one table -- so the kernel runs in that mode over tokens
// [0, pos_start + M) with the context split over the whole chip, and a small kernel folds each
// row's pieces (and applies the gate).
int g_prefill_two_phase = 1;                   // 0: never; 1: by the rule in prefill_impl; 2: whenever the geometry allows (tests); 3: as 2, with register staging also for 16-bit pages
int g_prefill_d256_waves = 1;                  // head_dim 256 chunk kernel: 0 one wave per SIMD does both products, 1 a score wave and a value wave per SIMD
int g_prefill_mass_direct = 1;                 // one-walk mass pass over 16-bit pages: 1 the kernel that takes tiles straight into LDS, 0 the register-staging kernel
int g_prefill_mass_parts = 0;                  // that kernel's parts per walk: 0 by its rule, n > 0 forced (tests)
int g_prefill_pieces = 1;                      // head_dim 256, pieces for the walks of the last round: 0 never, 1 when they are worth it, 2 whenever there are any (tests)
int g_prefill_split = -1;                      // -1: by the rule below; 0: never; n > 0: every chunk of up to n rows (tests)
constexpr int kSplitMinPos = 2048, kSplitMaxM = 1024, kSplitMaxPieces = 128;

// grid = rows (query token x query head), block = 64: lane s owns the (m, l) of piece s (at most 128
// pieces: two per lane), so the weights come in one round of loads; then the lanes own dims
// [l VEC, l VEC + VEC) and fold the o rows eight at a time.  Pieces are unnormalised (o, m, l) in the
// base-2 exponent domain; an empty piece carries l = 0 and may hold anything else.
__device__ __forceinline__ float pm_lane(float v, int l)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
#else
    (void)l;
    return v;
#endif
}

template <int D>
__global__ __launch_bounds__(64) void prefill_merge_kernel(const float *__restrict__ part_o, const float *__restrict__ part_m,
                                                           const float *__restrict__ part_l, uint16_t *__restrict__ out,
                                                           int nsplits, int io_dtype, const uint16_t *__restrict__ gate,
                                                           size_t gate_stride, float *__restrict__ lse_rows)
{
    constexpr int VEC = D / 64;
    typedef float fvec __attribute__((ext_vector_type(VEC)));
    const size_t row = blockIdx.x;
    const int lane = threadIdx.x, d = lane * VEC;
    float pm[2], pl[2], w[2];
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const int sidx = lane + 64 * r;
        pl[r] = sidx < nsplits ? part_l[row * nsplits + sidx] : 0.0f;
        pm[r] = sidx < nsplits ? part_m[row * nsplits + sidx] : -INFINITY;
    }
    float M = fmaxf(pl[0] > 0.0f ? pm[0] : -INFINITY, pl[1] > 0.0f ? pm[1] : -INFINITY);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off));
    float L = 0.0f;
#pragma unroll
    for (int r = 0; r < 2; r++) {
        w[r] = pl[r] > 0.0f ? __builtin_amdgcn_exp2f(pm[r] - M) : 0.0f;
        L = fmaf(pl[r], w[r], L);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) L += __shfl_xor(L, off);
    if (lse_rows && lane == 0) lse_rows[row] = L > 0.0f ? M + __builtin_log2f(L) : INFINITY;
    fvec acc = {};
    const float *obase = part_o + row * nsplits * D + d;
    for (int j = 0; j < nsplits; j += 8) {
        fvec o[8];
        float wj[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int sj = min(j + u, nsplits - 1);
            const float ws = sj < 64 ? pm_lane(w[0], sj) : pm_lane(w[1], sj - 64);
            wj[u] = j + u < nsplits ? ws : 0.0f;
            o[u] = *(const fvec *)(obase + (size_t)sj * D);
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (wj[u] != 0.0f) {
#pragma unroll
                for (int x = 0; x < VEC; x++) acc[x] = fmaf(o[u][x], wj[u], acc[x]);
            }
    }
    // with a gate the row is always rewritten: the reference gates whatever the attention kernel
    // left in out, also when no token took part (paged_attention.cu:551, 633-634)
    uint16_t *dst = out + row * D + d;
    uint16_t vals[VEC];
    if (L > 0.0f) {
#pragma unroll
        for (int x = 0; x < VEC; x++) vals[x] = f_to_elem16(acc[x] / L, io_dtype);
    } else {
        if (!gate) return;
#pragma unroll
        for (int x = 0; x < VEC; x++) vals[x] = dst[x];
    }
    if (gate) {
        const uint16_t *gp = gate + row * gate_stride + d;
#pragma unroll
        for (int x = 0; x < VEC; x++) vals[x] = gated_elem16(vals[x], gp[x], io_dtype);
    }
#pragma unroll
    for (int x = 0; x < VEC; x++) dst[x] = vals[x];
}

// ---- head_dim 256: walks beyond a whole number of rounds are cut into pieces --------------------------
// prefill_d256_kernel holds one workgroup per CU, so W walks of about equal length take ceil(W / 256) rounds
// however few workgroups the last round has.  The walks of that last round (the shortest: they are dispatched
// last) are cut into k = floor(256 / their number) pieces each, which still fit one round and take a k-th of
// the time; their rows are then folded from the pieces by prefill_piece_merge_kernel.  gh query heads per
// workgroup (the largest divisor of the heads per kv head that divides 128), so that no row of a workgroup idles.
constexpr int kD256MaxPieces = 32;                  // per walk: the merge gives a piece a lane of half a wave
struct D256Shape { int gh, tpw, nqt, walks, n_full, tail, kparts; };
static D256Shape d256_shape(const Lay &a, int pos_start, int M, int pieces)      // pieces: 0 none, 1 by the rule, 2 whenever a last round exists
{
    D256Shape s;
    const int G = a.QH / a.KVH;
    s.gh = 1;
    for (int d = 1; d <= G && d <= 128; d++)
        if (G % d == 0 && 128 % d == 0) s.gh = d;
    s.tpw = 128 / s.gh;
    s.nqt = (M + s.tpw - 1) / s.tpw;
    s.walks = s.nqt * a.KVH * (G / s.gh);
    s.tail = s.walks % 256;
    s.kparts = (pieces && s.tail > 0) ? 256 / s.tail : 1;
    if (s.kparts > kD256MaxPieces) s.kparts = kD256MaxPieces;
    // a piece should be worth its start-up and the merge: eight tiles or more of the longest walk that is cut
    // (the last round holds the shortest walks: the first row blocks of the chunk)
    const int qt_tail = s.nqt - 1 - (s.walks - s.tail) / (a.KVH * (G / s.gh));
    const int rows_to = (qt_tail + 1) * s.tpw < M ? (qt_tail + 1) * s.tpw : M;
    const int tiles = (pos_start + rows_to + kPfBN - 1) / kPfBN;
    if (pieces == 1 && s.kparts > tiles / 8) s.kparts = tiles / 8;
    if (s.kparts < 2) { s.kparts = 1; s.tail = 0; }
    s.n_full = s.walks - s.tail;
    return s;
}
static size_t d256_pieces_need(const D256Shape &s) { return (size_t)s.tail * 128 * s.kparts * (256 + 2) * sizeof(float); }

// grid = tail walks x 128 rows, block = 64: the row's pieces (at most 8) folded as in prefill_merge_kernel
__global__ __launch_bounds__(64) void prefill_piece_merge_kernel(PrefillArgs A, int io_dtype)
{
    constexpr int D = 256, VEC = 4;
    typedef float fvec __attribute__((ext_vector_type(VEC)));
    const int walk = A.n_full + (int)blockIdx.x / 128, r = (int)blockIdx.x % 128;
    const int lane = threadIdx.x, d = lane * VEC;
    const int G = A.QH / A.KVH, GH = A.gh, NHG = G / GH;
    const int kvh = walk % A.KVH, hg = (walk / A.KVH) % NHG, qt = A.nqt - 1 - walk / (A.KVH * NHG);
    const int rt = r / GH, tq = qt * A.tpw + rt;
    if (rt >= A.tpw || tq >= A.M) return;
    const size_t row = (size_t)tq * A.QH + kvh * G + hg * GH + (r - rt * GH);
    const size_t p0 = (size_t)blockIdx.x * A.kparts;
    const float pl = lane < A.kparts ? A.part_l[p0 + lane] : 0.0f;
    const float pm = (lane < A.kparts && pl > 0.0f) ? A.part_m[p0 + lane] : -INFINITY;
    float M = pm;
#pragma unroll
    for (int off = kD256MaxPieces / 2; off > 0; off >>= 1) M = fmaxf(M, __shfl_xor(M, off));
    const float w = pl > 0.0f ? __builtin_amdgcn_exp2f(pm - M) : 0.0f;
    float L = pl * w;
#pragma unroll
    for (int off = kD256MaxPieces / 2; off > 0; off >>= 1) L += __shfl_xor(L, off);
    M = pm_lane(M, 0);
    L = pm_lane(L, 0);
    if (A.lse_rows && lane == 0) A.lse_rows[row] = L > 0.0f ? M + __builtin_log2f(L) : INFINITY;
    fvec acc = {};
    for (int j = 0; j < A.kparts; j++) {
        const float wj = pm_lane(w, j);
        if (wj != 0.0f) {                                    // an empty piece may hold anything
            const fvec o = *(const fvec *)(A.part_o + (p0 + j) * D + d);
#pragma unroll
            for (int x = 0; x < VEC; x++) acc[x] = fmaf(o[x], wj, acc[x]);
        }
    }
    uint16_t *dst = (uint16_t *)A.out + row * D + d;
    uint16_t vals[VEC];
    if (L > 0.0f) {
#pragma unroll
        for (int x = 0; x < VEC; x++) vals[x] = f_to_elem16(acc[x] / L, io_dtype);
    } else {
        if (!A.gate) return;
#pragma unroll
        for (int x = 0; x < VEC; x++) vals[x] = dst[x];
    }
    if (A.gate) {
        const uint16_t *gp = A.gate + row * A.gate_stride + d;
#pragma unroll
        for (int x = 0; x < VEC; x++) vals[x] = gated_elem16(vals[x], gp[x], io_dtype);
    }
    *(uint2 *)dst = make_uint2((uint32_t)vals[0] | ((uint32_t)vals[1] << 16), (uint32_t)vals[2] | ((uint32_t)vals[3] << 16));
}

// context splits: two workgroups per CU over the whole grid -- one resident round -- of whole tiles each
static void prefill_split_shape(const Lay &a, int pos_start, int M, int *chunk_tiles, int *nsplits)
{
    const int tpw = 128 / (a.QH / a.KVH);
    const int per_split = ((M + tpw - 1) / tpw) * a.KVH;
    const int tiles = (pos_start + M + kPfBN - 1) / kPfBN;
    int ns = (512 + per_split - 1) / per_split;
    if (ns > kSplitMaxPieces) ns = kSplitMaxPieces;
    if (ns > tiles) ns = tiles;
    if (ns < 1) ns = 1;
    *chunk_tiles = (tiles + ns - 1) / ns;
    *nsplits = (tiles + *chunk_tiles - 1) / *chunk_tiles;
}

// When it pays (measured, 32 Q / 8 KV x 128 bf16): the chunk kernel takes 27 us per 1 024 tokens of
// context whatever the chunk length up to 1 024 rows (one workgroup per CU at most); the split pass
// keeps every CU busy.  Rows behind 2k / 32k / 128k tokens, chunk kernel -> split:
//   16: 59 -> 18, 878 -> 42, 3 992 -> 115 us;  256: 66 -> 37, 868 -> 211, 3 857 -> 799 us;
//   1 024: 92 -> 98, 928 -> 715, 3 896 -> 2 566 us.
// (with the two-phase kernels walking their context in parts, prefill_split_ppd_parts, behind 32k tokens: 64 rows 70 -> 55,
// 256 rows 211 -> 141, 1 024 rows 715 -> 487 us; int8 pages 64 rows 81 -> 60, 256 rows 242 -> 168 us)
static bool d256_direct(const Lay &a);
static int prefill_split_ppd_parts(const Lay &a, int pos_start, int M);
static bool prefill_split_applies(const Lay &a, int pos_start, int M)
{
    if (g_prefill_split == 0 || pos_start < kSplitMinPos) return false;
    if (g_prefill_split > 0) return M <= g_prefill_split;
    // head_dim 256 on 16-bit pages: the chunk kernel cuts its walks into up to 32 pieces each and fills the chip that
    // way, faster than this path's kernel at every chunk length (16 rows behind 32k tokens 69 against 73 us, 256 rows
    // 210 against 596, 1 024 rows 895 against 1 993)
    if (d256_direct(a) && g_prefill_pieces != 0) return false;
    return M <= 512 || (M <= kSplitMaxM && pos_start >= 2 * kSplitMinPos);
}

// head_dim 256 on 16-bit pages takes prefill_d256_kernel (tiles straight into LDS)
static bool d256_direct(const Lay &a)
{
    return a.D == 256 && (a.dtype == DRK_BF16 || a.dtype == DRK_F16) && a.bs >= 16 && ilog2_exact((unsigned)a.bs) >= 4 &&
           g_prefill_two_phase != 0 && g_prefill_two_phase != 3;
}

// Whether the chunk kernel that prefill_impl takes for this chunk folds the softmax scale into Q (rounded to the
// 16-bit type): the two-phase kernels and the head_dim 256 kernels do, the four-wave kernel and the split path
// (taken when the caller passes its workspace) do not.  The mass pass scores the way the attention call did.
static bool chunk_kernel_scales_q(const Lay &a, int pos_start, int M)
{
    if (prefill_split_applies(a, pos_start, M)) return prefill_split_ppd_parts(a, pos_start, M) != 0;
    if (d256_direct(a)) return true;
    const int G = a.QH / a.KVH;
    if (a.D == 128 && G <= 256 && a.bs >= 16 && ilog2_exact((unsigned)a.bs) >= 4 && g_prefill_two_phase != 0) {
        const int tpw2 = 256 / G;
        const long wgs2 = (long)((M + tpw2 - 1) / tpw2) * a.KVH;
        return wgs2 >= 192 || g_prefill_two_phase > 1;
    }
    return false;
}

// A chunk at head_dim 128 with at least 256 rows per kv head takes the two-phase kernels on that path
// too: every walk in parts, one workgroup per CU, the same (o, m, l) pieces and the same merge.  Returns the number of
// parts per walk (never more than the pieces the workspace was sized for), or 0 for the four-wave kernel.
static int prefill_split_ppd_parts(const Lay &a, int pos_start, int M)
{
    if (!(a.D == 128 && a.bs >= 16 && ilog2_exact((unsigned)a.bs) >= 4)) return 0;
    if (g_prefill_two_phase == 0) return 0;
    const int G = a.QH / a.KVH;
    if (G > 256 || (long)M * G < 256) return 0;
    const int tpw2 = 256 / G;
    const long walks = (long)((M + tpw2 - 1) / tpw2) * a.KVH;
    int ct, ns;
    prefill_split_shape(a, pos_start, M, &ct, &ns);
    const int shortest = (pos_start + 1 + kPfBN - 1) / kPfBN;          // tiles of the first row block's walk, at least
    long kp = 256 / walks;
    if (kp > shortest / 8) kp = shortest / 8;
    if (kp > ns) kp = ns;
    return kp >= 2 ? (int)kp : 0;
}

static size_t prefill_split_need(const Lay &a, int pos_start, int M)
{
    int ct, ns;
    prefill_split_shape(a, pos_start, M, &ct, &ns);
    return (size_t)M * a.QH * ns * (a.D + 2) * sizeof(float);
}

static int prefill_split(const Lay &a, const void *q, const void *pool, const int32_t *table, void *out, int layer,
                         int pos_start, int M, float scale, int io_dtype, void *workspace, hipStream_t st,
                         const void *gate, size_t gate_stride, float *lse_rows)
{
    int ct, ns;
    prefill_split_shape(a, pos_start, M, &ct, &ns);
    float *part_o = (float *)workspace;
    float *part_m = part_o + (size_t)M * a.QH * ns * a.D;
    float *part_l = part_m + (size_t)M * a.QH * ns;
    int rc = launch_shared_prefix(a, q, pool, table, nullptr, M, pos_start + M, layer, scale, io_dtype, part_o, part_m, part_l, st,
                                  ct, ns, pos_start);
    if (rc) return rc;
    const dim3 grid((unsigned)((size_t)M * a.QH));
    if (a.D == 128)
        hipLaunchKernelGGL(prefill_merge_kernel<128>, grid, dim3(64), 0, st, part_o, part_m, part_l, (uint16_t *)out, ns, io_dtype,
                           (const uint16_t *)gate, gate_stride, lse_rows);
    else
        hipLaunchKernelGGL(prefill_merge_kernel<256>, grid, dim3(64), 0, st, part_o, part_m, part_l, (uint16_t *)out, ns, io_dtype,
                           (const uint16_t *)gate, gate_stride, lse_rows);
    DRK_LAUNCH_CHECK("prefill_merge_kernel");
    return DRK_OK;
}

} // namespace drk

using namespace drk;

extern "C" {

void drk_debug_set_prefill_split(int max_rows) { g_prefill_split = max_rows < 0 ? -1 : max_rows; }
void drk_debug_set_prefill_d256_waves(int mode) { g_prefill_d256_waves = mode != 0 ? 1 : 0; }
void drk_debug_set_prefill_mass_direct(int on) { g_prefill_mass_direct = on != 0 ? 1 : 0; }
void drk_debug_set_prefill_mass_parts(int parts) { g_prefill_mass_parts = parts < 0 ? 0 : (parts > 4096 ? 4096 : parts); }
void drk_debug_set_prefill_pieces(int mode) { g_prefill_pieces = mode < 0 ? 1 : (mode > 2 ? 2 : mode); }
static int prefill_mass_impl(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *d_block_table,
                             int layer, int pos_start, int M, float scale, int io_dtype, const float *d_row_lse,
                             float *d_block_mass, int mass_len, int accumulate, void *stream)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    if (pos_start < 0 || M < 0 || mass_len < 0) return fail(DRK_ERR_INVALID, "prefill_mass: negative pos_start, M or mass_len");
    if (!q || !pool || !d_block_table || !d_block_mass) return fail(DRK_ERR_INVALID, "prefill_mass: NULL pointer");
    if (io_dtype != DRK_F16 && io_dtype != DRK_BF16) return fail(DRK_ERR_INVALID, "prefill_mass: io_dtype must be F16 or BF16");
    if ((a.dtype == DRK_F16 || a.dtype == DRK_BF16) && io_dtype != a.dtype)
        return fail(DRK_ERR_INVALID, "prefill_mass: io_dtype %d differs from the pool's %d", io_dtype, a.dtype);
    if (layer < 0 || layer >= a.L) return fail(DRK_ERR_INVALID, "prefill_mass: layer %d outside [0,%d)", layer, a.L);
    if (!((a.D == 128 || a.D == 256) && a.QH % a.KVH == 0 && a.QH / a.KVH <= 128 && (a.bs % 16) == 0 && scale > 0.0f))
        return fail(DRK_ERR_UNSUPPORTED, "prefill_mass: needs head_dim 128 or 256, at most 128 query heads per kv head, block_size %% 16 == 0, scale > 0");
    if (a.KVH > 65535) return fail(DRK_ERR_INVALID, "prefill_mass: more than 65535 kv heads");
    if (M > 0 && mass_len < (pos_start + M + a.bs - 1) / a.bs)
        return fail(DRK_ERR_INVALID, "prefill_mass: mass_len %d is less than the %d blocks of pos_start + M", mass_len,
                    (pos_start + M + a.bs - 1) / a.bs);
    hipStream_t st = (hipStream_t)stream;
    if (!accumulate && mass_len > 0) {
        hipLaunchKernelGGL(pf_zero_kernel, dim3((mass_len + 255) / 256), dim3(256), 0, st, d_block_mass, mass_len);
        DRK_LAUNCH_CHECK("pf_zero_kernel");
    }
    if (M == 0) return DRK_OK;
    PrefillArgs A;
    A.pool_layer = (const uint8_t *)pool + (size_t)layer * a.layer_stride;
    A.table = d_block_table;
    A.q = (const uint8_t *)q;
    A.out = nullptr;
    A.pos_start = pos_start; A.M = M; A.QH = a.QH; A.KVH = a.KVH; A.NB = a.NB; A.bs = a.bs;
    A.tpw = 128 / (a.QH / a.KVH);
    A.bs_shift = ilog2_exact((unsigned)a.bs);
    A.head_stride = a.head_stride; A.kv_plane = a.kv_plane; A.block_stride = a.block_stride; A.scale_plane = a.scale_plane;
    A.scale_log2e = scale * kLog2eP;
    A.seq_lens = nullptr; A.shared = 0; A.chunk_tiles = 0; A.nsplits = 0; A.part_o = A.part_m = A.part_l = nullptr;
    A.gate = nullptr; A.gate_stride = 0;
    A.lse_rows = const_cast<float *>(d_row_lse);             // read only here: the rows' log-sum-exps, or NULL (first walk finds them)
    // 16-bit pages: the kernel that takes its tiles straight into LDS -- one walk when the rows' log-sum-exps are
    // given, else two by the same workgroup (whole walks then: the first must see every key)
    // (the table of page sums in LDS holds the blocks of one part: a context of more blocks than it holds is cut into
    // parts for that reason alone -- which the two-walk call cannot do)
    const int massd_cap = (a.D == 128 ? kMassdBlocks<128> : kMassdBlocks<256>) - 8;      // a part's range is rounded to tiles and to blocks
    const int massd_min_parts = ((pos_start + M + a.bs - 1) / a.bs + massd_cap - 1) / massd_cap;
    const bool q8 = a.dtype == DRK_INT8 || a.dtype == DRK_FP8_E4M3;       // 8-bit pages: head_dim 128, the one-walk call
    if (g_prefill_mass_direct && (a.dtype == DRK_BF16 || a.dtype == DRK_F16 || (q8 && a.D == 128 && d_row_lse)) && A.bs_shift >= 4 &&
        (d_row_lse || massd_min_parts == 1) && a.QH / a.KVH <= 128) {
        A.tpw = 256 / (a.QH / a.KVH);
        A.nqt = (M + A.tpw - 1) / A.tpw;
        // few walks (a short chunk): every walk's tiles in parts, so that the workgroups fill the chip once (one
        // per CU: the LDS ring), a part no shorter than eight tiles
        const int walks = A.nqt * a.KVH;
        const int tiles = (pos_start + M + kPfBN - 1) / kPfBN;
        A.kparts = !d_row_lse ? 1 : std::max(massd_min_parts, g_prefill_mass_parts > 0 ? g_prefill_mass_parts
                                                                                        : std::max(1, std::min(256 / walks, tiles / 8)));
        A.gh = 0; A.n_full = 0;
        const dim3 gridd((unsigned)(walks * A.kparts));
        const int kind = !d_row_lse ? 2 : (chunk_kernel_scales_q(a, pos_start, M) ? 1 : 0);
#define DRK_PMD(DT, DD)                                                                                                   \
        do {                                                                                                             \
            if (kind == 2) hipLaunchKernelGGL((prefill_massd_kernel<DT, DT, DD, false, true>), gridd, dim3(512), 0, st, A, d_block_mass, mass_len);  \
            else if (kind == 1) hipLaunchKernelGGL((prefill_massd_kernel<DT, DT, DD, true, false>), gridd, dim3(512), 0, st, A, d_block_mass, mass_len);  \
            else hipLaunchKernelGGL((prefill_massd_kernel<DT, DT, DD, false, false>), gridd, dim3(512), 0, st, A, d_block_mass, mass_len);  \
        } while (0)
#define DRK_PMD8(KV, IO)                                                                                                  \
        do {                                                                                                             \
            if (kind == 1) hipLaunchKernelGGL((prefill_massd_kernel<DRK_F16, IO, 128, true, false, KV>), gridd, dim3(512), 0, st, A, d_block_mass, mass_len);  \
            else hipLaunchKernelGGL((prefill_massd_kernel<DRK_F16, IO, 128, false, false, KV>), gridd, dim3(512), 0, st, A, d_block_mass, mass_len);  \
        } while (0)
        if (a.dtype == DRK_INT8 && io_dtype == DRK_BF16) DRK_PMD8(DRK_INT8, DRK_BF16);
        else if (a.dtype == DRK_INT8) DRK_PMD8(DRK_INT8, DRK_F16);
        else if (a.dtype == DRK_FP8_E4M3 && io_dtype == DRK_BF16) DRK_PMD8(DRK_FP8_E4M3, DRK_BF16);
        else if (a.dtype == DRK_FP8_E4M3) DRK_PMD8(DRK_FP8_E4M3, DRK_F16);
        else if (a.dtype == DRK_BF16 && a.D == 128) DRK_PMD(DRK_BF16, 128);
        else if (a.dtype == DRK_BF16) DRK_PMD(DRK_BF16, 256);
        else if (a.D == 128) DRK_PMD(DRK_F16, 128);
        else DRK_PMD(DRK_F16, 256);
#undef DRK_PMD8
#undef DRK_PMD
        DRK_LAUNCH_CHECK("prefill_massd_kernel");
        return DRK_OK;
    }
    // few walks and the rows' log-sum-exps given: every walk's tiles in parts, about 512 workgroups (two per CU at
    // head_dim 128), a part no shorter than eight tiles
    A.gh = 0; A.nqt = 0; A.n_full = 0;
    {
        const int walks = ((M + A.tpw - 1) / A.tpw) * a.KVH;
        const int tiles = (pos_start + M + kPfBN - 1) / kPfBN;
        A.kparts = !d_row_lse ? 1 : (g_prefill_mass_parts > 0 ? g_prefill_mass_parts : std::max(1, std::min(512 / walks, tiles / 8)));
    }
    dim3 grid(((M + A.tpw - 1) / A.tpw) * a.KVH * A.kparts);
#define DRK_PM(DT, KV, IO)                                                                                                      \
    do {                                                                                                                       \
        if (a.D == 128) hipLaunchKernelGGL((prefill_mass_kernel<DT, KV, IO, 128>), grid, dim3(256), 0, st, A, d_block_mass, mass_len); \
        else hipLaunchKernelGGL((prefill_mass_kernel<DT, KV, IO, 256>), grid, dim3(256), 0, st, A, d_block_mass, mass_len);    \
    } while (0)
    if (a.dtype == DRK_BF16) DRK_PM(DRK_BF16, DRK_BF16, DRK_BF16);
    else if (a.dtype == DRK_F16) DRK_PM(DRK_F16, DRK_F16, DRK_F16);
    else if (a.dtype == DRK_INT8 && io_dtype == DRK_BF16) DRK_PM(DRK_F16, DRK_INT8, DRK_BF16);
    else if (a.dtype == DRK_INT8) DRK_PM(DRK_F16, DRK_INT8, DRK_F16);
    else if (io_dtype == DRK_BF16) DRK_PM(DRK_F16, DRK_FP8_E4M3, DRK_BF16);
    else DRK_PM(DRK_F16, DRK_FP8_E4M3, DRK_F16);
#undef DRK_PM
    DRK_LAUNCH_CHECK("prefill_mass_kernel");
    return DRK_OK;
}

int drk_paged_prefill_attention_mass(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *d_block_table,
                                     int layer, int pos_start, int M, float scale, int io_dtype, float *d_block_mass,
                                     int mass_len, int accumulate, void *stream)
{
    return prefill_mass_impl(g, q, pool, d_block_table, layer, pos_start, M, scale, io_dtype, nullptr, d_block_mass, mass_len,
                             accumulate, stream);
}

int drk_paged_prefill_attention_mass_lse(const drk_kv_layout *g, const void *q, const void *pool,
                                         const int32_t *d_block_table, int layer, int pos_start, int M, float scale,
                                         int io_dtype, const float *d_row_lse, float *d_block_mass, int mass_len,
                                         int accumulate, void *stream)
{
    if (!d_row_lse) return fail(DRK_ERR_INVALID, "prefill_mass: d_row_lse is NULL");
    return prefill_mass_impl(g, q, pool, d_block_table, layer, pos_start, M, scale, io_dtype, d_row_lse, d_block_mass, mass_len,
                             accumulate, stream);
}

void drk_debug_set_prefill_two_phase(int mode) { g_prefill_two_phase = mode < 0 ? 1 : (mode > 3 ? 3 : mode); }

size_t drk_prefill_workspace_bytes(const drk_kv_layout *g, int pos_start, int M)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK || M <= 0 || pos_start < 0) return 0;
    const bool mfma = !g_force_portable && (a.D == 128 || a.D == 256) && a.QH % a.KVH == 0 && a.QH / a.KVH <= 128 &&
                      (a.bs % 16) == 0;
    if (mfma) {
        if (prefill_split_applies(a, pos_start, M)) return prefill_split_need(a, pos_start, M);
        if (d256_direct(a) && g_prefill_pieces) return d256_pieces_need(d256_shape(a, pos_start, M, g_prefill_pieces));
        return 0;
    }
    return drk_decode_workspace_bytes(g, M, pos_start + M);
}

size_t drk_prefill_workspace_bytes_max(const drk_kv_layout *g, int max_seq_len, int max_rows)
{
    Lay a;
    if (make_lay(g, &a) != DRK_OK || max_seq_len <= 0 || max_rows <= 0) return 0;
    if (max_rows > max_seq_len) max_rows = max_seq_len;
    const bool mfma = !g_force_portable && (a.D == 128 || a.D == 256) && a.QH % a.KVH == 0 && a.QH / a.KVH <= 128 &&
                      (a.bs % 16) == 0;
    if (!mfma) return drk_decode_workspace_bytes(g, max_rows, max_seq_len);
    // the pieces per row grow with the context: the chunk that ends at max_seq_len needs the most for its length
    size_t need = 0;
    // (the debug switch drk_debug_set_prefill_split(n) lets chunks of up to n rows take the split path)
    const int widest = g_prefill_split > kSplitMaxM ? g_prefill_split : kSplitMaxM;
    const int top = max_rows < widest ? max_rows : widest;
    for (int M = 1; M <= top; M++) {
        const size_t n = drk_prefill_workspace_bytes(g, max_seq_len - M, M);
        if (n > need) need = n;
    }
    if (d256_direct(a) && g_prefill_pieces) {
        // the pieces of the last round's walks: at most 256 pieces of 128 rows whatever the chunk's length
        const size_t n = (size_t)256 * 128 * (256 + 2) * sizeof(float);
        if (n > need) need = n;
    }
    return need;
}

// paged_prefill_attention_kernel, paged_attention.cu:465-554, 621-630.
// head_dim 128 or 256, block_size a multiple of 16: the MFMA kernel above (no workspace; any
// group size; 8-bit pages are dequantised on their way into LDS).  Anything else: row t of the
// chunk runs as one causal "branch" of the portable decode kernel -- the reference's algorithm
// verbatim (paged_attention.cu:481, 506-549) -- and needs the workspace.
static int prefill_impl(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *d_block_table,
                        void *out, int layer, int pos_start, int M, float scale, int io_dtype, void *workspace,
                        size_t workspace_bytes, void *stream, const void *gate, size_t gate_stride, float *lse_rows = nullptr)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    if (pos_start < 0 || M < 0) return fail(DRK_ERR_INVALID, "prefill: negative pos_start or M");
    if (M == 0) return DRK_OK;
    if (!q || !pool || !d_block_table || !out) return fail(DRK_ERR_INVALID, "prefill: NULL pointer");
    if (io_dtype != DRK_F16 && io_dtype != DRK_BF16) return fail(DRK_ERR_INVALID, "prefill: io_dtype must be F16 or BF16");
    if ((a.dtype == DRK_F16 || a.dtype == DRK_BF16) && io_dtype != a.dtype)
        return fail(DRK_ERR_INVALID, "prefill: io_dtype %d differs from the pool's %d", io_dtype, a.dtype);
    if (layer < 0 || layer >= a.L) return fail(DRK_ERR_INVALID, "prefill: layer %d outside [0,%d)", layer, a.L);
    // the MFMA kernels fold the scale into the exponent's base-2 factor and assume it positive; a softmax scale
    // is 1/sqrt(head_dim) or close to it
    if (!(scale > 0.0f)) return fail(DRK_ERR_INVALID, "prefill: scale must be positive (got %g)", (double)scale);

    const bool mfma = !g_force_portable && (a.D == 128 || a.D == 256) && a.QH % a.KVH == 0 &&
                      a.QH / a.KVH <= 128 && (a.bs % 16) == 0;
    if (!mfma && lse_rows)
        return fail(DRK_ERR_UNSUPPORTED, "prefill: row log-sum-exps need head_dim 128 or 256 and block_size %% 16 == 0");
    if (!mfma)
        return launch_decode(g, q, pool, d_block_table, 0, nullptr, 0, pos_start, M, pos_start + M, out, layer, scale,
                             io_dtype, 0, workspace, workspace_bytes, stream, gate, gate_stride);
    if (a.KVH > 65535) return fail(DRK_ERR_INVALID, "prefill: more than 65535 kv heads");
    if (gate && (gate_stride < (size_t)a.D || (gate_stride % 8) || ((uintptr_t)gate % 16)))
        return fail(DRK_ERR_INVALID, "prefill: gate rows must be 16-byte aligned and at least head_dim apart");
    // a short chunk behind a long context: split the context over the chip (needs the workspace
    // drk_prefill_workspace_bytes reports; without it the chunk kernel below does the work)
    int split_parts = 0;                                     // > 0: the two-phase kernel below, every walk in that many parts
    if (prefill_split_applies(a, pos_start, M) && workspace && ((uintptr_t)workspace % 16) == 0 &&
        workspace_bytes >= prefill_split_need(a, pos_start, M)) {
        split_parts = prefill_split_ppd_parts(a, pos_start, M);
        if (split_parts == 0)
            return prefill_split(a, q, pool, d_block_table, out, layer, pos_start, M, scale, io_dtype, workspace,
                                 (hipStream_t)stream, gate, gate_stride, lse_rows);
    }
    PrefillArgs A;
    A.kparts = 1;
    A.pool_layer = (const uint8_t *)pool + (size_t)layer * a.layer_stride;
    A.table = d_block_table;
    A.q = (const uint8_t *)q;
    A.out = (uint8_t *)out;
    A.pos_start = pos_start; A.M = M; A.QH = a.QH; A.KVH = a.KVH; A.NB = a.NB; A.bs = a.bs;
    A.tpw = 128 / (a.QH / a.KVH);
    A.bs_shift = ilog2_exact((unsigned)a.bs);
    A.head_stride = a.head_stride; A.kv_plane = a.kv_plane; A.block_stride = a.block_stride; A.scale_plane = a.scale_plane;
    A.scale_log2e = scale * kLog2eP;
    dim3 grid(((M + A.tpw - 1) / A.tpw) * a.KVH);
    A.seq_lens = nullptr; A.shared = 0; A.chunk_tiles = 0; A.nsplits = 0; A.part_o = A.part_m = A.part_l = nullptr;
    A.gate = (const uint16_t *)gate; A.gate_stride = gate_stride;
    A.lse_rows = lse_rows;
    hipStream_t st = (hipStream_t)stream;
    // Long chunks of head_dim 128 take the two-phase kernel (256 rows per workgroup, one workgroup per CU)
    // when that still gives at least three quarters of the CUs a workgroup.  That kernel takes its pages
    // without a branch, which wants a block size that is a power of two and at least 16.
    const int G = a.QH / a.KVH;
    if (a.D == 128 && G <= 256 && A.bs_shift >= 4 && g_prefill_two_phase != 0) {
        const int tpw2 = 256 / G;
        const long wgs2 = (long)((M + tpw2 - 1) / tpw2) * a.KVH;
        if (wgs2 >= 192 || g_prefill_two_phase > 1 || split_parts > 0) {
            A.tpw = tpw2;
            if (split_parts > 0) {                           // pieces into the caller's workspace, then the split path's merge
                A.kparts = split_parts;
                A.part_o = (float *)workspace;
                A.part_m = A.part_o + (size_t)M * a.QH * split_parts * a.D;
                A.part_l = A.part_m + (size_t)M * a.QH * split_parts;
            }
            dim3 grid2((unsigned)(wgs2 * A.kparts));
            if ((a.dtype == DRK_BF16 || a.dtype == DRK_F16) && g_prefill_two_phase != 3) {    // 16-bit pages: global -> LDS directly
                if (a.dtype == DRK_BF16) hipLaunchKernelGGL((prefill_ppd_kernel<DRK_BF16, DRK_BF16>), grid2, dim3(512), 0, st, A);
                else hipLaunchKernelGGL((prefill_ppd_kernel<DRK_F16, DRK_F16>), grid2, dim3(512), 0, st, A);
                DRK_LAUNCH_CHECK("prefill_ppd_kernel");
                if (split_parts > 0) {
                    hipLaunchKernelGGL(prefill_merge_kernel<128>, dim3((unsigned)((size_t)M * a.QH)), dim3(64), 0, st, A.part_o, A.part_m,
                                       A.part_l, (uint16_t *)out, split_parts, io_dtype, (const uint16_t *)gate, gate_stride, lse_rows);
                    DRK_LAUNCH_CHECK("prefill_merge_kernel");
                }
                return DRK_OK;
            }
#define DRK_PP_LAUNCH(DT, KV, IO) hipLaunchKernelGGL((prefill_pp_kernel<DT, KV, IO>), grid2, dim3(512), 0, st, A)
            if (a.dtype == DRK_BF16) DRK_PP_LAUNCH(DRK_BF16, DRK_BF16, DRK_BF16);
            else if (a.dtype == DRK_F16) DRK_PP_LAUNCH(DRK_F16, DRK_F16, DRK_F16);
            else if (a.dtype == DRK_INT8 && io_dtype == DRK_BF16) DRK_PP_LAUNCH(DRK_F16, DRK_INT8, DRK_BF16);
            else if (a.dtype == DRK_INT8) DRK_PP_LAUNCH(DRK_F16, DRK_INT8, DRK_F16);
            else if (io_dtype == DRK_BF16) DRK_PP_LAUNCH(DRK_F16, DRK_FP8_E4M3, DRK_BF16);
            else DRK_PP_LAUNCH(DRK_F16, DRK_FP8_E4M3, DRK_F16);
#undef DRK_PP_LAUNCH
            DRK_LAUNCH_CHECK("prefill_pp_kernel");
            if (split_parts > 0) {
                hipLaunchKernelGGL(prefill_merge_kernel<128>, dim3((unsigned)((size_t)M * a.QH)), dim3(64), 0, st, A.part_o, A.part_m,
                                   A.part_l, (uint16_t *)out, split_parts, io_dtype, (const uint16_t *)gate, gate_stride, lse_rows);
                DRK_LAUNCH_CHECK("prefill_merge_kernel");
            }
            return DRK_OK;
        }
    }
    // head_dim 256 on 16-bit pages: one wave per SIMD, tiles straight into LDS (same grid, same rows per workgroup)
    if (d256_direct(a)) {
        // pieces for the walks of the last round when the caller brought the workspace for them
        D256Shape sh = d256_shape(a, pos_start, M, g_prefill_pieces);
        if (sh.kparts > 1 && (!workspace || ((uintptr_t)workspace % 16) || workspace_bytes < d256_pieces_need(sh)))
            sh = d256_shape(a, pos_start, M, 0);
        A.gh = sh.gh; A.tpw = sh.tpw; A.nqt = sh.nqt; A.n_full = sh.n_full; A.kparts = sh.kparts;
        if (sh.kparts > 1) {
            A.part_o = (float *)workspace;
            A.part_m = A.part_o + (size_t)sh.tail * 128 * sh.kparts * 256;
            A.part_l = A.part_m + (size_t)sh.tail * 128 * sh.kparts;
        }
        const dim3 gridp((unsigned)(sh.n_full + sh.tail * sh.kparts));
        if (g_prefill_d256_waves) {
            if (a.dtype == DRK_BF16) hipLaunchKernelGGL((prefill_d256w_kernel<DRK_BF16, DRK_BF16>), gridp, dim3(512), 0, st, A);
            else hipLaunchKernelGGL((prefill_d256w_kernel<DRK_F16, DRK_F16>), gridp, dim3(512), 0, st, A);
        } else {
            if (a.dtype == DRK_BF16) hipLaunchKernelGGL((prefill_d256_kernel<DRK_BF16, DRK_BF16>), gridp, dim3(256), 0, st, A);
            else hipLaunchKernelGGL((prefill_d256_kernel<DRK_F16, DRK_F16>), gridp, dim3(256), 0, st, A);
        }
        DRK_LAUNCH_CHECK("prefill_d256_kernel");
        if (sh.kparts > 1) {
            hipLaunchKernelGGL(prefill_piece_merge_kernel, dim3((unsigned)(sh.tail * 128)), dim3(64), 0, st, A, io_dtype);
            DRK_LAUNCH_CHECK("prefill_piece_merge_kernel");
        }
        return DRK_OK;
    }
#define DRK_PF_LAUNCH(DT, KV, IO)                                                                                        \
    do {                                                                                                                \
        if (a.D == 128) hipLaunchKernelGGL((prefill_mfma_kernel<DT, false, KV, IO, 128>), grid, dim3(256), 0, st, A);   \
        else hipLaunchKernelGGL((prefill_mfma_kernel<DT, false, KV, IO, 256>), grid, dim3(256), 0, st, A);              \
    } while (0)
    if (a.dtype == DRK_BF16) DRK_PF_LAUNCH(DRK_BF16, DRK_BF16, DRK_BF16);
    else if (a.dtype == DRK_F16) DRK_PF_LAUNCH(DRK_F16, DRK_F16, DRK_F16);
    else if (a.dtype == DRK_INT8 && io_dtype == DRK_BF16) DRK_PF_LAUNCH(DRK_F16, DRK_INT8, DRK_BF16);
    else if (a.dtype == DRK_INT8) DRK_PF_LAUNCH(DRK_F16, DRK_INT8, DRK_F16);
    else if (io_dtype == DRK_BF16) DRK_PF_LAUNCH(DRK_F16, DRK_FP8_E4M3, DRK_BF16);
    else DRK_PF_LAUNCH(DRK_F16, DRK_FP8_E4M3, DRK_F16);
#undef DRK_PF_LAUNCH
    DRK_LAUNCH_CHECK("prefill_mfma_kernel");
    return DRK_OK;
}

int drk_paged_prefill_attention(const drk_kv_layout *g, const void *q, const void *pool,
                                const int32_t *d_block_table, void *out, int layer, int pos_start, int M,
                                float scale, int io_dtype, void *workspace, size_t workspace_bytes,
                                void *stream)
{
    return prefill_impl(g, q, pool, d_block_table, out, layer, pos_start, M, scale, io_dtype, workspace,
                        workspace_bytes, stream, nullptr, 0);
}

// steps 8 + 9 of full_attention_forward_paged_prefill (paged_attention.cu:621-634) in one launch
int drk_paged_prefill_attention_gated(const drk_kv_layout *g, const void *q, const void *pool,
                                      const int32_t *d_block_table, void *out, int layer, int pos_start, int M,
                                      float scale, int io_dtype, const void *gate, size_t gate_stride,
                                      void *workspace, size_t workspace_bytes, void *stream)
{
    if (!gate) return fail(DRK_ERR_INVALID, "prefill: gate is NULL");
    return prefill_impl(g, q, pool, d_block_table, out, layer, pos_start, M, scale, io_dtype, workspace,
                        workspace_bytes, stream, gate, gate_stride);
}

// the same call (gate may be NULL) that also leaves every row's log2-sum-exp, for the single-walk mass pass
int drk_paged_prefill_attention_lse(const drk_kv_layout *g, const void *q, const void *pool,
                                    const int32_t *d_block_table, void *out, int layer, int pos_start, int M,
                                    float scale, int io_dtype, const void *gate, size_t gate_stride, float *d_row_lse,
                                    void *workspace, size_t workspace_bytes, void *stream)
{
    if (!d_row_lse) return fail(DRK_ERR_INVALID, "prefill: d_row_lse is NULL");
    return prefill_impl(g, q, pool, d_block_table, out, layer, pos_start, M, scale, io_dtype, workspace,
                        workspace_bytes, stream, gate, gate_stride, d_row_lse);
}

} // extern "C"
