// drk_stream_tile.hpp -- the pieces of one 16-token group of a 64-token tile that the
// persistent decode kernels share: loads of a wave's K and V runs from the pool, the K
// rows' way through LDS into the matrix cores' A-operand layout (8-bit codes become fp16
// on the way), the V operands by byte permutes, and the two products.
#pragma once

#include "drk_common.hpp"

#include <math.h>

namespace drk {

constexpr int kSTile = 64;
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

// Geometry of one instantiation: head_dim D (128 or 256) and the storage type.
template <int DT, int D> struct StreamGeo {
    static constexpr bool q8 = KvTraits<DT>::q8;
    static constexpr int RB = D * (q8 ? 1 : 2);        // bytes of one token row of one kv head in the pool
    static constexpr int NK = RB / 64;                 // 128-bit loads per lane for a 16-token K run
    static constexpr int PITCH = D * 2 + 16;           // LDS pitch of a staged (16-bit) K row: 272 / 528
    static constexpr int NQK = D / 32;                 // v_mfma_f32_16x16x32 per tile and wave
    static constexpr int NCH = D / 128;                // 8-dim chunks a lane holds of each of its V rows
    static constexpr int NPV = D / 16;                 // v_mfma_f32_16x16x16 per tile and wave
};

// one wave's 16-token group of a tile, as loaded from the pool: 16 x RB contiguous bytes
template <int DT, int D> struct KRegs { uint4 r[StreamGeo<DT, D>::NK]; };

// The 16-token run of one kv head at offset `off` of the layer, in units of 16 bytes (kNone:
// the run has no page).  A missing run is loaded from offset 0 -- always mapped -- instead of being
// predicated off: its K only feeds scores that are masked anyway, and its V is cleared
// by the consumer where a stale bit pattern could matter.
template <int DT, int D>
__device__ __forceinline__ KRegs<DT, D> load_k(const uint8_t *__restrict__ layer, uint32_t off, int lane)
{
    KRegs<DT, D> k;
    const uint8_t *p = layer + ((size_t)(off == 0xffffffffu ? 0u : off) << 4) + (size_t)lane * 16;
#pragma unroll
    for (int j = 0; j < StreamGeo<DT, D>::NK; j++) k.r[j] = ld_stream128(p + 1024 * j);
    return k;
}

// stage the wave's 16 K rows as 16-bit values, one row per PITCH bytes
template <int DT, int D>
__device__ __forceinline__ void stage_k(uint8_t *lds, const KRegs<DT, D> &k, int lane)
{
    using G = StreamGeo<DT, D>;
#pragma unroll
    for (int j = 0; j < G::NK; j++) {
        const int bp = lane * 16 + 1024 * j;                 // byte position inside the run
        const int row = bp / G::RB, col = bp % G::RB;
        if constexpr (G::q8) {
            uint32_t h[8];
            if constexpr (DT == DRK_INT8) {
                int8x4_to_f16x4(k.r[j].x, h[0], h[1]);
                int8x4_to_f16x4(k.r[j].y, h[2], h[3]);
                int8x4_to_f16x4(k.r[j].z, h[4], h[5]);
                int8x4_to_f16x4(k.r[j].w, h[6], h[7]);
            } else {
                fp8x4_to_f16x4(k.r[j].x, h[0], h[1]);
                fp8x4_to_f16x4(k.r[j].y, h[2], h[3]);
                fp8x4_to_f16x4(k.r[j].z, h[4], h[5]);
                fp8x4_to_f16x4(k.r[j].w, h[6], h[7]);
            }
            uint8_t *dst = lds + row * G::PITCH + col * 2;
            *(uint4 *)(dst) = make_uint4(h[0], h[1], h[2], h[3]);
            *(uint4 *)(dst + 16) = make_uint4(h[4], h[5], h[6], h[7]);
        } else {
            *(uint4 *)(lds + row * G::PITCH + col) = k.r[j];
        }
    }
}

typedef _Float16 w_f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 w_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 w_f16x4 __attribute__((ext_vector_type(4)));
typedef short w_s16x4 __attribute__((ext_vector_type(4)));
typedef float w_f32x4 __attribute__((ext_vector_type(4)));

template <int DOT>
__device__ __forceinline__ w_f32x4 w_mfma_qk(const uint4 &a, const uint4 &b, w_f32x4 c)
{
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (DOT == DRK_BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(w_bf16x8, a), __builtin_bit_cast(w_bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(w_f16x8, a), __builtin_bit_cast(w_f16x8, b), c, 0, 0, 0);
#else
    (void)a; (void)b;
    return c;
#endif
}
template <int DOT>
__device__ __forceinline__ w_f32x4 w_mfma_pv(const uint2 &a, const uint2 &b, w_f32x4 c)
{
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (DOT == DRK_BF16)
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(w_s16x4, a), __builtin_bit_cast(w_s16x4, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(w_f16x4, a), __builtin_bit_cast(w_f16x4, b), c, 0, 0, 0);
#else
    (void)a; (void)b;
    return c;
#endif
}

// V of one 16-token group as the second product wants it: lane (g = lane/16, c = lane%16)
// holds rows 4g..4g+3, dims 128 ch + 8c .. + 7 for each chunk ch
template <int DT, int D, bool Q8 = KvTraits<DT>::q8> struct VRegs { uint4 r[4][StreamGeo<DT, D>::NCH]; };
template <int DT, int D> struct VRegs<DT, D, true> { uint2 r[4][StreamGeo<DT, D>::NCH]; };

template <int DT, int D>
__device__ __forceinline__ VRegs<DT, D> load_v(const uint8_t *__restrict__ layer, uint32_t off, uint32_t kv_plane, int lane)
{
    using G = StreamGeo<DT, D>;
    VRegs<DT, D> v;
    const uint8_t *p = layer + ((size_t)(off == 0xffffffffu ? 0u : off) << 4) + kv_plane + (size_t)(lane >> 4) * (4 * G::RB);
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int ch = 0; ch < G::NCH; ch++) {
            if constexpr (G::q8) v.r[j][ch] = ld_stream64(p + j * G::RB + ch * 128 + (lane & 15) * 8);
            else v.r[j][ch] = ld_stream128(p + j * G::RB + ch * 256 + (lane & 15) * 16);
        }
    return v;
}

// B operands of the second product for one chunk: vb[e] = V[4g..4g+3][128 ch + 8c + e] as four 16-bit values
template <int DT>
__device__ __forceinline__ void v_operands(const uint2 &r0, const uint2 &r1, const uint2 &r2, const uint2 &r3, uint2 (&vb)[8])
{
#pragma unroll
    for (int h = 0; h < 2; h++) {                         // low / high dword of the 8 codes: dims 4h..4h+3
        const uint32_t a0 = h ? r0.y : r0.x, a1 = h ? r1.y : r1.x, a2 = h ? r2.y : r2.x, a3 = h ? r3.y : r3.x;
        const uint32_t i01a = s_perm(a1, a0, 0x05010400u), i01b = s_perm(a1, a0, 0x07030602u);   // t0 t1 pairs of dims 0,1 | 2,3
        const uint32_t i23a = s_perm(a3, a2, 0x05010400u), i23b = s_perm(a3, a2, 0x07030602u);   // t2 t3
        uint32_t lo[4], hi[4];
        if constexpr (DT == DRK_INT8) {
            int8x4_to_f16x4(i01a, lo[0], lo[1]);
            int8x4_to_f16x4(i01b, lo[2], lo[3]);
            int8x4_to_f16x4(i23a, hi[0], hi[1]);
            int8x4_to_f16x4(i23b, hi[2], hi[3]);
        } else {
            fp8x4_to_f16x4(i01a, lo[0], lo[1]);
            fp8x4_to_f16x4(i01b, lo[2], lo[3]);
            fp8x4_to_f16x4(i23a, hi[0], hi[1]);
            fp8x4_to_f16x4(i23b, hi[2], hi[3]);
        }
#pragma unroll
        for (int e = 0; e < 4; e++) vb[4 * h + e] = make_uint2(lo[e], hi[e]);
    }
}
template <int DT>
__device__ __forceinline__ void v_operands(const uint4 &r0, const uint4 &r1, const uint4 &r2, const uint4 &r3, uint2 (&vb)[8])
{
    const uint32_t w0[4] = {r0.x, r0.y, r0.z, r0.w}, w1[4] = {r1.x, r1.y, r1.z, r1.w};
    const uint32_t w2[4] = {r2.x, r2.y, r2.z, r2.w}, w3[4] = {r3.x, r3.y, r3.z, r3.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        vb[2 * i] = make_uint2(s_perm(w1[i], w0[i], 0x05040100u), s_perm(w3[i], w2[i], 0x05040100u));
        vb[2 * i + 1] = make_uint2(s_perm(w1[i], w0[i], 0x07060302u), s_perm(w3[i], w2[i], 0x07060302u));
    }
}

// ---- a workgroup's unit descriptors to and from a plan in global memory ---------------------------------
// UD is the kernel's 16-byte unit descriptor; udesc / gdesc are its tables in LDS, complete (a barrier has passed).
template <typename UD, int MAXU>
__device__ __forceinline__ void plan_store(uint8_t *plan, int nunits, const UD *udesc, const uint2 (*gdesc)[4])
{
    static_assert(sizeof(UD) == 16, "unit descriptors are 16 bytes");
    uint8_t *rec = plan + (size_t)blockIdx.x * plan_record_bytes(MAXU);
    if (threadIdx.x == 0) *(int4 *)rec = make_int4(nunits, 0, 0, 0);
    for (int i = threadIdx.x; i < nunits * 3; i += blockDim.x) {
        const int u = i / 3, part = i - 3 * u;
        if (part == 0) *(uint4 *)(rec + 16 + 16 * u) = *(const uint4 *)&udesc[u];
        else *(uint4 *)(rec + 16 + 16 * MAXU + 32 * u + 16 * (part - 1)) = *(const uint4 *)&gdesc[u][2 * (part - 1)];
    }
}
// returns the number of units (the same for every thread); holds a barrier
template <typename UD, int MAXU>
__device__ __forceinline__ int plan_load(const uint8_t *plan, UD *udesc, uint2 (*gdesc)[4])
{
    const uint8_t *rec = plan + (size_t)blockIdx.x * plan_record_bytes(MAXU);
    int nunits = __builtin_amdgcn_readfirstlane(*(const int *)rec);
    nunits = nunits < 0 ? 0 : (nunits > MAXU ? MAXU : nunits);
    for (int i = threadIdx.x; i < nunits * 3; i += blockDim.x) {
        const int u = i / 3, part = i - 3 * u;
        if (part == 0) *(uint4 *)&udesc[u] = *(const uint4 *)(rec + 16 + 16 * u);
        else *(uint4 *)&gdesc[u][2 * (part - 1)] = *(const uint4 *)(rec + 16 + 16 * MAXU + 32 * u + 16 * (part - 1));
    }
    __syncthreads();
    return nunits;
}

// ---- global memory straight into LDS ------------------------------------------------------------
__device__ __forceinline__ uint32_t lds_addr32(const void *p)
{
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void *)p;
}
// 16 bytes per lane from base + lane_offset straight into LDS: lane i's land at lds_addr + 16 i (base and lds_addr
// are the same for the whole wave).  Written as assembly so that the compiler does not know of the store into LDS:
// it would wait for every outstanding load ahead of the next LDS read.  The caller waits itself (vm_wait_all)
// before it reads the bytes.  The LDS address travels in M0, which the compiler reserves for instructions of its
// own that need it and loads right before each of them; its remark about the clobber is switched off here.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void lds_dma16(const void *base, uint32_t lane_offset, uint32_t lds_addr)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" : : "v"(lane_offset), "s"(base), "s"(lds_addr) : "memory", "m0");
#else
    (void)base; (void)lane_offset; (void)lds_addr;
#endif
}
#pragma clang diagnostic pop
// every load of the wave has arrived (loads return in order; direct loads have then written LDS)
__device__ __forceinline__ void vm_wait_all()
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
}

} // namespace drk
