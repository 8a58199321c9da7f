// drk_codec.hpp -- what the append-side kernels share: byte offsets of page rows and
// scales, the int8 / fp8 codecs, and the store of one 16-byte source chunk into a page.
#pragma once
#include "drk_common.hpp"

namespace drk {

__device__ __forceinline__ size_t row_off(const Lay &a, int layer, int blk, int kv, int h, int p)
{
    return lay_block_base(a, layer, blk) + (size_t)kv * a.kv_plane + (size_t)h * a.head_stride +
           (size_t)p * a.row_bytes;
}
__device__ __forceinline__ size_t scale_off(const Lay &a, int layer, int blk, int kv, int h, int p)
{
    return lay_block_base(a, layer, blk) + 2 * (size_t)a.kv_plane + (size_t)kv * a.scale_plane +
           ((size_t)h * a.bs + p) * 2;
}

struct Div {            // divisor with a power-of-two fast path
    unsigned d;
    int shift;
};
static inline Div mk_div(unsigned d) { return Div{d, ilog2_exact(d)}; }
__device__ __forceinline__ unsigned dv(unsigned x, Div v) { return udiv(x, v.d, v.shift); }

__device__ __forceinline__ void unpack8(const uint4 &v, int src_dtype, float *x)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        x[2 * i] = elem16_to_f((uint16_t)(w[i] & 0xffffu), src_dtype);
        x[2 * i + 1] = elem16_to_f((uint16_t)(w[i] >> 16), src_dtype);
    }
}

// E4M3FN code of x: round-half-even, |x| >= 448 and +-inf saturate to +-448,
// NaN stays NaN.  The clamp runs before the hardware conversion so that the
// conversion never sees an out-of-range input.
__device__ __forceinline__ uint32_t fp8_pair(float x0, float x1)
{
    x0 = (x0 != x0) ? x0 : fminf(fmaxf(x0, -448.0f), 448.0f);
    x1 = (x1 != x1) ? x1 : fminf(fmaxf(x1, -448.0f), 448.0f);
#if defined(__HIP_DEVICE_COMPILE__)
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(x0, x1, 0, false) & 0xffffu;
#else
    (void)x0; (void)x1;
    return 0;
#endif
}

// maximum over each aligned group of 16 lanes, by DPP (quad swaps, half-row and row mirrors)
template <int CTRL>
__device__ __forceinline__ float codec_dpp(float v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
#else
    return v;
#endif
}
__device__ __forceinline__ float row16_max(float v)
{
    v = fmaxf(v, codec_dpp<0xB1>(v));
    v = fmaxf(v, codec_dpp<0x4E>(v));
    v = fmaxf(v, codec_dpp<0x141>(v));
    v = fmaxf(v, codec_dpp<0x140>(v));
    return v;
}

// The int8 scale of a row from its largest magnitude, and the reciprocal the codes are made with:
//   scale = fp16(amax / 127), saturated to the largest finite fp16;  rcp = 1 / scale  (0 for a zero scale),
// both divisions correctly rounded in fp32.  IEEE = the compiler's full division sequences (about two dozen
// instructions for the two); otherwise one multiply by the rounded reciprocal plus one residual correction
// each, which gives the same bits for every input that occurs here: amax is the magnitude of a bf16 or fp16
// number, and the scale is an fp16 number (so its significand is never all ones, the one case in which the
// corrected reciprocal of a 1-ulp estimate can be off).  drk_debug_check_int8_scale_math compares the two
// forms over all of those inputs on the device.
template <bool IEEE>
__device__ __forceinline__ void int8_row_scale(float amax, uint16_t &scale_bits, float &rcp)
{
    float s32;
    if (IEEE) {
        s32 = __fdiv_rn(amax, 127.0f);
    } else {
        const float c = 1.0f / 127.0f;
        const float q = __fmul_rn(amax, c);
        s32 = __fmaf_rn(__fmaf_rn(-q, 127.0f, amax), c, q);
        s32 = amax == INFINITY ? amax : s32;                  // inf - inf in the residual
    }
    uint16_t sh = __half_as_ushort(__float2half_rn(s32));
    if ((sh & 0x7fffu) == 0x7c00u) sh = 0x7bffu;
    const float sf = f16_bits_to_f(sh);
    if (IEEE) {
        rcp = sf > 0.0f ? __fdiv_rn(1.0f, sf) : 0.0f;
    } else {
#if defined(__HIP_DEVICE_COMPILE__)
        const float y = __builtin_amdgcn_rcpf(sf);            // within 1 ulp
        rcp = sf > 0.0f ? __fmaf_rn(__fmaf_rn(-sf, y, 1.0f), y, y) : 0.0f;
#else
        rcp = 0.0f;
#endif
    }
    scale_bits = sh;
}

// int8 codes of 8 values: code = clamp(rint(x * rcp), -127, 127).  The clamp bounds are integers, so it may run
// before the rounding, and adding 1.5 * 2^23 rounds to the nearest integer, ties to even, exactly as rint does --
// and leaves the code's two's-complement byte as the low byte of the sum.
__device__ __forceinline__ void int8_codes8(const float *x, float rcp, uint32_t &lo, uint32_t &hi)
{
    uint32_t u[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float r = __fmul_rn(x[i], rcp);
        r = fminf(fmaxf(r, -127.0f), 127.0f);
        u[i] = __float_as_uint(__fadd_rn(r, 12582912.0f));
    }
    lo = s_perm(s_perm(u[3], u[2], 0x04000c0cu), s_perm(u[1], u[0], 0x0c0c0400u), 0x07060100u);
    hi = s_perm(s_perm(u[7], u[6], 0x04000c0cu), s_perm(u[5], u[4], 0x0c0c0400u), 0x07060100u);
}
__device__ __forceinline__ void fp8_codes8(const float *x, uint32_t &lo, uint32_t &hi)
{
    lo = fp8_pair(x[0], x[1]) | (fp8_pair(x[2], x[3]) << 16);
    hi = fp8_pair(x[4], x[5]) | (fp8_pair(x[6], x[7]) << 16);
}

// The 8 codes of chunk c of a row: the even lane of each lane pair takes its neighbour's
// 8 bytes (chunks of one row sit in consecutive lanes, so both belong to the same row) and
// stores 16 (fp8 bulk append 4.60 -> 5.02 TB/s against 8-byte stores from every lane);
// every lane of the wave must call this.
__device__ __forceinline__ void store_codes(uint8_t *__restrict__ row, unsigned c, unsigned rc, uint32_t lo, uint32_t hi,
                                            bool ok)
{
#if defined(__HIP_DEVICE_COMPILE__)
    if (rc < 2) {                                            // a row of one chunk has no neighbour
        if (ok) st_stream64(row, make_uint2(lo, hi));
        return;
    }
    const uint32_t lo_n = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)lo, 0xB1, 0xf, 0xf, false);
    const uint32_t hi_n = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)hi, 0xB1, 0xf, 0xf, false);
    if (ok && !(c & 1u)) st_stream128(row + (size_t)c * 8, make_uint4(lo, hi, lo_n, hi_n));
#else
    (void)row; (void)c; (void)rc; (void)lo; (void)hi; (void)ok;
#endif
}

// Store one source chunk (8 elements of type src_dtype, `val`) into the page row at byte
// offset poff as chunk c of its row.  rc = chunks per row; the rc lanes that hold one row
// are consecutive lanes of one wave (rc is a power of two <= 64), and every lane of the
// wave must call this (the int8 row maximum is a lane exchange); ok = this lane stores.
// QMODE 0: copy.  1: int8 codes + fp16 scale per row (soff).  2: fp8 e4m3 codes.
template <int QMODE>
__device__ __forceinline__ void store_page_chunk(uint8_t *__restrict__ pool, size_t poff, size_t soff, unsigned c,
                                                 unsigned rc, const uint4 &val, int src_dtype, bool ok)
{
    if (QMODE == 0) {
        if (ok) st_stream128(pool + poff + (size_t)c * 16, val);
    } else {
        float x[8];
        unpack8(val, src_dtype, x);
        if (QMODE == 1) {
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(x[i]));
            if (rc == 16) {                                   // head_dim 128: one row = one DPP row of 16 lanes
                amax = row16_max(amax);
            } else {
                for (unsigned off = rc >> 1; off > 0; off >>= 1)
                    amax = fmaxf(amax, __shfl_xor(amax, (int)off));
            }
            uint16_t sh;
            float rcp;
            int8_row_scale<false>(amax, sh, rcp);
            uint32_t lo, hi;
            int8_codes8(x, rcp, lo, hi);
            store_codes(pool + poff, c, rc, lo, hi, ok);
            if (ok && c == 0) *(uint16_t *)(pool + soff) = sh;
        } else {
            uint32_t lo, hi;
            fp8_codes8(x, lo, hi);
            store_codes(pool + poff, c, rc, lo, hi, ok);
        }
    }
}

} // namespace drk
