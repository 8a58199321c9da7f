// drk_common.hpp -- shared between the translation units of libdrk_kv.so:
// error reporting, the device-side view of the pool layout, element helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stddef.h>

#include "drk_kv.h"
#include "drk_debug.h"

namespace drk {

// ---- error reporting ----------------------------------------------------
int fail(int code, const char *fmt, ...);
#define DRK_HIP(call)                                                          \
    do {                                                                       \
        hipError_t e__ = (call);                                               \
        if (e__ != hipSuccess)                                                 \
            return drk::fail(DRK_ERR_HIP, "%s: %s", #call, hipGetErrorString(e__)); \
    } while (0)
// kernel launches report through hipGetLastError
#define DRK_LAUNCH_CHECK(name)                                                 \
    do {                                                                       \
        hipError_t e__ = hipGetLastError();                                    \
        if (e__ != hipSuccess)                                                 \
            return drk::fail(DRK_ERR_HIP, "launch %s: %s", name, hipGetErrorString(e__)); \
    } while (0)

// ---- layout, precomputed in bytes ---------------------------------------
// Contract: see the comment above drk_kv_layout in drk_kv.h.
struct Lay {
    int L, KVH, QH, D, bs, NB, dtype, E;
    unsigned row_bytes;          // D*E
    unsigned head_stride;        // bs*D*E: one head's rows inside a K or V plane
    unsigned kv_plane;           // KVH*bs*D*E
    unsigned scale_plane;        // INT8: KVH*bs*2, else 0
    unsigned block_stride;       // 2*kv_plane + 2*scale_plane
    size_t layer_stride;         // NB*block_stride
};

int make_lay(const drk_kv_layout *g, Lay *out);   // validates, returns DRK_*

__host__ __device__ inline size_t lay_block_base(const Lay &a, int layer, int blk)
{
    return (size_t)layer * a.layer_stride + (size_t)blk * a.block_stride;
}

inline int ilog2_exact(unsigned v)                 // -1 when v is not a power of two
{
    if (v == 0 || (v & (v - 1))) return -1;
    int s = 0;
    while ((1u << s) != v) s++;
    return s;
}

// ---- shared between the decode and prefill translation units ---------------
// The unit descriptors of the persistent decode kernels, built once and read by every launch on the same tables and
// lengths (the layers of one step).  mode 1: the launch only builds and stores them; 2: it reads them.  One record per
// workgroup: {units, 0, 0, 0}, max_units unit descriptors of 16 bytes, max_units x 4 page descriptors of 8 bytes.
struct DecodePlan {
    uint8_t *ptr = nullptr;
    int mode = 0;
    // optional (plain tiled kernel, 16-bit pages): the step's new token of every branch, [B][KVH][D] in the pages'
    // own type, written at position seq_len - 1 by the workgroup that owns the branch's last tile before it reads it
    const uint8_t *new_k = nullptr, *new_v = nullptr;
};
constexpr size_t plan_record_bytes(int max_units) { return 16 + 48 * (size_t)max_units; }
size_t decode_plan_need(const Lay &a, int B, int max_seq_len, const drk_prefix_group *groups, int n_groups);
extern int g_force_portable;
extern int g_skip_merge;
int launch_decode(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *tables,
                  int table_stride, const int32_t *d_seq_lens, int seq_len_host, int causal_base, int B,
                  int max_seq_len, void *out, int layer, float scale, int io_dtype, int split_tokens,
                  void *workspace, size_t workspace_bytes, void *stream, const void *gate = nullptr,
                  size_t gate_stride = 0, DecodePlan plan = {});
// bulk / per-branch append (drk_pages.hip); branch mode (d_pos != NULL) writes at d_pos[i] + pos_start
int launch_append(const drk_kv_layout *g, void *pool, const int32_t *tables, int table_stride, const int32_t *d_pos,
                  int pos_start, int ntokens, int layer, int layer_count, const void *src_k, const void *src_v,
                  int src_dtype, void *stream);
// out[row][d] *= sigmoid(gate[row * gate_stride + d]), rows of D elements (drk_layer.hip)
int launch_sigmoid_gate(const void *x, const void *gate, void *out, size_t rows, int D, size_t gate_stride_elems,
                        int dtype, hipStream_t st);

// persistent stream-K decode (drk_decode_stream.hip)
constexpr int kStreamMaxUnits = 256;                          // 64-token tiles one workgroup may own (descriptor table in LDS)
constexpr int kStreamMaxSplitTokens = kStreamMaxUnits * 64;   // the longest explicit split: 16 384 tokens
extern int g_stream_wgs;
extern int g_stream_stop_after_descriptors;
extern int g_shared_splits;
extern int g_prefix_stream;
bool stream_decode_supported(const Lay &a, int B);
size_t stream_workspace_need(const Lay &a, int B, int max_seq_len, int split_tokens, int start_tile = 0);
int launch_decode_stream(const Lay &a, const void *q, const void *pool, const int32_t *tables, int table_stride,
                         const int32_t *d_seq_lens, int seq_len_host, int B, int max_seq_len, void *out, int layer,
                         float scale, int io_dtype, int split_tokens, void *workspace, bool merge_only, hipStream_t st,
                         int start_tile = 0, const float *pre_o = nullptr, const float *pre_m = nullptr,
                         const float *pre_l = nullptr, int pre_splits = 0, const void *gate = nullptr,
                         size_t gate_stride = 0, float *lse_groups = nullptr, float *lse_rows = nullptr,
                         int lse_stride = 0, DecodePlan plan = {});
size_t stream_plan_need(const Lay &a, int B, int max_seq_len);
int launch_block_mass(const float *lse_groups, const float *lse_rows, const int32_t *d_seq_lens, int B, int QH,
                      int lse_stride, int bs, float *mass, int mass_stride, int accumulate, hipStream_t st);
// branches over a shared prefix: prefix pass + tails + one merge (drk_decode.hip); table_stride 0 = one table for all
int launch_decode_shared(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *tables,
                         int table_stride, const int32_t *d_seq_lens, int B, int max_seq_len, int shared_tokens,
                         void *out, int layer, float scale, int io_dtype, void *workspace, size_t workspace_bytes,
                         void *stream, const void *gate = nullptr, size_t gate_stride = 0);
// branches that share pages as a tree: one launch over shared and private tiles (drk_decode_group.hip)
extern int g_grouped_mode;
bool grouped_decode_supported(const Lay &a, int B);
size_t grouped_workspace_need(const Lay &a, int B, int max_seq_len, const drk_prefix_group *groups, int n_groups);
size_t grouped_workspace_need_max(const Lay &a, int B, int max_seq_len, int max_depth);
bool grouped_decode_writes_new_rows(const Lay &a);        // the grouped kernel for this layout takes DecodePlan::new_k / new_v
int launch_decode_grouped(const drk_kv_layout *g, const void *q, const void *pool, const int32_t *tables, int table_stride,
                          const int32_t *d_seq_lens, int B, int max_seq_len, const drk_prefix_group *groups, int n_groups,
                          void *out, int layer, float scale, int io_dtype, void *workspace, size_t workspace_bytes,
                          void *stream, const void *gate = nullptr, size_t gate_stride = 0, DecodePlan plan = {});
size_t grouped_plan_need(const Lay &a, int B, int max_seq_len, const drk_prefix_group *groups, int n_groups);
// shared-prefix pass on the matrix cores (drk_prefill.hip)
void shared_prefix_shape(const Lay &a, int B, int shared, int *chunk_tiles, int *nsplits);
int launch_shared_prefix(const Lay &a, const void *q, const void *pool, const int32_t *table0,
                         const int32_t *d_seq_lens, int B, int shared, int layer, float scale, int io_dtype,
                         float *part_o, float *part_m, float *part_l, hipStream_t st, int chunk_tiles = 0,
                         int nsplits = 0, int causal_pos_start = 0);

// ---- element helpers (device) -------------------------------------------
// Streaming ("non-temporal") 128- and 64-bit accesses for data that is touched once
// per launch: the page pool is far larger than the caches, and on MI355X a read
// stream marked this way sustains about 10 % more HBM bandwidth than a plain one.
typedef uint32_t drk_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t drk_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 ld_stream128(const void *p)
{
    const drk_u32x4 v = __builtin_nontemporal_load((const drk_u32x4 *)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 ld_stream64(const void *p)
{
    const drk_u32x2 v = __builtin_nontemporal_load((const drk_u32x2 *)p);
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ void st_stream128(void *p, uint4 v)
{
    drk_u32x4 w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, (drk_u32x4 *)p);
}
__device__ __forceinline__ void st_stream64(void *p, uint2 v)
{
    drk_u32x2 w = {v.x, v.y};
    __builtin_nontemporal_store(w, (drk_u32x2 *)p);
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float f16_bits_to_f(uint16_t h)
{
    return __half2float(__ushort_as_half(h));
}
__device__ __forceinline__ float elem16_to_f(uint16_t x, int dtype)
{
    return dtype == DRK_BF16 ? __uint_as_float((uint32_t)x << 16) : f16_bits_to_f(x);
}
// round-to-nearest-even fp32 -> bf16 bits
__device__ __forceinline__ uint16_t f_to_bf16_bits(float f)
{
    uint32_t u = __float_as_uint(f);
    if (f != f) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ uint16_t f_to_elem16(float f, int dtype)
{
    return dtype == DRK_BF16 ? f_to_bf16_bits(f) : __half_as_ushort(__float2half_rn(f));
}

// Correctly rounded fp32 square root: the fp32 device routine is the hardware
// approximation (about one unit in the last place); the fp64 one is exact to the last
// bit, and rounding it to fp32 is the correctly rounded fp32 result (53 >= 2*24 + 2).
__device__ __forceinline__ float sqrt_rn(float x) { return (float)sqrt((double)x); }

// sigmoid_gate_kernel, layer.cu:406-431: v / (1 + exp(-g)), every operation rounded once
__device__ __forceinline__ float sigmoid_gate_value(float v, float g)
{
    return __fdiv_rn(v, __fadd_rn(1.0f, expf(-g)));
}
// the attention epilogue with the gate folded in: the 16-bit attention output times
// sigmoid(gate), rounded to 16 bits again -- the two roundings the separate kernels make
__device__ __forceinline__ uint16_t gated_elem16(uint16_t x16, uint16_t g16, int dtype)
{
    return f_to_elem16(sigmoid_gate_value(elem16_to_f(x16, dtype), elem16_to_f(g16, dtype)), dtype);
}

// ---- 8-bit page codes -> fp16, shared by the decode and prefill kernels ----
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
constexpr uint32_t kBf16Ones = 0x3F803F80u;

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

// unsigned divide with a power-of-two fast path chosen on the host
__device__ __forceinline__ unsigned udiv(unsigned x, unsigned d, int shift)
{
    return shift >= 0 ? (x >> shift) : (x / d);
}

} // namespace drk
