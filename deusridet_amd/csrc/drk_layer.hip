// drk_layer.hip -- the steps of a full-attention layer either side of the page
// kernels (full_attention_forward_paged, paged_attention.cu:314-376): split of the
// interleaved Q|gate projection, per-head RMSNorm, partial half-half RoPE, sigmoid gate.
//
// Stand-alone forms with the reference's call shapes (head_norm, apply_rope,
// sigmoid_gate, split) and the fused form: ONE launch reads the raw projections of
// T tokens, writes the normalised + rotated Q rows, and appends the normalised +
// rotated K rows and the V rows into their pages (quantising for int8 / fp8 pools),
// where the reference launches split, head_norm x2, rope and the page write.
//
// Mapping (all kernels): a head row of D 16-bit elements is held by D/8 consecutive
// lanes, 8 elements = 16 bytes per lane; D/8 is a power of two <= 64, so a row never
// straddles a wave and every row reduction is an xor butterfly over those lanes.
// The arithmetic is written out operation by operation (fused multiply-adds where
// nvcc's default contraction fuses them) so that the CPU restatement used by the tests
// matches to the bit whenever both use the same cos/sin table.
#include "drk_common.hpp"
#include "drk_codec.hpp"

#include <math.h>

namespace drk {

constexpr int kLThreads = 256;

__device__ __forceinline__ uint4 pack8(const float *y, int dtype)
{
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
        w[i] = (uint32_t)f_to_elem16(y[2 * i], dtype) | ((uint32_t)f_to_elem16(y[2 * i + 1], dtype) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// head_norm_kernel, layer_attention.cu:86-127: out = fp16((x * rsqrt(mean(x^2) + eps)) * w).
// nl = lanes per row.  Every lane of the wave calls this.
__device__ __forceinline__ uint4 norm_chunk(const uint4 &val, const uint4 &wv, unsigned nl, int D, float eps, int dtype)
{
    float x[8], w[8], y[8];
    unpack8(val, dtype, x);
    unpack8(wv, dtype, w);
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) ss = __fmaf_rn(x[i], x[i], ss);
    for (unsigned off = nl >> 1; off > 0; off >>= 1) ss = __fadd_rn(ss, __shfl_xor(ss, (int)off));
    const float inv_rms = __fdiv_rn(1.0f, sqrt_rn(__fadd_rn(__fdiv_rn(ss, (float)D), eps)));
#pragma unroll
    for (int i = 0; i < 8; i++) y[i] = __fmul_rn(__fmul_rn(x[i], inv_rms), w[i]);
    return pack8(y, dtype);
}

// rope_kernel, layer_attention.cu:32-69: pairs (i, i + rd/2), i < rd/2, rotated by
// pos * theta^(-2i/rd).  hp = (rd/2)/8 = lanes per half; chunk c < hp holds x0 of 8
// pairs, chunk c + hp their x1.  table_row = (cos, sin) per pair for this position, or
// NULL: computed here with the reference's fp32 expressions.  Every lane of the wave
// calls this (lane exchange); chunks c >= 2*hp come back unchanged.
__device__ __forceinline__ uint4 rope_chunk(const uint4 &val, unsigned c, unsigned hp, int rotary_dim, int pos,
                                            float theta, const float *__restrict__ table_row, int dtype)
{
    uint4 oth;
    oth.x = (uint32_t)__shfl_xor((int)val.x, (int)hp);
    oth.y = (uint32_t)__shfl_xor((int)val.y, (int)hp);
    oth.z = (uint32_t)__shfl_xor((int)val.z, (int)hp);
    oth.w = (uint32_t)__shfl_xor((int)val.w, (int)hp);
    if (c >= 2 * hp) return val;
    const bool low = c < hp;
    const unsigned pair0 = (low ? c : c - hp) * 8;
    float own[8], other[8], y[8];
    unpack8(val, dtype, own);
    unpack8(oth, dtype, other);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float cs, sn;
        if (table_row) {
            const float2 t = *(const float2 *)(table_row + (pair0 + i) * 2);
            cs = t.x;
            sn = t.y;
        } else {
            const float freq = __fdiv_rn(1.0f, powf(theta, __fdiv_rn(2.0f * (float)(pair0 + i), (float)rotary_dim)));
            const float angle = __fmul_rn((float)pos, freq);
            cs = cosf(angle);
            sn = sinf(angle);
        }
        // x0' = x0 c - x1 s ; x1' = x1 c + x0 s
        y[i] = low ? __fmaf_rn(own[i], cs, -__fmul_rn(other[i], sn)) : __fmaf_rn(own[i], cs, __fmul_rn(other[i], sn));
    }
    return pack8(y, dtype);
}

// layer.cu:406-431: x * sigmoid(g) on 16-bit values
__device__ __forceinline__ uint4 gate_chunk(const uint4 &xv, const uint4 &gv, int dtype)
{
    float x[8], g[8], y[8];
    unpack8(xv, dtype, x);
    unpack8(gv, dtype, g);
#pragma unroll
    for (int i = 0; i < 8; i++) y[i] = sigmoid_gate_value(x[i], g[i]);
    return pack8(y, dtype);
}

__global__ __launch_bounds__(kLThreads) void rope_table_kernel(float *__restrict__ table, int n_pos, int np,
                                                              int rotary_dim, float theta)
{
    const size_t i = (size_t)blockIdx.x * kLThreads + threadIdx.x;
    if (i >= (size_t)n_pos * np) return;
    const int pos = (int)(i / np), pair = (int)(i - (size_t)pos * np);
    const float freq = __fdiv_rn(1.0f, powf(theta, __fdiv_rn(2.0f * (float)pair, (float)rotary_dim)));
    const float angle = __fmul_rn((float)pos, freq);
    *(float2 *)(table + i * 2) = make_float2(cosf(angle), sinf(angle));
}

__global__ __launch_bounds__(kLThreads) void head_norm_kernel(const uint8_t *__restrict__ x, const uint8_t *__restrict__ w,
                                                             uint8_t *__restrict__ out, size_t items, unsigned nl, int D,
                                                             float eps, int dtype)
{
    const size_t it = (size_t)blockIdx.x * kLThreads + threadIdx.x;
    const bool live = it < items;
    const unsigned c = (unsigned)(it & (nl - 1));
    const uint4 val = live ? *(const uint4 *)(x + it * 16) : make_uint4(0, 0, 0, 0);
    const uint4 wv = *(const uint4 *)(w + (size_t)c * 16);
    const uint4 y = norm_chunk(val, wv, nl, D, eps, dtype);
    if (live) *(uint4 *)(out + it * 16) = y;
}

// rows of one token: QH query heads of q, then KVH heads of k; in place
__global__ __launch_bounds__(kLThreads) void rope_kernel(uint8_t *__restrict__ q, uint8_t *__restrict__ k, int T, int QH, int KVH,
                                                        unsigned nl, int nl_shift, unsigned hp, int rotary_dim,
                                                        const int32_t *__restrict__ d_pos, int pos_start, float theta,
                                                        const float *__restrict__ table, int table_positions, int dtype)
{
    const size_t it = (size_t)blockIdx.x * kLThreads + threadIdx.x;
    const unsigned rpt = (unsigned)(QH + KVH);
    const size_t items = (size_t)T * rpt * nl;
    const bool live = it < items;
    const unsigned c = (unsigned)(it & (nl - 1));
    const size_t row = it >> nl_shift;
    const unsigned t = live ? (unsigned)(row / rpt) : 0u, r = live ? (unsigned)(row - (size_t)t * rpt) : 0u;
    uint8_t *p = r < (unsigned)QH ? q + (((size_t)t * QH + r) * nl + c) * 16 : k + (((size_t)t * KVH + (r - QH)) * nl + c) * 16;
    const int pos = live ? (d_pos ? d_pos[t] : pos_start + (int)t) : 0;
    const float *trow = (table && pos >= 0 && pos < table_positions) ? table + (size_t)pos * (rotary_dim / 2) * 2 : nullptr;
    const uint4 val = live ? *(const uint4 *)p : make_uint4(0, 0, 0, 0);
    const uint4 y = rope_chunk(val, c, hp, rotary_dim, pos, theta, trow, dtype);
    if (live && c < 2 * hp) *(uint4 *)p = y;
}

// paged_split_q_gate, paged_attention.cu:288-298, 386-404
__global__ __launch_bounds__(kLThreads) void split_q_gate_kernel(const uint8_t *__restrict__ qg, uint8_t *__restrict__ q,
                                                                uint8_t *__restrict__ gate, size_t rows, unsigned nl,
                                                                int nl_shift)
{
    const size_t it = (size_t)blockIdx.x * kLThreads + threadIdx.x;
    if (it >= rows * nl) return;
    const size_t row = it >> nl_shift;
    const unsigned c = (unsigned)(it & (nl - 1));
    const uint8_t *src = qg + (row * 2 * nl + c) * 16;
    *(uint4 *)(q + it * 16) = *(const uint4 *)src;
    *(uint4 *)(gate + it * 16) = *(const uint4 *)(src + (size_t)nl * 16);
}

// x, out: [rows][D]; gate: row stride gate_stride elements (2*D when it still sits in the Q|gate projection)
__global__ __launch_bounds__(kLThreads) void sigmoid_gate_kernel(const uint8_t *__restrict__ x, const uint8_t *__restrict__ gate,
                                                                uint8_t *__restrict__ out, size_t chunks, unsigned nl,
                                                                int nl_shift, size_t gate_stride_bytes, int dtype)
{
    const size_t it = (size_t)blockIdx.x * kLThreads + threadIdx.x;
    if (it >= chunks) return;
    const size_t row = it >> nl_shift;
    const unsigned c = (unsigned)(it & (nl - 1));
    const uint4 xv = *(const uint4 *)(x + it * 16);
    const uint4 gv = *(const uint4 *)(gate + row * gate_stride_bytes + (size_t)c * 16);
    *(uint4 *)(out + it * 16) = gate_chunk(xv, gv, dtype);
}

// The fused step.  Rows of token t: QH rows of Q (from qg, row stride 2*D), KVH rows of K,
// KVH rows of V.  Q rows: norm, rope -> q_out.  K rows: norm, rope -> page (quantised for
// 8-bit pools).  V rows -> page.  Every lane runs every stage (the stages exchange data
// between lanes) and a per-lane flag selects what is kept.
struct FusedArgs {
    const uint8_t *qg, *k, *v, *q_norm_w, *k_norm_w;
    uint8_t *q_out, *pool;
    const int32_t *tables, *d_pos;
    const float *rope_table;
    int table_stride, pos_start, T, layer, QH, KVH, rotary_dim, table_positions, dtype;
    unsigned nl, hp;
    int nl_shift;
    float eps, theta;
    Div bs_div;
};

template <int QMODE>
__global__ __launch_bounds__(kLThreads) void qk_norm_rope_append_kernel(Lay a, FusedArgs A)
{
    const size_t it = (size_t)blockIdx.x * kLThreads + threadIdx.x;
    const unsigned rpt = (unsigned)(A.QH + 2 * A.KVH), nl = A.nl;
    const size_t items = (size_t)A.T * rpt * nl;
    const bool live = it < items;
    const unsigned c = (unsigned)(it & (nl - 1));
    const size_t row = it >> A.nl_shift;
    const unsigned t = live ? (unsigned)(row / rpt) : 0u, r = live ? (unsigned)(row - (size_t)t * rpt) : 0u;
    const int kind = r < (unsigned)A.QH ? 0 : (r < (unsigned)(A.QH + A.KVH) ? 1 : 2);     // Q, K, V
    const unsigned h = kind == 0 ? r : (kind == 1 ? r - A.QH : r - A.QH - A.KVH);
    const uint8_t *src = kind == 0 ? A.qg + (((size_t)t * A.QH + h) * 2 * nl + c) * 16
                       : (kind == 1 ? A.k : A.v) + (((size_t)t * A.KVH + h) * nl + c) * 16;
    uint4 val = live ? ld_stream128(src) : make_uint4(0, 0, 0, 0);
    const uint4 wv = *(const uint4 *)((kind == 0 ? A.q_norm_w : A.k_norm_w) + (size_t)c * 16);
    const int pos = live ? (A.d_pos ? A.d_pos[t] : A.pos_start + (int)t) : -1;

    const uint4 normed = norm_chunk(val, wv, nl, a.D, A.eps, A.dtype);
    if (kind != 2) val = normed;
    const float *trow = (A.rope_table && pos >= 0 && pos < A.table_positions)
                            ? A.rope_table + (size_t)pos * (A.rotary_dim / 2) * 2 : nullptr;
    const uint4 rotated = rope_chunk(val, c, A.hp, A.rotary_dim, pos, A.theta, trow, A.dtype);
    if (kind != 2) val = rotated;

    if (live && kind == 0) *(uint4 *)(A.q_out + (((size_t)t * A.QH + h) * nl + c) * 16) = val;

    bool ok = false;
    size_t poff = 0, soff = 0;
    if (live && kind != 0 && pos >= 0) {
        const int32_t *tab = A.tables + (size_t)(A.d_pos ? t : 0) * A.table_stride;
        const unsigned lb = dv((unsigned)pos, A.bs_div);
        const int blk = tab[lb];
        if (blk >= 0 && blk < a.NB) {
            ok = true;
            const int p = pos - (int)(lb * A.bs_div.d);
            poff = row_off(a, A.layer, blk, kind - 1, (int)h, p);
            if (QMODE == 1) soff = scale_off(a, A.layer, blk, kind - 1, (int)h, p);
        }
    }
    store_page_chunk<QMODE>(A.pool, poff, soff, c, nl, val, A.dtype, ok);
}

static int row_shape(int D, unsigned *nl, int *nl_shift, const char *who)
{
    if (D < 8 || D > 512 || (D % 8) || ilog2_exact((unsigned)D / 8) < 0)
        return fail(DRK_ERR_UNSUPPORTED, "%s: head_dim %d is not a power of two in [8, 512]", who, D);
    *nl = (unsigned)D / 8;
    *nl_shift = ilog2_exact(*nl);
    return DRK_OK;
}
static int rope_shape(int D, int rotary_dim, unsigned *hp, const char *who)
{
    if (rotary_dim < 16 || rotary_dim > D || (rotary_dim % 16) || ilog2_exact((unsigned)rotary_dim / 16) < 0)
        return fail(DRK_ERR_UNSUPPORTED, "%s: rotary_dim %d must be 16 * 2^k and at most head_dim %d", who, rotary_dim, D);
    *hp = (unsigned)rotary_dim / 16;
    return DRK_OK;
}
static int check16(int dtype, const char *who)
{
    if (dtype != DRK_F16 && dtype != DRK_BF16) return fail(DRK_ERR_INVALID, "%s: dtype must be F16 or BF16", who);
    return DRK_OK;
}
static inline unsigned blocks_for(size_t items) { return (unsigned)((items + kLThreads - 1) / kLThreads); }

int launch_sigmoid_gate(const void *x, const void *gate, void *out, size_t rows, int D, size_t gate_stride_elems,
                        int dtype, hipStream_t st)
{
    unsigned nl;
    int sh, rc;
    if ((rc = row_shape(D, &nl, &sh, "sigmoid_gate"))) return rc;
    const size_t chunks = rows * nl;
    if (chunks == 0) return DRK_OK;
    hipLaunchKernelGGL(sigmoid_gate_kernel, dim3(blocks_for(chunks)), dim3(kLThreads), 0, st, (const uint8_t *)x,
                       (const uint8_t *)gate, (uint8_t *)out, chunks, nl, sh, gate_stride_elems * 2, dtype);
    DRK_LAUNCH_CHECK("sigmoid_gate_kernel");
    return DRK_OK;
}

} // namespace drk

using namespace drk;

extern "C" {

int drk_rope_table_fill(float *d_table, int n_pos, int rotary_dim, float theta, void *stream)
{
    if (!d_table || n_pos < 1 || rotary_dim < 2 || (rotary_dim & 1) || !(theta > 0.0f))
        return fail(DRK_ERR_INVALID, "rope_table_fill: bad argument");
    const int np = rotary_dim / 2;
    hipLaunchKernelGGL(rope_table_kernel, dim3(blocks_for((size_t)n_pos * np)), dim3(kLThreads), 0, (hipStream_t)stream,
                       d_table, n_pos, np, rotary_dim, theta);
    DRK_LAUNCH_CHECK("rope_table_kernel");
    return DRK_OK;
}

// head_norm, layer_attention.cu:129-135
int drk_head_norm(const void *x, const void *weight, void *out, int num_rows, int head_dim, float eps, int dtype,
                  void *stream)
{
    unsigned nl;
    int sh, rc;
    if ((rc = check16(dtype, "head_norm")) || (rc = row_shape(head_dim, &nl, &sh, "head_norm"))) return rc;
    if (!x || !weight || !out || num_rows < 0) return fail(DRK_ERR_INVALID, "head_norm: bad argument");
    if (num_rows == 0) return DRK_OK;
    const size_t items = (size_t)num_rows * nl;
    hipLaunchKernelGGL(head_norm_kernel, dim3(blocks_for(items)), dim3(kLThreads), 0, (hipStream_t)stream,
                       (const uint8_t *)x, (const uint8_t *)weight, (uint8_t *)out, items, nl, head_dim, eps, dtype);
    DRK_LAUNCH_CHECK("head_norm_kernel");
    return DRK_OK;
}

// apply_rope, layer_attention.cu:71-79 (one token, *d_pos) and paged_rope_batch_kernel,
// paged_attention.cu:412-451 (T tokens at pos_start + t)
int drk_apply_rope(void *q, void *k, int T, int num_q_heads, int num_kv_heads, int head_dim, int rotary_dim,
                   const int32_t *d_pos, int pos_start, float theta, const float *d_rope_table, int table_positions,
                   int dtype, void *stream)
{
    unsigned nl, hp;
    int sh, rc;
    if ((rc = check16(dtype, "apply_rope")) || (rc = row_shape(head_dim, &nl, &sh, "apply_rope")) ||
        (rc = rope_shape(head_dim, rotary_dim, &hp, "apply_rope")))
        return rc;
    if (T < 0 || num_q_heads < 0 || num_kv_heads < 0 || (num_q_heads > 0 && !q) || (num_kv_heads > 0 && !k) ||
        pos_start < 0 || !(theta > 0.0f))
        return fail(DRK_ERR_INVALID, "apply_rope: bad argument");
    const size_t items = (size_t)T * (num_q_heads + num_kv_heads) * nl;
    if (items == 0) return DRK_OK;
    hipLaunchKernelGGL(rope_kernel, dim3(blocks_for(items)), dim3(kLThreads), 0, (hipStream_t)stream, (uint8_t *)q,
                       (uint8_t *)k, T, num_q_heads, num_kv_heads, nl, sh, hp, rotary_dim, d_pos, pos_start, theta,
                       d_rope_table, d_rope_table ? table_positions : 0, dtype);
    DRK_LAUNCH_CHECK("rope_kernel");
    return DRK_OK;
}

int drk_split_q_gate(const void *qg, void *q, void *gate, int T, int num_heads, int head_dim, void *stream)
{
    unsigned nl;
    int sh, rc;
    if ((rc = row_shape(head_dim, &nl, &sh, "split_q_gate"))) return rc;
    if (!qg || !q || !gate || T < 0 || num_heads < 0) return fail(DRK_ERR_INVALID, "split_q_gate: bad argument");
    const size_t rows = (size_t)T * num_heads;
    if (rows == 0) return DRK_OK;
    hipLaunchKernelGGL(split_q_gate_kernel, dim3(blocks_for(rows * nl)), dim3(kLThreads), 0, (hipStream_t)stream,
                       (const uint8_t *)qg, (uint8_t *)q, (uint8_t *)gate, rows, nl, sh);
    DRK_LAUNCH_CHECK("split_q_gate_kernel");
    return DRK_OK;
}

// sigmoid_gate, layer.cu:433-439; gate rows may be strided (gate_stride elements between rows)
int drk_sigmoid_gate(const void *x, const void *gate, void *out, size_t num_rows, int head_dim, size_t gate_stride,
                     int dtype, void *stream)
{
    int rc;
    if ((rc = check16(dtype, "sigmoid_gate"))) return rc;
    if (!x || !gate || !out || gate_stride < (size_t)head_dim || (gate_stride % 8))
        return fail(DRK_ERR_INVALID, "sigmoid_gate: bad argument");
    return launch_sigmoid_gate(x, gate, out, num_rows, head_dim, gate_stride, dtype, (hipStream_t)stream);
}

int drk_qk_norm_rope_append(const drk_kv_layout *g, void *pool, const int32_t *d_tables, int table_stride,
                            const int32_t *d_pos, int pos_start, int T, int layer, const void *qg, const void *k,
                            const void *v, const void *q_norm_w, const void *k_norm_w, float eps, int rotary_dim,
                            float theta, const float *d_rope_table, int table_positions, void *q_out, int src_dtype,
                            void *stream)
{
    Lay a;
    int rc = make_lay(g, &a);
    if (rc) return rc;
    FusedArgs A;
    if ((rc = check16(src_dtype, "qk_norm_rope_append")) || (rc = row_shape(a.D, &A.nl, &A.nl_shift, "qk_norm_rope_append")) ||
        (rc = rope_shape(a.D, rotary_dim, &A.hp, "qk_norm_rope_append")))
        return rc;
    if (!pool || !d_tables || !qg || !k || !v || !q_norm_w || !k_norm_w || !q_out)
        return fail(DRK_ERR_INVALID, "qk_norm_rope_append: NULL pointer");
    if (layer < 0 || layer >= a.L) return fail(DRK_ERR_INVALID, "qk_norm_rope_append: layer %d outside [0,%d)", layer, a.L);
    if (T < 0 || pos_start < 0 || table_stride < 0 || !(theta > 0.0f))
        return fail(DRK_ERR_INVALID, "qk_norm_rope_append: bad argument");
    if ((a.dtype == DRK_F16 || a.dtype == DRK_BF16) && src_dtype != a.dtype)
        return fail(DRK_ERR_INVALID, "qk_norm_rope_append: src_dtype %d differs from the pool's %d", src_dtype, a.dtype);
    if (T == 0) return DRK_OK;
    A.qg = (const uint8_t *)qg; A.k = (const uint8_t *)k; A.v = (const uint8_t *)v;
    A.q_norm_w = (const uint8_t *)q_norm_w; A.k_norm_w = (const uint8_t *)k_norm_w;
    A.q_out = (uint8_t *)q_out; A.pool = (uint8_t *)pool;
    A.tables = d_tables; A.d_pos = d_pos; A.rope_table = d_rope_table;
    A.table_stride = table_stride; A.pos_start = pos_start; A.T = T; A.layer = layer; A.QH = a.QH; A.KVH = a.KVH;
    A.rotary_dim = rotary_dim; A.table_positions = d_rope_table ? table_positions : 0; A.dtype = src_dtype;
    A.eps = eps; A.theta = theta;
    A.bs_div = mk_div((unsigned)a.bs);
    const size_t items = (size_t)T * (a.QH + 2 * a.KVH) * A.nl;
    const dim3 grid(blocks_for(items));
    hipStream_t st = (hipStream_t)stream;
    if (a.dtype == DRK_INT8) hipLaunchKernelGGL(qk_norm_rope_append_kernel<1>, grid, dim3(kLThreads), 0, st, a, A);
    else if (a.dtype == DRK_FP8_E4M3) hipLaunchKernelGGL(qk_norm_rope_append_kernel<2>, grid, dim3(kLThreads), 0, st, a, A);
    else hipLaunchKernelGGL(qk_norm_rope_append_kernel<0>, grid, dim3(kLThreads), 0, st, a, A);
    DRK_LAUNCH_CHECK("qk_norm_rope_append_kernel");
    return DRK_OK;
}

} // extern "C"
