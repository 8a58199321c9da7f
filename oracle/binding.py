"""ctypes binding of oracle/liboracle.so (see drk_oracle.h).

TEST INFRASTRUCTURE ONLY.  The shipped package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# DRK_ORACLE_SAN=asan / tsan: the sanitizer build of oracle/Makefile (SAN=1 / SAN=thread), made beforehand
_SAN = os.environ.get("DRK_ORACLE_SAN", "")
_SO = os.path.join(_HERE, "liboracle%s.so" % ("_" + _SAN if _SAN in ("asan", "tsan") else ""))

F16, BF16, INT8, FP8 = 0, 1, 2, 3


class Layout(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("L", "KVH", "QH", "D", "bs", "NB", "dtype")]


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-B", "-C", _HERE, os.path.basename(_SO)] +
                              ({"asan": ["SAN=1"], "tsan": ["SAN=thread"]}.get(_SAN, [])))
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    build()
    L = C.CDLL(_SO)
    P = C.POINTER(Layout)
    vp, i32, sz, f32, f64 = C.c_void_p, C.c_int32, C.c_size_t, C.c_float, C.c_double
    sig = {
        "orc_h2f": (f32, [C.c_uint16]), "orc_f2h": (C.c_uint16, [f32]),
        "orc_bf2f": (f32, [C.c_uint16]), "orc_f2bf": (C.c_uint16, [f32]),
        "orc_f2fp8": (C.c_uint8, [f32]), "orc_fp82f": (f32, [C.c_uint8]),
        "orc_elem_bytes": (sz, [P]), "orc_kv_plane_bytes": (sz, [P]),
        "orc_block_stride_bytes": (sz, [P]), "orc_layer_stride_bytes": (sz, [P]),
        "orc_pool_bytes": (sz, [P]),
        "orc_k_off": (sz, [P, i32, i32, i32, i32, i32]),
        "orc_v_off": (sz, [P, i32, i32, i32, i32, i32]),
        "orc_kscale_off": (sz, [P, i32, i32, i32, i32]),
        "orc_vscale_off": (sz, [P, i32, i32, i32, i32]),
        "orc_max_blocks_for_budget": (i32, [P, sz]),
        "orc_append_token": (None, [P, vp, vp, i32, i32, vp, vp, i32]),
        "orc_append_batch": (None, [P, vp, vp, i32, i32, i32, vp, vp, i32]),
        "orc_extract": (None, [P, vp, vp, vp, vp, i32, i32, i32]),
        "orc_inject": (None, [P, vp, vp, vp, vp, i32, i32, i32]),
        "orc_copy_block": (None, [P, vp, i32, i32]),
        "orc_block_image": (None, [P, vp, i32, vp]),
        "orc_block_from_image": (None, [P, vp, i32, vp]),
        "orc_block_attention_mass": (None, [P, vp, vp, vp, i32, vp, i32, i32, f64, i32, vp, i32]),
        "orc_split_q_gate": (None, [vp, vp, vp, i32, i32, i32]),
        "orc_head_norm": (None, [vp, vp, vp, i32, i32, f32, i32]),
        "orc_rope_table": (None, [vp, i32, i32, f32]),
        "orc_apply_rope": (None, [vp, i32, i32, i32, i32, vp, vp, i32]),
        "orc_sigmoid_gate": (None, [vp, vp, vp, sz, i32]),
        "orc_quant_row_int8": (None, [vp, i32, i32, vp, vp]),
        "orc_quant_row_fp8": (None, [vp, i32, i32, vp]),
        "orc_decode_ref_order": (i32, [P, vp, vp, vp, vp, i32, i32, f32, i32]),
        "orc_decode_f64": (i32, [P, vp, vp, vp, vp, i32, i32, f64, i32]),
        "orc_prefill_ref_order": (None, [P, vp, vp, vp, vp, i32, i32, i32, f32, i32]),
        "orc_prefill_f64": (None, [P, vp, vp, vp, vp, i32, i32, i32, f64, i32]),
        "orc_decode_splitk": (None, [P, vp, vp, vp, vp, i32, i32, f32, i32, i32]),
        "orc_decode_branches": (None, [P, vp, vp, vp, i32, vp, i32, vp, i32, f32, i32, i32]),
        "orc_importance_update": (None, [vp, vp, i32, f32]),
        "orc_least_important": (i32, [vp, vp, i32]),
        "orc_cm_create": (vp, [i32, i32, i32]), "orc_cm_destroy": (None, [vp]),
        "orc_cm_alloc_block": (i32, [vp]), "orc_cm_free_block": (None, [vp, i32]),
        "orc_cm_free_count": (i32, [vp]), "orc_cm_refcount": (i32, [vp, i32]),
        "orc_cm_free_stack": (i32, [vp, vp, i32]),
        "orc_cm_ensure": (i32, [vp, i32, i32]), "orc_cm_ensure_range": (i32, [vp, i32, i32, i32]),
        "orc_cm_evict_blocks": (i32, [vp, i32]), "orc_cm_ensure_free_blocks": (i32, [vp, i32]),
        "orc_cm_fork": (i32, [vp, i32, i32]), "orc_cm_release": (None, [vp, i32]),
        "orc_cm_touch": (None, [vp, i32, i32]), "orc_cm_set_scores": (None, [vp, vp, i32]),
        "orc_cm_max_logical": (i32, [vp]), "orc_cm_gpu_blocks_used": (i32, [vp]),
        "orc_cm_table": (C.POINTER(C.c_int32), [vp, i32]),
        "orc_cm_location": (C.POINTER(C.c_int8), [vp, i32]),
        "orc_cm_seq_len": (i32, [vp, i32]), "orc_cm_set_seq_len": (None, [vp, i32, i32]),
        "orc_cm_lru": (i32, [vp, vp, vp, i32]), "orc_cm_drain_copies": (i32, [vp, vp, vp, i32]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    _lib = L
    return L


def ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def layout(L, KVH, QH, D, bs, NB, dtype):
    return Layout(L, KVH, QH, D, bs, NB, dtype)


def elem_bytes(g):
    return lib().orc_elem_bytes(C.byref(g))


def pool_bytes(g):
    return lib().orc_pool_bytes(C.byref(g))


def new_pool(g):
    return np.zeros(pool_bytes(g), dtype=np.uint8)


def append_batch(g, pool, table, layer, pos_start, k, v, src_dtype):
    """k, v: uint16 arrays [M, KVH, D]."""
    M = k.shape[0]
    lib().orc_append_batch(C.byref(g), ptr(pool), ptr(table), layer, pos_start, M, ptr(k), ptr(v), src_dtype)


def append_token(g, pool, table, layer, pos, k, v, src_dtype):
    lib().orc_append_token(C.byref(g), ptr(pool), ptr(table), layer, pos, ptr(k), ptr(v), src_dtype)


def extract(g, pool, table, start, n, num_layers):
    eb = elem_bytes(g)
    dt = np.uint16 if eb == 2 else np.uint8
    dst = np.empty((num_layers, 2, n, g.KVH, g.D), dtype=dt)
    sc = np.empty((num_layers, 2, n, g.KVH), dtype=np.uint16) if g.dtype == INT8 else None
    lib().orc_extract(C.byref(g), ptr(dst), ptr(sc), ptr(pool), ptr(table), start, n, num_layers)
    return dst, sc


def inject(g, pool, src, src_scales, table, start, n, num_layers):
    lib().orc_inject(C.byref(g), ptr(pool), ptr(src), ptr(src_scales), ptr(table), start, n, num_layers)


def copy_block(g, pool, src, dst):
    lib().orc_copy_block(C.byref(g), ptr(pool), src, dst)


def block_image(g, pool, blk):
    """bytes of the .kv file image of physical block blk (all layers)"""
    out = np.empty(g.L * lib().orc_block_stride_bytes(C.byref(g)), np.uint8)
    lib().orc_block_image(C.byref(g), ptr(pool), blk, ptr(out))
    return out


def block_from_image(g, pool, blk, image):
    image = np.ascontiguousarray(image, dtype=np.uint8)
    lib().orc_block_from_image(C.byref(g), ptr(pool), blk, ptr(image))


def decode_ref_order(g, q, pool, table, layer, seq_len, scale, io_dtype, out=None):
    out = np.zeros((g.QH, g.D), dtype=np.uint16) if out is None else out
    lib().orc_decode_ref_order(C.byref(g), ptr(q), ptr(pool), ptr(table), ptr(out), layer, seq_len, scale, io_dtype)
    return out


def decode_f64(g, q, pool, table, layer, seq_len, scale, io_dtype):
    out = np.zeros((g.QH, g.D), dtype=np.float64)
    lib().orc_decode_f64(C.byref(g), ptr(q), ptr(pool), ptr(table), ptr(out), layer, seq_len, scale, io_dtype)
    return out


def decode_splitk(g, q, pool, table, layer, seq_len, scale, io_dtype, split_tokens):
    out = np.zeros((g.QH, g.D), dtype=np.uint16)
    lib().orc_decode_splitk(C.byref(g), ptr(q), ptr(pool), ptr(table), ptr(out), layer, seq_len, scale, io_dtype, split_tokens)
    return out


def prefill_ref_order(g, q, pool, table, layer, pos_start, scale, io_dtype):
    M = q.shape[0]
    out = np.zeros((M, g.QH, g.D), dtype=np.uint16)
    lib().orc_prefill_ref_order(C.byref(g), ptr(q), ptr(pool), ptr(table), ptr(out), layer, pos_start, M, scale, io_dtype)
    return out


def prefill_f64(g, q, pool, table, layer, pos_start, scale, io_dtype):
    M = q.shape[0]
    out = np.zeros((M, g.QH, g.D), dtype=np.float64)
    lib().orc_prefill_f64(C.byref(g), ptr(q), ptr(pool), ptr(table), ptr(out), layer, pos_start, M, scale, io_dtype)
    return out


def decode_branches(g, q, pool, tables, seq_lens, layer, scale, io_dtype, threads=1):
    B = q.shape[0]
    out = np.zeros((B, g.QH, g.D), dtype=np.uint16)
    tables = np.ascontiguousarray(tables, dtype=np.int32)
    seq_lens = np.ascontiguousarray(seq_lens, dtype=np.int32)
    lib().orc_decode_branches(C.byref(g), ptr(q), ptr(pool), ptr(tables), tables.shape[1], ptr(seq_lens), B,
                              ptr(out), layer, scale, io_dtype, threads)
    return out


def quant_row_int8(x, src_dtype):
    codes = np.empty(x.shape[0], dtype=np.int8)
    sc = np.empty(1, dtype=np.uint16)
    lib().orc_quant_row_int8(ptr(x), x.shape[0], src_dtype, ptr(codes), ptr(sc))
    return codes, sc[0]


def quant_row_fp8(x, src_dtype):
    codes = np.empty(x.shape[0], dtype=np.uint8)
    lib().orc_quant_row_fp8(ptr(x), x.shape[0], src_dtype, ptr(codes))
    return codes


def block_attention_mass(g, q, pool, tables, seq_lens, layer, scale, io_dtype, mass_stride):
    """fp64 attention mass per (branch, logical block): [B][mass_stride]"""
    tables = np.ascontiguousarray(tables, dtype=np.int32)
    seq_lens = np.ascontiguousarray(seq_lens, dtype=np.int32)
    q = np.ascontiguousarray(q, dtype=np.uint16)
    B = seq_lens.shape[0]
    mass = np.zeros((B, mass_stride), np.float64)
    lib().orc_block_attention_mass(C.byref(g), ptr(q), ptr(pool), ptr(tables), tables.shape[1], ptr(seq_lens), B, layer,
                                   float(scale), io_dtype, ptr(mass), mass_stride)
    return mass


def split_q_gate(qg, T, H, D):
    """qg uint16 [T][H][2D] -> (q, gate), each [T][H][D]"""
    qg = np.ascontiguousarray(qg, dtype=np.uint16)
    q = np.empty((T, H, D), np.uint16)
    gate = np.empty((T, H, D), np.uint16)
    lib().orc_split_q_gate(ptr(qg), ptr(q), ptr(gate), T, H, D)
    return q, gate


def head_norm(x, w, eps, dtype):
    """x uint16 [rows][D], w uint16 [D]"""
    x = np.ascontiguousarray(x, dtype=np.uint16)
    w = np.ascontiguousarray(w, dtype=np.uint16)
    D = x.shape[-1]
    out = np.empty_like(x)
    lib().orc_head_norm(ptr(x), ptr(w), ptr(out), x.size // D, D, float(eps), dtype)
    return out


def rope_table(n_pos, rotary_dim, theta):
    t = np.empty((n_pos, rotary_dim // 2, 2), np.float32)
    lib().orc_rope_table(ptr(t), n_pos, rotary_dim, float(theta))
    return t


def apply_rope(x, pos, table, rotary_dim, dtype):
    """x uint16 [T][H][D] (a rotated copy is returned), pos int32 [T]"""
    x = np.array(x, dtype=np.uint16, order="C", copy=True)
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    T, H, D = x.shape
    lib().orc_apply_rope(ptr(x), T, H, D, rotary_dim, ptr(pos), ptr(table), dtype)
    return x


def sigmoid_gate(x, gate, dtype):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    gate = np.ascontiguousarray(gate, dtype=np.uint16)
    out = np.empty_like(x)
    lib().orc_sigmoid_gate(ptr(x), ptr(gate), ptr(out), x.size, dtype)
    return out


class CacheManager:
    """Oracle bookkeeping (BlockPool + CacheManager + branches)."""

    def __init__(self, NB, bs, max_branches=1):
        self.NB, self.bs, self.max_branches = NB, bs, max_branches
        self._h = lib().orc_cm_create(NB, bs, max_branches)
        self.max_logical = lib().orc_cm_max_logical(self._h)

    def __del__(self):
        if getattr(self, "_h", None):
            lib().orc_cm_destroy(self._h)
            self._h = None

    def alloc_block(self): return lib().orc_cm_alloc_block(self._h)
    def free_block(self, i): lib().orc_cm_free_block(self._h, i)
    def free_count(self): return lib().orc_cm_free_count(self._h)
    def refcount(self, i): return lib().orc_cm_refcount(self._h, i)
    def ensure(self, b, pos): return bool(lib().orc_cm_ensure(self._h, b, pos))
    def ensure_range(self, b, pos, M): return bool(lib().orc_cm_ensure_range(self._h, b, pos, M))
    def evict_blocks(self, n): return lib().orc_cm_evict_blocks(self._h, n)
    def ensure_free_blocks(self, n): return bool(lib().orc_cm_ensure_free_blocks(self._h, n))
    def fork(self, parent, pos): return lib().orc_cm_fork(self._h, parent, pos)
    def release(self, b): lib().orc_cm_release(self._h, b)
    def touch(self, b, l): lib().orc_cm_touch(self._h, b, l)
    def gpu_blocks_used(self): return lib().orc_cm_gpu_blocks_used(self._h)
    def seq_len(self, b): return lib().orc_cm_seq_len(self._h, b)
    def set_seq_len(self, b, n): lib().orc_cm_set_seq_len(self._h, b, n)

    def set_scores(self, scores):
        if scores is None:
            lib().orc_cm_set_scores(self._h, None, 0)
        else:
            s = np.ascontiguousarray(scores, dtype=np.float32)
            lib().orc_cm_set_scores(self._h, ptr(s), s.shape[0])

    def free_stack(self):
        out = np.empty(self.NB, dtype=np.int32)
        n = lib().orc_cm_free_stack(self._h, ptr(out), self.NB)
        return out[:n].copy()

    def table(self, b):
        p = lib().orc_cm_table(self._h, b)
        return np.ctypeslib.as_array(p, shape=(self.max_logical,)).copy()

    def location(self, b):
        p = lib().orc_cm_location(self._h, b)
        return np.ctypeslib.as_array(p, shape=(self.max_logical,)).copy()

    def lru(self):
        cap = self.max_logical * self.max_branches
        bo = np.empty(cap, dtype=np.int32)
        lo = np.empty(cap, dtype=np.int32)
        n = lib().orc_cm_lru(self._h, ptr(bo), ptr(lo), cap)
        return list(zip(bo[:n].tolist(), lo[:n].tolist()))

    def drain_copies(self):
        cap = 4096
        so = np.empty(cap, dtype=np.int32)
        dn = np.empty(cap, dtype=np.int32)
        n = lib().orc_cm_drain_copies(self._h, ptr(so), ptr(dn), cap)
        return list(zip(so[:n].tolist(), dn[:n].tolist()))
