"""ctypes binding of the C ABI declared in include/drk_kv.h.

Loads deusridet_amd/lib/libdrk_kv.so.  If the library is missing this module
raises ImportError: nothing here computes anything on its own.
"""
import ctypes as C
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdrk_kv.so")

F16, BF16, INT8, FP8_E4M3 = 0, 1, 2, 3
OK, ERR_INVALID, ERR_HIP, ERR_UNSUPPORTED, ERR_WORKSPACE = 0, -1, -2, -3, -4
STATIC_SCRATCH_BYTES = 32 << 20


class DrkError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"drk error {code}: {text}")
        self.code = code


class Layout(C.Structure):
    """drk_kv_layout"""
    _fields_ = [(n, C.c_int32) for n in (
        "num_layers", "num_kv_heads", "num_q_heads", "head_dim", "block_size",
        "max_phys_blocks", "dtype", "reserved")]


def layout(L, KVH, QH, D, bs, NB, dtype):
    return Layout(L, KVH, QH, D, bs, NB, dtype, 0)


MAX_PREFIX_GROUPS = 16             # DRK_MAX_PREFIX_GROUPS


class PrefixGroup(C.Structure):
    """drk_prefix_group: branches [first_branch, +n_branches) hold tokens [tok_begin, tok_end) in the same pages"""
    _fields_ = [(n, C.c_int32) for n in ("first_branch", "n_branches", "tok_begin", "tok_end")]


def prefix_groups(groups):
    """ctypes array of drk_prefix_group from (first_branch, n_branches, tok_begin, tok_end) tuples"""
    arr = (PrefixGroup * max(len(groups), 1))()
    for i, gr in enumerate(groups):
        arr[i] = PrefixGroup(*[int(x) for x in gr])
    return arr


_vp, _i32, _sz, _f32 = C.c_void_p, C.c_int32, C.c_size_t, C.c_float
_LP = C.POINTER(Layout)
_GP = C.POINTER(PrefixGroup)

# name -> (restype, argtypes); mirrors include/drk_kv.h and include/drk_debug.h one to one
SIGNATURES = {
    "drk_abi_version": (_i32, []),
    "drk_last_error": (C.c_char_p, []),
    "drk_strerror": (C.c_char_p, [_i32]),
    "drk_device_count": (_i32, [C.POINTER(_i32)]),
    "drk_kv_layout_check": (_i32, [_LP]),
    "drk_kv_elem_bytes": (_sz, [_LP]),
    "drk_kv_plane_bytes": (_sz, [_LP]),
    "drk_kv_block_stride_bytes": (_sz, [_LP]),
    "drk_kv_layer_stride_bytes": (_sz, [_LP]),
    "drk_kv_pool_bytes": (_sz, [_LP]),
    "drk_kv_k_offset": (_sz, [_LP, _i32, _i32]),
    "drk_kv_v_offset": (_sz, [_LP, _i32, _i32]),
    "drk_kv_max_blocks_for_budget": (_i32, [_LP, _sz]),
    "drk_dev_malloc": (_i32, [C.POINTER(_vp), _sz]),
    "drk_dev_free": (_i32, [_vp]),
    "drk_dev_memset_async": (_i32, [_vp, _i32, _sz, _vp]),
    "drk_memcpy_h2d_async": (_i32, [_vp, _vp, _sz, _vp]),
    "drk_memcpy_d2d_async": (_i32, [_vp, _vp, _sz, _vp]),
    "drk_memcpy_d2h": (_i32, [_vp, _vp, _sz, _vp]),
    "drk_positions_advance": (_i32, [_vp, _vp, _i32, _i32, _vp]),
    "drk_graph_begin_capture": (_i32, [_vp]),
    "drk_graph_end_capture": (_i32, [_vp, C.POINTER(_vp)]),
    "drk_graph_launch": (_i32, [_vp, _vp]),
    "drk_graph_destroy": (_i32, [_vp]),
    "drk_device_synchronize": (_i32, []),
    "drk_host_malloc": (_i32, [C.POINTER(_vp), _sz]),
    "drk_host_free": (_i32, [_vp]),
    "drk_kv_block_total_bytes": (_sz, [_LP]),
    "drk_kv_block_to_host": (_i32, [_LP, _vp, _i32, _vp, _vp]),
    "drk_kv_block_from_host": (_i32, [_LP, _vp, _i32, _vp, _vp]),
    "drk_stream_create": (_i32, [C.POINTER(_vp)]),
    "drk_stream_destroy": (_i32, [_vp]),
    "drk_stream_synchronize": (_i32, [_vp]),
    "drk_stream_is_capturing": (_i32, [_vp, C.POINTER(_i32)]),
    "drk_event_create": (_i32, [C.POINTER(_vp)]),
    "drk_event_destroy": (_i32, [_vp]),
    "drk_event_record": (_i32, [_vp, _vp]),
    "drk_event_synchronize": (_i32, [_vp]),
    "drk_stream_wait_event": (_i32, [_vp, _vp]),
    "drk_kv_append_token": (_i32, [_LP, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _vp]),
    "drk_kv_append_batch": (_i32, [_LP, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _vp, _i32, _vp]),
    "drk_kv_append_branches": (_i32, [_LP, _vp, _vp, _i32, _vp, _i32, _i32, _i32, _vp, _vp, _i32, _vp]),
    "drk_kv_extract": (_i32, [_LP, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "drk_kv_inject": (_i32, [_LP, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "drk_kv_copy_blocks": (_i32, [_LP, _vp, _vp, _i32, _vp]),
    "drk_decode_workspace_bytes": (_sz, [_LP, _i32, _i32]),
    "drk_decode_workspace_bytes_for_split": (_sz, [_LP, _i32, _i32, _i32]),
    "drk_decode_default_split": (_i32, [_LP, _i32, _i32]),
    "drk_debug_force_portable_decode": (None, [_i32]),
    "drk_debug_set_decode_kernel": (None, [_i32]),
    "drk_debug_set_stream_workgroups": (None, [_i32]),
    "drk_debug_set_stream_descriptors_only": (None, [_i32]),
    "drk_debug_set_shared_splits": (None, [_i32]),
    "drk_debug_set_prefix_stream": (None, [_i32]),
    "drk_debug_set_skip_merge": (None, [_i32]),
    "drk_debug_set_decode_lds_pad": (None, [_i32]),
    "drk_debug_set_append_chunks": (None, [_i32, _i32, _i32]),
    "drk_debug_check_int8_scale_math": (_i32, [_vp, _vp]),
    "drk_debug_set_quant_append_pairs": (None, [_i32]),
    "drk_debug_set_prefill_split": (None, [_i32]),
    "drk_debug_set_prefill_pieces": (None, [_i32]),
    "drk_debug_set_prefill_d256_waves": (None, [_i32]),
    "drk_debug_set_prefill_mass_direct": (None, [_i32]),
    "drk_debug_set_prefill_mass_parts": (None, [_i32]),
    "drk_debug_set_prefill_two_phase": (None, [_i32]),
    "drk_probe_read_bandwidth": (_i32, [_vp, _sz, _i32, _vp, C.POINTER(C.c_float)]),
    "drk_probe_read_bandwidth_permuted": (_i32, [_vp, _sz, _i32, _i32, _vp, C.POINTER(C.c_float)]),
    "drk_probe_mfma_rate": (_i32, [_i32, _vp, C.POINTER(C.c_float)]),
    "drk_probe_mfma_valu_coexec": (_i32, [_i32, _vp, C.POINTER(C.c_float), C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "drk_probe_phase_coexec": (_i32, [_i32, _i32, _vp, C.POINTER(C.c_float), C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "drk_prefill_workspace_bytes_max": (_sz, [_LP, _i32, _i32]),
    "drk_paged_decode_attention": (_i32, [_LP, _vp, _vp, _vp, _vp, _i32, _i32, _f32, _i32, _vp, _sz, _vp]),
    "drk_paged_decode_attention_branches": (_i32, [_LP, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _i32,
                                                   _f32, _i32, _i32, _vp, _sz, _vp]),
    "drk_paged_decode_attention_branches_static": (_i32, [_LP, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _i32,
                                                          _f32, _i32, _vp]),
    "drk_decode_shared_workspace_bytes": (_sz, [_LP, _i32, _i32, _i32]),
    "drk_paged_decode_attention_shared": (_i32, [_LP, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _i32, _vp, _i32, _f32,
                                                 _i32, _vp, _sz, _vp]),
    "drk_decode_grouped_workspace_bytes": (_sz, [_LP, _i32, _i32, _GP, _i32]),
    "drk_decode_grouped_workspace_bytes_max": (_sz, [_LP, _i32, _i32, _i32]),
    "drk_paged_decode_attention_grouped": (_i32, [_LP, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _GP, _i32, _vp, _i32, _f32,
                                                  _i32, _vp, _sz, _vp, _sz, _vp]),
    "drk_decode_plan_bytes": (_sz, [_LP, _i32, _i32, _i32]),
    "drk_decode_plan_build": (_i32, [_LP, _vp, _i32, _vp, _i32, _i32, _GP, _i32, _vp, _sz, _vp]),
    "drk_paged_decode_attention_planned": (_i32, [_LP, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _GP, _i32, _vp, _vp, _i32, _f32,
                                                  _i32, _vp, _sz, _vp, _sz, _vp]),
    "drk_kv_append_decode_planned": (_i32, [_LP, _vp, _vp, _i32, _vp, _i32, _i32, _GP, _i32, _vp, _vp, _vp, _i32, _vp, _vp, _i32,
                                            _f32, _i32, _vp, _sz, _vp, _sz, _vp]),
    "drk_debug_set_grouped_decode": (None, [_i32]),
    "drk_debug_grouped_grid": (_i32, [_i32, _i32, _i32, _i32]),
    "drk_debug_grouped_region_split": (None, [_i32, _i32, _i32, _i32, _i32, C.POINTER(C.c_int)]),
    "drk_prefill_workspace_bytes": (_sz, [_LP, _i32, _i32]),
    "drk_paged_prefill_attention": (_i32, [_LP, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _i32, _vp, _sz, _vp]),
    "drk_rope_table_fill": (_i32, [_vp, _i32, _i32, _f32, _vp]),
    "drk_head_norm": (_i32, [_vp, _vp, _vp, _i32, _i32, _f32, _i32, _vp]),
    "drk_apply_rope": (_i32, [_vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp, _i32, _f32, _vp, _i32, _i32, _vp]),
    "drk_split_q_gate": (_i32, [_vp, _vp, _vp, _i32, _i32, _i32, _vp]),
    "drk_sigmoid_gate": (_i32, [_vp, _vp, _vp, _sz, _i32, _sz, _i32, _vp]),
    "drk_qk_norm_rope_append": (_i32, [_LP, _vp, _vp, _i32, _vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _f32,
                                       _i32, _f32, _vp, _i32, _vp, _i32, _vp]),
    "drk_paged_decode_attention_gated": (_i32, [_LP, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _i32, _f32, _i32,
                                                _vp, _sz, _vp, _sz, _vp]),
    "drk_paged_prefill_attention_gated": (_i32, [_LP, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _i32, _vp, _sz,
                                                 _vp, _sz, _vp]),
    "drk_decode_mass_workspace_bytes": (_sz, [_LP, _i32, _i32]),
    "drk_paged_decode_attention_mass": (_i32, [_LP, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _i32, _f32, _i32, _vp,
                                               _i32, _i32, _vp, _sz, _vp]),
    "drk_paged_decode_attention_mass_gated": (_i32, [_LP, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _vp, _i32, _f32, _i32,
                                                     _vp, _sz, _vp, _i32, _i32, _vp, _sz, _vp]),
    "drk_paged_prefill_attention_mass": (_i32, [_LP, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _i32, _vp, _i32, _i32, _vp]),
    "drk_paged_prefill_attention_lse": (_i32, [_LP, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _i32, _vp, _sz, _vp, _vp, _sz,
                                               _vp]),
    "drk_paged_prefill_attention_mass_lse": (_i32, [_LP, _vp, _vp, _vp, _i32, _i32, _i32, _f32, _i32, _vp, _vp, _i32, _i32,
                                                    _vp]),
    "drk_importance_update": (_i32, [_vp, _vp, _i32, _f32, _vp]),
    "drk_importance_fold_clear": (_i32, [_vp, _vp, _i32, _f32, _vp]),
}

_lib = None


def lib():
    """The loaded library (raises ImportError when it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C deusridet_amd/csrc`")
        # A process must hold ONE HIP runtime.  PyTorch-ROCm ships its own libamdhip64;
        # when this library is loaded first it binds /opt/rocm's copy instead, torch then
        # brings a second one, and HIP calls of the later-initialised copy fail with
        # "no ROCm-capable device is detected".  Loading torch first makes both share
        # torch's copy; a process without torch simply uses /opt/rocm's.
        if "torch" not in sys.modules:
            try:
                import torch  # noqa: F401
            except ImportError:
                pass
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def check(code):
    if code != OK:
        raise DrkError(code, lib().drk_last_error().decode())
    return code


def call(name, *args):
    """Call an int-returning entry point and raise DrkError on failure."""
    return check(getattr(lib(), name)(*args))


# ---- plumbing for callers that keep device memory in torch tensors -------------------
def p(t):
    """Device pointer of a torch tensor as a ctypes void pointer (None stays None)."""
    return C.c_void_p(t.data_ptr()) if t is not None else None


def time_partial_kernels(call_one, n, warm=6):
    """Average milliseconds of the kernels that read the pages in one decode call, merge left out: n calls back
    to back on torch's current stream (which the calls must use), one event pair around each."""
    import torch
    for i in range(warm):
        call_one(i)
    lib().drk_debug_set_skip_merge(1)
    try:
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for i, (e0, e1) in enumerate(ev):
            e0.record()
            call_one(i)
            e1.record()
        torch.cuda.synchronize()
    finally:
        lib().drk_debug_set_skip_merge(0)
    call_one(0)                                      # leave real results behind
    return sum(e0.elapsed_time(e1) for e0, e1 in ev) / n


def stream_ptr():
    """The hipStream_t of torch's current stream, as the entry points take it."""
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)
