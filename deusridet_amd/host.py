"""ctypes binding of the C shim over the C++ host classes (include/drk_host.h,
deusridet_amd/lib/libdeusridet_memoria.so).  Method names follow the C++
classes, which follow the reference's (src/memoria/cache_manager.h:52-169,
block_pool.h:58-123, importance_scorer.h:25-67, machina/paged_attention.h:27-73).
Raises ImportError when the library has not been built."""
import ctypes as C
import os

import numpy as np

from . import cabi

_HERE = os.path.dirname(os.path.abspath(__file__))
# DRK_HOST_SAN=asan / tsan: the sanitizer build of deusridet_amd/host/Makefile (SAN=1 / SAN=thread), made beforehand
_SAN = os.environ.get("DRK_HOST_SAN", "")
LIB_PATH = os.path.join(_HERE, "lib", "libdeusridet_memoria%s.so" % ("_" + _SAN if _SAN in ("asan", "tsan") else ""))

_vp, _i32, _sz, _f32 = C.c_void_p, C.c_int32, C.c_size_t, C.c_float
_ip = C.POINTER(C.c_int32)

SIGNATURES = {
    "drkh_set_attention_geometry": (_i32, [_i32] * 6),
    "drkh_scorer_create": (_vp, []), "drkh_scorer_destroy": (None, [_vp]),
    "drkh_scorer_init": (_i32, [_vp, _i32, _f32]), "drkh_scorer_init_detached": (_i32, [_vp, _i32, _f32]),
    "drkh_scorer_update": (None, [_vp, _vp, _i32]), "drkh_scorer_least_important": (_i32, [_vp, _vp, _i32]),
    "drkh_scorer_score": (_f32, [_vp, _i32]), "drkh_scorer_sync_to_host": (None, [_vp]),
    "drkh_scorer_load_host_scores": (None, [_vp, _vp, _i32]),
    "drkh_cm_create": (_vp, []), "drkh_cm_destroy": (None, [_vp]),
    "drkh_cm_init": (_i32, [_vp, _sz, _i32, _vp, _i32]),
    "drkh_cm_init_ssd": (_i32, [_vp, _sz, C.c_char_p, _i32, _vp, _vp, _i32]),
    "drkh_cm_ssd_blocks_used": (_i32, [_vp]),
    "drkh_cm_prefetch_block": (None, [_vp, _i32, _i32]),
    "drkh_swapper_create": (_vp, []),
    "drkh_swapper_destroy": (None, [_vp]),
    "drkh_swapper_init": (_i32, [_vp, _vp, C.c_char_p, _i32]),
    "drkh_swapper_shutdown": (None, [_vp]),
    "drkh_swapper_drain": (None, [_vp]),
    "drkh_swapper_pending": (_i32, [_vp]),
    "drkh_swapper_prefetch": (None, [_vp, _i32, C.c_char_p]),
    "drkh_swapper_is_prefetched": (_i32, [_vp, _i32]),
    "drkh_swapper_block_bytes": (_sz, [_vp]),
    "drkh_swapper_swap": (_i32, [_vp, _i32, _i32, _i32, C.c_char_p]),
    "drkh_swapper_swap_many": (_i32, [_vp, _i32, _vp, _vp, _vp, _vp, _vp, _vp]),
    "drkh_swapper_remove_writer_stream": (None, [_vp, _vp]),
    "drkh_cm_init_detached": (_i32, [_vp, _i32, _i32, _vp, _i32]),
    "drkh_cm_ensure_blocks_for": (_i32, [_vp, _i32, _i32]),
    "drkh_cm_ensure_blocks_for_range": (_i32, [_vp, _i32, _i32, _i32]),
    "drkh_cm_sync_block_table": (None, [_vp, _vp]),
    "drkh_cm_forget_stream": (None, [_vp, _vp]),
    "drkh_cm_d_block_table": (_vp, [_vp, _i32]), "drkh_cm_h_block_table": (_ip, [_vp, _i32]),
    "drkh_cm_table_stride": (_i32, [_vp]),
    "drkh_cm_seq_len": (_i32, [_vp, _i32]), "drkh_cm_set_seq_len": (None, [_vp, _i32, _i32]),
    "drkh_cm_num_logical_blocks": (_i32, [_vp, _i32]),
    "drkh_cm_fork_branch": (_i32, [_vp, _i32, _i32]), "drkh_cm_release_branch": (None, [_vp, _i32]),
    "drkh_cm_touch_block": (None, [_vp, _i32, _i32]),
    "drkh_cm_common_prefix_tokens": (_i32, [_vp, _vp, _i32]),
    "drkh_cm_common_prefix_groups": (_i32, [_vp, _vp, _i32, _i32, _i32, _vp, _i32]), "drkh_cm_block_location": (_i32, [_vp, _i32, _i32]),
    "drkh_cm_evict_blocks": (_i32, [_vp, _i32]), "drkh_cm_ensure_free_blocks": (_i32, [_vp, _i32]),
    "drkh_cm_gpu_blocks_used": (_i32, [_vp]), "drkh_cm_free_blocks": (_i32, [_vp]),
    "drkh_cm_lru_snapshot": (_i32, [_vp, _vp, _vp, _i32]),
    "drkh_cm_take_pending_copies": (_i32, [_vp, _vp, _vp, _i32]),
    "drkh_pool_alloc_block": (_i32, [_vp]), "drkh_pool_free_block": (None, [_vp, _i32]),
    "drkh_pool_free_count": (_i32, [_vp]), "drkh_pool_max_blocks": (_i32, [_vp]),
    "drkh_pool_block_size": (_i32, [_vp]), "drkh_pool_refcount": (_i32, [_vp, _i32]),
    "drkh_pool_ptr": (_vp, [_vp]), "drkh_pool_k_offset": (_sz, [_vp, _i32, _i32]),
    "drkh_pool_v_offset": (_sz, [_vp, _i32, _i32]), "drkh_pool_total_bytes": (_sz, [_vp]),
    "drkh_pool_free_stack": (_i32, [_vp, _vp, _i32]),
    "drkh_paged_kv_cache_write": (None, [_vp, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp]),
    "drkh_paged_kv_cache_write_batch": (None, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp]),
    "drkh_paged_kv_cache_write_branches": (None, [_vp, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _i32, _i32, _vp]),
    "drkh_paged_gqa_decode_attention": (None, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _f32, _vp]),
    "drkh_paged_gqa_decode_attention_branches": (None, [_vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _i32, _i32,
                                                        _i32, _f32, _vp]),
    "drkh_paged_gqa_decode_attention_shared": (None, [_vp, _vp, _vp, _i32, _vp, _i32, _i32, _i32, _vp, _i32, _i32, _i32,
                                                      _f32, _vp]),
    "drkh_paged_gqa_decode_grouped_supported": (_i32, [_i32]),
    "drkh_paged_gqa_decode_attention_grouped": (None, [_vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _i32, _vp, _i32, _i32, _i32,
                                                       _f32, _vp]),
    "drkh_paged_prefill_attention": (None, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _f32, _vp]),
    "drkh_paged_attention_reserve_workspace": (_i32, [_i32, _i32, _i32, _i32, _vp]),
    "drkh_paged_attention_workspace_bytes": (_sz, [_i32, _i32, _i32, _i32]),
    "drkh_set_rope_table": (None, [_vp, _i32]),
    "drkh_full_attention_forward_paged": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                                 C.POINTER(_vp), _vp, _vp]),
    "drkh_full_attention_forward_paged_prefill": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                                         _i32, C.POINTER(_vp), _vp]),
    "drkh_paged_attention_release_workspace": (None, []),
    "drkh_kvs_create": (_vp, []),
    "drkh_kvs_destroy": (None, [_vp]),
    "drkh_kvs_init": (_i32, [_vp, _vp, _i32, _vp, _vp, _i32, _i32]),
    "drkh_kvs_begin_prefill": (_i32, [_vp, _i32, _vp]),
    "drkh_kvs_prefill_layer": (None, [_vp, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp]),
    "drkh_kvs_end_prefill": (None, [_vp, _i32, _vp]),
    "drkh_kvs_current_pos": (_i32, [_vp]),
    "drkh_kvs_open_branches": (_i32, [_vp, _i32]),
    "drkh_kvs_set_branch_count": (_i32, [_vp, _i32]),
    "drkh_kvs_close_branches": (None, [_vp]),
    "drkh_kvs_num_branches": (_i32, [_vp]),
    "drkh_kvs_branch_id": (_i32, [_vp, _i32]),
    "drkh_kvs_branch_pos": (_i32, [_vp, _i32]),
    "drkh_kvs_shared_tokens": (_i32, [_vp]),
    "drkh_kvs_set_shared_prefix_policy": (None, [_vp, _i32, _i32]),
    "drkh_kvs_begin_decode_step": (_i32, [_vp, _vp]),
    "drkh_kvs_decode_layer": (None, [_vp, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "drkh_kvs_end_decode_step": (None, [_vp, _vp]),
    "drkh_kvs_capture_decode_step": (_i32, [_vp, _vp, _vp, _vp]),
    "drkh_kvs_replay_decode_step": (_i32, [_vp, _vp]),
    "drkh_scorer_d_new_scores": (_vp, [_vp]),
    "drkh_scorer_apply_new_scores": (None, [_vp, _vp]),
    "drkh_scorer_apply_new_scores_range": (None, [_vp, _i32, _i32, _vp]),
    "drkh_paged_gqa_decode_attention_branches_scored": (None, [_vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _i32, _i32, _i32,
                                                               _f32, _vp, _i32, _vp]),
    "drkh_set_rope": (_i32, [_i32, _f32, _f32]),
    "drkh_sigmoid_gate": (None, [_vp, _vp, _vp, _i32, _vp]),
    "drkh_apply_rope": (None, [_vp, _vp, _i32, _i32, _i32, _i32, _vp, _f32, _vp]),
    "drkh_head_norm": (None, [_vp, _vp, _vp, _i32, _i32, _f32, _vp]),
    "drkh_paged_qk_norm_rope_write_batch": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                                   _vp, _i32, _vp]),
    "drkh_paged_qk_norm_rope_write_branches": (None, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _i32,
                                                      _i32, _vp, _i32, _vp]),
    "drkh_paged_gqa_decode_attention_gated_branches": (None, [_vp, _vp, _vp, _i32, _vp, _i32, _i32, _vp, _i32, _vp, _i32,
                                                              _i32, _i32, _f32, _vp]),
    "drkh_paged_prefill_attention_gated": (None, [_vp, _vp, _vp, _vp, _i32, _vp, _i32, _i32, _i32, _i32, _i32, _f32, _vp]),
    "drkh_invoke_extract_kv_from_pages": (None, [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "drkh_invoke_inject_kv_to_pages": (None, [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
}

_lib = None


def lib():
    global _lib
    if _lib is None:
        cabi.lib()
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: run __graft_entry__.build() or make -C deusridet_amd/host")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def set_attention_geometry(num_fa_layers, num_attn_heads, num_kv_heads, head_dim, kv_dtype=cabi.F16, io_dtype=-1):
    return bool(lib().drkh_set_attention_geometry(num_fa_layers, num_attn_heads, num_kv_heads, head_dim, kv_dtype,
                                                  io_dtype))


def _destroy(obj, fn):
    """Free a native handle once; at interpreter shutdown the module may already be torn down."""
    h, obj._h = getattr(obj, "_h", None), None
    if h and lib is not None:
        getattr(lib(), fn)(h)


class ImportanceScorer:
    def __init__(self):
        self._h = lib().drkh_scorer_create()

    def __del__(self):
        _destroy(self, "drkh_scorer_destroy")

    def init(self, max_blocks, decay=0.95): return bool(lib().drkh_scorer_init(self._h, max_blocks, decay))
    def init_detached(self, max_blocks, decay=0.95): return bool(lib().drkh_scorer_init_detached(self._h, max_blocks, decay))
    def update(self, d_scores_ptr, n): lib().drkh_scorer_update(self._h, d_scores_ptr, n)
    def score(self, b): return lib().drkh_scorer_score(self._h, b)
    def sync_to_host(self): lib().drkh_scorer_sync_to_host(self._h)
    def d_new_scores(self): return lib().drkh_scorer_d_new_scores(self._h)
    def apply_new_scores(self, stream=None): lib().drkh_scorer_apply_new_scores(self._h, stream)
    def apply_new_scores_range(self, first, count, stream=None): lib().drkh_scorer_apply_new_scores_range(self._h, first, count, stream)

    def least_important(self, ids):
        a = np.ascontiguousarray(ids, dtype=np.int32)
        return lib().drkh_scorer_least_important(self._h, _p(a), a.shape[0])

    def load_host_scores(self, scores):
        a = np.ascontiguousarray(scores, dtype=np.float32)
        lib().drkh_scorer_load_host_scores(self._h, _p(a), a.shape[0])


LAYERS_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_void_p)


class KvStream:
    """conscientia/kv_stream.h; io = (qg, k, v, q_norm, k_norm, q_scratch, attn_out) device pointers."""

    def __init__(self):
        self._h = lib().drkh_kvs_create()

    def __del__(self):
        _destroy(self, "drkh_kvs_destroy")

    def init(self, cm, max_context_len, scorer=None, rope_table=None, table_positions=0, max_prefill_rows=2048):
        self._cm, self._scorer = cm, scorer
        return bool(lib().drkh_kvs_init(self._h, cm._h, max_context_len, scorer._h if scorer else None, rope_table,
                                        table_positions, max_prefill_rows))

    def begin_prefill(self, M, stream=None): return bool(lib().drkh_kvs_begin_prefill(self._h, M, stream))
    def prefill_layer(self, layer, io, M, stream=None): lib().drkh_kvs_prefill_layer(self._h, layer, *io, M, stream)
    def end_prefill(self, M, stream=None): lib().drkh_kvs_end_prefill(self._h, M, stream)
    def current_pos(self): return lib().drkh_kvs_current_pos(self._h)
    def open_branches(self, n): return lib().drkh_kvs_open_branches(self._h, n)
    def set_branch_count(self, n): return lib().drkh_kvs_set_branch_count(self._h, n)
    def shared_tokens(self): return lib().drkh_kvs_shared_tokens(self._h)
    def set_shared_prefix_policy(self, min_branches, min_tokens): lib().drkh_kvs_set_shared_prefix_policy(self._h, min_branches, min_tokens)
    def close_branches(self): lib().drkh_kvs_close_branches(self._h)
    def num_branches(self): return lib().drkh_kvs_num_branches(self._h)
    def branch_id(self, i): return lib().drkh_kvs_branch_id(self._h, i)
    def branch_pos(self, i): return lib().drkh_kvs_branch_pos(self._h, i)
    def begin_decode_step(self, stream=None): return bool(lib().drkh_kvs_begin_decode_step(self._h, stream))
    def decode_layer(self, layer, io, stream=None): lib().drkh_kvs_decode_layer(self._h, layer, *io, stream)
    def end_decode_step(self, stream=None): lib().drkh_kvs_end_decode_step(self._h, stream)

    def capture_decode_step(self, layers, stream=None):
        """layers(stream_ptr) enqueues one step (decode_layer per full-attention layer)."""
        cb = LAYERS_FN(lambda s, _u: layers(C.c_void_p(s)))
        return bool(lib().drkh_kvs_capture_decode_step(self._h, C.cast(cb, C.c_void_p), None, stream))

    def replay_decode_step(self, stream=None): return bool(lib().drkh_kvs_replay_decode_step(self._h, stream))


class KVSwapper:
    """src/memoria/kv_swapper.h:50-114; init() takes the CacheManager whose pool it serves."""

    def __init__(self):
        self._h = lib().drkh_swapper_create()

    def __del__(self):
        _destroy(self, "drkh_swapper_destroy")

    def init(self, cm, ssd_dir, staging_blocks=2):
        return bool(lib().drkh_swapper_init(self._h, cm._h, str(ssd_dir).encode(), staging_blocks))

    def shutdown(self): lib().drkh_swapper_shutdown(self._h)
    def drain(self): lib().drkh_swapper_drain(self._h)
    def pending(self): return lib().drkh_swapper_pending(self._h)
    def prefetch(self, idx, path): lib().drkh_swapper_prefetch(self._h, idx, str(path).encode())
    def is_prefetched(self, idx): return bool(lib().drkh_swapper_is_prefetched(self._h, idx))
    def block_bytes(self): return lib().drkh_swapper_block_bytes(self._h)
    def remove_writer_stream(self, stream): lib().drkh_swapper_remove_writer_stream(self._h, stream)

    def swap_many(self, requests):
        """requests: (direction 0 out / 1 in, logical idx, physical block or -1 for a prefetch, path); submitted in order,
        then drained.  Returns (completion order, ok per request)."""
        n = len(requests)
        d = np.array([r[0] for r in requests], dtype=np.int32)
        lg = np.array([r[1] for r in requests], dtype=np.int32)
        ph = np.array([r[2] for r in requests], dtype=np.int32)
        paths = (C.c_char_p * n)(*[str(r[3]).encode() for r in requests])
        order, ok = np.full(n, -1, dtype=np.int32), np.zeros(n, dtype=np.int32)
        done = lib().drkh_swapper_swap_many(self._h, n, _p(d), _p(lg), _p(ph), C.cast(paths, C.c_void_p), _p(order), _p(ok))
        return [int(x) for x in order[:done]], [bool(x) for x in ok]
    def swap_out(self, idx, phys, path): return bool(lib().drkh_swapper_swap(self._h, 0, idx, phys, str(path).encode()))
    def swap_in(self, idx, phys, path): return bool(lib().drkh_swapper_swap(self._h, 1, idx, phys, str(path).encode()))


class CacheManager:
    GPU, INVALID, SSD = 0, -1, -2

    def __init__(self):
        self._h = lib().drkh_cm_create()
        self._scorer = None

    def __del__(self):
        _destroy(self, "drkh_cm_destroy")

    def init(self, kv_budget_bytes, block_size=256, scorer=None, max_branches=1):
        self._scorer = scorer
        return bool(lib().drkh_cm_init(self._h, int(kv_budget_bytes), block_size, scorer._h if scorer else None,
                                       max_branches))

    def init_ssd(self, kv_budget_bytes, cache_dir, block_size, swapper, scorer=None, max_branches=1):
        self._scorer, self._swapper = scorer, swapper
        return bool(lib().drkh_cm_init_ssd(self._h, int(kv_budget_bytes), str(cache_dir).encode(), block_size,
                                           swapper._h if swapper else None, scorer._h if scorer else None, max_branches))

    def ssd_blocks_used(self): return lib().drkh_cm_ssd_blocks_used(self._h)
    def prefetch_block(self, branch, logical): lib().drkh_cm_prefetch_block(self._h, branch, logical)

    def init_detached(self, max_blocks, block_size, scorer=None, max_branches=1):
        self._scorer = scorer
        return bool(lib().drkh_cm_init_detached(self._h, max_blocks, block_size, scorer._h if scorer else None,
                                                max_branches))

    def ensure_blocks_for(self, branch, pos): return bool(lib().drkh_cm_ensure_blocks_for(self._h, branch, pos))
    def ensure_blocks_for_range(self, branch, pos, M): return bool(lib().drkh_cm_ensure_blocks_for_range(self._h, branch, pos, M))
    def sync_block_table(self, stream=None): lib().drkh_cm_sync_block_table(self._h, stream)
    def forget_stream(self, stream): lib().drkh_cm_forget_stream(self._h, stream)
    def d_block_table(self, branch=0): return lib().drkh_cm_d_block_table(self._h, branch)
    def table_stride(self): return lib().drkh_cm_table_stride(self._h)
    def seq_len(self, branch=0): return lib().drkh_cm_seq_len(self._h, branch)
    def set_seq_len(self, branch, n): lib().drkh_cm_set_seq_len(self._h, branch, n)
    def num_logical_blocks(self, branch=0): return lib().drkh_cm_num_logical_blocks(self._h, branch)
    def fork_branch(self, parent, pos): return lib().drkh_cm_fork_branch(self._h, parent, pos)
    def release_branch(self, branch): lib().drkh_cm_release_branch(self._h, branch)
    def touch_block(self, branch, logical): lib().drkh_cm_touch_block(self._h, branch, logical)

    def common_prefix_groups(self, branches, max_group_branches=16, min_tokens=64, max_groups=16):
        """the fork tree of the branches as (first_branch, n_branches, tok_begin, tok_end) tuples, parents first"""
        a = np.ascontiguousarray(branches, dtype=np.int32)
        out = np.zeros((max_groups, 4), dtype=np.int32)
        n = lib().drkh_cm_common_prefix_groups(self._h, _p(a), a.shape[0], max_group_branches, min_tokens, _p(out), max_groups)
        return [tuple(int(x) for x in out[i]) for i in range(n)]

    def common_prefix_tokens(self, branches):
        a = np.ascontiguousarray(branches, dtype=np.int32)
        return lib().drkh_cm_common_prefix_tokens(self._h, _p(a), a.shape[0])

    def block_location(self, branch, logical): return lib().drkh_cm_block_location(self._h, branch, logical)
    def evict_blocks(self, n): return lib().drkh_cm_evict_blocks(self._h, n)
    def ensure_free_blocks(self, n): return bool(lib().drkh_cm_ensure_free_blocks(self._h, n))
    def gpu_blocks_used(self): return lib().drkh_cm_gpu_blocks_used(self._h)
    def free_blocks(self): return lib().drkh_cm_free_blocks(self._h)

    def h_block_table(self, branch=0):
        p = lib().drkh_cm_h_block_table(self._h, branch)
        return np.ctypeslib.as_array(p, shape=(self.table_stride(),)).copy()

    def lru_snapshot(self):
        cap = self.pool_max_blocks() * 64 + 16
        bo, lo = np.empty(cap, dtype=np.int32), np.empty(cap, dtype=np.int32)
        n = lib().drkh_cm_lru_snapshot(self._h, _p(bo), _p(lo), cap)
        return list(zip(bo[:n].tolist(), lo[:n].tolist()))

    def take_pending_copies(self):
        cap = 65536
        so, dn = np.empty(cap, dtype=np.int32), np.empty(cap, dtype=np.int32)
        n = lib().drkh_cm_take_pending_copies(self._h, _p(so), _p(dn), cap)
        return list(zip(so[:n].tolist(), dn[:n].tolist()))

    # BlockPool
    def pool_alloc_block(self): return lib().drkh_pool_alloc_block(self._h)
    def pool_free_block(self, i): lib().drkh_pool_free_block(self._h, i)
    def pool_free_count(self): return lib().drkh_pool_free_count(self._h)
    def pool_max_blocks(self): return lib().drkh_pool_max_blocks(self._h)
    def pool_block_size(self): return lib().drkh_pool_block_size(self._h)
    def pool_refcount(self, i): return lib().drkh_pool_refcount(self._h, i)
    def pool_ptr(self): return lib().drkh_pool_ptr(self._h)
    def pool_k_offset(self, layer, block): return lib().drkh_pool_k_offset(self._h, layer, block)
    def pool_v_offset(self, layer, block): return lib().drkh_pool_v_offset(self._h, layer, block)
    def pool_total_bytes(self): return lib().drkh_pool_total_bytes(self._h)

    def pool_free_stack(self):
        cap = self.pool_max_blocks()
        out = np.empty(max(cap, 1), dtype=np.int32)
        n = lib().drkh_pool_free_stack(self._h, _p(out), cap)
        return out[:n].copy()
