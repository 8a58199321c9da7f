"""The built libraries load without a GPU and export every symbol that
include/drk_kv.h, include/drk_debug.h and include/drk_host.h declare; the layout arithmetic (host
only) agrees with the oracle's.  No kernel is launched here."""
import ctypes as C
import os
import re

import pytest

from deusridet_amd import cabi, host
from oracle import binding as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header, prefix):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"\w+)\s*\(", text)))


def test_drk_kv_symbols_are_exported_and_bound():
    names = declared("drk_kv.h", "drk_")
    assert len(names) > 30
    assert not [n for n in names if n.startswith(("drk_debug_", "drk_probe_"))], \
        "diagnostic switches and measurement probes belong in drk_debug.h, out of the boundary a drop-in binds"
    debug = declared("drk_debug.h", "drk_debug_") + declared("drk_debug.h", "drk_probe_")
    assert len(debug) >= 14
    names = sorted(names + debug)
    raw = C.CDLL(cabi.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in drk_kv.h / drk_debug.h but not exported"
    assert sorted(cabi.SIGNATURES) == names, "the ctypes table and the header differ"
    assert cabi.lib().drk_abi_version() == 1


def test_drk_host_symbols_are_exported_and_bound():
    names = declared("drk_host.h", "drkh_")
    raw = C.CDLL(host.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in drk_host.h but not exported"
    assert sorted(host.SIGNATURES) == names


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
def test_layout_arithmetic_matches_oracle(dtype):
    L = cabi.lib()
    for geom in [(1, 4, 16, 128, 16, 256), (36, 8, 32, 128, 16, 16954), (16, 4, 24, 256, 256, 14)]:
        g, og = cabi.layout(*geom, dtype), orc.layout(*geom, dtype)
        o = orc.lib()
        assert L.drk_kv_layout_check(C.byref(g)) == 0
        assert L.drk_kv_elem_bytes(C.byref(g)) == o.orc_elem_bytes(C.byref(og))
        assert L.drk_kv_plane_bytes(C.byref(g)) == o.orc_kv_plane_bytes(C.byref(og))
        assert L.drk_kv_block_stride_bytes(C.byref(g)) == o.orc_block_stride_bytes(C.byref(og))
        assert L.drk_kv_layer_stride_bytes(C.byref(g)) == o.orc_layer_stride_bytes(C.byref(og))
        assert L.drk_kv_pool_bytes(C.byref(g)) == o.orc_pool_bytes(C.byref(og))
        for layer, blk in [(0, 0), (geom[0] - 1, geom[5] - 1), (0, 7)]:
            assert L.drk_kv_k_offset(C.byref(g), layer, blk) == o.orc_k_off(C.byref(og), layer, blk, 0, 0, 0)
            assert L.drk_kv_v_offset(C.byref(g), layer, blk) == o.orc_v_off(C.byref(og), layer, blk, 0, 0, 0)
        for budget in (10 ** 9, 40 * 10 ** 9, 123456789):
            assert L.drk_kv_max_blocks_for_budget(C.byref(g), budget) == o.orc_max_blocks_for_budget(C.byref(og), budget)


def test_errors_are_reported_without_a_gpu():
    L = cabi.lib()
    bad = cabi.layout(1, 4, 6, 128, 16, 8, cabi.F16)           # 6 q heads over 4 kv heads
    assert L.drk_kv_layout_check(C.byref(bad)) == cabi.ERR_INVALID
    assert L.drk_kv_pool_bytes(C.byref(bad)) == 0
    assert L.drk_strerror(cabi.ERR_WORKSPACE) == b"workspace missing or too small"
    g = cabi.layout(1, 4, 16, 128, 16, 8, cabi.F16)
    need = L.drk_decode_workspace_bytes(C.byref(g), 1, 512)
    assert need >= 16 * (512 // L.drk_decode_default_split(C.byref(g), 1, 512)) * 130 * 4 and need % (130 * 4) == 0


def test_decode_refuses_a_split_longer_than_the_kernels_run():
    """split_tokens above 16 384 would overrun the persistent kernel's descriptor table: the call
    returns DRK_ERR_INVALID before anything is launched (no GPU needed: the pointers are never used)."""
    g = cabi.layout(1, 8, 32, 128, 16, 4096, cabi.BF16)
    fake = C.c_void_p(0x1000)
    L = cabi.lib()
    for split, want in ((16384 + 64, cabi.ERR_INVALID), (100, cabi.ERR_INVALID)):
        rc = L.drk_paged_decode_attention_branches(C.byref(g), fake, fake, fake, 4096, fake, 2, 65536, fake, 0, 0.1, cabi.BF16,
                                                   split, fake, 1 << 30, None)
        assert rc == want, (split, rc)
    assert b"split_tokens" in L.drk_last_error()
