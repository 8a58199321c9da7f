"""The fixtures of tests/golden against the oracle, the host library (CPU) and the HIP
path (GPU, through the C ABI).  The fixtures come from tests/golden/make_golden.py, which
uses neither of the three: a published number format, the reference's documented free
stack, IEEE arithmetic of stated widths, and fp64 attention of BASELINE config 1.

Bars: codes, scales, ids and gathered K/V bit for bit; attention within
|err| <= 2e-2 + 1e-2 * |want| (the oracle's fp64 path: 1e-6)."""
import ctypes as C
import importlib.util
import json
import os

import numpy as np
import pytest

from deusridet_amd import cabi, host
from oracle import binding as orc
from tests import util as U

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with open(os.path.join(GOLD, name)) as f:
        return json.load(f)


def generator():
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLD, "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def f16_exact(v):
    return abs(v) <= 65504.0 and float(np.float32(np.float16(v))) == v


# ------------------------------------------------------------------ CPU: oracle and host
def test_e4m3fn_table_and_encode_cases_oracle():
    t = load("e4m3fn_table.json")
    lib = orc.lib()
    for code, want in enumerate(t["values"]):
        got = lib.orc_fp82f(code)
        assert (np.isnan(got) if want is None else got == want), (code, got, want)
    for v, code in t["encode"]:
        assert lib.orc_f2fp8(float(np.float32(v))) == code, (v, code)
    assert lib.orc_f2fp8(float("inf")) == t["saturating"]["inf"] and lib.orc_f2fp8(float("-inf")) == t["saturating"]["-inf"]


def test_int8_rows_oracle():
    for row in load("int8_rows.json")["rows"]:
        x = np.array(row["x_f16_bits"], dtype=np.uint16)
        codes, scale = orc.quant_row_int8(x, orc.F16)
        assert int(scale) == row["scale_f16_bits"] and codes.tolist() == row["codes"]


def test_block_pool_trace_host_and_oracle():
    t = load("block_pool_trace.json")
    assert host.set_attention_geometry(2, 4, 2, 16, cabi.F16)
    cm = host.CacheManager()
    assert cm.init_detached(t["max_blocks"], 4, None, 1)
    suts = [(cm.pool_alloc_block, cm.pool_free_block, cm.pool_free_count)]
    o = orc.CacheManager(t["max_blocks"], 4)
    suts.append((o.alloc_block, o.free_block, o.free_count))
    for alloc, free, count in suts:
        for op in t["ops"]:
            if op["op"] == "alloc":
                assert alloc() == op["returns"]
            else:
                free(op["id"])
            assert count() == op["free_count"]


def _config1():
    t = load("config1_decode.json")
    gen = generator()
    table, k, v, q = gen.config1_inputs()
    assert gen.inputs_digest(table, k, v, q) == t["inputs_sha256"] and table.tolist() == t["table"]
    return t, table, k, v, q, np.array(t["out_f32"], dtype=np.float32)


def test_config1_oracle():
    t, table, k, v, q, want = _config1()
    c = t["config"]
    og = orc.layout(c["L"], c["KVH"], c["QH"], c["D"], c["bs"], c["NB"], orc.F16)
    pool = orc.new_pool(og)
    orc.append_batch(og, pool, table, 0, 0, k, v, orc.F16)
    flat, _ = orc.extract(og, pool, table, 0, c["tokens"], 1)
    assert np.array_equal(flat[0, 0], k) and np.array_equal(flat[0, 1], v)          # gathered K/V bit for bit
    f64 = orc.decode_f64(og, q, pool, table, 0, c["tokens"], t["scale"], orc.F16)
    assert np.max(np.abs(f64 - want)) <= 1e-6
    ref = U.from_bits(orc.decode_ref_order(og, q, pool, table, 0, c["tokens"], t["scale"], orc.F16), cabi.F16)
    ok, ma, _ = U.rel_abs_ok(ref, want)
    assert ok, ma


# ------------------------------------------------------------------ GPU: the HIP path
@pytest.mark.gpu
def test_config1_gpu(dev):
    t, table, k, v, q, want = _config1()
    c = t["config"]
    g = cabi.layout(c["L"], c["KVH"], c["QH"], c["D"], c["bs"], c["NB"], cabi.F16)
    lib = cabi.lib()
    dpool = U.dev_zeros(lib.drk_kv_pool_bytes(C.byref(g)))
    dtab, dk, dv, dq = U.dev_i32(table), U.dev_bytes(k), U.dev_bytes(v), U.dev_bytes(q)
    cabi.call("drk_kv_append_batch", C.byref(g), U.p(dpool), U.p(dtab), 0, 1, 0, c["tokens"], U.p(dk), U.p(dv), cabi.F16,
              U.stream_ptr())
    flat = U.dev_zeros(2 * k.nbytes)
    cabi.call("drk_kv_extract", C.byref(g), U.p(flat), None, U.p(dpool), U.p(dtab), 0, c["tokens"], 1, U.stream_ptr())
    wsb = lib.drk_decode_workspace_bytes(C.byref(g), 1, c["tokens"])
    ws, out = U.dev_zeros(max(wsb, 16)), U.dev_zeros(q.nbytes)
    cabi.call("drk_paged_decode_attention", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out), 0, c["tokens"],
              float(t["scale"]), cabi.F16, U.p(ws), wsb, U.stream_ptr())
    U.sync()
    got_flat = U.host(flat, np.uint16, (2,) + k.shape)
    assert np.array_equal(got_flat[0], k) and np.array_equal(got_flat[1], v)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(U.host(out, np.uint16, q.shape), cabi.F16), want)
    assert ok, ma


def _append_rows(rows_bits, D, dtype):
    """rows [M, D] of fp16 bit patterns through the quantising append; returns codes [M, D] and scales [M]"""
    M = rows_bits.shape[0]
    bs = 16
    NB = (M + bs - 1) // bs
    g = cabi.layout(1, 1, 1, D, bs, NB, dtype)
    lib = cabi.lib()
    dpool = U.dev_zeros(lib.drk_kv_pool_bytes(C.byref(g)))
    table = np.arange(NB, dtype=np.int32)
    src = np.ascontiguousarray(rows_bits.reshape(M, 1, D))
    d, dtab = U.dev_bytes(src), U.dev_i32(table)
    cabi.call("drk_kv_append_batch", C.byref(g), U.p(dpool), U.p(dtab), 0, 1, 0, M, U.p(d), U.p(d), cabi.F16, U.stream_ptr())
    U.sync()
    # the page layout, read directly: per block [K codes bs x D][V codes][K scales bs x fp16][V scales] (int8)
    blocks = U.host(dpool, np.uint8).reshape(NB, -1)
    plane = bs * D
    codes = np.stack([blocks[:, :plane].reshape(NB * bs, D)[:M], blocks[:, plane:2 * plane].reshape(NB * bs, D)[:M]])
    if dtype == cabi.INT8:
        sc = np.ascontiguousarray(blocks[:, 2 * plane:]).view(np.uint16).reshape(NB, 2, bs)
        scales = np.stack([sc[:, 0].reshape(-1)[:M], sc[:, 1].reshape(-1)[:M]])
    else:
        scales = np.zeros((2, M), np.uint16)
    assert np.array_equal(codes[0], codes[1]) and np.array_equal(scales[0], scales[1])       # K and V took the same rows
    return codes[0], scales[0]


@pytest.mark.gpu
def test_e4m3fn_encode_cases_gpu(dev):
    t = load("e4m3fn_table.json")
    cases = [(v, code) for v, code in t["encode"] if f16_exact(v)]
    cases += [(float("inf"), t["saturating"]["inf"]), (float("-inf"), t["saturating"]["-inf"])]
    assert len(cases) > 500            # every value, every midpoint, the saturating ones that fp16 can hold
    D = 128
    vals = np.array([v for v, _ in cases], dtype=np.float32)
    want = np.array([code for _, code in cases], dtype=np.uint8)
    pad = (-vals.size) % D
    bits = np.concatenate([vals.astype(np.float16).view(np.uint16), np.zeros(pad, np.uint16)]).reshape(-1, D)
    codes, _ = _append_rows(bits, D, cabi.FP8_E4M3)
    assert np.array_equal(codes.reshape(-1)[:vals.size], want)


@pytest.mark.gpu
def test_int8_rows_gpu(dev):
    for row in load("int8_rows.json")["rows"]:
        x = np.array(row["x_f16_bits"], dtype=np.uint16)
        codes, scales = _append_rows(np.tile(x, (3, 1)), x.size, cabi.INT8)          # the same row at three positions
        for i in range(3):
            assert int(scales[i]) == row["scale_f16_bits"] and codes[i].view(np.int8).tolist() == row["codes"]
