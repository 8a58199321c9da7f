"""GPU parity: append / extract / inject / block copy through the C ABI against
the CPU oracle, bit for bit (paged_attention.cu:73-167, cache_kernels.cu:30-187)."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi
from oracle import binding as orc
from tests import util as U

pytestmark = pytest.mark.gpu

GEOMS = [
    # L, KVH, QH, D, bs, NB
    (1, 4, 16, 128, 16, 256),      # BASELINE config 1
    (3, 8, 32, 128, 16, 96),       # config 2 geometry, small pool
    (2, 4, 24, 256, 256, 6),       # the reference's own model geometry (block_pool.h:34-38)
    (2, 2, 4, 64, 32, 24),
    (1, 3, 6, 96, 16, 40),         # non power-of-two heads / dim
]


def _append_case(dev, geom, dtype, M, pos_start, seed, layer_count=None):
    L, KVH, QH, D, bs, NB = geom
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(seed)
    src_dtype = dtype if dtype in (cabi.F16, cabi.BF16) else cabi.BF16
    n_logical = (pos_start + M + bs - 1) // bs
    table = U.shuffled_table(rng, NB, n_logical)
    lc = layer_count or 1
    layer0 = L - lc
    k = U.normal_bits(rng, (lc, M, KVH, D), src_dtype)
    v = U.normal_bits(rng, (lc, M, KVH, D), src_dtype)
    # oracle
    opool = orc.new_pool(og)
    for li in range(lc):
        orc.append_batch(og, opool, table, layer0 + li, pos_start, k[li], v[li], src_dtype)
    # product
    dpool = U.dev_zeros(orc.pool_bytes(og))
    dt, dk, dv = U.dev_i32(table), U.dev_bytes(k), U.dev_bytes(v)
    cabi.call("drk_kv_append_batch", C.byref(g), U.p(dpool), U.p(dt), layer0, lc, pos_start, M,
              U.p(dk), U.p(dv), src_dtype, U.stream_ptr())
    U.sync()
    return g, og, table, opool, dpool, (k, v)


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
def test_append_batch_bit_exact(dev, geom, dtype):
    bs = geom[4]
    M = min(3 * bs + 5, (geom[5] - 1) * bs - 7)
    g, og, table, opool, dpool, _ = _append_case(dev, geom, dtype, M=M, pos_start=7, seed=11)
    assert np.array_equal(U.host(dpool, np.uint8), opool)


def test_config1_append_and_gather(dev):
    """BASELINE config 1: 512 tokens, 256 x 16-token blocks, 4 KV heads x 128, fp16."""
    geom = (1, 4, 16, 128, 16, 256)
    g, og, table, opool, dpool, (k, v) = _append_case(dev, geom, cabi.F16, M=512, pos_start=0, seed=1)
    assert np.array_equal(U.host(dpool, np.uint8), opool)
    # gathered K/V, bit exact, against the oracle and against the source itself
    flat = U.dev_zeros(2 * 512 * 4 * 128 * 2)
    dtab = U.dev_i32(table)
    cabi.call("drk_kv_extract", C.byref(g), U.p(flat), None, U.p(dpool), U.p(dtab), 0, 512, 1, U.stream_ptr())
    U.sync()
    got = U.host(flat, np.uint16, (1, 2, 512, 4, 128))
    want, _ = orc.extract(og, opool, table, 0, 512, 1)
    assert np.array_equal(got, want)
    assert np.array_equal(got[0, 0], k[0]) and np.array_equal(got[0, 1], v[0])


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
def test_append_multi_layer_one_launch(dev, dtype):
    geom = (4, 8, 32, 128, 16, 64)
    g, og, table, opool, dpool, _ = _append_case(dev, geom, dtype, M=100, pos_start=33, seed=5, layer_count=3)
    assert np.array_equal(U.host(dpool, np.uint8), opool)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
def test_append_token_and_branches_equal_batch(dev, dtype):
    """M single-token appends == one batch append; B branches in one launch ==
    B single appends (write_batch(M) == M x write, paged_attention.cu:73-167)."""
    L, KVH, QH, D, bs, NB = 2, 4, 16, 128, 16, 64
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    src_dtype = dtype if dtype in (cabi.F16, cabi.BF16) else cabi.BF16
    rng = np.random.default_rng(3)
    B = 5
    tables = np.stack([U.shuffled_table(rng, NB, 8) for _ in range(B)])
    # make the branches' blocks disjoint
    perm = rng.permutation(NB).astype(np.int32)
    for b in range(B):
        tables[b, :8] = perm[b * 8:(b + 1) * 8]
    pos = np.array([0, 15, 16, 77, 127], dtype=np.int32)
    k = U.normal_bits(rng, (L, B, KVH, D), src_dtype)
    v = U.normal_bits(rng, (L, B, KVH, D), src_dtype)
    opool = orc.new_pool(og)
    for l in range(L):
        for b in range(B):
            orc.append_token(og, opool, tables[b], l, int(pos[b]), k[l, b], v[l, b], src_dtype)
    dpool = U.dev_zeros(orc.pool_bytes(og))
    dtab, dpos, dk, dv = U.dev_i32(tables), U.dev_i32(pos), U.dev_bytes(k), U.dev_bytes(v)
    cabi.call("drk_kv_append_branches", C.byref(g), U.p(dpool), U.p(dtab), tables.shape[1], U.p(dpos), B, 0, L,
              U.p(dk), U.p(dv), src_dtype, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(dpool, np.uint8), opool)
    # the single-token entry point, branch by branch, layer by layer
    dpool2 = U.dev_zeros(orc.pool_bytes(og))
    row = KVH * D * 2
    for l in range(L):
        for b in range(B):
            off = (l * B + b) * row
            cabi.call("drk_kv_append_token", C.byref(g), U.p(dpool2), U.p(dtab[b]), l, U.p(dpos[b:b + 1]),
                      C.c_void_p(dk.data_ptr() + off), C.c_void_p(dv.data_ptr() + off), src_dtype, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(dpool2, np.uint8), opool)


@pytest.fixture(params=["32B_per_thread", "16B_per_thread"])
def quant_form(request):
    """the quantising append has two kernels: 32 source bytes per thread (the default) and 16"""
    cabi.lib().drk_debug_set_quant_append_pairs(1 if request.param == "32B_per_thread" else 0)
    yield request.param
    cabi.lib().drk_debug_set_quant_append_pairs(1)


@pytest.mark.parametrize("dtype", [cabi.INT8, cabi.FP8_E4M3])
@pytest.mark.parametrize("src_dtype", [cabi.F16, cabi.BF16])
def test_quantising_append_bit_exact(dev, quant_form, dtype, src_dtype):
    """int8 codes + fp16 scales / fp8 codes equal the oracle's, with 1% outliers x20
    (BASELINE config 4) and a few crafted rows: zeros, ties, huge values."""
    L, KVH, QH, D, bs, NB = 2, 8, 32, 128, 16, 48
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(44)
    M = 200
    table = U.shuffled_table(rng, NB, (M + bs - 1) // bs + 1)
    x = rng.standard_normal((2, L, M, KVH, D)).astype(np.float32)
    x = np.where(rng.random(x.shape) < 0.01, x * 20.0, x)
    x[0, 0, 0, 0] = 0.0                                   # all-zero row
    x[0, 0, 1, 0] = np.arange(D, dtype=np.float32) - 63.5  # half-way points when the scale is 0.5
    x[0, 0, 1, 0, 0] = 63.5
    x[0, 0, 2, 0] = 30000.0                                # saturating for fp8
    x[0, 0, 3, 0] = 1e-7                                   # scale underflows fp16
    x[1, 0, 4, 1, :8] = [448, 449, 464, 465, 480, -448, -464, 1e4]
    kb, vb = U.to_bits(x[0], src_dtype), U.to_bits(x[1], src_dtype)
    opool = orc.new_pool(og)
    for l in range(L):
        orc.append_batch(og, opool, table, l, 3, kb[l], vb[l], src_dtype)
    dpool = U.dev_zeros(orc.pool_bytes(og))
    dtab, dk, dv = U.dev_i32(table), U.dev_bytes(kb), U.dev_bytes(vb)      # keep the buffers alive
    cabi.call("drk_kv_append_batch", C.byref(g), U.p(dpool), U.p(dtab), 0, L, 3, M, U.p(dk), U.p(dv), src_dtype,
              U.stream_ptr())
    U.sync()
    got = U.host(dpool, np.uint8)
    bad = np.nonzero(got != opool)[0]
    assert bad.size == 0, f"{bad.size} bytes differ, first at {bad[:8]}"


@pytest.mark.parametrize("geom", [(2, 2, 4, 64, 32, 24), (1, 3, 6, 32, 16, 40), (2, 4, 24, 256, 256, 6), (1, 1, 1, 16, 16, 8),
                                  (1, 2, 2, 512, 16, 12), (1, 5, 5, 128, 16, 20)])
@pytest.mark.parametrize("dtype", [cabi.INT8, cabi.FP8_E4M3])
def test_quantising_append_other_head_dims(dev, quant_form, geom, dtype):
    """Rows of 1 to 32 lanes (head_dim 16 .. 512), odd head counts, a start inside a block: pool bytes
    equal the oracle's for both kernels of the quantising append."""
    bs = geom[4]
    M = min(3 * bs + 5, (geom[5] - 1) * bs - 7)
    g, og, table, opool, dpool, _ = _append_case(dev, geom, dtype, M=M, pos_start=7, seed=geom[3] + dtype, layer_count=geom[0])
    assert np.array_equal(U.host(dpool, np.uint8), opool)


def test_int8_scale_math_self_check(dev):
    """The quantising kernels divide by multiply-and-correct; on the device that form and the IEEE
    divisions give the same scale bits and the same reciprocal bits for every bf16 / fp16 magnitude."""
    import torch
    count = torch.zeros(1, dtype=torch.int32, device="cuda")
    cabi.call("drk_debug_check_int8_scale_math", U.p(count), U.stream_ptr())
    U.sync()
    assert int(count.item()) == 0


@pytest.mark.parametrize("src_dtype", [cabi.F16, cabi.BF16])
def test_int8_scales_exhaustive(dev, quant_form, src_dtype):
    """Every non-NaN 16-bit magnitude as the largest element of a row: scale and codes of the int8
    append equal the oracle's (which divides in IEEE fp32)."""
    D = 128
    top = 0x7C00 if src_dtype == cabi.F16 else 0x7F80                  # +inf
    mags = np.arange(top + 1, dtype=np.uint16)
    M = mags.size
    rng = np.random.default_rng(8)
    vals = U.from_bits(mags, src_dtype).astype(np.float64)
    finite = np.where(np.isfinite(vals), vals, 60000.0 if src_dtype == cabi.F16 else 3e38)
    rows = U.to_bits((finite[:, None] * rng.uniform(-1.0, 1.0, (M, D))).astype(np.float32), src_dtype)
    rows[:, 5] = mags | np.where(rng.random(M) < 0.5, 0x8000, 0).astype(np.uint16)
    assert np.all(np.abs(U.from_bits(rows, src_dtype)).max(axis=1) == vals)
    L, KVH, QH, bs = 1, 1, 1, 16
    NB = (M + bs - 1) // bs
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, cabi.INT8)
    table = np.arange(NB, dtype=np.int32)
    src = np.ascontiguousarray(rows.reshape(M, 1, D))
    opool = orc.new_pool(og)
    orc.append_batch(og, opool, table, 0, 0, src, src, src_dtype)
    dpool = U.dev_zeros(orc.pool_bytes(og))
    d, dtab = U.dev_bytes(src), U.dev_i32(table)
    cabi.call("drk_kv_append_batch", C.byref(g), U.p(dpool), U.p(dtab), 0, 1, 0, M, U.p(d), U.p(d), src_dtype,
              U.stream_ptr())
    U.sync()
    got = U.host(dpool, np.uint8)
    bad = np.nonzero(got != opool)[0]
    assert bad.size == 0, f"{bad.size} bytes differ, first at {bad[:8]}"


@pytest.mark.parametrize("src_dtype", [cabi.F16, cabi.BF16])
def test_fp8_codes_exhaustive(dev, quant_form, src_dtype):
    """Every finite 16-bit input pattern through the fp8 append equals the oracle's
    E4M3FN round-half-even code (hardware conversion vs the C restatement)."""
    D = 128
    bits = np.arange(65536, dtype=np.uint16)
    vals = U.from_bits(bits, src_dtype)
    bits = bits[np.isfinite(vals)]
    pad = (-bits.size) % D
    bits = np.concatenate([bits, np.zeros(pad, dtype=np.uint16)])
    M = bits.size // D
    L, KVH, QH, bs = 1, 1, 1, 16
    NB = (M + bs - 1) // bs
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, cabi.FP8_E4M3)
    table = np.arange(NB, dtype=np.int32)
    src = bits.reshape(M, 1, D)
    opool = orc.new_pool(og)
    orc.append_batch(og, opool, table, 0, 0, src, src, src_dtype)
    dpool = U.dev_zeros(orc.pool_bytes(og))
    d, dtab = U.dev_bytes(src), U.dev_i32(table)
    cabi.call("drk_kv_append_batch", C.byref(g), U.p(dpool), U.p(dtab), 0, 1, 0, M, U.p(d), U.p(d), src_dtype,
              U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(dpool, np.uint8), opool)


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
def test_extract_inject_roundtrip_and_holes(dev, geom, dtype):
    """inject then extract returns the input bit for bit; a hole is skipped by
    inject and zero-filled by extract (cache_kernels.cu:64-68, 120)."""
    L, KVH, QH, D, bs, NB = geom
    if dtype in (cabi.INT8, cabi.FP8_E4M3) and D % 16:
        pytest.skip("1-byte rows must be a multiple of 16 bytes")
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(9)
    T = min(2 * bs + 9, (NB - 2) * bs)
    start = 5
    n_logical = (start + T + bs - 1) // bs
    table = U.shuffled_table(rng, NB, n_logical)
    if n_logical >= 2:
        table[1] = -1                                          # a hole
    eb = 2 if dtype in (cabi.F16, cabi.BF16) else 1
    flat = rng.integers(0, 256, size=(L, 2, T, KVH, D * eb), dtype=np.uint8)
    scales = rng.integers(0, 65536, size=(L, 2, T, KVH), dtype=np.uint16) if dtype == cabi.INT8 else None
    opool = orc.new_pool(og)
    orc.inject(og, opool, flat, scales, table, start, T, L)
    dpool = U.dev_zeros(orc.pool_bytes(og))
    dtab = U.dev_i32(table)
    dsc = U.dev_bytes(scales) if scales is not None else None
    dflat = U.dev_bytes(flat)
    cabi.call("drk_kv_inject", C.byref(g), U.p(dpool), U.p(dflat), U.p(dsc), U.p(dtab), start, T, L, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(dpool, np.uint8), opool)
    out = U.dev_bytes(np.full(flat.size, 0xAB, dtype=np.uint8))
    osc = U.dev_bytes(np.full(L * 2 * T * KVH, 0xABAB, dtype=np.uint16)) if scales is not None else None
    cabi.call("drk_kv_extract", C.byref(g), U.p(out), U.p(osc), U.p(dpool), U.p(dtab), start, T, L, U.stream_ptr())
    U.sync()
    want, wsc = orc.extract(og, opool, table, start, T, L)
    got = U.host(out, np.uint8).reshape(flat.shape)
    assert np.array_equal(got, want.view(np.uint8).reshape(flat.shape))
    tok = np.arange(start, start + T)
    hole = (table[tok // bs] < 0)
    assert np.all(got[:, :, hole] == 0)
    assert np.array_equal(got[:, :, ~hole], flat[:, :, ~hole])
    if scales is not None:
        assert np.array_equal(U.host(osc, np.uint16).reshape(scales.shape), wsc)


@pytest.mark.parametrize("dtype", [cabi.BF16, cabi.INT8])
def test_copy_blocks(dev, dtype):
    L, KVH, QH, D, bs, NB = 3, 8, 32, 128, 16, 32
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(2)
    opool = rng.integers(0, 256, size=orc.pool_bytes(og), dtype=np.uint8)
    dpool = U.dev_bytes(opool)
    pairs = np.array([[3, 17], [5, 5], [0, 31], [-1, 4], [9, 2]], dtype=np.int32)
    for s, d in pairs:
        if s >= 0 and d >= 0 and s != d:
            orc.copy_block(og, opool, int(s), int(d))
    dpairs = U.dev_i32(pairs)
    cabi.call("drk_kv_copy_blocks", C.byref(g), U.p(dpool), U.p(dpairs), len(pairs), U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(dpool, np.uint8), opool)


def test_importance_update(dev):
    rng = np.random.default_rng(0)
    n = 1000
    s = rng.random(n).astype(np.float32)
    new = rng.random(n).astype(np.float32)
    want = s.copy()
    orc.lib().orc_importance_update(orc.ptr(want), orc.ptr(new), n, 0.95)
    ds, dn = U.dev_bytes(s), U.dev_bytes(new)
    cabi.call("drk_importance_update", U.p(ds), U.p(dn), n, 0.95, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(ds, np.float32), want)


def test_bad_arguments_are_refused(dev):
    g = cabi.layout(1, 4, 16, 128, 16, 8, cabi.F16)
    d = U.dev_zeros(64)
    L = cabi.lib()
    assert L.drk_kv_append_batch(C.byref(g), U.p(d), U.p(d), 1, 1, 0, 1, U.p(d), U.p(d), cabi.F16, None) == cabi.ERR_INVALID
    assert L.drk_kv_append_batch(C.byref(g), None, U.p(d), 0, 1, 0, 1, U.p(d), U.p(d), cabi.F16, None) == cabi.ERR_INVALID
    assert L.drk_kv_append_batch(C.byref(g), U.p(d), U.p(d), 0, 1, 0, 1, U.p(d), U.p(d), cabi.BF16, None) == cabi.ERR_INVALID
    bad = cabi.layout(1, 3, 16, 128, 16, 8, cabi.F16)
    assert L.drk_kv_layout_check(C.byref(bad)) == cabi.ERR_INVALID
    assert b"multiple" in L.drk_last_error()
