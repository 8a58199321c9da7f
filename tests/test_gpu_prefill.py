"""GPU parity: chunked causal prefill over pages (paged_attention.cu:465-554) --
the MFMA kernels (the 128-row one and the two-phase 256-row one) and the row-wise
path against the fp64 oracle, tolerance |err| <= 2e-2 + 1e-2*|want|."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi
from oracle import binding as orc
from tests import util as U

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["by_rule", "two_phase", "two_phase_through_registers"])
def chunk_kernel(request):
    """Every case runs three times: with the library's own choice of chunk kernel, with the two-phase
    kernels taken wherever their geometry allows (head_dim 128, blocks of 16 * 2^k tokens; 16-bit pages go
    from global memory straight into LDS, 8-bit pages through registers), and with the register kind for
    16-bit pages too, whatever the chunk's length.  Head_dim 256 on 16-bit pages takes its own direct-to-LDS kernel
    in the first two runs and the register-staging kernel in the third."""
    lib = cabi.lib()
    lib.drk_debug_set_prefill_two_phase({"by_rule": 1, "two_phase": 2, "two_phase_through_registers": 3}[request.param])
    yield request.param
    lib.drk_debug_set_prefill_two_phase(1)


def run_prefill(g, dq, dpool, dtab, layer, pos_start, M, scale, dtype, QH, D):
    lib = cabi.lib()
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M)
    ws = U.dev_zeros(max(wsb, 16))
    out = U.dev_bytes(np.full(M * QH * D * 2, 0x7B, dtype=np.uint8))
    cabi.call("drk_paged_prefill_attention", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out), layer, pos_start, M,
              float(scale), dtype, U.p(ws), wsb, U.stream_ptr())
    U.sync()
    return U.host(out, np.uint16, (M, QH, D))


def build(geom, dtype, total, seed, holes=(), mul=1.0):
    L, KVH, QH, D, bs, NB = geom
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(seed)
    nblk = (total + bs - 1) // bs
    table = U.shuffled_table(rng, NB, nblk, nblk + 2)
    opool = orc.new_pool(og)
    k = U.normal_bits(rng, (total, KVH, D), dtype, mul)
    v = U.normal_bits(rng, (total, KVH, D), dtype, mul)
    orc.append_batch(og, opool, table, L - 1, 0, k, v, dtype)
    for h in holes:
        table[h] = -1
    return g, og, rng, table, opool


@pytest.fixture(params=["mfma", "rowwise"])
def path(request):
    cabi.lib().drk_debug_force_portable_decode(1 if request.param == "rowwise" else 0)
    yield request.param
    cabi.lib().drk_debug_force_portable_decode(0)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("pos_start,M", [(0, 1), (0, 32), (0, 200), (37, 45), (64, 64), (100, 129), (509, 77), (1000, 256)])
def test_prefill_matches_oracle(dev, path, dtype, pos_start, M):
    geom = (2, 4, 16, 128, 16, 100)
    g, og, rng, table, opool = build(geom, dtype, pos_start + M, seed=pos_start * 7 + M)
    QH, D = geom[2], geom[3]
    q = U.normal_bits(rng, (M, QH, D), dtype)
    scale = 1 / np.sqrt(D)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    got = U.from_bits(run_prefill(g, dq, dpool, dtab, 1, pos_start, M, scale, dtype, QH, D), dtype)
    want = orc.prefill_f64(og, q, opool, table, 1, pos_start, scale, dtype)
    ok, ma, _ = U.rel_abs_ok(got, want)
    assert ok, ma


def test_first_row_of_first_chunk_is_v0_bitwise(dev, path):
    geom = (1, 4, 16, 128, 16, 16)
    g, og, rng, table, opool = build(geom, cabi.BF16, 40, seed=3)
    q = U.normal_bits(rng, (40, 16, 128), cabi.BF16)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    got = run_prefill(g, dq, dpool, dtab, 0, 0, 40, 0.1, cabi.BF16, 16, 128)
    flat, _ = orc.extract(og, opool, table, 0, 1, 1)
    assert np.array_equal(got[0], np.repeat(flat[0, 1, 0], 4, axis=0))


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
def test_chunked_prefill_config5_small(dev, dtype):
    """BASELINE config 5 in small: chunks appended into 16-token pages, causal
    attention over all prior pages plus the chunk, 32 Q / 8 KV heads x 128; every
    chunk's rows must equal decode attention at that row's length."""
    L, KVH, QH, D, bs, NB = 1, 8, 32, 128, 16, 80
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(55)
    chunk, nchunks = 160, 6
    total = chunk * nchunks
    table = U.shuffled_table(rng, NB, (total + bs - 1) // bs)
    dpool = U.dev_zeros(orc.pool_bytes(og))
    dtab = U.dev_i32(table)
    opool = orc.new_pool(og)
    scale = 1 / np.sqrt(D)
    for c in range(nchunks):
        k = U.normal_bits(rng, (chunk, KVH, D), dtype)
        v = U.normal_bits(rng, (chunk, KVH, D), dtype)
        q = U.normal_bits(rng, (chunk, QH, D), dtype)
        dk, dv, dq = U.dev_bytes(k), U.dev_bytes(v), U.dev_bytes(q)
        cabi.call("drk_kv_append_batch", C.byref(g), U.p(dpool), U.p(dtab), 0, 1, c * chunk, chunk, U.p(dk), U.p(dv),
                  dtype, U.stream_ptr())
        orc.append_batch(og, opool, table, 0, c * chunk, k, v, dtype)
        got = U.from_bits(run_prefill(g, dq, dpool, dtab, 0, c * chunk, chunk, scale, dtype, QH, D), dtype)
        rows = [0, 1, 31, 32, 77, chunk - 1]
        for t in rows:
            want = orc.decode_f64(og, q[t], opool, table, 0, c * chunk + t + 1, scale, dtype)
            ok, ma, _ = U.rel_abs_ok(got[t], want)
            assert ok, (c, t, ma)
    assert np.array_equal(U.host(dpool, np.uint8), opool)


def test_prefill_with_holes_and_stale_rows(dev, path):
    geom = (1, 4, 16, 128, 16, 64)
    pos_start, M = 130, 70
    g, og, rng, table, opool = build(geom, cabi.BF16, pos_start + M, seed=9, holes=(1, 5))
    # NaN patterns in the slots of the last page past the end
    flat = np.full((1, 2, 8, 4, 128), 0x7FC0, dtype=np.uint16)
    orc.inject(og, opool, flat, None, table, pos_start + M, 8, 1)
    q = U.normal_bits(rng, (M, 16, 128), cabi.BF16)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    scale = 1 / np.sqrt(128)
    got = U.from_bits(run_prefill(g, dq, dpool, dtab, 0, pos_start, M, scale, cabi.BF16, 16, 128), cabi.BF16)
    want = orc.prefill_f64(og, q, opool, table, 0, pos_start, scale, cabi.BF16)
    ok, ma, _ = U.rel_abs_ok(got, want)
    assert ok, ma


def test_mfma_and_rowwise_paths_agree(dev):
    geom = (1, 8, 32, 128, 16, 120)
    pos_start, M = 1024, 512
    g, og, rng, table, opool = build(geom, cabi.BF16, pos_start + M, seed=21, mul=0.7)
    q = U.normal_bits(rng, (M, 32, 128), cabi.BF16, 0.7)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    scale = 1 / np.sqrt(128)
    a = U.from_bits(run_prefill(g, dq, dpool, dtab, 0, pos_start, M, scale, cabi.BF16, 32, 128), cabi.BF16)
    cabi.lib().drk_debug_force_portable_decode(1)
    try:
        b = U.from_bits(run_prefill(g, dq, dpool, dtab, 0, pos_start, M, scale, cabi.BF16, 32, 128), cabi.BF16)
    finally:
        cabi.lib().drk_debug_force_portable_decode(0)
    ok, ma, _ = U.rel_abs_ok(a, b)
    assert ok, ma


def build_io(geom, dtype, io, total, seed, holes=(), mul=1.0):
    """like build(), for a pool whose storage type differs from the type K/V arrive in"""
    L, KVH, QH, D, bs, NB = geom
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(seed)
    nblk = (total + bs - 1) // bs
    table = U.shuffled_table(rng, NB, nblk, nblk + 2)
    opool = orc.new_pool(og)
    opool[:] = 0xFF                                               # stale bytes everywhere first
    k = U.normal_bits(rng, (total, KVH, D), io, mul)
    v = U.normal_bits(rng, (total, KVH, D), io, mul)
    orc.append_batch(og, opool, table, L - 1, 0, k, v, io)
    for h in holes:
        table[h] = -1
    return g, og, rng, table, opool


@pytest.mark.parametrize("geom,dtype,io", [((1, 8, 32, 128, 16, 100), cabi.INT8, cabi.BF16), ((1, 8, 32, 128, 16, 100), cabi.FP8_E4M3, cabi.BF16),
                                           ((1, 8, 32, 128, 16, 100), cabi.INT8, cabi.F16), ((1, 8, 32, 128, 16, 100), cabi.FP8_E4M3, cabi.F16),
                                           ((2, 4, 24, 256, 256, 8), cabi.F16, cabi.F16), ((1, 2, 32, 128, 16, 100), cabi.BF16, cabi.BF16),
                                           ((1, 4, 4, 128, 16, 100), cabi.BF16, cabi.BF16), ((1, 2, 6, 256, 16, 100), cabi.INT8, cabi.BF16),
                                           ((1, 2, 10, 128, 32, 60), cabi.F16, cabi.F16), ((1, 2, 16, 128, 16, 100), cabi.FP8_E4M3, cabi.F16)])
@pytest.mark.parametrize("pos_start,M", [(0, 1), (0, 70), (37, 45), (509, 77), (1000, 300)])
def test_prefill_of_8bit_pages_and_other_head_shapes(dev, geom, dtype, io, pos_start, M):
    """The MFMA prefill kernel away from the headline shape: 8-bit pages (codes dequantised on their
    way into LDS; int8: code * scale rounded to fp16 once), head_dim 256, and 4, 6, 16, 1, 3, 5, 8 query
    heads per kv head (a workgroup's 128 rows are 128 / G tokens x G heads).  A hole in the table,
    stale bytes behind the end.  Against the fp64 oracle, the gated form against plain + gate, and
    not the bits of the row-wise path."""
    L, KVH, QH, D, bs, NB = geom
    holes = (1,) if pos_start + M > 3 * bs else ()
    g, og, rng, table, opool = build_io(geom, dtype, io, pos_start + M, seed=pos_start * 5 + M + D, holes=holes, mul=0.7)
    q = U.normal_bits(rng, (M, QH, D), io, 0.7)
    qg = U.normal_bits(rng, (M, QH, 2 * D), io, 2.0)
    scale = 1 / np.sqrt(D)
    dq, dpool, dtab, dqg = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table), U.dev_bytes(qg)
    raw = run_prefill(g, dq, dpool, dtab, L - 1, pos_start, M, scale, io, QH, D)
    want = orc.prefill_f64(og, q, opool, table, L - 1, pos_start, scale, io)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(raw, io), want)
    assert ok, ma
    lib = cabi.lib()
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M)
    assert wsb < 64 << 20
    ws = U.dev_zeros(max(wsb, 16))
    out = U.dev_zeros(M * QH * D * 2)
    gptr = C.c_void_p(dqg.data_ptr() + D * 2)
    cabi.call("drk_paged_prefill_attention_gated", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out), L - 1, pos_start, M,
              float(scale), io, gptr, 2 * D, U.p(ws), wsb, U.stream_ptr())
    U.sync()
    gated = orc.sigmoid_gate(raw, np.ascontiguousarray(qg[:, :, D:]), io)
    assert U.ulp_distance(U.host(out, np.uint16, (M, QH, D)), gated).max() <= 1
    # and it is not the row-wise path that produced the bits
    lib.drk_debug_force_portable_decode(1)
    try:
        other = run_prefill(g, dq, dpool, dtab, L - 1, pos_start, M, scale, io, QH, D)
    finally:
        lib.drk_debug_force_portable_decode(0)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(other, io), want)
    assert ok, ma
    if M > 1:
        assert not np.array_equal(other, raw)


@pytest.mark.parametrize("seed", range(12))
def test_random_prefill_shapes(dev, seed):
    """A seeded draw over what the MFMA kernel takes: head_dim 128 / 256, 1..16 query heads per kv head
    (powers of two and not), blocks of 16..256 tokens, every storage type, any chunk position and
    length, holes, stale bytes -- against fp64 on the stored values."""
    rng = np.random.default_rng(2000 + seed)
    D = int(rng.choice([128, 256]))
    KVH = int(rng.choice([1, 2, 4]))
    G = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 12, 16]))
    bs = int(rng.choice([16, 32, 48, 64, 256]))
    dtype = int(rng.choice([cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3]))
    io = dtype if dtype in (cabi.F16, cabi.BF16) else int(rng.choice([cabi.F16, cabi.BF16]))
    pos_start = int(rng.choice([0, 1, 63, 64, 65, int(rng.integers(0, 900))]))
    M = int(rng.choice([1, 31, 32, 33, 127, 128, 129, int(rng.integers(1, 400))]))
    total = pos_start + M
    nblk = (total + bs - 1) // bs
    holes = tuple(int(h) for h in rng.choice(nblk, size=min(nblk - 1, int(rng.integers(0, 3))), replace=False)) if nblk > 1 else ()
    geom = (2, KVH, KVH * G, D, bs, nblk + 3)
    g, og, rng2, table, opool = build_io(geom, dtype, io, total, seed=seed, holes=holes, mul=0.7)
    q = U.normal_bits(rng2, (M, KVH * G, D), io, 0.7)
    scale = 1 / np.sqrt(D)
    got = run_prefill(g, U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table), 1, pos_start, M, scale, io, KVH * G, D)
    want = orc.prefill_f64(og, q, opool, table, 1, pos_start, scale, io)
    # a row that sees no token (every page before it is a hole) keeps the bytes the caller left in out
    seen = np.array([any(table[t // bs] >= 0 for t in range(pos_start + r + 1)) for r in range(M)])
    assert np.all(got[~seen].view(np.uint8) == 0x7B)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(got[seen], io), want[seen])
    assert ok, f"max abs err {ma:.4g} ({D=} {KVH=} {G=} {bs=} {dtype=} {pos_start=} {M=} {holes=})"


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("bs,G,pos_start,M,holes", [
    (16, 4, 700, 150, (3, 44)), (32, 1, 1, 300, (0,)), (64, 3, 640, 64, (9,)), (128, 8, 1023, 33, ()), (256, 2, 900, 257, (1,)),
    (16, 16, 0, 600, (5, 6, 7, 8)), (32, 5, 2047, 2, ()), (16, 4, 4096, 256, (100, 255))])
def test_ring_of_tiles_wraps_over_holes_and_ragged_ends(dev, chunk_kernel, dtype, bs, G, pos_start, M, holes):
    """16-bit pages with head_dim 128 on the kernel that loads tiles straight into LDS (the forced two-phase run of
    this case; the other two runs take the same inputs through the other kernels): walks of 10 to 70 tiles, so that
    the ring of tile buffers wraps many times, with missing pages (whole tiles of them with 16-token blocks), chunks
    that end inside a page and inside a tile, every block size the kernel takes and group sizes that are not powers of
    two.  Rows behind holes only keep the caller's bytes; everything else against fp64 on the stored values."""
    KVH, D = 2, 128
    total = pos_start + M
    nblk = (total + bs - 1) // bs
    holes = tuple(h for h in holes if h < nblk)
    geom = (2, KVH, KVH * G, D, bs, nblk + 3)
    g, og, rng, table, opool = build(geom, dtype, total, seed=bs * 1000 + G, holes=holes, mul=0.7)
    q = U.normal_bits(rng, (M, KVH * G, D), dtype, 0.7)
    scale = 1 / np.sqrt(D)
    got = run_prefill(g, U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table), 1, pos_start, M, scale, dtype, KVH * G, D)
    want = orc.prefill_f64(og, q, opool, table, 1, pos_start, scale, dtype)
    seen = np.array([any(table[t // bs] >= 0 for t in range(pos_start + r + 1)) for r in range(M)])
    assert np.all(got[~seen].view(np.uint8) == 0x7B)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(got[seen], dtype), want[seen])
    assert ok, f"max abs err {ma:.4g} ({chunk_kernel=} {bs=} {G=} {pos_start=} {M=} {holes=})"


@pytest.fixture(params=["score_and_value_waves", "one_wave_per_simd"])
def d256_waves(request):
    """The two head_dim 256 chunk kernels for 16-bit pages: eight waves, a score wave and a value wave per 32 rows
    (the library's default), and four waves that do both products."""
    lib = cabi.lib()
    lib.drk_debug_set_prefill_d256_waves(1 if request.param == "score_and_value_waves" else 0)
    yield request.param
    lib.drk_debug_set_prefill_d256_waves(1)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("bs,G,pos_start,M,holes", [
    (256, 6, 900, 257, (1,)), (16, 2, 0, 300, (3, 4, 5, 6, 17)), (64, 6, 1500, 100, (20,)), (32, 1, 33, 130, ()),
    (128, 12, 2047, 22, (0,)), (16, 6, 640, 64, (40, 43))])
def test_head_dim_256_over_holes_and_ragged_ends(dev, chunk_kernel, d256_waves, dtype, bs, G, pos_start, M, holes):
    """16-bit pages with head_dim 256 (the reference model's: 24 query over 4 kv heads, blocks of 256 tokens) on the
    kernels that load tiles straight into LDS (the first two runs of this case, each with both arrangements of waves;
    the third takes the register-staging kernel): walks of up to 35 tiles over missing pages, chunk ends inside a page and inside a
    tile, query tiles of 21, 64, 128, 10 tokens.  Rows behind holes only keep the caller's bytes; everything else
    against fp64 on the stored values."""
    KVH, D = 2, 256
    total = pos_start + M
    nblk = (total + bs - 1) // bs
    holes = tuple(h for h in holes if h < nblk)
    geom = (2, KVH, KVH * G, D, bs, nblk + 3)
    g, og, rng, table, opool = build(geom, dtype, total, seed=bs * 1000 + G + 7, holes=holes, mul=0.7)
    q = U.normal_bits(rng, (M, KVH * G, D), dtype, 0.7)
    scale = 1 / np.sqrt(D)
    got = run_prefill(g, U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table), 1, pos_start, M, scale, dtype, KVH * G, D)
    want = orc.prefill_f64(og, q, opool, table, 1, pos_start, scale, dtype)
    seen = np.array([any(table[t // bs] >= 0 for t in range(pos_start + r + 1)) for r in range(M)])
    assert np.all(got[~seen].view(np.uint8) == 0x7B)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(got[seen], dtype), want[seen])
    assert ok, f"max abs err {ma:.4g} ({chunk_kernel=} {bs=} {G=} {pos_start=} {M=} {holes=})"


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("bs,KVH,G,pos_start,M,holes", [
    (256, 4, 6, 900, 257, (1,)), (16, 2, 2, 0, 300, (3, 4, 5, 6, 17)), (64, 2, 6, 1500, 100, (20,)), (32, 2, 1, 33, 130, ()),
    (128, 1, 12, 2047, 22, (0,)), (16, 2, 6, 640, 64, (40, 43)), (16, 4, 6, 64, 2048, (7,)), (16, 3, 5, 3, 50, ())])
def test_head_dim_256_walks_cut_into_pieces(dev, d256_waves, dtype, bs, KVH, G, pos_start, M, holes):
    """The workgroups of the head_dim 256 kernel's last round take pieces of their walks (ranges of tiles) and a merge
    folds them: forced here for every shape (2 to 8 pieces, walks shorter than their number of pieces, the reference
    model's 24 / 4 heads on a full 2 048-row chunk: 384 walks, the last 128 in two pieces each), against fp64 and
    against the same call with whole walks; rows behind holes only keep the caller's bytes."""
    lib = cabi.lib()
    D = 256
    total = pos_start + M
    nblk = (total + bs - 1) // bs
    holes = tuple(h for h in holes if h < nblk)
    geom = (2, KVH, KVH * G, D, bs, nblk + 3)
    g, og, rng, table, opool = build(geom, dtype, total, seed=bs * 1000 + G + 11, holes=holes, mul=0.7)
    q = U.normal_bits(rng, (M, KVH * G, D), dtype, 0.7)
    scale = 1 / np.sqrt(D)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    try:
        lib.drk_debug_set_prefill_two_phase(1)              # whatever the fixture chose: the kernel that loads tiles straight into LDS
        lib.drk_debug_set_prefill_pieces(2)
        assert lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M) > 0
        got = run_prefill(g, dq, dpool, dtab, 1, pos_start, M, scale, dtype, KVH * G, D)
        lib.drk_debug_set_prefill_pieces(0)
        whole = run_prefill(g, dq, dpool, dtab, 1, pos_start, M, scale, dtype, KVH * G, D)
    finally:
        lib.drk_debug_set_prefill_pieces(1)
    seen = np.array([any(table[t // bs] >= 0 for t in range(pos_start + r + 1)) for r in range(M)])
    assert np.all(got[~seen].view(np.uint8) == 0x7B)
    a, b = U.from_bits(got[seen], dtype), U.from_bits(whole[seen], dtype)
    assert np.abs(a - b).max() <= 2e-2 * max(1.0, np.abs(b).max())
    if M <= 300:
        want = orc.prefill_f64(og, q, opool, table, 1, pos_start, scale, dtype)
        ok, ma, _ = U.rel_abs_ok(a, want[seen])
        assert ok, f"max abs err {ma:.4g}"
    else:                                                   # the long chunk: a sample of rows against fp64
        rows = np.array([0, 1, 63, 64, 1000, 1343, 1344, 2047])
        for rsel in rows:
            w1 = orc.decode_f64(og, q[rsel], opool, table, 1, pos_start + int(rsel) + 1, scale, dtype)
            ok, ma, _ = U.rel_abs_ok(U.from_bits(got[rsel], dtype), w1)
            assert ok, (int(rsel), ma)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("bs,KVH,G,pos_start,M,holes,pieces", [
    (256, 4, 6, 900, 257, (1,), 0), (16, 2, 2, 0, 300, (3, 4, 5, 6, 17), 2), (64, 2, 6, 1500, 100, (20,), 0),
    (128, 1, 12, 2047, 22, (0,), 2), (16, 4, 6, 4096, 2048, (7, 200), 1), (16, 3, 5, 3, 50, (), 2)])
def test_head_dim_256_wave_arrangements_give_the_same_bits(dev, dtype, bs, KVH, G, pos_start, M, holes, pieces):
    """The eight-wave kernel splits the work of the four-wave kernel between two waves per 32 rows and keeps its
    arithmetic and its order: outputs and row log-sum-exps of the two are the same bits, with whole walks, with the
    library's rule for pieces (a 2 048-row chunk behind 4 096 tokens) and with pieces forced."""
    lib = cabi.lib()
    D, QH = 256, KVH * G
    total = pos_start + M
    nblk = (total + bs - 1) // bs
    holes = tuple(h for h in holes if h < nblk)
    g, og, rng, table, opool = build((2, KVH, QH, D, bs, nblk + 3), dtype, total, seed=bs * 77 + G, holes=holes, mul=0.7)
    q = U.normal_bits(rng, (M, QH, D), dtype, 0.7)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    res = []
    try:
        lib.drk_debug_set_prefill_two_phase(1)
        lib.drk_debug_set_prefill_pieces(pieces)
        wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M)
        ws = U.dev_zeros(max(wsb, 16))
        for waves in (1, 0):
            lib.drk_debug_set_prefill_d256_waves(waves)
            out = U.dev_bytes(np.full(M * QH * D * 2, 0x7B, dtype=np.uint8))
            lse = U.dev_bytes(np.full(M * QH * 4, 0x7B, dtype=np.uint8))
            cabi.call("drk_paged_prefill_attention_lse", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out), 1, pos_start, M,
                      float(1 / np.sqrt(D)), dtype, None, 0, U.p(lse), U.p(ws), wsb, U.stream_ptr())
            U.sync()
            res.append((U.host(out, np.uint16, (M, QH, D)), U.host(lse, np.uint32, (M, QH))))
    finally:
        lib.drk_debug_set_prefill_pieces(1)
        lib.drk_debug_set_prefill_d256_waves(1)
    assert np.array_equal(res[0][0], res[1][0])
    assert np.array_equal(res[0][1], res[1][1])
    assert not np.all(res[0][0].view(np.uint8) == 0x7B)


@pytest.mark.parametrize("geom,dtype,io", [((2, 8, 32, 128, 16, 300), cabi.BF16, cabi.BF16), ((2, 4, 24, 256, 256, 20), cabi.F16, cabi.F16),
                                           ((2, 2, 8, 128, 32, 150), cabi.INT8, cabi.BF16), ((2, 2, 12, 128, 16, 300), cabi.FP8_E4M3, cabi.F16)])
@pytest.mark.parametrize("pos_start,M", [(2048, 1), (2049, 17), (3000, 64), (4095, 65), (2500, 130), (2048, 256)])
def test_short_chunks_behind_a_long_context(dev, geom, dtype, io, pos_start, M):
    """A chunk of up to 1 024 tokens behind 2 048 or more runs with the context split over the chip (the
    kernel's shared-prefix mode with rows = query tokens, then a merge): against the fp64 oracle, against
    the chunk kernel, the gated form against plain + gate; a hole in the table, stale bytes behind the end."""
    L, KVH, QH, D, bs, NB = geom
    lib = cabi.lib()
    g, og, rng, table, opool = build_io(geom, dtype, io, pos_start + M, seed=pos_start + M + D, holes=(2,), mul=0.7)
    q = U.normal_bits(rng, (M, QH, D), io, 0.7)
    qg = U.normal_bits(rng, (M, QH, 2 * D), io, 2.0)
    scale = 1 / np.sqrt(D)
    dq, dpool, dtab, dqg = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table), U.dev_bytes(qg)
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M)
    assert wsb > 0                                                  # the split path asks for room for its partial results
    raw = run_prefill(g, dq, dpool, dtab, L - 1, pos_start, M, scale, io, QH, D)
    got = U.from_bits(raw, io)
    want = orc.prefill_f64(og, q, opool, table, L - 1, pos_start, scale, io)
    ok, ma, _ = U.rel_abs_ok(got, want)
    assert ok, ma
    lib.drk_debug_set_prefill_split(0)
    lib.drk_debug_set_prefill_pieces(0)                    # head_dim 256 would cut its walks into pieces otherwise
    try:
        assert lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M) == 0
        chunk = U.from_bits(run_prefill(g, dq, dpool, dtab, L - 1, pos_start, M, scale, io, QH, D), io)
    finally:
        lib.drk_debug_set_prefill_split(-1)
        lib.drk_debug_set_prefill_pieces(1)
    assert np.max(np.abs(chunk - got)) <= 2e-2                      # two summation orders of the same sums
    ws = U.dev_zeros(wsb)
    out = U.dev_zeros(M * QH * D * 2)
    gptr = C.c_void_p(dqg.data_ptr() + D * 2)
    cabi.call("drk_paged_prefill_attention_gated", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out), L - 1, pos_start, M,
              float(scale), io, gptr, 2 * D, U.p(ws), wsb, U.stream_ptr())
    U.sync()
    gated = orc.sigmoid_gate(raw, np.ascontiguousarray(qg[:, :, D:]), io)
    assert U.ulp_distance(U.host(out, np.uint16, (M, QH, D)), gated).max() <= 1


def test_prefill_refuses_a_scale_that_is_not_positive_and_sizes_follow_the_debug_switch(dev):
    """The size a caller reserves once must cover what the split path asks for also when the debug switch widens
    that path; a softmax scale of zero or less is refused before anything is launched."""
    lib = cabi.lib()
    geom = (1, 8, 32, 128, 16, 600)
    g = cabi.layout(*geom, cabi.BF16)
    try:
        lib.drk_debug_set_prefill_split(1500)
        top = lib.drk_prefill_workspace_bytes_max(C.byref(g), 8192, 2048)
        assert top >= lib.drk_prefill_workspace_bytes(C.byref(g), 8192 - 1500, 1500) > 0
    finally:
        lib.drk_debug_set_prefill_split(-1)
    buf = U.dev_zeros(64 * 32 * 128 * 2)
    pool = U.dev_zeros(lib.drk_kv_pool_bytes(C.byref(g)))
    tab = U.dev_i32(np.arange(600, dtype=np.int32))
    for scale in (0.0, -0.1, float("nan")):
        rc = lib.drk_paged_prefill_attention(C.byref(g), U.p(buf), U.p(pool), U.p(tab), U.p(buf), 0, 0, 64, scale, cabi.BF16,
                                             None, 0, U.stream_ptr())
        assert rc == cabi.ERR_INVALID and b"scale" in lib.drk_last_error()
