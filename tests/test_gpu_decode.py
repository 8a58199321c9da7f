"""GPU parity: paged GQA decode attention (and the row-wise prefill built on it)
through the C ABI against the CPU oracle (paged_attention.cu:179-282, 465-554).

Tolerance, from the task statement: |got - want| <= 2e-2 + 1e-2*|want| against an
fp64 softmax(QK^T*scale)V evaluated on the same stored K/V."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi
from oracle import binding as orc
from tests import util as U

pytestmark = pytest.mark.gpu

REL, ABS = 1e-2, 2e-2


class Case:
    """A filled pool on host (oracle) and device, B branches with disjoint pages."""

    def __init__(self, geom, dtype, seq_lens, seed, mul=1.0, io_dtype=None, holes=(), outliers=False, stale=0):
        L, KVH, QH, D, bs, NB = geom
        self.geom, self.dtype = geom, dtype
        self.io = io_dtype if io_dtype is not None else (dtype if dtype in (cabi.F16, cabi.BF16) else cabi.BF16)
        self.g, self.og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
        rng = np.random.default_rng(seed)
        self.rng = rng
        self.seq_lens = np.asarray(seq_lens, dtype=np.int32)
        B = len(seq_lens)
        nblk = [(int(s) + bs - 1) // bs for s in seq_lens]
        self.stride = max(max(nblk), 1) + 2
        perm = rng.permutation(NB).astype(np.int32)
        assert sum(nblk) <= NB
        self.tables = np.full((B, self.stride), -1, dtype=np.int32)
        o = 0
        for b in range(B):
            self.tables[b, :nblk[b]] = perm[o:o + nblk[b]]
            o += nblk[b]
        self.opool = orc.new_pool(self.og)
        # stale garbage everywhere first: positions past seq_len must not matter
        self.opool[:] = stale
        self.layer = L - 1
        for b in range(B):
            n = int(seq_lens[b])
            if n == 0:
                continue
            kf = rng.standard_normal((n, KVH, D)).astype(np.float32) * np.float32(mul)
            vf = rng.standard_normal((n, KVH, D)).astype(np.float32) * np.float32(mul)
            if outliers:
                kf = np.where(rng.random(kf.shape) < 0.01, kf * 20, kf)
                vf = np.where(rng.random(vf.shape) < 0.01, vf * 20, vf)
            k, v = U.to_bits(kf, self.io), U.to_bits(vf, self.io)
            orc.append_batch(self.og, self.opool, self.tables[b], self.layer, 0, k, v, self.io)
        for (b, lb) in holes:
            self.tables[b, lb] = -1
        self.q = U.normal_bits(rng, (B, QH, D), self.io, mul)
        self.scale = 1.0 / np.sqrt(D)
        self.dpool = U.dev_bytes(self.opool)
        self.dtab = U.dev_i32(self.tables)
        self.dq = U.dev_bytes(self.q)
        self.dlens = U.dev_i32(self.seq_lens)

    def want_f64(self):
        return np.stack([orc.decode_f64(self.og, self.q[b], self.opool, self.tables[b], self.layer,
                                        int(self.seq_lens[b]), self.scale, self.io)
                         for b in range(len(self.seq_lens))])

    def run_branches(self, split=0, fill=0x7B):
        B = len(self.seq_lens)
        QH, D = self.geom[2], self.geom[3]
        mx = int(self.seq_lens.max())
        L = cabi.lib()
        ws_bytes = (L.drk_decode_workspace_bytes_for_split(C.byref(self.g), B, mx, split) if split
                    else L.drk_decode_workspace_bytes(C.byref(self.g), B, mx))
        ws = U.dev_zeros(max(ws_bytes, 16))
        out = U.dev_bytes(np.full(B * QH * D * 2, fill, dtype=np.uint8))
        cabi.call("drk_paged_decode_attention_branches", C.byref(self.g), U.p(self.dq), U.p(self.dpool),
                  U.p(self.dtab), self.stride, U.p(self.dlens), B, mx, U.p(out), self.layer,
                  float(self.scale), self.io, split, U.p(ws), ws_bytes, U.stream_ptr())
        U.sync()
        return U.host(out, np.uint16, (B, QH, D))

    def run_single(self, b):
        QH, D = self.geom[2], self.geom[3]
        n = int(self.seq_lens[b])
        L = cabi.lib()
        ws_bytes = L.drk_decode_workspace_bytes(C.byref(self.g), 1, max(n, 1))
        ws = U.dev_zeros(max(ws_bytes, 16))
        out = U.dev_bytes(np.full(QH * D * 2, 0x7B, dtype=np.uint8))
        cabi.call("drk_paged_decode_attention", C.byref(self.g), U.p(self.dq[b * QH * D * 2:]), U.p(self.dpool),
                  U.p(self.dtab[b]), U.p(out), self.layer, n, float(self.scale), self.io, U.p(ws), ws_bytes,
                  U.stream_ptr())
        U.sync()
        return U.host(out, np.uint16, (QH, D))


def _check(case, got):
    want = case.want_f64()
    ok, max_abs, max_rel = U.rel_abs_ok(U.from_bits(got, case.io), want, REL, ABS)
    assert ok, f"max abs err {max_abs:.4g}, max rel err {max_rel:.4g}"
    return max_abs


@pytest.fixture(params=["stream", "tiled", "portable"])
def kernel(request):
    cabi.lib().drk_debug_force_portable_decode(1 if request.param == "portable" else 0)
    cabi.lib().drk_debug_set_decode_kernel(2 if request.param == "tiled" else 0)
    yield request.param
    cabi.lib().drk_debug_force_portable_decode(0)
    cabi.lib().drk_debug_set_decode_kernel(0)


def test_config1_decode(dev, kernel):
    """BASELINE config 1: 512 tokens, fp16, 16 Q heads over 4 KV heads x 128."""
    case = Case((1, 4, 16, 128, 16, 256), cabi.F16, [512], seed=1)
    got = case.run_single(0)
    _check(case, got[None])
    # and against the restatement of the reference's own summation order
    ref = orc.decode_ref_order(case.og, case.q[0], case.opool, case.tables[0], 0, 512, case.scale, cabi.F16)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(got, cabi.F16), U.from_bits(ref, cabi.F16), REL, ABS)
    assert ok, ma


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("n", [1, 2, 15, 16, 17, 63, 64, 65, 127, 129, 1000, 2049, 4100])
def test_decode_lengths(dev, kernel, dtype, n):
    case = Case((2, 8, 32, 128, 16, 300), dtype, [n], seed=100 + n, mul=0.5)
    _check(case, case.run_single(0)[None])


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
def test_seq_len_one_returns_v0_bitwise(dev, kernel, dtype):
    """softmax over one token is 1, so out == V[0] exactly."""
    case = Case((1, 4, 16, 128, 16, 8), dtype, [1], seed=7)
    got = case.run_single(0)
    flat, _ = orc.extract(case.og, case.opool, case.tables[0], 0, 1, 1)
    v0 = flat[0, 1, 0]                                  # [KVH, D]
    assert np.array_equal(got, np.repeat(v0, 4, axis=0))


def test_equal_keys_give_mean_of_values(dev, kernel):
    L, KVH, QH, D, bs, NB = 1, 4, 16, 128, 16, 64
    case = Case((L, KVH, QH, D, bs, NB), cabi.BF16, [300], seed=8)
    rng = np.random.default_rng(5)
    krow = U.normal_bits(rng, (1, KVH, D), cabi.BF16)
    k = np.repeat(krow, 300, axis=0)
    v = U.normal_bits(rng, (300, KVH, D), cabi.BF16)
    case.opool[:] = 0
    orc.append_batch(case.og, case.opool, case.tables[0], case.layer, 0, k, v, cabi.BF16)
    case.dpool = U.dev_bytes(case.opool)
    got = U.from_bits(case.run_single(0), cabi.BF16)
    mean_v = U.from_bits(v, cabi.BF16).astype(np.float64).mean(axis=0)      # [KVH, D]
    ok, ma, _ = U.rel_abs_ok(got, np.repeat(mean_v, 4, axis=0), REL, ABS)
    assert ok, ma


def test_same_q_in_a_group_gives_same_out(dev, kernel):
    case = Case((1, 4, 16, 128, 16, 64), cabi.F16, [200], seed=9)
    case.q[0, 1] = case.q[0, 0]
    case.q[0, 2] = case.q[0, 0]
    case.dq = U.dev_bytes(case.q)
    got = case.run_single(0)
    assert np.array_equal(got[0], got[1]) and np.array_equal(got[0], got[2])


def test_physical_placement_does_not_change_bits(dev, kernel):
    """Same logical content in different physical blocks => identical output bits."""
    geom = (1, 8, 32, 128, 16, 128)
    a = Case(geom, cabi.BF16, [700], seed=21)
    b = Case(geom, cabi.BF16, [700], seed=21)
    rng = np.random.default_rng(99)
    new_tab = U.shuffled_table(rng, geom[5], (700 + 15) // 16, b.stride)
    flat, _ = orc.extract(a.og, a.opool, a.tables[0], 0, 700, 1)
    b.opool[:] = 0
    orc.inject(b.og, b.opool, flat, None, new_tab, 0, 700, 1)
    b.tables[0] = new_tab
    b.dpool, b.dtab = U.dev_bytes(b.opool), U.dev_i32(b.tables)
    b.q, b.dq = a.q, a.dq
    assert not np.array_equal(a.tables, b.tables)
    assert np.array_equal(a.run_single(0), b.run_single(0))


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
def test_branches_match_single_calls_and_oracle(dev, kernel, dtype):
    """8 branches of ragged length in one launch (BASELINE config 2 shape, small)."""
    lens = [1024, 77, 3000, 1, 2048, 555, 16, 1999]
    case = Case((2, 8, 32, 128, 16, 700), dtype, lens, seed=31, mul=0.5)
    got = case.run_branches(split=256)
    _check(case, got)
    auto = case.run_branches(split=0)
    _check(case, auto)


def test_split_size_changes_nothing_beyond_rounding(dev, kernel):
    case = Case((1, 8, 32, 128, 16, 300), cabi.BF16, [4000], seed=41)
    outs = [U.from_bits(case.run_branches(split=s), cabi.BF16) for s in (64, 512, 4096)]
    _check(case, case.run_branches(split=64))
    for o in outs[1:]:
        ok, ma, _ = U.rel_abs_ok(o, outs[0], REL, ABS)
        assert ok, ma


def test_holes_are_skipped(dev, kernel):
    """An evicted page (table entry -1) takes no part; the reference leaves this
    case undefined (paged_attention.cu:220 indexes with -1), extract zero-fills."""
    case = Case((1, 4, 16, 128, 16, 128), cabi.F16, [600, 300], seed=51, holes=[(0, 3), (0, 20), (1, 0)])
    got = case.run_branches(split=128)
    _check(case, got)


def test_all_holes_or_empty_leaves_out_untouched(dev, kernel):
    """l == 0 => `out` is not written (paged_attention.cu:266)."""
    case = Case((1, 4, 16, 128, 16, 64), cabi.F16, [32, 0, 40], seed=52, holes=[(0, 0), (0, 1)])
    got = case.run_branches(split=64, fill=0x7B)
    assert np.all(got[0] == 0x7B7B) and np.all(got[1] == 0x7B7B)
    want = orc.decode_f64(case.og, case.q[2], case.opool, case.tables[2], 0, 40, case.scale, cabi.F16)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(got[2], cabi.F16), want, REL, ABS)
    assert ok, ma


def test_stale_rows_past_the_end_do_not_leak(dev, kernel):
    """Slots of the last page beyond seq_len hold NaN/Inf bit patterns; the output
    must not change."""
    case = Case((1, 4, 16, 128, 16, 64), cabi.BF16, [70], seed=53)
    clean = case.run_single(0)
    flat = np.full((1, 2, 10, 4, 128), 0x7FC0, dtype=np.uint16)          # bf16 NaN
    orc.inject(case.og, case.opool, flat, None, case.tables[0], 70, 10, 1)
    case.dpool = U.dev_bytes(case.opool)
    assert np.array_equal(case.run_single(0), clean)


@pytest.mark.parametrize("geom", [(2, 4, 24, 256, 256, 8), (1, 2, 4, 64, 32, 40), (1, 2, 16, 128, 16, 80),
                                  (1, 4, 4, 128, 16, 80)])
@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
def test_other_geometries(dev, geom, dtype):
    """Group sizes 6, 2, 8, 1 and head dims 256, 64 (the reference's own model is
    24 Q / 4 KV heads x 256, block 256: block_pool.h:34-38)."""
    case = Case(geom, dtype, [900, 130], seed=61, mul=0.7)
    _check(case, case.run_branches())


@pytest.mark.parametrize("geom", [(1, 2, 32, 128, 16, 120), (1, 2, 24, 128, 16, 120), (1, 4, 12, 128, 32, 60), (1, 2, 10, 256, 16, 120),
                                  (1, 2, 8, 256, 32, 60), (1, 1, 16, 256, 16, 120), (1, 3, 3, 256, 16, 120)])
@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
def test_stream_kernel_group_sizes_and_head_dims(dev, geom, dtype):
    """The tiled kernel takes head_dim 128 and 256 with 1..16 query heads per kv head (here 16, 12,
    3, 5, 4, 16, 1), every storage type: ragged branches, a hole, stale bytes past the end, against
    the fp64 oracle; and its bits are not the portable kernel's (it really is the one that ran)."""
    case = Case(geom, dtype, [900, 130, 64, 1, 333], seed=62, mul=0.7, holes=[(0, 3)], stale=0xFF, outliers=dtype in (cabi.INT8, cabi.FP8_E4M3))
    got = case.run_branches()
    _check(case, got)
    _check(case, case.run_branches(split=128))
    cabi.lib().drk_debug_force_portable_decode(1)
    try:
        other = case.run_branches()
    finally:
        cabi.lib().drk_debug_force_portable_decode(0)
    _check(case, other)
    assert not np.array_equal(got, other)
    for b in (0, 3):
        assert np.array_equal(case.run_single(b), got[b])               # one sequence per call: same bits


@pytest.mark.parametrize("seed", range(16))
def test_random_geometries_lengths_and_holes(dev, seed):
    """A seeded draw over what the tiled kernel takes: head_dim 128 / 256, 1..16 query heads per kv head,
    blocks of 16..256 tokens, every storage type, 1..9 branches of ragged lengths (some empty), a few
    holes in the tables, stale bytes in unused rows -- against fp64 on the stored values."""
    rng = np.random.default_rng(1000 + seed)
    D = int(rng.choice([128, 256]))
    KVH = int(rng.choice([1, 2, 4, 8]))
    G = int(rng.choice([1, 2, 3, 4, 5, 6, 8, 12, 16]))
    bs = int(rng.choice([16, 32, 48, 64, 256]))
    dtype = int(rng.choice([cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3]))
    io = dtype if dtype in (cabi.F16, cabi.BF16) else int(rng.choice([cabi.F16, cabi.BF16]))
    B = int(rng.integers(1, 10))
    lens = rng.integers(0, 1400, size=B)
    lens[rng.integers(0, B)] = int(rng.choice([1, 63, 64, 65, 1023, 1024, 1025]))
    nblk = sum((int(n) + bs - 1) // bs for n in lens)
    holes = []
    for _ in range(int(rng.integers(0, 4))):
        b = int(rng.integers(0, B))
        if lens[b] > bs:
            holes.append((b, int(rng.integers(0, (int(lens[b]) + bs - 1) // bs))))
    case = Case((2, KVH, KVH * G, D, bs, nblk + 3), dtype, lens, seed=seed, io_dtype=io, holes=holes,
                outliers=bool(seed & 1), stale=0x7F if dtype in (cabi.F16, cabi.BF16) else 0x3C)
    got = case.run_branches()
    for b in range(B):        # a branch with no visible token leaves its rows as they were
        if lens[b] == 0 or all((b, lb) in holes for lb in range((int(lens[b]) + bs - 1) // bs)):
            assert np.all(got[b].view(np.uint8) == 0x7B)
            continue
        want = orc.decode_f64(case.og, case.q[b], case.opool, case.tables[b], case.layer, int(lens[b]), case.scale, case.io)
        ok, ma, mr = U.rel_abs_ok(U.from_bits(got[b], case.io), want, REL, ABS)
        assert ok, f"branch {b}: max abs err {ma:.4g}, max rel err {mr:.4g} ({D=} {KVH=} {G=} {bs=} {dtype=} lens={lens.tolist()} {holes=})"


@pytest.mark.parametrize("dtype", [cabi.INT8, cabi.FP8_E4M3])
@pytest.mark.parametrize("io", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("portable", [0, 1])
def test_quantised_pools(dev, dtype, io, portable):
    """Dequantisation inside attention: the fp64 oracle runs on the same codes
    (BASELINE config 4 in small: K/V with 1 % outliers x20, ragged lengths, a hole,
    stale bytes after the end)."""
    cabi.lib().drk_debug_force_portable_decode(portable)
    try:
        case = Case((1, 8, 32, 128, 16, 400), dtype, [1500, 260, 64, 1, 2047], seed=71, io_dtype=io, outliers=True,
                    holes=[(0, 7)], stale=0xFF)
        _check(case, case.run_branches())
        _check(case, case.run_branches(split=128))
    finally:
        cabi.lib().drk_debug_force_portable_decode(0)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
def test_prefill_rows_are_causal_decodes(dev, kernel, dtype):
    """Row t of a chunk == decode with seq_len = pos_start + t + 1
    (paged_attention.cu:481)."""
    L, KVH, QH, D, bs, NB = 1, 4, 16, 128, 16, 64
    pos_start, M = 37, 45
    case = Case((L, KVH, QH, D, bs, NB), dtype, [pos_start + M], seed=81)
    q = U.normal_bits(case.rng, (M, QH, D), dtype)
    dq = U.dev_bytes(q)
    lib = cabi.lib()
    wsb = lib.drk_prefill_workspace_bytes(C.byref(case.g), pos_start, M)
    ws = U.dev_zeros(max(wsb, 16))
    out = U.dev_zeros(M * QH * D * 2)
    cabi.call("drk_paged_prefill_attention", C.byref(case.g), U.p(dq), U.p(case.dpool), U.p(case.dtab[0]), U.p(out),
              0, pos_start, M, float(case.scale), dtype, U.p(ws), wsb, U.stream_ptr())
    U.sync()
    got = U.from_bits(U.host(out, np.uint16, (M, QH, D)), dtype)
    want = orc.prefill_f64(case.og, q, case.opool, case.tables[0], 0, pos_start, case.scale, dtype)
    ok, ma, _ = U.rel_abs_ok(got, want, REL, ABS)
    assert ok, ma


def test_workspace_too_small_is_refused(dev):
    case = Case((1, 4, 16, 128, 16, 64), cabi.F16, [100], seed=91)
    ws = U.dev_zeros(64)
    out = U.dev_zeros(16 * 128 * 2)
    rc = cabi.lib().drk_paged_decode_attention(C.byref(case.g), U.p(case.dq), U.p(case.dpool), U.p(case.dtab[0]),
                                               U.p(out), 0, 100, 0.1, cabi.F16, U.p(ws), 64, None)
    assert rc == cabi.ERR_WORKSPACE


_SHARED_CASES = {}


def _shared_case(dtype, shared, extra, heads):
    """The pool, tables and queries of a shared-prefix case and the fp64 oracle's outputs: the same for every kernel the
    case runs on, built once (nothing writes to them afterwards)."""
    key = (dtype, shared, tuple(extra), tuple(heads))
    if key in _SHARED_CASES:
        return _SHARED_CASES[key]
    L, bs = 1, 16
    KVH, QH, D = heads
    io = dtype if dtype in (cabi.F16, cabi.BF16) else cabi.BF16
    B = len(extra)
    lens = np.array([shared + e for e in extra], dtype=np.int32)
    n_shared_blk = shared // bs
    priv_blk = [(int(l) + bs - 1) // bs - n_shared_blk for l in lens]
    NB = n_shared_blk + sum(priv_blk) + 8
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(shared + B)
    perm = rng.permutation(NB).astype(np.int32)
    stride = n_shared_blk + max(priv_blk) + 2
    tables = np.full((B, stride), -1, dtype=np.int32)
    o = n_shared_blk
    for b in range(B):
        tables[b, :n_shared_blk] = perm[:n_shared_blk]
        tables[b, n_shared_blk:n_shared_blk + priv_blk[b]] = perm[o:o + priv_blk[b]]
        o += priv_blk[b]
    opool = orc.new_pool(og)
    k = U.normal_bits(rng, (shared, KVH, D), io, 0.7)
    v = U.normal_bits(rng, (shared, KVH, D), io, 0.7)
    orc.append_batch(og, opool, tables[0], 0, 0, k, v, io)
    for b in range(B):
        n = int(lens[b]) - n_shared_blk * bs
        if n > 0:
            # a branch's private part starts at the first non-shared block boundary
            kk = U.normal_bits(rng, (n, KVH, D), io, 0.7)
            vv = U.normal_bits(rng, (n, KVH, D), io, 0.7)
            orc.append_batch(og, opool, tables[b], 0, n_shared_blk * bs, kk, vv, io)
    if shared >= 1024:                                   # a page of the prefix is missing (evicted) in every branch
        tables[:, 2] = -1
        tables[:, n_shared_blk - 5] = -1
    q = U.normal_bits(rng, (B, QH, D), io, 0.7)
    scale = 1 / np.sqrt(D)
    want = np.stack([orc.decode_f64(og, q[b], opool, tables[b], 0, int(lens[b]), scale, io) for b in range(B)])
    _SHARED_CASES[key] = (bs, KVH, QH, D, io, B, lens, n_shared_blk, g, og, stride, tables, opool, q, scale, want)
    return _SHARED_CASES[key]


@pytest.fixture(params=["grouped", "producer_consumer", "every_wave_stages"])
def prefix_kernel(request):
    """Shared pages are read by the grouped kernel (shared and private tiles in one launch: head_dim 128, up to
    64 rows per kv head) or by a prefix pass + the tail kernel; the prefix pass has two kernels for up to 64 rows
    per kv head of head_dim 128."""
    cabi.lib().drk_debug_set_grouped_decode(0 if request.param == "grouped" else 1)
    cabi.lib().drk_debug_set_prefix_stream(0 if request.param == "every_wave_stages" else 1)
    yield request.param
    cabi.lib().drk_debug_set_prefix_stream(1)
    cabi.lib().drk_debug_set_grouped_decode(0)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
@pytest.mark.parametrize("shared,extra,heads", [(1024, [0, 1, 63, 64, 65, 500, 1000, 17], (8, 32, 128)), (960 + 16, [5, 300], (8, 32, 128)),
                                                (64, [0], (8, 32, 128)), (4096, list(range(0, 400, 10)), (8, 32, 128)),
                                                (1024, [3, 200, 64, 700, 1], (2, 16, 128)), (512, [9, 100, 33], (4, 24, 256)),
                                                (8192 + 64, [(37 * i) % 900 for i in range(16)], (8, 32, 128)),
                                                (192, [0, 5, 70], (1, 16, 128))])
def test_shared_prefix_decode(dev, prefix_kernel, dtype, shared, extra, heads):
    """Branches whose leading pages are the same physical blocks (BASELINE config 3
    in small): the shared pass + private tails must agree with the fp64 oracle run
    per branch, and with the plain per-branch call.  Also with 8 and 6 query heads per kv head,
    head_dim 256, and 8-bit pages."""
    bs, KVH, QH, D, io, B, lens, n_shared_blk, g, og, stride, tables, opool, q, scale, want = _shared_case(dtype, shared, extra, heads)
    dq, dpool, dtab, dl = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(tables), U.dev_i32(lens)
    lib = cabi.lib()
    mx = int(lens.max())
    shared_arg = n_shared_blk * bs
    wsb = lib.drk_decode_shared_workspace_bytes(C.byref(g), B, mx, shared_arg)
    ws = U.dev_zeros(wsb)
    out = U.dev_bytes(np.full(B * QH * D * 2, 0x7B, dtype=np.uint8))
    cabi.call("drk_paged_decode_attention_shared", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), stride, U.p(dl), B, mx,
              shared_arg, U.p(out), 0, float(scale), io, U.p(ws), wsb, U.stream_ptr())
    out2 = U.dev_zeros(B * QH * D * 2)
    cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), stride, U.p(dl), B, mx,
              U.p(out2), 0, float(scale), io, 0, U.p(ws), wsb, U.stream_ptr())
    U.sync()
    got = U.from_bits(U.host(out, np.uint16, (B, QH, D)), io)
    plain = U.from_bits(U.host(out2, np.uint16, (B, QH, D)), io)
    ok, ma, _ = U.rel_abs_ok(got, want, REL, ABS)
    assert ok, ma
    ok, ma, _ = U.rel_abs_ok(got, plain, REL, ABS)
    assert ok, ma
    # a workspace sized for the longest prefix the caller may ever pass serves every shorter one
    # (the pieces the private tails need grow as the prefix shrinks)
    assert wsb <= lib.drk_decode_shared_workspace_bytes(C.byref(g), B, mx, mx)
    wsb_max = lib.drk_decode_shared_workspace_bytes(C.byref(g), B, mx, mx)
    ws_max = U.dev_zeros(wsb_max)
    if shared_arg >= 128:
        out3 = U.dev_zeros(B * QH * D * 2)
        cabi.call("drk_paged_decode_attention_shared", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), stride, U.p(dl), B, mx,
                  shared_arg - 64, U.p(out3), 0, float(scale), io, U.p(ws_max), wsb_max, U.stream_ptr())
        U.sync()
        ok, ma, _ = U.rel_abs_ok(U.from_bits(U.host(out3, np.uint16, (B, QH, D)), io), want, REL, ABS)
        assert ok, ma


def test_more_branches_than_one_launch_takes(dev):
    """150 branches: the tiled kernel takes 64 per launch, so the call runs three launches through
    the same workspace; each branch must come out as if it had been called alone."""
    lens = [int(x) for x in np.random.default_rng(5).integers(1, 300, size=150)]
    case = Case((1, 8, 32, 128, 16, 150 * 20), cabi.BF16, lens, seed=63, mul=0.7)
    got = case.run_branches()
    _check(case, got)
    for b in (0, 63, 64, 127, 128, 149):                     # another split of the context: equal up to summation order
        ok, ma, _ = U.rel_abs_ok(U.from_bits(case.run_single(b), case.io), U.from_bits(got[b], case.io).astype(np.float64), REL, ABS)
        assert ok, (b, ma)
