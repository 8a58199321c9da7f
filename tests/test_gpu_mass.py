"""GPU parity of the attention-mass output of the decode path (the per-block importance
values ImportanceScorer::update consumes, importance_scorer.h:37-41) against the fp64
oracle.  Floating point: |err| <= 2e-3 + 2e-3 * |want| on masses that range over
[0, num_q_heads]; the attention output itself must keep the bits of the plain call."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi
from oracle import binding as orc
from tests import util as U

pytestmark = pytest.mark.gpu


def _case(dtype, bs, seed, B=4, ctx=900, holes=True, heads=(8, 32, 128)):
    L = 2
    KVH, QH, D = heads
    nblk = (ctx + bs - 1) // bs
    NB = B * nblk + 2
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    io = dtype if dtype in (cabi.F16, cabi.BF16) else cabi.BF16
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, ctx + 1, size=B).astype(np.int32)
    lens[0] = ctx
    if B > 2:
        lens[2] = 0
    perm = rng.permutation(NB).astype(np.int32)
    stride = nblk + 3
    tables = np.full((B, stride), -1, np.int32)
    tables[:, :nblk] = perm[:B * nblk].reshape(B, nblk)
    opool = orc.new_pool(og)
    for b in range(B):
        n = int(lens[b])
        if n:
            # a few sharp keys so that the mass is far from uniform
            kf = rng.standard_normal((n, KVH, D)).astype(np.float32) * 0.5
            kf[rng.integers(0, n, size=max(1, n // 50))] *= 4.0
            orc.append_batch(og, opool, tables[b], 1, 0, U.to_bits(kf, io), U.normal_bits(rng, (n, KVH, D), io, 0.5), io)
    if holes:
        tables[0, 1] = -1
    q = U.normal_bits(rng, (B, QH, D), io, 0.7)
    return g, og, io, lens, tables, stride, opool, q, (B, QH, D, ctx)


def _run(g, io, lens, tables, stride, opool, q, shape, mass0=None, accumulate=0):
    B, QH, D, ctx = shape
    lib = cabi.lib()
    dpool, dq, dtab, dlens = U.dev_bytes(opool), U.dev_bytes(q), U.dev_i32(tables), U.dev_i32(lens)
    wsb = lib.drk_decode_mass_workspace_bytes(C.byref(g), B, ctx)
    assert wsb > lib.drk_decode_workspace_bytes(C.byref(g), B, ctx) - 4096
    ws = U.dev_zeros(wsb)
    out, out_plain = U.dev_zeros(B * QH * D * 2), U.dev_zeros(B * QH * D * 2)
    mass = U.dev_bytes(mass0 if mass0 is not None else np.full((B, stride), 7.0, np.float32))
    scale = 1.0 / np.sqrt(D)
    cabi.call("drk_paged_decode_attention_mass", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), stride, U.p(dlens), B, ctx,
              U.p(out), 1, scale, io, U.p(mass), stride, accumulate, U.p(ws), wsb, U.stream_ptr())
    cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), stride, U.p(dlens), B, ctx,
              U.p(out_plain), 1, scale, io, 0, U.p(ws), wsb, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(out, np.uint16), U.host(out_plain, np.uint16))
    return U.host(mass, np.float32, (B, stride)).copy()


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
@pytest.mark.parametrize("bs", [16, 64])
def test_block_mass_matches_fp64(dev, dtype, bs):
    g, og, io, lens, tables, stride, opool, q, shape = _case(dtype, bs, seed=100 + bs)
    got = _run(g, io, lens, tables, stride, opool, q, shape)
    want = orc.block_attention_mass(og, q, opool, tables, lens, 1, 1.0 / np.sqrt(shape[2]), io, stride)
    assert np.all(np.abs(got - want) <= 2e-3 + 2e-3 * np.abs(want)), float(np.abs(got - want).max())
    QH = shape[1]
    sums = got.sum(axis=1)
    assert np.allclose(sums[lens > 0], QH, atol=2e-2) and sums[2] == 0.0          # an empty branch: all zero
    assert got[0, 1] == 0.0                                                        # the hole
    nblk = (lens + bs - 1) // bs
    for b in range(len(lens)):
        assert not got[b, nblk[b]:].any()                                          # overwritten with zeros past the length


@pytest.mark.parametrize("heads", [(4, 24, 256), (2, 32, 128)])
def test_block_mass_other_head_shapes(dev, heads):
    """The reference's own model (24 Q / 4 KV heads x 256, block 256) and 16 query heads per kv head."""
    g, og, io, lens, tables, stride, opool, q, shape = _case(cabi.F16, 256, seed=9, B=3, ctx=1500, holes=False, heads=heads)
    got = _run(g, io, lens, tables, stride, opool, q, shape)
    want = orc.block_attention_mass(og, q, opool, tables, lens, 1, 1.0 / np.sqrt(shape[2]), io, stride)
    assert np.all(np.abs(got - want) <= 2e-3 + 2e-3 * np.abs(want)), float(np.abs(got - want).max())
    assert np.allclose(got.sum(axis=1)[lens > 0], shape[1], atol=2e-2)


def test_block_mass_accumulates_over_layers(dev):
    g, og, io, lens, tables, stride, opool, q, shape = _case(cabi.BF16, 16, seed=7, holes=False)
    base = np.random.default_rng(3).random((shape[0], stride)).astype(np.float32)
    once = _run(g, io, lens, tables, stride, opool, q, shape)
    acc = _run(g, io, lens, tables, stride, opool, q, shape, mass0=base, accumulate=1)
    assert np.allclose(acc, base + once, rtol=0, atol=1e-5)


@pytest.mark.parametrize("dtype,heads,bs", [(cabi.BF16, (8, 32, 128), 16), (cabi.F16, (4, 24, 256), 64), (cabi.INT8, (8, 32, 128), 16)])
@pytest.mark.parametrize("with_plan", [False, True])
def test_block_mass_with_the_gate_and_the_plan_folded_in(dev, dtype, heads, bs, with_plan):
    """drk_paged_decode_attention_mass_gated -- the step's unit descriptors read from a plan, the sigmoid gate applied in
    the merge -- against drk_paged_decode_attention_mass followed by drk_sigmoid_gate: same output bits, same masses."""
    g, og, io, lens, tables, stride, opool, q, shape = _case(dtype, bs, seed=31, heads=heads)
    B, QH, D, ctx = shape
    lib = cabi.lib()
    rng = np.random.default_rng(8)
    gate = U.normal_bits(rng, (B, QH, 2 * D), io, 1.0)          # rows 2 D apart, as the second halves of a Q | gate projection
    dpool, dq, dtab, dlens, dgate = U.dev_bytes(opool), U.dev_bytes(q), U.dev_i32(tables), U.dev_i32(lens), U.dev_bytes(gate)
    wsb = lib.drk_decode_mass_workspace_bytes(C.byref(g), B, ctx)
    ws = U.dev_zeros(wsb)
    scale = 1.0 / np.sqrt(D)
    plan = None
    if with_plan:
        pb = lib.drk_decode_plan_bytes(C.byref(g), B, ctx, 0)
        assert pb > 0
        plan = U.dev_zeros(pb)
        cabi.call("drk_decode_plan_build", C.byref(g), U.p(dtab), stride, U.p(dlens), B, ctx, None, 0, U.p(plan), pb, U.stream_ptr())
    out_a, out_b = U.dev_zeros(B * QH * D * 2), U.dev_zeros(B * QH * D * 2)
    mass_a = U.dev_bytes(np.full((B, stride), 7.0, np.float32))
    mass_b = U.dev_bytes(np.full((B, stride), 7.0, np.float32))
    gate_ptr = C.c_void_p(U.p(dgate).value + D * 2)
    cabi.call("drk_paged_decode_attention_mass", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), stride, U.p(dlens), B, ctx,
              U.p(out_a), 1, scale, io, U.p(mass_a), stride, 0, U.p(ws), wsb, U.stream_ptr())
    cabi.call("drk_sigmoid_gate", U.p(out_a), gate_ptr, U.p(out_a), B * QH, D, 2 * D, io, U.stream_ptr())
    cabi.call("drk_paged_decode_attention_mass_gated", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), stride, U.p(dlens), B, ctx,
              U.p(plan) if plan is not None else None, U.p(out_b), 1, scale, io, gate_ptr, 2 * D, U.p(mass_b), stride, 0,
              U.p(ws), wsb, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(out_a, np.uint16), U.host(out_b, np.uint16))
    ma, mb = U.host(mass_a, np.float32), U.host(mass_b, np.float32)
    assert np.allclose(ma, mb, rtol=1e-5, atol=1e-5) and not np.all(ma == 7.0)


def test_block_mass_argument_errors(dev):
    g, og, io, lens, tables, stride, opool, q, shape = _case(cabi.BF16, 16, seed=8, B=2, ctx=100, holes=False)
    B, QH, D, ctx = shape
    x = U.dev_zeros(1 << 16)
    with pytest.raises(cabi.DrkError):       # mass rows shorter than the blocks of max_seq_len
        cabi.call("drk_paged_decode_attention_mass", C.byref(g), U.p(x), U.p(x), U.p(x), stride, U.p(x), B, ctx, U.p(x), 0,
                  0.1, io, U.p(x), 3, 0, U.p(x), 1 << 16, U.stream_ptr())
    g2 = cabi.layout(1, 4, 24, 64, 16, 8, cabi.F16)        # a geometry the tiled kernels do not take (head_dim 64)
    assert cabi.lib().drk_decode_mass_workspace_bytes(C.byref(g2), 1, 100) == 0
    with pytest.raises(cabi.DrkError):
        cabi.call("drk_paged_decode_attention_mass", C.byref(g2), U.p(x), U.p(x), U.p(x), 8, U.p(x), 1, 100, U.p(x), 0,
                  0.1, cabi.F16, U.p(x), 8, 0, U.p(x), 1 << 16, U.stream_ptr())


# ---- perception frames: the mass a chunk of query tokens gives to the pages of the context ----------------

@pytest.fixture(params=["tiles_straight_into_lds", "tiles_through_registers"])
def mass_kernel(request):
    """The two one-walk mass kernels (8-bit pages: the first at head_dim 128 with a power-of-two block size, staged
    through registers on their way into LDS; the second otherwise)."""
    lib = cabi.lib()
    lib.drk_debug_set_prefill_mass_direct(1 if request.param == "tiles_straight_into_lds" else 0)
    yield request.param
    lib.drk_debug_set_prefill_mass_direct(1)


_FRAME_CASES, _FRAME_WANTS = {}, {}


def _frame_case(dtype, bs, seed, pos_start, M, heads=(8, 32, 128), holes=()):
    """The case and, through _frame_want, its fp64 masses are the same for every kernel choice a test runs them on:
    built once per set of arguments (nothing below writes to what it returns)."""
    key = (dtype, bs, seed, pos_start, M, tuple(heads), tuple(holes))
    if key not in _FRAME_CASES:
        _FRAME_CASES[key] = _build_frame_case(dtype, bs, seed, pos_start, M, heads, holes)
    return _FRAME_CASES[key]


def _build_frame_case(dtype, bs, seed, pos_start, M, heads=(8, 32, 128), holes=()):
    L = 2
    KVH, QH, D = heads
    total = pos_start + M
    nblk = (total + bs - 1) // bs
    NB = nblk + 3
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    io = dtype if dtype in (cabi.F16, cabi.BF16) else cabi.BF16
    rng = np.random.default_rng(seed)
    table = np.full(nblk + 2, -1, np.int32)
    table[:nblk] = rng.permutation(NB).astype(np.int32)[:nblk]
    opool = orc.new_pool(og)
    kf = rng.standard_normal((total, KVH, D)).astype(np.float32) * 0.5
    kf[rng.integers(0, total, size=max(1, total // 50))] *= 4.0             # a few sharp keys: mass far from uniform
    orc.append_batch(og, opool, table, 1, 0, U.to_bits(kf, io), U.normal_bits(rng, (total, KVH, D), io, 0.5), io)
    for h in holes:
        table[h] = -1
    q = U.normal_bits(rng, (M, QH, D), io, 0.7)
    return g, og, io, table, opool, q


def _frame_want(og, io, table, opool, q, pos_start, scale):
    """fp64: every row of the frame is a branch of length pos_start + t + 1 over the same table"""
    key = (id(opool), id(q), pos_start, float(scale))
    if key not in _FRAME_WANTS:
        _FRAME_WANTS[key] = (_compute_frame_want(og, io, table, opool, q, pos_start, scale), opool, q)   # the arrays stay alive with their ids
    return _FRAME_WANTS[key][0].copy()


def _compute_frame_want(og, io, table, opool, q, pos_start, scale):
    M = q.shape[0]
    tables = np.ascontiguousarray(np.broadcast_to(table, (M, table.size)))
    lens = (pos_start + 1 + np.arange(M)).astype(np.int32)
    return orc.block_attention_mass(og, q, opool, tables, lens, 1, scale, io, table.size).sum(axis=0)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
@pytest.mark.parametrize("bs,pos_start,M,heads", [(16, 0, 1, (8, 32, 128)), (16, 0, 70, (8, 32, 128)), (16, 333, 45, (8, 32, 128)),
                                                  (32, 500, 130, (2, 12, 128)), (256, 100, 33, (4, 24, 256)), (48, 64, 64, (2, 2, 128))])
def test_frame_mass_matches_fp64(dev, mass_kernel, dtype, bs, pos_start, M, heads):
    """drk_paged_prefill_attention_mass against the fp64 oracle (rows of the frame as causal branches): 8-bit
    pages, head_dim 256, 1 / 4 / 6 query heads per kv head, block sizes that are not powers of two, a missing
    page, stale entries in the output array; the entries add up to M x num_q_heads minus nothing."""
    total = pos_start + M
    holes = (1,) if total > 3 * bs else ()
    g, og, io, table, opool, q = _frame_case(dtype, bs, seed=bs + pos_start + M, pos_start=pos_start, M=M, heads=heads, holes=holes)
    scale = 1.0 / np.sqrt(heads[2])
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    mass = U.dev_bytes(np.full(table.size, 7.0, np.float32))
    cabi.call("drk_paged_prefill_attention_mass", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 1, pos_start, M, float(scale), io,
              U.p(mass), table.size, 0, U.stream_ptr())
    U.sync()
    got = U.host(mass, np.float32).astype(np.float64)
    want = _frame_want(og, io, table, opool, q, pos_start, scale)
    assert np.all(np.abs(got - want) <= 2e-3 * M + 2e-3 * np.abs(want)), np.abs(got - want).max()
    # every row that sees a token gives all of its probability away
    seen = sum(1 for t in range(M) if any(table[p // bs] >= 0 for p in range(pos_start + t + 1)))
    assert abs(got.sum() - seen * heads[1]) <= 1e-3 * M * heads[1]
    # accumulate: a second layer's pass adds to the first's
    cabi.call("drk_paged_prefill_attention_mass", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 1, pos_start, M, float(scale), io,
              U.p(mass), table.size, 1, U.stream_ptr())
    U.sync()
    assert np.all(np.abs(U.host(mass, np.float32) - 2 * want) <= 4e-3 * M + 4e-3 * np.abs(want))


@pytest.fixture(params=["by_rule", "two_phase", "two_phase_through_registers", "context_split"])
def chunk_path(request):
    """the chunk kernels that can leave the rows' log-sum-exps: the four-wave kernel and the head_dim 256 one (by the
    rule, for these sizes), the two-phase kernels, and the context-split pass with its merge"""
    lib = cabi.lib()
    if request.param == "context_split":
        lib.drk_debug_set_prefill_split(4096)
    else:
        lib.drk_debug_set_prefill_two_phase({"by_rule": 1, "two_phase": 2, "two_phase_through_registers": 3}[request.param])
    yield request.param
    lib.drk_debug_set_prefill_two_phase(1)
    lib.drk_debug_set_prefill_split(-1)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
@pytest.mark.parametrize("bs,pos_start,M,heads", [(16, 0, 70, (8, 32, 128)), (16, 333, 45, (8, 32, 128)), (32, 2500, 130, (2, 12, 128)),
                                                  (256, 2100, 33, (4, 24, 256)), (16, 64, 300, (2, 2, 128)), (16, 7, 200, (1, 5, 256)),
                                                  (64, 1000, 260, (2, 14, 128))])
def test_frame_mass_from_the_attention_calls_row_sums(dev, chunk_path, mass_kernel, dtype, bs, pos_start, M, heads):
    """The attention call leaves every row's log-sum-exp, the mass pass then walks the keys once: same masses as the
    two-walk pass within the tolerance of the fp64 oracle, same attention output as the call without the extra result.
    Both one-walk kernels: the one that takes 256 rows per workgroup and its tiles straight into LDS (8-bit pages: by
    way of registers; head counts that leave idle rows, walks that end inside a tile and inside a page, holes) and the
    register-staging one."""
    total = pos_start + M
    holes = (1,) if total > 3 * bs else ()
    g, og, io, table, opool, q = _frame_case(dtype, bs, seed=bs + pos_start + M, pos_start=pos_start, M=M, heads=heads, holes=holes)
    KVH, QH, D = heads
    scale = 1.0 / np.sqrt(D)
    lib = cabi.lib()
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M)
    ws = U.dev_zeros(max(wsb, 16))
    out0 = U.dev_bytes(np.full(M * QH * D * 2, 0x7B, dtype=np.uint8))
    out1 = U.dev_bytes(np.full(M * QH * D * 2, 0x7B, dtype=np.uint8))
    lse = U.dev_bytes(np.full(M * QH, 123.0, np.float32))
    cabi.call("drk_paged_prefill_attention", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out0), 1, pos_start, M, float(scale), io,
              U.p(ws), wsb, U.stream_ptr())
    cabi.call("drk_paged_prefill_attention_lse", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out1), 1, pos_start, M, float(scale),
              io, None, 0, U.p(lse), U.p(ws), wsb, U.stream_ptr())
    mass = U.dev_bytes(np.full(table.size, 7.0, np.float32))
    cabi.call("drk_paged_prefill_attention_mass_lse", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 1, pos_start, M, float(scale), io,
              U.p(lse), U.p(mass), table.size, 0, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(out0, np.uint16), U.host(out1, np.uint16))
    got = U.host(mass, np.float32).astype(np.float64)
    want = _frame_want(og, io, table, opool, q, pos_start, scale)
    assert np.all(np.abs(got - want) <= 2e-3 * M + 3e-3 * np.abs(want)), np.abs(got - want).max()
    seen = sum(1 for t in range(M) if any(table[p // bs] >= 0 for p in range(pos_start + t + 1)))
    assert abs(got.sum() - seen * QH) <= 2e-3 * M * QH
    rows = U.host(lse, np.float32).reshape(M, QH)
    for t in range(M):                                     # rows without a visible token say so
        sees = any(table[p // bs] >= 0 for p in range(pos_start + t + 1))
        assert np.all(np.isfinite(rows[t])) if sees else np.all(np.isposinf(rows[t]))


@pytest.mark.parametrize("dtype,bs,pos_start,M,heads", [(cabi.BF16, 16, 1500, 100, (8, 32, 128)), (cabi.F16, 256, 2500, 70, (4, 24, 256)),
                                                        (cabi.F16, 64, 900, 300, (2, 14, 128)), (cabi.INT8, 16, 1500, 100, (8, 32, 128)),
                                                        (cabi.FP8_E4M3, 32, 1100, 260, (2, 8, 128))])
def test_frame_mass_where_every_block_has_a_page(dev, mass_kernel, dtype, bs, pos_start, M, heads):
    """No holes: the kernel for 16-bit pages takes its lean steps through the interior of every walk (no validity flags,
    no masks) and the general ones at the ends.  The two-walk call and the one-walk call against fp64."""
    lib = cabi.lib()
    g, og, io, table, opool, q = _frame_case(dtype, bs, seed=3 * bs + M, pos_start=pos_start, M=M, heads=heads, holes=())
    KVH, QH, D = heads
    scale = 1.0 / np.sqrt(D)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M)
    ws = U.dev_zeros(max(wsb, 16))
    out = U.dev_bytes(np.zeros(M * QH * D * 2, dtype=np.uint8))
    lse = U.dev_bytes(np.zeros(M * QH, np.float32))
    cabi.call("drk_paged_prefill_attention_lse", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out), 1, pos_start, M, float(scale),
              io, None, 0, U.p(lse), U.p(ws), wsb, U.stream_ptr())
    one = U.dev_bytes(np.full(table.size, 7.0, np.float32))
    two = U.dev_bytes(np.full(table.size, 7.0, np.float32))
    cabi.call("drk_paged_prefill_attention_mass_lse", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 1, pos_start, M, float(scale),
              io, U.p(lse), U.p(one), table.size, 0, U.stream_ptr())
    cabi.call("drk_paged_prefill_attention_mass", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 1, pos_start, M, float(scale), io,
              U.p(two), table.size, 0, U.stream_ptr())
    U.sync()
    want = _frame_want(og, io, table, opool, q, pos_start, scale)
    for got in (U.host(one, np.float32).astype(np.float64), U.host(two, np.float32).astype(np.float64)):
        assert np.all(np.abs(got - want) <= 2e-3 * M + 3e-3 * np.abs(want)), np.abs(got - want).max()
        assert abs(got.sum() - M * QH) <= 2e-3 * M * QH


@pytest.mark.parametrize("parts", [0, 3, 40])
@pytest.mark.parametrize("dtype,bs,pos_start,M,heads,holes", [
    (cabi.BF16, 16, 3000, 20, (8, 32, 128), (7, 150)), (cabi.F16, 256, 2100, 33, (4, 24, 256), (2,)),
    (cabi.F16, 32, 700, 260, (2, 14, 128), ()), (cabi.BF16, 64, 0, 130, (1, 6, 256), (1,)),
    (cabi.INT8, 16, 3000, 20, (8, 32, 128), (7, 150)), (cabi.FP8_E4M3, 48, 1500, 40, (2, 8, 128), (3,))])
def test_frame_mass_with_the_context_in_parts(dev, mass_kernel, parts, dtype, bs, pos_start, M, heads, holes):
    """A short frame behind a long context has few walks; the one-walk kernels cut them into parts (by their rule:
    16-tile parts for the first case; forced: 3 and 40 per walk, more parts than some walks have tiles) -- the kernel
    with 256 rows per workgroup and the register-staging one, which block sizes that are no power of two take.
    Masses against fp64 and against the same call with whole walks."""
    lib = cabi.lib()
    g, og, io, table, opool, q = _frame_case(dtype, bs, seed=bs + M, pos_start=pos_start, M=M, heads=heads, holes=holes)
    KVH, QH, D = heads
    scale = 1.0 / np.sqrt(D)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M)
    ws = U.dev_zeros(max(wsb, 16))
    out = U.dev_bytes(np.zeros(M * QH * D * 2, dtype=np.uint8))
    lse = U.dev_bytes(np.zeros(M * QH, np.float32))
    cabi.call("drk_paged_prefill_attention_lse", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out), 1, pos_start, M, float(scale),
              io, None, 0, U.p(lse), U.p(ws), wsb, U.stream_ptr())
    got = []
    try:
        for p in (parts, 1):
            lib.drk_debug_set_prefill_mass_parts(p)
            mass = U.dev_bytes(np.full(table.size, 7.0, np.float32))
            cabi.call("drk_paged_prefill_attention_mass_lse", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 1, pos_start, M, float(scale),
                      io, U.p(lse), U.p(mass), table.size, 0, U.stream_ptr())
            U.sync()
            got.append(U.host(mass, np.float32).astype(np.float64))
    finally:
        lib.drk_debug_set_prefill_mass_parts(0)
    want = _frame_want(og, io, table, opool, q, pos_start, scale)
    assert np.all(np.abs(got[0] - want) <= 2e-3 * M + 3e-3 * np.abs(want)), np.abs(got[0] - want).max()
    assert np.all(np.abs(got[0] - got[1]) <= 1e-4 * M + 1e-4 * np.abs(got[1])), np.abs(got[0] - got[1]).max()
    for h in holes:
        assert got[0][h] == 0.0


@pytest.mark.parametrize("dtype,heads,total", [(cabi.BF16, (1, 2, 128), 8192 * 16 + 700), (cabi.F16, (1, 1, 256), 6144 * 16 + 300)])
def test_frame_mass_behind_more_blocks_than_the_kernels_table_holds(dev, dtype, heads, total):
    """A context of more 16-token blocks than the one-walk kernel's table of page sums in LDS holds (8 192 at head_dim
    128, 6 144 at 256): the walk is cut into parts for that reason alone.  Five rows behind 131k / 98k tokens against
    fp64; the masses of the whole context add up to rows x heads."""
    bs, M = 16, 5
    pos_start = total - M
    g, og, io, table, opool, q = _frame_case(dtype, bs, seed=77, pos_start=pos_start, M=M, heads=heads, holes=(3, 4000))
    KVH, QH, D = heads
    scale = 1.0 / np.sqrt(D)
    lib = cabi.lib()
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M)
    ws = U.dev_zeros(max(wsb, 16))
    out = U.dev_bytes(np.zeros(M * QH * D * 2, dtype=np.uint8))
    lse = U.dev_bytes(np.zeros(M * QH, np.float32))
    cabi.call("drk_paged_prefill_attention_lse", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out), 1, pos_start, M, float(scale),
              io, None, 0, U.p(lse), U.p(ws), wsb, U.stream_ptr())
    got = []
    try:
        for parts in (0, 1):                                # the rule's parts; "one part" asked for: still as many as the table needs
            lib.drk_debug_set_prefill_mass_parts(parts)
            mass = U.dev_bytes(np.full(table.size, 7.0, np.float32))
            cabi.call("drk_paged_prefill_attention_mass_lse", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 1, pos_start, M, float(scale),
                      io, U.p(lse), U.p(mass), table.size, 0, U.stream_ptr())
            U.sync()
            got.append(U.host(mass, np.float32).astype(np.float64))
    finally:
        lib.drk_debug_set_prefill_mass_parts(0)
    want = _frame_want(og, io, table, opool, q, pos_start, scale)
    for m in got:
        assert np.all(np.abs(m - want) <= 2e-3 * M + 3e-3 * np.abs(want)), np.abs(m - want).max()
        assert abs(m.sum() - M * QH) <= 2e-3 * M * QH
        assert m[3] == 0.0 and m[4000] == 0.0


def test_frame_mass_of_a_long_chunk(dev):
    """A 300-token frame behind 3 000 tokens (several row tiles per kv head meeting in every page)."""
    pos_start, M, bs = 3000, 300, 16
    g, og, io, table, opool, q = _frame_case(cabi.BF16, bs, seed=5, pos_start=pos_start, M=M, holes=(7, 150))
    scale = 1.0 / np.sqrt(128)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    mass = U.dev_zeros(table.size * 4)
    cabi.call("drk_paged_prefill_attention_mass", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 1, pos_start, M, float(scale), io,
              U.p(mass), table.size, 0, U.stream_ptr())
    U.sync()
    got = U.host(mass, np.float32).astype(np.float64)
    want = _frame_want(og, io, table, opool, q, pos_start, scale)
    assert np.all(np.abs(got - want) <= 2e-3 * M + 2e-3 * np.abs(want)), np.abs(got - want).max()
    assert got[7] == 0.0 and got[150] == 0.0


def test_frame_mass_argument_errors(dev):
    g, og, io, table, opool, q = _frame_case(cabi.BF16, 16, seed=1, pos_start=10, M=5)
    dq, dpool, dtab = U.dev_bytes(q), U.dev_bytes(opool), U.dev_i32(table)
    mass = U.dev_zeros(64)
    lib = cabi.lib()
    args = (C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 1, 10, 5, 0.1, io, U.p(mass))
    assert lib.drk_paged_prefill_attention_mass(*args, 0, 0, None) == cabi.ERR_INVALID          # mass_len too small
    assert lib.drk_paged_prefill_attention_mass(C.byref(g), None, U.p(dpool), U.p(dtab), 1, 10, 5, 0.1, io, U.p(mass), 4, 0, None) == cabi.ERR_INVALID
    assert lib.drk_paged_prefill_attention_mass(C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), 9, 10, 5, 0.1, io, U.p(mass), 4, 0, None) == cabi.ERR_INVALID
