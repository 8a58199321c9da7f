"""GPU parity of the layer steps either side of the page kernels (split of the Q|gate
projection, per-head RMSNorm, partial RoPE, sigmoid gate: paged_attention.cu:288-376,
386-451, 563-638; layer_attention.cu:32-135; layer.cu:406-439) and of their fused forms.

Bar: the norm, the rotation with a given cos/sin table, the split and every fused form
are bit-exact against the CPU oracle; what evaluates exp / cos / sin / pow on the
device (the gate, the table fill, the table-free rotation) is within one unit in the
last place of the 16-bit type, resp. 2e-6 absolute for the fp32 table."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi
from oracle import binding as orc
from tests import util as U

pytestmark = pytest.mark.gpu

EPS, THETA = 1e-6, 1.0e7     # RMS_EPS, ROPE_THETA of the reference model (machina.conf defaults)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_head_norm_bit_exact(dev, dtype, D):
    rng = np.random.default_rng(60 + D)
    rows = 1037
    x = U.normal_bits(rng, (rows, D), dtype, 1.5)
    x[5] = 0                                                    # a zero row
    w = U.normal_bits(rng, (D,), dtype)
    dx, dw, dout = U.dev_bytes(x), U.dev_bytes(w), U.dev_zeros(x.nbytes)
    cabi.call("drk_head_norm", U.p(dx), U.p(dw), U.p(dout), rows, D, EPS, dtype, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(dout, np.uint16, (rows, D)), orc.head_norm(x, w, EPS, dtype))
    # in place, as the reference calls it (paged_attention.cu:345-348)
    cabi.call("drk_head_norm", U.p(dx), U.p(dw), U.p(dx), rows, D, EPS, dtype, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(dx, np.uint16, (rows, D)), orc.head_norm(x, w, EPS, dtype))


def test_rope_table_fill_matches_libm(dev):
    import torch
    n, rd = 5000, 64
    t = torch.zeros(n * (rd // 2) * 2, dtype=torch.float32, device="cuda")
    cabi.call("drk_rope_table_fill", U.p(t), n, rd, THETA, U.stream_ptr())
    U.sync()
    got = t.cpu().numpy().reshape(n, rd // 2, 2)
    want = orc.rope_table(n, rd, THETA)
    # powf may differ by an ulp or two between the two libraries; the angle carries that times pos
    pos = np.arange(n, dtype=np.float64)[:, None, None]
    freq = (THETA ** (-2.0 * np.arange(rd // 2) / rd))[None, :, None]
    assert (np.abs(got.astype(np.float64) - want) <= 2e-6 + 4e-7 * pos * freq).all()
    assert np.array_equal(got[0], want[0])


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("D,rd", [(128, 32), (256, 64), (128, 128), (64, 16)])
@pytest.mark.parametrize("mode", ["batch", "branches"])
def test_apply_rope_with_table_bit_exact(dev, dtype, D, rd, mode):
    import torch
    rng = np.random.default_rng(61)
    T, QH, KVH, npos = 19, 6, 2, 700
    tab = orc.rope_table(npos, rd, THETA)
    q = U.normal_bits(rng, (T, QH, D), dtype)
    k = U.normal_bits(rng, (T, KVH, D), dtype)
    if mode == "batch":
        pos_start, pos, dpos = 123, 123 + np.arange(T, dtype=np.int32), None
    else:
        pos_start, pos = 0, rng.integers(0, npos, size=T).astype(np.int32)
        dpos = U.dev_i32(pos)
    dq, dk = U.dev_bytes(q), U.dev_bytes(k)
    dtab = torch.from_numpy(tab).cuda()
    cabi.call("drk_apply_rope", U.p(dq), U.p(dk), T, QH, KVH, D, rd, U.p(dpos), pos_start, THETA, U.p(dtab), npos,
              dtype, U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(dq, np.uint16, (T, QH, D)), orc.apply_rope(q, pos, tab, rd, dtype))
    assert np.array_equal(U.host(dk, np.uint16, (T, KVH, D)), orc.apply_rope(k, pos, tab, rd, dtype))


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
def test_apply_rope_without_table_within_one_ulp(dev, dtype):
    """The reference's call shape (layer_attention.cu:71-79): one token, position read on the device."""
    rng = np.random.default_rng(62)
    QH, KVH, D, rd = 24, 4, 256, 64
    tab = orc.rope_table(600, rd, THETA)
    for pos in (0, 1, 77, 599):
        q = U.normal_bits(rng, (1, QH, D), dtype)
        k = U.normal_bits(rng, (1, KVH, D), dtype)
        dq, dk, dpos = U.dev_bytes(q), U.dev_bytes(k), U.dev_i32(np.array([pos]))
        cabi.call("drk_apply_rope", U.p(dq), U.p(dk), 1, QH, KVH, D, rd, U.p(dpos), 0, THETA, None, 0, dtype,
                  U.stream_ptr())
        U.sync()
        p = np.array([pos], np.int32)
        assert U.ulp_distance(U.host(dq, np.uint16, (1, QH, D)), orc.apply_rope(q, p, tab, rd, dtype)).max() <= 1
        assert U.ulp_distance(U.host(dk, np.uint16, (1, KVH, D)), orc.apply_rope(k, p, tab, rd, dtype)).max() <= 1
        if pos == 0:
            assert np.array_equal(U.host(dq, np.uint16, (1, QH, D)), q)


def test_split_q_gate(dev):
    rng = np.random.default_rng(63)
    T, H, D = 7, 24, 256
    qg = rng.integers(0, 65536, size=(T, H, 2 * D)).astype(np.uint16)
    dqg, dq, dg = U.dev_bytes(qg), U.dev_zeros(qg.nbytes // 2), U.dev_zeros(qg.nbytes // 2)
    cabi.call("drk_split_q_gate", U.p(dqg), U.p(dq), U.p(dg), T, H, D, U.stream_ptr())
    U.sync()
    q, gate = orc.split_q_gate(qg, T, H, D)
    assert np.array_equal(U.host(dq, np.uint16, (T, H, D)), q)
    assert np.array_equal(U.host(dg, np.uint16, (T, H, D)), gate)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
def test_sigmoid_gate_within_one_ulp_and_strided(dev, dtype):
    rng = np.random.default_rng(64)
    rows, D = 333, 128
    x = U.normal_bits(rng, (rows, D), dtype, 2.0)
    qg = U.normal_bits(rng, (rows, 2 * D), dtype, 3.0)         # gate = second half of each row
    gate = np.ascontiguousarray(qg[:, D:])
    want = orc.sigmoid_gate(x, gate, dtype)
    dx, dqg, dg, dout = U.dev_bytes(x), U.dev_bytes(qg), U.dev_bytes(gate), U.dev_zeros(x.nbytes)
    cabi.call("drk_sigmoid_gate", U.p(dx), U.p(dg), U.p(dout), rows, D, D, dtype, U.stream_ptr())
    U.sync()
    dense = U.host(dout, np.uint16, (rows, D)).copy()
    assert U.ulp_distance(dense, want).max() <= 1
    gptr = C.c_void_p(dqg.data_ptr() + D * 2)
    cabi.call("drk_sigmoid_gate", U.p(dx), gptr, U.p(dx), rows, D, 2 * D, dtype, U.stream_ptr())   # in place, strided gate
    U.sync()
    assert np.array_equal(U.host(dx, np.uint16, (rows, D)), dense)


def _fused_case(dtype, mode, seed, holes=False):
    """Returns everything for one fused call and the oracle's composition of the separate steps."""
    L, KVH, QH, D, bs, NB = 2, 4, 16, 128, 16, 64
    rd, npos = 32, 900
    src = dtype if dtype in (cabi.F16, cabi.BF16) else cabi.BF16
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(seed)
    T = 37 if mode == "batch" else 9
    qg = U.normal_bits(rng, (T, QH, 2 * D), src, 1.3)
    k = U.normal_bits(rng, (T, KVH, D), src, 0.7)
    v = U.normal_bits(rng, (T, KVH, D), src)
    if dtype in (cabi.INT8, cabi.FP8_E4M3):                     # some outliers, as in the compressed-KV workload
        kf = U.from_bits(k, src)
        kf[rng.random(kf.shape) < 0.01] *= 20.0
        k = U.to_bits(kf, src)
    qw, kw = U.normal_bits(rng, (D,), src), U.normal_bits(rng, (D,), src)
    tab = orc.rope_table(npos, rd, THETA)
    if mode == "batch":
        pos_start = 45
        pos = pos_start + np.arange(T, dtype=np.int32)
        tables = U.shuffled_table(rng, NB, (pos_start + T + bs - 1) // bs)[None, :]
        if holes:
            tables[0, 3] = -1
    else:
        pos_start = 0
        pos = rng.integers(0, 6 * bs, size=T).astype(np.int32)
        perm = rng.permutation(NB).astype(np.int32)
        tables = perm[:T * 7].reshape(T, 7).copy()              # 7 logical blocks per branch, all distinct
        if holes:
            tables[2, pos[2] // bs] = -1
    # oracle: the reference's sequence of separate steps
    q0, gate = orc.split_q_gate(qg, T, QH, D)
    qn = orc.head_norm(q0, qw, EPS, src).reshape(T, QH, D)
    kn = orc.head_norm(k, kw, EPS, src).reshape(T, KVH, D)
    qr = orc.apply_rope(qn, pos, tab, rd, src)
    kr = orc.apply_rope(kn, pos, tab, rd, src)
    opool = orc.new_pool(og)
    for t in range(T):
        row = tables[t] if mode == "branches" else tables[0]
        orc.append_token(og, opool, row, 1, int(pos[t]), kr[t], v[t], src)
    return dict(g=g, og=og, T=T, QH=QH, KVH=KVH, D=D, rd=rd, npos=npos, src=src, qg=qg, k=k, v=v, qw=qw, kw=kw, tab=tab,
                pos=pos, pos_start=pos_start, tables=tables, mode=mode, q_want=qr, pool_want=opool, gate=gate, kr=kr)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
@pytest.mark.parametrize("mode", ["batch", "branches"])
@pytest.mark.parametrize("holes", [False, True])
def test_fused_norm_rope_append_equals_the_separate_steps(dev, dtype, mode, holes):
    import torch
    c = _fused_case(dtype, mode, seed=70, holes=holes)
    dpool = U.dev_zeros(orc.pool_bytes(c["og"]))
    dqg, dk, dv, dqw, dkw = (U.dev_bytes(c[n]) for n in ("qg", "k", "v", "qw", "kw"))
    dtab = torch.from_numpy(c["tab"]).cuda()
    dtables = U.dev_i32(c["tables"])
    dpos = U.dev_i32(c["pos"]) if mode == "branches" else None
    dq = U.dev_zeros(c["T"] * c["QH"] * c["D"] * 2)
    qg_before = U.host(dqg, np.uint16).copy()
    cabi.call("drk_qk_norm_rope_append", C.byref(c["g"]), U.p(dpool), U.p(dtables), c["tables"].shape[1], U.p(dpos),
              c["pos_start"], c["T"], 1, U.p(dqg), U.p(dk), U.p(dv), U.p(dqw), U.p(dkw), EPS, c["rd"], THETA,
              U.p(dtab), c["npos"], U.p(dq), c["src"], U.stream_ptr())
    U.sync()
    assert np.array_equal(U.host(dq, np.uint16, (c["T"], c["QH"], c["D"])), c["q_want"])
    assert np.array_equal(U.host(dpool, np.uint8), c["pool_want"])
    assert np.array_equal(U.host(dqg, np.uint16), qg_before)            # the projection (and its gate halves) is only read


@pytest.mark.parametrize("dtype", [cabi.BF16, cabi.INT8])
def test_fused_equals_the_librarys_own_separate_kernels(dev, dtype):
    """split + head_norm x2 + apply_rope + append_branches, all on the GPU, table-free rotation
    (device cos/sin on both sides): same bits as the one fused launch."""
    c = _fused_case(dtype, "branches", seed=71)
    T, QH, KVH, D, src = c["T"], c["QH"], c["KVH"], c["D"], c["src"]
    st = U.stream_ptr()
    dqg, dk, dv, dqw, dkw = (U.dev_bytes(c[n]) for n in ("qg", "k", "v", "qw", "kw"))
    dtables, dpos = U.dev_i32(c["tables"]), U.dev_i32(c["pos"])
    # fused
    pool_a, q_a = U.dev_zeros(orc.pool_bytes(c["og"])), U.dev_zeros(T * QH * D * 2)
    cabi.call("drk_qk_norm_rope_append", C.byref(c["g"]), U.p(pool_a), U.p(dtables), c["tables"].shape[1], U.p(dpos), 0,
              T, 1, U.p(dqg), U.p(dk), U.p(dv), U.p(dqw), U.p(dkw), EPS, c["rd"], THETA, None, 0, U.p(q_a), src, st)
    # separate
    pool_b, q_b, gate_b = U.dev_zeros(orc.pool_bytes(c["og"])), U.dev_zeros(T * QH * D * 2), U.dev_zeros(T * QH * D * 2)
    k_b = U.dev_bytes(c["k"])
    cabi.call("drk_split_q_gate", U.p(dqg), U.p(q_b), U.p(gate_b), T, QH, D, st)
    cabi.call("drk_head_norm", U.p(q_b), U.p(dqw), U.p(q_b), T * QH, D, EPS, src, st)
    cabi.call("drk_head_norm", U.p(k_b), U.p(dkw), U.p(k_b), T * KVH, D, EPS, src, st)
    cabi.call("drk_apply_rope", U.p(q_b), U.p(k_b), T, QH, KVH, D, c["rd"], U.p(dpos), 0, THETA, None, 0, src, st)
    cabi.call("drk_kv_append_branches", C.byref(c["g"]), U.p(pool_b), U.p(dtables), c["tables"].shape[1], U.p(dpos), T, 1,
              1, U.p(k_b), U.p(dv), src, st)
    U.sync()
    assert np.array_equal(U.host(q_a, np.uint16), U.host(q_b, np.uint16))
    assert np.array_equal(U.host(pool_a, np.uint8), U.host(pool_b, np.uint8))
    assert np.array_equal(U.host(gate_b, np.uint16, (T, QH, D)), c["gate"])


def _decode_inputs(dtype, seed, B=5, ctx=700, heads=(8, 32, 128)):
    L, bs = 1, 16
    KVH, QH, D = heads
    nblk = (ctx + bs - 1) // bs
    NB = B * nblk + 3
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(seed)
    io = dtype if dtype in (cabi.F16, cabi.BF16) else cabi.BF16
    lens = rng.integers(1, ctx + 1, size=B).astype(np.int32)
    lens[0] = ctx
    perm = rng.permutation(NB).astype(np.int32)
    tables = perm[:B * nblk].reshape(B, nblk).copy()
    opool = orc.new_pool(og)
    for b in range(B):
        k = U.normal_bits(rng, (int(lens[b]), KVH, D), io, 0.5)
        v = U.normal_bits(rng, (int(lens[b]), KVH, D), io, 0.5)
        orc.append_batch(og, opool, tables[b], 0, 0, k, v, io)
    q = U.normal_bits(rng, (B, QH, D), io, 0.5)
    qg = U.normal_bits(rng, (B, QH, 2 * D), io, 2.0)
    return g, og, io, lens, tables, opool, q, qg, (B, QH, D, ctx)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8])
@pytest.mark.parametrize("kernel,heads", [("stream", (8, 32, 128)), ("portable", (8, 32, 128)),
                                          ("stream", (4, 24, 256)), ("stream", (2, 32, 128))])   # the last two: the reference's model; 16 heads per kv head
def test_gated_decode_equals_decode_then_gate(dev, dtype, kernel, heads):
    g, og, io, lens, tables, opool, q, qg, (B, QH, D, ctx) = _decode_inputs(dtype, 80, heads=heads)
    lib = cabi.lib()
    lib.drk_debug_force_portable_decode(1 if kernel == "portable" else 0)
    try:
        st = U.stream_ptr()
        dpool, dq, dqg = U.dev_bytes(opool), U.dev_bytes(q), U.dev_bytes(qg)
        dtab, dlens = U.dev_i32(tables), U.dev_i32(lens)
        wsb = lib.drk_decode_workspace_bytes(C.byref(g), B, ctx)
        ws = U.dev_zeros(wsb)
        out_a, out_b = U.dev_zeros(B * QH * D * 2), U.dev_zeros(B * QH * D * 2)
        gptr = C.c_void_p(dqg.data_ptr() + D * 2)                       # the gate halves inside the projection
        cabi.call("drk_paged_decode_attention_gated", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), tables.shape[1], U.p(dlens),
                  B, ctx, U.p(out_a), 0, 1.0 / np.sqrt(D), io, gptr, 2 * D, U.p(ws), wsb, st)
        cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), tables.shape[1],
                  U.p(dlens), B, ctx, U.p(out_b), 0, 1.0 / np.sqrt(D), io, 0, U.p(ws), wsb, st)
        U.sync()
        plain = U.host(out_b, np.uint16, (B, QH, D)).copy()
        cabi.call("drk_sigmoid_gate", U.p(out_b), gptr, U.p(out_b), B * QH, D, 2 * D, io, st)
        U.sync()
    finally:
        lib.drk_debug_force_portable_decode(0)
    got = U.host(out_a, np.uint16, (B, QH, D))
    assert np.array_equal(got, U.host(out_b, np.uint16, (B, QH, D)))      # same bits as the two separate launches
    want = orc.sigmoid_gate(plain, np.ascontiguousarray(qg[:, :, D:]), io)
    assert U.ulp_distance(got, want).max() <= 1                           # device exp against libm's


def test_gated_decode_gates_rows_without_tokens_too(dev):
    """seq_len 0: the attention kernel leaves out alone (paged_attention.cu:266) and the gate
    that follows multiplies what was there (368-370)."""
    g, og, io, lens, tables, opool, q, qg, (B, QH, D, ctx) = _decode_inputs(cabi.BF16, 81)
    lens[1] = 0
    rng = np.random.default_rng(5)
    before = U.normal_bits(rng, (B, QH, D), io)
    lib = cabi.lib()
    dpool, dq, dqg, dout = U.dev_bytes(opool), U.dev_bytes(q), U.dev_bytes(qg), U.dev_bytes(before)
    dtab, dlens = U.dev_i32(tables), U.dev_i32(lens)
    wsb = lib.drk_decode_workspace_bytes(C.byref(g), B, ctx)
    ws = U.dev_zeros(wsb)
    gptr = C.c_void_p(dqg.data_ptr() + D * 2)
    cabi.call("drk_paged_decode_attention_gated", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), tables.shape[1], U.p(dlens),
              B, ctx, U.p(dout), 0, 1.0 / np.sqrt(D), io, gptr, 2 * D, U.p(ws), wsb, U.stream_ptr())
    U.sync()
    got = U.host(dout, np.uint16, (B, QH, D))
    want = orc.sigmoid_gate(before[1], np.ascontiguousarray(qg[1, :, D:]), io)
    assert U.ulp_distance(got[1], want).max() <= 1


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16])
@pytest.mark.parametrize("kernel", ["mfma", "portable"])
def test_gated_prefill_equals_prefill_then_gate(dev, dtype, kernel):
    L, KVH, QH, D, bs, NB = 1, 8, 32, 128, 16, 40
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(82)
    pos_start, M = 150, 75
    table = U.shuffled_table(rng, NB, (pos_start + M + bs - 1) // bs)
    opool = orc.new_pool(og)
    orc.append_batch(og, opool, table, 0, 0, U.normal_bits(rng, (pos_start + M, KVH, D), dtype, 0.5),
                     U.normal_bits(rng, (pos_start + M, KVH, D), dtype, 0.5), dtype)
    q = U.normal_bits(rng, (M, QH, D), dtype, 0.5)
    qg = U.normal_bits(rng, (M, QH, 2 * D), dtype, 2.0)
    lib = cabi.lib()
    lib.drk_debug_force_portable_decode(1 if kernel == "portable" else 0)
    try:
        st = U.stream_ptr()
        dpool, dq, dqg, dtab = U.dev_bytes(opool), U.dev_bytes(q), U.dev_bytes(qg), U.dev_i32(table)
        wsb = max(lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M), 16)
        ws = U.dev_zeros(wsb)
        out_a, out_b = U.dev_zeros(M * QH * D * 2), U.dev_zeros(M * QH * D * 2)
        gptr = C.c_void_p(dqg.data_ptr() + D * 2)
        cabi.call("drk_paged_prefill_attention_gated", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out_a), 0, pos_start, M,
                  1.0 / np.sqrt(D), dtype, gptr, 2 * D, U.p(ws), wsb, st)
        cabi.call("drk_paged_prefill_attention", C.byref(g), U.p(dq), U.p(dpool), U.p(dtab), U.p(out_b), 0, pos_start, M,
                  1.0 / np.sqrt(D), dtype, U.p(ws), wsb, st)
        cabi.call("drk_sigmoid_gate", U.p(out_b), gptr, U.p(out_b), M * QH, D, 2 * D, dtype, st)
        U.sync()
    finally:
        lib.drk_debug_force_portable_decode(0)
    assert np.array_equal(U.host(out_a, np.uint16), U.host(out_b, np.uint16))


def test_layer_step_argument_errors(dev):
    x = U.dev_zeros(4096)
    with pytest.raises(cabi.DrkError):
        cabi.call("drk_head_norm", U.p(x), U.p(x), U.p(x), 4, 96, EPS, cabi.F16, U.stream_ptr())       # 96 / 8 is no power of two
    with pytest.raises(cabi.DrkError):
        cabi.call("drk_apply_rope", U.p(x), U.p(x), 1, 1, 1, 128, 48, None, 0, THETA, None, 0, cabi.F16, U.stream_ptr())
    with pytest.raises(cabi.DrkError):
        cabi.call("drk_sigmoid_gate", U.p(x), U.p(x), U.p(x), 4, 128, 64, cabi.F16, U.stream_ptr())     # gate rows overlap
    with pytest.raises(cabi.DrkError):
        cabi.call("drk_head_norm", U.p(x), U.p(x), U.p(x), 4, 128, EPS, cabi.INT8, U.stream_ptr())
