"""Pins the CPU oracle (oracle/drk_oracle.c) before anything is compared with it.

The reference holds no test, fixture or golden vector for this path, so each
function is pinned by what the mathematics fixes: library routines (numpy's
float16, torch's bfloat16 / float8_e4m3fn casts, np.rint), closed forms,
brute force on tiny inputs and invariants, chosen so that a dropped term, a
wrong index or a transposed operand fails."""
import ctypes as C

import numpy as np
import pytest

from oracle import binding as orc
from tests import util as U


# ---------------------------------------------------------------- conversions
def test_f16_conversions_match_numpy_exhaustively():
    lib = orc.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.orc_h2f(int(b)) for b in bits], dtype=np.float32)
    fin = np.isfinite(want)
    assert np.array_equal(got[fin], want[fin])
    assert np.all(np.isnan(got[np.isnan(want)]))
    # float -> half, RNE: every half value, every midpoint between neighbours, and noise
    rng = np.random.default_rng(0)
    xs = [want[fin]]
    pos = np.sort(want[fin & (want >= 0)])
    xs.append(((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32))
    xs.append((rng.standard_normal(20000) * 10 ** rng.uniform(-9, 5, 20000)).astype(np.float32))
    xs.append(np.array([65504, 65519.9, 65520, 65536, 1e9, -1e9, 5.96e-8, 2.98e-8, 2.9802322e-8, 0.0, -0.0], dtype=np.float32))
    x = np.concatenate(xs)
    x = np.concatenate([x, -x])
    with np.errstate(over="ignore"):
        want_h = x.astype(np.float16).view(np.uint16)
    got_h = np.array([lib.orc_f2h(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got_h, want_h)


def test_bf16_conversions_match_torch():
    import torch
    lib = orc.lib()
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(30000) * 10 ** rng.uniform(-20, 20, 30000)).astype(np.float32)
    # exact ties: low 16 bits == 0x8000
    ties = (rng.integers(0, 2 ** 16, 2000).astype(np.uint32) << 16 | 0x8000).view(np.float32)
    x = np.concatenate([x, ties[np.isfinite(ties)]])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([lib.orc_f2bf(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(U.f32_to_bf16_bits(x), want)          # the tests' own numpy helper too
    back = np.array([lib.orc_bf2f(int(b)) for b in want], dtype=np.float32)
    assert np.array_equal(back, torch.from_numpy(want.view(np.int16)).view(torch.bfloat16).float().numpy())


def test_fp8_e4m3_matches_torch_in_range_and_saturates_by_spec():
    import torch
    lib = orc.lib()
    # decode: all 256 codes
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    got = np.array([lib.orc_fp82f(int(c)) for c in codes], dtype=np.float32)
    fin = np.isfinite(want)
    assert np.array_equal(got[fin], want[fin]) and np.all(np.isnan(got[~fin]))
    # encode: every fp16 and bf16 bit pattern with |x| <= 448 must equal torch's RNE cast
    for to_f in (lambda b: b.view(np.float16).astype(np.float32), U.bf16_bits_to_f32):
        x = to_f(np.arange(65536, dtype=np.uint16))
        x = x[np.isfinite(x) & (np.abs(x) <= 448)]
        want_c = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        got_c = np.array([lib.orc_f2fp8(float(v)) for v in x], dtype=np.uint8)
        assert np.array_equal(got_c, want_c)
    # midpoints between adjacent fp8 values go to the even code
    vals = np.sort(want[fin & (want >= 0)])
    mids = ((vals[:-1].astype(np.float64) + vals[1:]) / 2).astype(np.float32)
    got_m = np.array([lib.orc_f2fp8(float(v)) for v in mids], dtype=np.uint8)
    assert np.all(got_m % 2 == 0)
    # saturation / specials, by this build's specification
    for v, c in [(448.0, 0x7E), (449.0, 0x7E), (464.0, 0x7E), (480.0, 0x7E), (1e30, 0x7E), (float("inf"), 0x7E),
                 (-448.0, 0xFE), (-1e9, 0xFE), (float("-inf"), 0xFE), (0.0, 0x00), (-0.0, 0x80),
                 (2.0 ** -9, 0x01), (2.0 ** -10, 0x00), (1.5 * 2.0 ** -10, 0x01), (2.0 ** -6, 0x08)]:
        assert lib.orc_f2fp8(v) == c, (v, hex(lib.orc_f2fp8(v)), hex(c))
    assert lib.orc_f2fp8(float("nan")) & 0x7F == 0x7F


# ---------------------------------------------------------------- addressing
def _np_offsets(L, KVH, D, bs, NB, E, int8):
    """independent numpy statement of the layout contract (block_pool.cpp:23-39)"""
    plane = KVH * bs * D * E
    sp = KVH * bs * 2 if int8 else 0
    bstride = 2 * plane + 2 * sp
    lstride = NB * bstride

    def k(l, b, h, p, d): return l * lstride + b * bstride + ((h * bs + p) * D + d) * E
    def v(l, b, h, p, d): return k(l, b, h, p, d) + plane
    def ks(l, b, h, p): return l * lstride + b * bstride + 2 * plane + (h * bs + p) * 2
    def vs(l, b, h, p): return ks(l, b, h, p) + sp
    return k, v, ks, vs, L * lstride


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16, orc.INT8, orc.FP8])
def test_addressing_is_a_bijection_onto_the_pool(dtype):
    L, KVH, QH, D, bs, NB = 2, 3, 6, 8, 4, 5
    g = orc.layout(L, KVH, QH, D, bs, NB, dtype)
    E = 2 if dtype in (orc.F16, orc.BF16) else 1
    k, v, ks, vs, total = _np_offsets(L, KVH, D, bs, NB, E, dtype == orc.INT8)
    lib = orc.lib()
    assert orc.pool_bytes(g) == total
    seen = np.zeros(total, dtype=np.int32)
    for l in range(L):
        for b in range(NB):
            for h in range(KVH):
                for p in range(bs):
                    for d in range(D):
                        ok = lib.orc_k_off(C.byref(g), l, b, h, p, d)
                        ov = lib.orc_v_off(C.byref(g), l, b, h, p, d)
                        assert ok == k(l, b, h, p, d) and ov == v(l, b, h, p, d)
                        seen[ok:ok + E] += 1
                        seen[ov:ov + E] += 1
                    if dtype == orc.INT8:
                        a, c = lib.orc_kscale_off(C.byref(g), l, b, h, p), lib.orc_vscale_off(C.byref(g), l, b, h, p)
                        assert a == ks(l, b, h, p) and c == vs(l, b, h, p)
                        seen[a:a + 2] += 1
                        seen[c:c + 2] += 1
    assert np.all(seen == 1)          # every byte of the pool is addressed exactly once


def test_budget_to_blocks():
    g = orc.layout(36, 8, 32, 128, 16, 1, orc.BF16)
    per_block = 36 * 2 * 8 * 16 * 128 * 2
    assert orc.lib().orc_max_blocks_for_budget(C.byref(g), 40 * 10 ** 9) == 40 * 10 ** 9 // per_block == 16954


# ---------------------------------------------------------------- append / gather
@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
def test_append_lands_where_the_layout_says_and_gathers_back(dtype):
    L, KVH, QH, D, bs, NB = 2, 4, 16, 16, 4, 12
    g = orc.layout(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(3)
    T, start = 19, 6
    table = U.shuffled_table(rng, NB, (start + T + bs - 1) // bs)
    k = rng.integers(0, 65536, (T, KVH, D)).astype(np.uint16)
    v = rng.integers(0, 65536, (T, KVH, D)).astype(np.uint16)
    pool = orc.new_pool(g)
    orc.append_batch(g, pool, table, 1, start, k, v, dtype)
    koff, voff, _, _, _ = _np_offsets(L, KVH, D, bs, NB, 2, False)
    p16 = pool.view(np.uint16)
    for t in range(T):
        pos = start + t
        b, p = int(table[pos // bs]), pos % bs
        for h in range(KVH):
            assert np.array_equal(p16[koff(1, b, h, p, 0) // 2:koff(1, b, h, p, 0) // 2 + D], k[t, h])
            assert np.array_equal(p16[voff(1, b, h, p, 0) // 2:voff(1, b, h, p, 0) // 2 + D], v[t, h])
    assert np.count_nonzero(pool.view(np.uint16)) <= 2 * T * KVH * D      # nothing else was written
    # M single appends == one batch
    pool2 = orc.new_pool(g)
    for t in range(T):
        orc.append_token(g, pool2, table, 1, start + t, k[t], v[t], dtype)
    assert np.array_equal(pool, pool2)
    flat, _ = orc.extract(g, pool, table, start, T, L)
    assert np.array_equal(flat[1, 0], k) and np.array_equal(flat[1, 1], v) and not flat[0].any()
    # inject(extract(x)) == x, and a permutation of physical blocks does not change the gather
    pool3 = orc.new_pool(g)
    table3 = U.shuffled_table(np.random.default_rng(8), NB, len(table))
    orc.inject(g, pool3, flat, None, table3, start, T, L)
    flat3, _ = orc.extract(g, pool3, table3, start, T, L)
    assert np.array_equal(flat3, flat)
    # hole: extract zero-fills, inject skips
    table3[1] = -1
    f4, _ = orc.extract(g, pool3, table3, start, T, L)
    tok = np.arange(start, start + T)
    assert not f4[:, :, tok // bs == 1].any() and np.array_equal(f4[:, :, tok // bs != 1], flat[:, :, tok // bs != 1])


def test_copy_block_copies_every_layer_and_nothing_else():
    g = orc.layout(3, 2, 2, 8, 4, 6, orc.INT8)
    rng = np.random.default_rng(4)
    pool = rng.integers(0, 256, orc.pool_bytes(g), dtype=np.uint8)
    before = pool.copy()
    orc.copy_block(g, pool, 1, 4)
    bsb = orc.lib().orc_block_stride_bytes(C.byref(g))
    view, old = pool.reshape(3, 6, bsb), before.reshape(3, 6, bsb)
    assert np.array_equal(view[:, 4], old[:, 1])
    keep = [0, 1, 2, 3, 5]
    assert np.array_equal(view[:, keep], old[:, keep])


# ---------------------------------------------------------------- codecs
@pytest.mark.parametrize("src", [orc.F16, orc.BF16])
def test_int8_codec_matches_numpy_restatement(src):
    rng = np.random.default_rng(5)
    rows = [rng.standard_normal(128).astype(np.float32) * s for s in (1e-6, 1e-3, 1.0, 50.0, 3e4)]
    rows.append(np.zeros(128, dtype=np.float32))
    r = rng.standard_normal(128).astype(np.float32)
    r[rng.random(128) < 0.02] *= 20
    rows.append(r)
    # exact ties: scale 0.5 (amax 63.5) puts x/s on k + 0.5 for x = k/2 + 0.25
    tie = (np.arange(128, dtype=np.float32) - 64) / 2 + 0.25
    tie[0] = 63.5
    rows.append(tie)
    for x in rows:
        b = U.to_bits(x, src)
        codes, sh = orc.quant_row_int8(b, src)
        xf = U.from_bits(b, src)
        amax = np.float32(np.abs(xf).max())
        with np.errstate(over="ignore"):
            s16 = (amax / np.float32(127)).astype(np.float16)
        if np.isinf(s16):
            s16 = np.float16(65504)
        sf = np.float32(s16)
        rcp = np.float32(1) / sf if sf > 0 else np.float32(0)
        want = np.clip(np.rint(xf * rcp), -127, 127).astype(np.int8)       # np.rint: half to even
        assert s16.view(np.uint16) == sh
        assert np.array_equal(codes, want)
    # the tie row really has ties and they went to even
    codes, sh = orc.quant_row_int8(U.to_bits(tie, src), src)
    assert sh == np.float16(0.5).view(np.uint16)
    assert np.all(codes[1:] % 2 == 0)


def test_fp8_row_codec_is_elementwise():
    x = np.linspace(-500, 500, 128, dtype=np.float32)
    b = U.to_bits(x, orc.BF16)
    codes = orc.quant_row_fp8(b, orc.BF16)
    want = np.array([orc.lib().orc_f2fp8(float(v)) for v in U.from_bits(b, orc.BF16)], dtype=np.uint8)
    assert np.array_equal(codes, want)


# ---------------------------------------------------------------- attention
def _numpy_attention(g, E, pool, table, layer, q, seq_len, scale, dtype):
    """fp64 softmax(QK^T*scale)V with its own gather (independent of orc_extract)."""
    L, KVH, QH, D, bs, NB = g.L, g.KVH, g.QH, g.D, g.bs, g.NB
    koff, voff, _, _, _ = _np_offsets(L, KVH, D, bs, NB, 2, False)
    p16 = pool.view(np.uint16)
    K = np.zeros((KVH, seq_len, D)); V = np.zeros((KVH, seq_len, D))
    for t in range(seq_len):
        b, p = int(table[t // bs]), t % bs
        for h in range(KVH):
            K[h, t] = U.from_bits(p16[koff(layer, b, h, p, 0) // 2:koff(layer, b, h, p, 0) // 2 + D], dtype)
            V[h, t] = U.from_bits(p16[voff(layer, b, h, p, 0) // 2:voff(layer, b, h, p, 0) // 2 + D], dtype)
    Q = U.from_bits(q, dtype).astype(np.float64)
    out = np.zeros((QH, D))
    for h in range(QH):
        kv = h // (QH // KVH)
        s = (K[kv] @ Q[h]) * scale
        w = np.exp(s - s.max())
        out[h] = (w / w.sum()) @ V[kv]
    return out


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
def test_attention_oracles_agree_with_numpy_fp64(dtype):
    L, KVH, QH, D, bs, NB = 2, 2, 6, 32, 4, 40
    g = orc.layout(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(6)
    n = 77
    table = U.shuffled_table(rng, NB, (n + bs - 1) // bs)
    pool = orc.new_pool(g)
    k = U.normal_bits(rng, (n, KVH, D), dtype)
    v = U.normal_bits(rng, (n, KVH, D), dtype)
    orc.append_batch(g, pool, table, 1, 0, k, v, dtype)
    q = U.normal_bits(rng, (QH, D), dtype)
    scale = 1 / np.sqrt(D)
    want = _numpy_attention(g, 2, pool, table, 1, q, n, scale, dtype)
    f64 = orc.decode_f64(g, q, pool, table, 1, n, scale, dtype)
    assert np.allclose(f64, want, rtol=1e-12, atol=1e-12)
    ref = U.from_bits(orc.decode_ref_order(g, q, pool, table, 1, n, scale, dtype), dtype)
    tol = 2e-3 if dtype == orc.F16 else 1.6e-2            # output rounding of the 16-bit type
    assert np.max(np.abs(ref - want)) < tol
    # a transposed GQA map (h % KVH instead of h // groups) would fail this:
    assert not np.allclose(f64[1], f64[QH // KVH], atol=1e-3)
    # split-K (any split) == unsplit within fp32 rounding; one split == unsplit path
    for split in (1, 5, 16, 64, 1000):
        sk = U.from_bits(orc.decode_splitk(g, q, pool, table, 1, n, scale, dtype, split), dtype)
        assert np.max(np.abs(sk - want)) < tol
    # prefill row t == decode with seq_len pos_start+t+1
    M, pos_start = 5, 60
    qm = U.normal_bits(rng, (M, QH, D), dtype)
    pf = orc.prefill_f64(g, qm, pool, table, 1, pos_start, scale, dtype)
    for t in range(M):
        assert np.allclose(pf[t], _numpy_attention(g, 2, pool, table, 1, qm[t], pos_start + t + 1, scale, dtype),
                           rtol=1e-12, atol=1e-12)
    pr = U.from_bits(orc.prefill_ref_order(g, qm, pool, table, 1, pos_start, scale, dtype), dtype)
    assert np.max(np.abs(pr - pf)) < tol
    # first row of a first chunk is V[0]
    p0 = orc.prefill_ref_order(g, qm[:1], pool, table, 1, 0, scale, dtype)
    assert np.array_equal(p0[0], np.repeat(v[0], QH // KVH, axis=0))


def test_attention_exact_cases():
    L, KVH, QH, D, bs, NB = 1, 2, 4, 16, 4, 16
    g = orc.layout(L, KVH, QH, D, bs, NB, orc.F16)
    rng = np.random.default_rng(7)
    table = U.shuffled_table(rng, NB, 8)
    n = 30
    v = U.normal_bits(rng, (n, KVH, D), orc.F16)
    krow = U.normal_bits(rng, (1, KVH, D), orc.F16)
    pool = orc.new_pool(g)
    orc.append_batch(g, pool, table, 0, 0, np.repeat(krow, n, 0), v, orc.F16)
    q = U.normal_bits(rng, (QH, D), orc.F16)
    # one token: out == V[0] bitwise
    out1 = orc.decode_ref_order(g, q, pool, table, 0, 1, 0.25, orc.F16)
    assert np.array_equal(out1, np.repeat(v[0], 2, axis=0))
    # identical keys: uniform weights -> mean of V
    out = orc.decode_f64(g, q, pool, table, 0, n, 0.25, orc.F16)
    mean_v = U.from_bits(v, orc.F16).astype(np.float64).mean(axis=0)
    assert np.allclose(out, np.repeat(mean_v, 2, axis=0), atol=1e-12)
    # holes are skipped; all holes -> out untouched
    table_h = table.copy(); table_h[2] = -1
    seen = orc.lib().orc_decode_f64(C.byref(g), orc.ptr(q), orc.ptr(pool), orc.ptr(table_h),
                                    orc.ptr(np.zeros((QH, D))), 0, n, 0.25, orc.F16)
    assert seen == n - bs
    sentinel = np.full((QH, D), 0x1234, dtype=np.uint16)
    orc.decode_ref_order(g, q, pool, np.full(8, -1, dtype=np.int32), 0, n, 0.25, orc.F16, out=sentinel)
    assert np.all(sentinel == 0x1234)


def test_quantised_attention_runs_on_dequantised_values():
    L, KVH, QH, D, bs, NB = 1, 2, 4, 16, 4, 16
    rng = np.random.default_rng(8)
    n = 21
    table = U.shuffled_table(rng, NB, 6)
    k = U.normal_bits(rng, (n, KVH, D), orc.BF16)
    v = U.normal_bits(rng, (n, KVH, D), orc.BF16)
    q = U.normal_bits(rng, (QH, D), orc.BF16)
    for dtype in (orc.INT8, orc.FP8):
        g = orc.layout(L, KVH, QH, D, bs, NB, dtype)
        pool = orc.new_pool(g)
        orc.append_batch(g, pool, table, 0, 0, k, v, orc.BF16)
        codes, scales = orc.extract(g, pool, table, 0, n, 1)
        if dtype == orc.INT8:
            deq = codes.view(np.int8).astype(np.float64) * scales.view(np.float16).astype(np.float64)[..., None]
        else:
            import torch
            deq = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).float().numpy().astype(np.float64)
        Q = U.from_bits(q, orc.BF16).astype(np.float64)
        want = np.zeros((QH, D))
        for h in range(QH):
            s = (deq[0, 0, :, h // 2] @ Q[h]) * 0.25
            w = np.exp(s - s.max())
            want[h] = (w / w.sum()) @ deq[0, 1, :, h // 2]
        got = orc.decode_f64(g, q, pool, table, 0, n, 0.25, orc.BF16)
        assert np.allclose(got, want, rtol=1e-12, atol=1e-12)


def test_importance_update_closed_form():
    lib = orc.lib()
    s = np.zeros(3, dtype=np.float32)
    news = [np.array([1, 2, 3], dtype=np.float32) * (i + 1) for i in range(4)]
    for nw in news:
        lib.orc_importance_update(orc.ptr(s), orc.ptr(nw), 3, 0.5)
    # s_n = sum decay^(n-k) new_k, exact in binary for decay = 0.5
    want = sum(nw * 0.5 ** (3 - i) for i, nw in enumerate(news))
    assert np.array_equal(s, want.astype(np.float32))
    ids = np.array([4, 2, 7, 1], dtype=np.int32)
    sc = np.array([9, 1.0, 1.0, 5, 3, 0, 0, 1.0], dtype=np.float32)
    assert lib.orc_least_important(orc.ptr(sc), orc.ptr(ids), 4) == 2      # first minimum in list order
    assert lib.orc_least_important(orc.ptr(sc), orc.ptr(ids), 0) == -1


# ---- layer steps either side of the kernels: split, head norm, RoPE, gate ----

def test_split_q_gate_is_the_reshape():
    rng = np.random.default_rng(50)
    T, H, D = 3, 5, 16
    qg = rng.integers(0, 65536, size=(T, H, 2 * D)).astype(np.uint16)
    q, gate = orc.split_q_gate(qg, T, H, D)
    r = qg.reshape(T, H, 2, D)
    assert np.array_equal(q, r[:, :, 0]) and np.array_equal(gate, r[:, :, 1])


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
@pytest.mark.parametrize("D", [64, 128, 256])
def test_head_norm_matches_fp64_closed_form(dtype, D):
    rng = np.random.default_rng(51 + D)
    rows, eps = 37, 1e-6
    x = U.normal_bits(rng, (rows, D), dtype, 2.0)
    w = U.normal_bits(rng, (D,), dtype, 1.0)
    got = orc.head_norm(x, w, eps, dtype)
    xf = U.from_bits(x, dtype).astype(np.float64)
    wf = U.from_bits(w, dtype).astype(np.float64)
    want = xf / np.sqrt((xf * xf).mean(axis=1, keepdims=True) + eps) * wf
    # two fp32 roundings sit between the exact value and the 16-bit result: one ulp
    assert U.ulp_distance(got, U.to_bits(want.astype(np.float32), dtype)).max() <= 1
    # a dropped 1/D, a misplaced eps or a missing weight are far outside that
    assert np.abs(U.from_bits(got, dtype) - want).max() < 0.02 * np.abs(want).max()
    # a zero row stays zero; a constant row with unit weights becomes +-1
    z = orc.head_norm(np.zeros((1, D), np.uint16), w, eps, dtype)
    assert not U.from_bits(z, dtype).any()
    c = orc.head_norm(U.to_bits(np.full((1, D), -3.0, np.float32), dtype), U.to_bits(np.ones(D, np.float32), dtype), eps, dtype)
    assert np.array_equal(U.from_bits(c, dtype), np.full((1, D), -1.0, np.float32))


def test_rope_table_matches_fp64_angles():
    rd, theta, n = 64, 1.0e7, 4096
    t = orc.rope_table(n, rd, theta)
    pos = np.arange(n, dtype=np.float64)[:, None]
    freq = theta ** (-2.0 * np.arange(rd // 2) / rd)
    ang = pos * freq[None, :]
    # the angle is formed in fp32 (as in the reference): its rounding error grows with pos
    tol = 2e-7 * np.maximum(1.0, ang) + 1e-6
    assert (np.abs(t[:, :, 0] - np.cos(ang)) <= tol).all()
    assert (np.abs(t[:, :, 1] - np.sin(ang)) <= tol).all()
    assert np.array_equal(t[0, :, 0], np.ones(rd // 2, np.float32)) and not t[0, :, 1].any()


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
def test_rope_is_a_rotation_of_half_half_pairs(dtype):
    rng = np.random.default_rng(53)
    T, H, D, rd, theta = 9, 3, 128, 32, 10000.0
    tab = orc.rope_table(600, rd, theta)
    x = U.normal_bits(rng, (T, H, D), dtype)
    pos = rng.integers(0, 600, size=T).astype(np.int32)
    pos[0] = 0
    got = orc.apply_rope(x, pos, tab, rd, dtype)
    assert np.array_equal(got[0], x[0])                      # position 0: identity, to the bit
    assert np.array_equal(got[:, :, rd:], x[:, :, rd:])      # dims past rotary_dim are not touched
    xf = U.from_bits(x, dtype).astype(np.float64)
    np_ = rd // 2
    c = tab[pos][:, None, :, 0].astype(np.float64)
    s = tab[pos][:, None, :, 1].astype(np.float64)
    want = xf.copy()
    want[:, :, :np_] = xf[:, :, :np_] * c - xf[:, :, np_:rd] * s
    want[:, :, np_:rd] = xf[:, :, np_:rd] * c + xf[:, :, :np_] * s
    assert U.ulp_distance(got, U.to_bits(want.astype(np.float32), dtype)).max() <= 1
    # direction: (1, 0) at angle a goes to (cos a, sin a)
    e = np.zeros((1, 1, D), np.float32)
    e[0, 0, 0] = 1.0
    r = U.from_bits(orc.apply_rope(U.to_bits(e, dtype), np.array([7], np.int32), tab, rd, dtype), dtype)
    assert abs(r[0, 0, 0] - tab[7, 0, 0]) < 4e-3 and abs(r[0, 0, np_] - tab[7, 0, 1]) < 4e-3
    assert np.sign(r[0, 0, np_]) == np.sign(tab[7, 0, 1])


@pytest.mark.parametrize("dtype", [orc.F16, orc.BF16])
def test_sigmoid_gate_matches_fp64_logistic(dtype):
    rng = np.random.default_rng(54)
    x = U.normal_bits(rng, (4096,), dtype, 2.0)
    g = U.normal_bits(rng, (4096,), dtype, 3.0)
    got = orc.sigmoid_gate(x, g, dtype)
    xf, gf = U.from_bits(x, dtype).astype(np.float64), U.from_bits(g, dtype).astype(np.float64)
    want = xf / (1.0 + np.exp(-gf))
    assert U.ulp_distance(got, U.to_bits(want.astype(np.float32), dtype)).max() <= 1
    half = orc.sigmoid_gate(x, np.zeros_like(g), dtype)      # gate 0: exactly x / 2
    assert np.array_equal(U.from_bits(half, dtype), U.from_bits(x, dtype) / 2)


def test_block_attention_mass_closed_forms():
    """Sum over a branch's blocks = number of query heads; equal keys spread the mass by token
    count; one dominant key collects it; a hole collects nothing."""
    L, KVH, QH, D, bs, NB = 1, 2, 8, 64, 16, 12
    g = orc.layout(L, KVH, QH, D, bs, NB, orc.BF16)
    rng = np.random.default_rng(55)
    n = 3 * bs + 5
    tables = np.array([[4, 9, 1, 7, -1], [2, 3, -1, 5, -1]], np.int32)
    lens = np.array([n, n], np.int32)
    pool = orc.new_pool(g)
    k = U.normal_bits(rng, (n, KVH, D), orc.BF16)
    v = U.normal_bits(rng, (n, KVH, D), orc.BF16)
    for b in range(2):
        orc.append_batch(g, pool, tables[b], 0, 0, k, v, orc.BF16)      # branch 1 has a hole at block 2
    q = U.normal_bits(rng, (2, QH, D), orc.BF16)
    m = orc.block_attention_mass(g, q, pool, tables, lens, 0, 0.125, orc.BF16, 5)
    assert np.allclose(m.sum(axis=1), QH, rtol=0, atol=1e-9)
    assert m[1, 2] == 0.0 and (m[:, 4] == 0.0).all() and (m[0, :4] > 0).all()
    # independent numpy softmax for branch 0
    kf = U.from_bits(k, orc.BF16).astype(np.float64)
    qf = U.from_bits(q[0], orc.BF16).astype(np.float64)
    want = np.zeros(5)
    for h in range(QH):
        s = kf[:, h // (QH // KVH)] @ qf[h] * 0.125
        p = np.exp(s - s.max())
        p /= p.sum()
        for t in range(n):
            want[t // bs] += p[t]
    assert np.allclose(m[0], want, rtol=1e-12, atol=1e-12)
    # equal keys: every token weighs 1/n
    pool2 = orc.new_pool(g)
    kc = np.broadcast_to(k[:1], k.shape).copy()
    orc.append_batch(g, pool2, tables[0], 0, 0, kc, v, orc.BF16)
    m2 = orc.block_attention_mass(g, q[:1], pool2, tables[:1], lens[:1], 0, 0.125, orc.BF16, 5)
    assert np.allclose(m2[0, :4], QH * np.array([bs, bs, bs, 5]) / n, atol=1e-9)
    # one dominant key (token 20, block 1) under a large scale
    kd = U.to_bits(np.zeros((n, KVH, D), np.float32), orc.BF16)
    kd[20] = U.to_bits(np.ones((KVH, D), np.float32), orc.BF16)
    qd = U.to_bits(np.ones((1, QH, D), np.float32), orc.BF16)
    pool3 = orc.new_pool(g)
    orc.append_batch(g, pool3, tables[0], 0, 0, kd, v, orc.BF16)
    m3 = orc.block_attention_mass(g, qd, pool3, tables[:1], lens[:1], 0, 1.0, orc.BF16, 5)
    assert abs(m3[0, 1] - QH) < 1e-9


@pytest.mark.parametrize("dtype", [orc.F16, orc.INT8])
def test_block_image_is_k_then_v_per_layer(dtype):
    """kv_swapper.cpp:183-198: for each layer the K plane of the block, then the V plane."""
    L, KVH, QH, D, bs, NB = 3, 2, 4, 16, 4, 5
    g = orc.layout(L, KVH, QH, D, bs, NB, dtype)
    lib = orc.lib()
    rng = np.random.default_rng(56)
    pool = rng.integers(0, 256, size=orc.pool_bytes(g)).astype(np.uint8)
    blk = 3
    img = orc.block_image(g, pool, blk)
    plane = lib.orc_kv_plane_bytes(C.byref(g))
    bstride = lib.orc_block_stride_bytes(C.byref(g))
    assert img.size == L * bstride
    for l in range(L):
        k0, v0 = lib.orc_k_off(C.byref(g), l, blk, 0, 0, 0), lib.orc_v_off(C.byref(g), l, blk, 0, 0, 0)
        assert np.array_equal(img[l * bstride:l * bstride + plane], pool[k0:k0 + plane])
        assert np.array_equal(img[l * bstride + plane:l * bstride + 2 * plane], pool[v0:v0 + plane])
        if dtype == orc.INT8:
            s0 = lib.orc_kscale_off(C.byref(g), l, blk, 0, 0)
            assert np.array_equal(img[l * bstride + 2 * plane:(l + 1) * bstride], pool[s0:s0 + bstride - 2 * plane])
    pool2 = np.zeros_like(pool)
    orc.block_from_image(g, pool2, 1, img)
    assert np.array_equal(orc.block_image(g, pool2, 1), img) and pool2.sum() == img.astype(np.int64).sum()
