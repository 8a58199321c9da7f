"""GPU: BASELINE's full sizes, checked through size-independent properties (the
CPU oracle would take minutes here): round trips, equality of independent
kernels, invariance under physical placement, closed-form attention results."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi
from tests import util as U

pytestmark = pytest.mark.gpu


def _torch():
    import torch
    return torch


def test_config2_full_size_properties(dev):
    """8 branches x 32k tokens, 32Q/8KV x128 bf16, pages shuffled over a 16 954-block
    pool (one layer of it resident here: the layer stride is the full 1.1 GB)."""
    torch = _torch()
    L, KVH, QH, D, bs, B, ctx = 2, 8, 32, 128, 16, 8, 32768
    NB = 16954
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    lib = cabi.lib()
    rng = np.random.default_rng(2)
    perm = rng.permutation(NB).astype(np.int32)
    nblk = ctx // bs
    tables = np.stack([perm[b * nblk:(b + 1) * nblk] for b in range(B)])
    pool = torch.zeros(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
    dtab = torch.from_numpy(tables).cuda()
    sp = U.stream_ptr()
    layer = 1
    gen = torch.Generator(device="cuda").manual_seed(7)
    srcs = []
    for b in range(B):
        k = (torch.randn(ctx, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        v = (torch.randn(ctx, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        cabi.call("drk_kv_append_batch", C.byref(g), U.p(pool), C.c_void_p(dtab[b].data_ptr()), layer, 1, 0, ctx,
                  U.p(k), U.p(v), cabi.BF16, sp)
        srcs.append((k, v))
    # 1. append then gather returns the source bit for bit (every branch, every token)
    flat = torch.empty(2 * 2 * ctx * KVH * D * 2, dtype=torch.uint8, device="cuda")
    for b in range(B):
        cabi.call("drk_kv_extract", C.byref(g), U.p(flat), None, U.p(pool), C.c_void_p(dtab[b].data_ptr()), 0, ctx, 2, sp)
        f = flat.view(torch.bfloat16).view(2, 2, ctx, KVH, D)
        assert torch.equal(f[1, 0], srcs[b][0]) and torch.equal(f[1, 1], srcs[b][1])
        assert not f[0].any()                                  # layer 0 was never written
    # 2. three independent kernels agree on the attention output
    q = (torch.randn(B, QH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
    lens = torch.full((B,), ctx, dtype=torch.int32, device="cuda")
    scale = 1 / np.sqrt(D)
    outs = {}
    for name, portable, which, split in (("stream", 0, 0, 0), ("tiled", 0, 2, 1024), ("portable", 1, 0, 2048)):
        lib.drk_debug_force_portable_decode(portable)
        lib.drk_debug_set_decode_kernel(which)
        wsb = max(lib.drk_decode_workspace_bytes(C.byref(g), B, ctx),
                  lib.drk_decode_workspace_bytes_for_split(C.byref(g), B, ctx, split) if split else 0)
        ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
        out = torch.zeros(B, QH, D, dtype=torch.bfloat16, device="cuda")
        try:
            cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(q), U.p(pool), U.p(dtab), nblk, U.p(lens), B,
                      ctx, U.p(out), layer, float(scale), cabi.BF16, split, U.p(ws), wsb, sp)
            U.sync()
        finally:
            lib.drk_debug_force_portable_decode(0)
            lib.drk_debug_set_decode_kernel(0)
        outs[name] = out.float().cpu().numpy()
    for name in ("tiled", "portable"):
        ok, ma, _ = U.rel_abs_ok(outs[name], outs["stream"])
        assert ok, (name, ma)
    # 3. torch's own fp32 attention on the gathered K/V of two branches
    for b in (0, B - 1):
        k, v = srcs[b][0].float(), srcs[b][1].float()                     # [ctx, KVH, D]
        qq = q[b].float().view(KVH, 4, D)
        s = torch.einsum("hgd,thd->hgt", qq, k) * scale
        want = torch.einsum("hgt,thd->hgd", torch.softmax(s, dim=-1), v).reshape(QH, D).cpu().numpy()
        ok, ma, _ = U.rel_abs_ok(outs["stream"][b], want)
        assert ok, (b, ma)
    # 4. moving every page to another physical block changes no bit of the output
    perm2 = np.roll(perm, 4321)
    tables2 = np.stack([perm2[b * nblk:(b + 1) * nblk] for b in range(B)])
    dtab2 = torch.from_numpy(tables2).cuda()
    pool2 = torch.zeros_like(pool)
    for b in range(B):
        cabi.call("drk_kv_append_batch", C.byref(g), U.p(pool2), C.c_void_p(dtab2[b].data_ptr()), layer, 1, 0, ctx,
                  U.p(srcs[b][0]), U.p(srcs[b][1]), cabi.BF16, sp)
    wsb = lib.drk_decode_workspace_bytes(C.byref(g), B, ctx)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    o1 = torch.zeros(B, QH, D, dtype=torch.bfloat16, device="cuda")
    o2 = torch.zeros_like(o1)
    for pl, tb, oo in ((pool, dtab, o1), (pool2, dtab2, o2)):
        cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(q), U.p(pl), U.p(tb), nblk, U.p(lens), B, ctx,
                  U.p(oo), layer, float(scale), cabi.BF16, 0, U.p(ws), wsb, sp)
    U.sync()
    assert torch.equal(o1, o2)


@pytest.mark.parametrize("dtype,tdt", [(cabi.INT8, "int8"), (cabi.FP8_E4M3, "fp8")])
def test_config4_full_length_quantised(dev, dtype, tdt):
    """One branch of 131 072 tokens with 1 % x20 outliers, quantised on append;
    attention must match torch fp32 attention on the DEQUANTISED pages, and the
    stream kernel must match the portable one."""
    torch = _torch()
    L, KVH, QH, D, bs, ctx = 1, 8, 32, 128, 16, 131072
    NB = ctx // bs + 4
    g = cabi.layout(L, KVH, QH, D, bs, NB, dtype)
    lib = cabi.lib()
    rng = np.random.default_rng(4)
    table = torch.from_numpy(rng.permutation(NB).astype(np.int32)).cuda()
    pool = torch.zeros(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(11)
    sp = U.stream_ptr()
    chunk = 16384
    for p0 in range(0, ctx, chunk):
        k = torch.randn(chunk, KVH, D, device="cuda", generator=gen)
        k = torch.where(torch.rand(k.shape, device="cuda", generator=gen) < 0.01, k * 20, k).to(torch.bfloat16)
        v = torch.randn(chunk, KVH, D, device="cuda", generator=gen)
        v = torch.where(torch.rand(v.shape, device="cuda", generator=gen) < 0.01, v * 20, v).to(torch.bfloat16)
        cabi.call("drk_kv_append_batch", C.byref(g), U.p(pool), U.p(table), 0, 1, p0, chunk, U.p(k), U.p(v), cabi.BF16, sp)
        U.sync()
    # dequantise what is stored (gather codes and scales through the C ABI)
    codes = torch.empty(2 * ctx * KVH * D, dtype=torch.uint8, device="cuda")
    scales = torch.empty(2 * ctx * KVH, dtype=torch.float16, device="cuda") if dtype == cabi.INT8 else None
    cabi.call("drk_kv_extract", C.byref(g), U.p(codes), U.p(scales), U.p(pool), U.p(table), 0, ctx, 1, sp)
    U.sync()
    if dtype == cabi.INT8:
        deq = codes.view(torch.int8).view(2, ctx, KVH, D).float() * scales.view(2, ctx, KVH, 1).float()
    else:
        deq = codes.view(torch.float8_e4m3fn).view(2, ctx, KVH, D).float()
    q = torch.randn(1, QH, D, device="cuda", generator=gen).to(torch.bfloat16)
    scale = 1 / np.sqrt(D)
    s = torch.einsum("hgd,thd->hgt", q[0].float().view(KVH, 4, D), deq[0]) * scale
    want = torch.einsum("hgt,thd->hgd", torch.softmax(s, dim=-1), deq[1]).reshape(QH, D).cpu().numpy()
    lens = torch.full((1,), ctx, dtype=torch.int32, device="cuda")
    res = {}
    for portable in (0, 1):
        lib.drk_debug_force_portable_decode(portable)
        try:
            wsb = lib.drk_decode_workspace_bytes(C.byref(g), 1, ctx)
            ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
            out = torch.zeros(1, QH, D, dtype=torch.bfloat16, device="cuda")
            cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(q), U.p(pool), U.p(table), NB, U.p(lens), 1,
                      ctx, U.p(out), 0, float(scale), cabi.BF16, 0, U.p(ws), wsb, sp)
            U.sync()
        finally:
            lib.drk_debug_force_portable_decode(0)
        res[portable] = out[0].float().cpu().numpy()
    for portable in (0, 1):
        ok, ma, _ = U.rel_abs_ok(res[portable], want)
        assert ok, (portable, ma)


def test_config5_full_chunk_prefill_rows(dev):
    """A 2 048-token chunk at position 30 720 (the last chunk of config 5): sampled
    rows of the MFMA prefill must equal decode attention at that row's length."""
    torch = _torch()
    L, KVH, QH, D, bs = 1, 8, 32, 128, 16
    total, M = 32768, 2048
    pos_start = total - M
    NB = total // bs
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    lib = cabi.lib()
    rng = np.random.default_rng(5)
    table = torch.from_numpy(rng.permutation(NB).astype(np.int32)).cuda()
    pool = torch.zeros(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(13)
    sp = U.stream_ptr()
    for p0 in range(0, total, 8192):
        k = torch.randn(8192, KVH, D, device="cuda", generator=gen).to(torch.bfloat16)
        v = torch.randn(8192, KVH, D, device="cuda", generator=gen).to(torch.bfloat16)
        cabi.call("drk_kv_append_batch", C.byref(g), U.p(pool), U.p(table), 0, 1, p0, 8192, U.p(k), U.p(v), cabi.BF16, sp)
        U.sync()
    q = torch.randn(M, QH, D, device="cuda", generator=gen).to(torch.bfloat16)
    out = torch.zeros_like(q)
    scale = 1 / np.sqrt(D)
    cabi.call("drk_paged_prefill_attention", C.byref(g), U.p(q), U.p(pool), U.p(table), U.p(out), 0, pos_start, M,
              float(scale), cabi.BF16, None, 0, sp)
    rows = [0, 1, 31, 32, 1000, 2047]
    lens = torch.tensor([pos_start + t + 1 for t in rows], dtype=torch.int32, device="cuda")
    tabs = table.repeat(len(rows), 1).contiguous()
    qd = q[rows].contiguous()
    od = torch.zeros_like(qd)
    wsb = lib.drk_decode_workspace_bytes(C.byref(g), len(rows), total)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(qd), U.p(pool), U.p(tabs), NB, U.p(lens), len(rows),
              total, U.p(od), 0, float(scale), cabi.BF16, 0, U.p(ws), wsb, sp)
    U.sync()
    ok, ma, _ = U.rel_abs_ok(out[rows].float().cpu().numpy(), od.float().cpu().numpy())
    assert ok, ma
    # fp32 causal attention in torch over the stored K and V (gathered through the C ABI): the sampled rows
    # of the chunk, for both chunk kernels
    flat = torch.empty(2 * total * KVH * D, dtype=torch.bfloat16, device="cuda")
    cabi.call("drk_kv_extract", C.byref(g), U.p(flat), None, U.p(pool), U.p(table), 0, total, 1, sp)
    U.sync()
    kv = flat.view(2, total, KVH, D).float()
    want = torch.empty(len(rows), QH, D, dtype=torch.float32, device="cuda")
    for i, t in enumerate(rows):
        n = pos_start + t + 1
        s = torch.einsum("hgd,thd->hgt", q[t].float().view(KVH, QH // KVH, D), kv[0, :n]) * scale
        want[i] = torch.einsum("hgt,thd->hgd", torch.softmax(s, dim=-1), kv[1, :n]).reshape(QH, D)
    want = want.cpu().numpy()
    for mode in (1, 0, 3):                                   # the library's choice (two-phase, global -> LDS), four-wave kernel, two-phase through registers
        lib.drk_debug_set_prefill_two_phase(mode)
        try:
            out2 = torch.zeros_like(q)
            cabi.call("drk_paged_prefill_attention", C.byref(g), U.p(q), U.p(pool), U.p(table), U.p(out2), 0, pos_start, M,
                      float(scale), cabi.BF16, None, 0, sp)
            U.sync()
        finally:
            lib.drk_debug_set_prefill_two_phase(1)
        ok, ma, _ = U.rel_abs_ok(out2[rows].float().cpu().numpy(), want)
        assert ok, (mode, ma)
    ok, ma, _ = U.rel_abs_ok(od.float().cpu().numpy(), want)
    assert ok, ma


def test_reference_model_shape_full_chunk_prefill_rows(dev):
    """The reference model's head shape (24 query over 4 kv heads x 256, blocks of 256 tokens, fp16): a 2 048-token chunk at
    position 30 720, sampled rows (first and last of a 21-token query tile among them) against fp32 causal attention in
    torch over the stored K and V, for the direct-to-LDS kernel (the library's choice) and the register-staging one."""
    torch = _torch()
    L, KVH, QH, D, bs = 1, 4, 24, 256, 256
    total, M = 32768, 2048
    pos_start = total - M
    NB = total // bs
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.F16)
    lib = cabi.lib()
    rng = np.random.default_rng(7)
    table = torch.from_numpy(rng.permutation(NB).astype(np.int32)).cuda()
    pool = torch.zeros(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(17)
    sp = U.stream_ptr()
    for p0 in range(0, total, 8192):
        k = (torch.randn(8192, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.float16)
        v = (torch.randn(8192, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.float16)
        cabi.call("drk_kv_append_batch", C.byref(g), U.p(pool), U.p(table), 0, 1, p0, 8192, U.p(k), U.p(v), cabi.F16, sp)
        U.sync()
    q = (torch.randn(M, QH, D, device="cuda", generator=gen) * 0.5).to(torch.float16)
    scale = 1 / np.sqrt(D)
    rows = [0, 1, 20, 21, 1000, 2046, 2047]
    flat = torch.empty(2 * total * KVH * D, dtype=torch.float16, device="cuda")
    cabi.call("drk_kv_extract", C.byref(g), U.p(flat), None, U.p(pool), U.p(table), 0, total, 1, sp)
    U.sync()
    kv = flat.view(2, total, KVH, D).float()
    want = torch.empty(len(rows), QH, D, dtype=torch.float32, device="cuda")
    for i, tq in enumerate(rows):
        n = pos_start + tq + 1
        s = torch.einsum("hgd,thd->hgt", q[tq].float().view(KVH, QH // KVH, D), kv[0, :n]) * scale
        want[i] = torch.einsum("hgt,thd->hgd", torch.softmax(s, dim=-1), kv[1, :n]).reshape(QH, D)
    want = want.cpu().numpy()
    for mode in (1, 3):
        lib.drk_debug_set_prefill_two_phase(mode)
        try:
            out = torch.zeros_like(q)
            cabi.call("drk_paged_prefill_attention", C.byref(g), U.p(q), U.p(pool), U.p(table), U.p(out), 0, pos_start, M,
                      float(scale), cabi.F16, None, 0, sp)
            U.sync()
        finally:
            lib.drk_debug_set_prefill_two_phase(1)
        ok, ma, _ = U.rel_abs_ok(out[rows].float().cpu().numpy(), want)
        assert ok, (mode, ma)


@pytest.mark.parametrize("shape", ["config5", "reference_model", "config5_int8", "config5_fp8"])
def test_full_chunk_frame_mass(dev, shape):
    """The attention mass of a full 2 048-token chunk at position 30 720 (config 5's shape over bf16, int8 and fp8
    pages, and the reference model's): the attention call leaves the rows' log-sum-exps, the one-walk pass adds every
    row's probabilities up by page.  Against fp32 softmax in torch over the stored K (dequantised for 8-bit pages; all
    2 048 x QH rows over 32 768 keys, summed per block), the pages of the whole context sum to rows x heads, and the
    register-staging kernel gives the same masses."""
    torch = _torch()
    io = None
    if shape == "config5":
        L, KVH, QH, D, bs, dt, tdt, amp = 1, 8, 32, 128, 16, cabi.BF16, torch.bfloat16, 1.0
    elif shape in ("config5_int8", "config5_fp8"):
        L, KVH, QH, D, bs, dt, tdt, amp = 1, 8, 32, 128, 16, (cabi.INT8 if shape == "config5_int8" else cabi.FP8_E4M3), torch.bfloat16, 1.0
        io = cabi.BF16
    else:
        L, KVH, QH, D, bs, dt, tdt, amp = 1, 4, 24, 256, 256, cabi.F16, torch.float16, 0.5
    total, M = 32768, 2048
    pos_start = total - M
    NB = total // bs
    g = cabi.layout(L, KVH, QH, D, bs, NB, dt)
    lib = cabi.lib()
    rng = np.random.default_rng(11)
    table = torch.from_numpy(rng.permutation(NB).astype(np.int32)).cuda()
    pool = torch.zeros(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(23)
    sp = U.stream_ptr()
    for p0 in range(0, total, 8192):
        k = (torch.randn(8192, KVH, D, device="cuda", generator=gen) * amp).to(tdt)
        v = (torch.randn(8192, KVH, D, device="cuda", generator=gen) * amp).to(tdt)
        cabi.call("drk_kv_append_batch", C.byref(g), U.p(pool), U.p(table), 0, 1, p0, 8192, U.p(k), U.p(v), io if io is not None else dt, sp)
        U.sync()
    q8 = io is not None
    if not q8:
        io = dt
    q = (torch.randn(M, QH, D, device="cuda", generator=gen) * amp).to(tdt)
    out = torch.zeros_like(q)
    scale = 1 / np.sqrt(D)
    lse = torch.zeros(M * QH, dtype=torch.float32, device="cuda")
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos_start, M)
    ws = torch.zeros(max(wsb, 16), dtype=torch.uint8, device="cuda")
    cabi.call("drk_paged_prefill_attention_lse", C.byref(g), U.p(q), U.p(pool), U.p(table), U.p(out), 0, pos_start, M,
              float(scale), io, None, 0, U.p(lse), U.p(ws), wsb, sp)
    got = {}
    try:
        for direct in (1, 0):
            lib.drk_debug_set_prefill_mass_direct(direct)
            mass = torch.full((NB,), 7.0, dtype=torch.float32, device="cuda")
            cabi.call("drk_paged_prefill_attention_mass_lse", C.byref(g), U.p(q), U.p(pool), U.p(table), 0, pos_start, M,
                      float(scale), io, U.p(lse), U.p(mass), NB, 0, sp)
            U.sync()
            got[direct] = mass.double().cpu().numpy()
    finally:
        lib.drk_debug_set_prefill_mass_direct(1)
    if q8:                                                   # codes and scales through the C ABI, dequantised here
        codes = torch.empty(2 * total * KVH * D, dtype=torch.uint8, device="cuda")
        scales = torch.empty(2 * total * KVH, dtype=torch.float16, device="cuda") if dt == cabi.INT8 else None
        cabi.call("drk_kv_extract", C.byref(g), U.p(codes), U.p(scales), U.p(pool), U.p(table), 0, total, 1, sp)
        U.sync()
        if dt == cabi.INT8:
            kk = codes.view(torch.int8).view(2, total, KVH, D)[0].float() * scales.view(2, total, KVH, 1)[0].float()
        else:
            kk = codes.view(torch.float8_e4m3fn).view(2, total, KVH, D)[0].float()
        del codes
    else:
        flat = torch.empty(2 * total * KVH * D, dtype=tdt, device="cuda")
        cabi.call("drk_kv_extract", C.byref(g), U.p(flat), None, U.p(pool), U.p(table), 0, total, 1, sp)
        U.sync()
        kk = flat.view(2, total, KVH, D)[0].float()
    G = QH // KVH
    keys = torch.arange(total, device="cuda")
    want = torch.zeros(total, dtype=torch.float64, device="cuda")
    for h in range(KVH):
        for r0 in range(0, M, 512):                          # 512 rows x G heads x 32 768 keys of fp32 scores at a time
            qq = q[r0:r0 + 512, h * G:(h + 1) * G].float()
            sc = torch.einsum("tgd,kd->tgk", qq, kk[:, h]) * scale
            vis = keys[None, None, :] <= (pos_start + r0 + torch.arange(qq.shape[0], device="cuda"))[:, None, None]
            sc = sc.masked_fill(~vis, float("-inf"))
            want += torch.softmax(sc, dim=-1).double().sum(dim=(0, 1))
    want = want.view(NB, bs).sum(dim=1).cpu().numpy()
    assert abs(want.sum() - M * QH) < 1e-3 * M * QH
    for direct in (1, 0):
        err = np.abs(got[direct] - want)
        assert np.all(err <= 2e-2 * np.abs(want) + 5e-2), (direct, err.max(), want[err.argmax()])
    assert abs(got[1].sum() - M * QH) <= 1e-4 * M * QH       # scored as the attention call scored: the rows' masses sum to 1
    assert abs(got[0].sum() - M * QH) <= 2e-3 * M * QH


@pytest.mark.parametrize("dtype", [cabi.BF16, cabi.INT8])
def test_pages_beyond_4GiB_of_a_layer(dev, dtype):
    """A pool whose single layer holds more than 4 GiB (a 288 GB part at 36 layers has 7 GiB per
    layer): pages at the top of it must be appended, gathered and attended exactly like the same
    tokens in a small pool -- same bits from the same production kernel, which must really be the
    tiled one (the portable kernel agrees within the attention tolerance only)."""
    torch = _torch()
    L, KVH, QH, D, bs = 1, 8, 32, 128, 16
    lib = cabi.lib()
    probe = cabi.layout(L, KVH, QH, D, bs, 1, dtype)
    per_block = lib.drk_kv_pool_bytes(C.byref(probe))
    NB_big = int(5.2 * 2 ** 30) // per_block
    lens_h = np.array([1500, 333], dtype=np.int32)
    nblk = [(int(n) + bs - 1) // bs for n in lens_h]
    stride = max(nblk) + 1
    NB_small = sum(nblk) + 3
    rng = np.random.default_rng(44)
    sp = U.stream_ptr()
    gen = torch.Generator(device="cuda").manual_seed(44)
    q = torch.randn(2, QH, D, device="cuda", generator=gen).to(torch.bfloat16)
    kv = [(torch.randn(int(n), KVH, D, device="cuda", generator=gen).to(torch.bfloat16),
           torch.randn(int(n), KVH, D, device="cuda", generator=gen).to(torch.bfloat16)) for n in lens_h]
    lens = torch.from_numpy(lens_h).cuda()
    outs, flats = {}, {}
    for name, NB in (("small", NB_small), ("big", NB_big)):
        g = cabi.layout(L, KVH, QH, D, bs, NB, dtype)
        assert lib.drk_kv_pool_bytes(C.byref(g)) > (4 << 30) or name == "small"
        ids = rng.permutation(NB_small) if name == "small" else NB - 1 - 5 * rng.permutation(NB_small)   # the top of the layer
        tab = np.full((2, stride), -1, dtype=np.int32)
        o = 0
        for b in range(2):
            tab[b, :nblk[b]] = ids[o:o + nblk[b]]
            o += nblk[b]
        dtab = torch.from_numpy(tab).cuda()
        pool = torch.empty(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
        for b in range(2):
            cabi.call("drk_kv_append_batch", C.byref(g), U.p(pool), C.c_void_p(dtab.data_ptr() + b * stride * 4), 0, 1, 0,
                      int(lens_h[b]), U.p(kv[b][0]), U.p(kv[b][1]), cabi.BF16, sp)
        E = 1 if dtype == cabi.INT8 else 2
        n0 = int(lens_h[0])
        flat = torch.empty(2 * n0 * KVH * D * E, dtype=torch.uint8, device="cuda")
        scales = torch.empty(2 * n0 * KVH, dtype=torch.float16, device="cuda") if dtype == cabi.INT8 else None
        cabi.call("drk_kv_extract", C.byref(g), U.p(flat), U.p(scales), U.p(pool), U.p(dtab), 0, n0, 1, sp)
        wsb = lib.drk_decode_workspace_bytes(C.byref(g), 2, int(lens_h.max()))
        ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
        out = torch.zeros(2, QH, D, dtype=torch.bfloat16, device="cuda")
        cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(q), U.p(pool), U.p(dtab), stride, U.p(lens), 2,
                  int(lens_h.max()), U.p(out), 0, float(1 / np.sqrt(D)), cabi.BF16, 0, U.p(ws), wsb, sp)
        U.sync()
        outs[name] = out.view(torch.int16).cpu().numpy()
        flats[name] = (flat.cpu().numpy(), scales.view(torch.int16).cpu().numpy() if scales is not None else None)
        if name == "big":
            lib.drk_debug_force_portable_decode(1)
            try:
                out2 = torch.zeros(2, QH, D, dtype=torch.bfloat16, device="cuda")
                wsb2 = lib.drk_decode_workspace_bytes(C.byref(g), 2, int(lens_h.max()))
                ws2 = torch.empty(wsb2, dtype=torch.uint8, device="cuda")
                cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(q), U.p(pool), U.p(dtab), stride, U.p(lens), 2,
                          int(lens_h.max()), U.p(out2), 0, float(1 / np.sqrt(D)), cabi.BF16, 0, U.p(ws2), wsb2, sp)
                U.sync()
            finally:
                lib.drk_debug_force_portable_decode(0)
            portable = out2.float().cpu().numpy()
        del pool
    assert np.array_equal(flats["big"][0], flats["small"][0])
    if dtype == cabi.INT8:
        assert np.array_equal(flats["big"][1], flats["small"][1])
    else:
        k0 = kv[0][0].view(torch.int16).cpu().numpy().reshape(-1)
        assert np.array_equal(flats["big"][0].view(np.int16)[:k0.size], k0)               # 16-bit pages: pure copies
    assert np.array_equal(outs["big"], outs["small"])
    got = torch.from_numpy(outs["big"]).view(torch.bfloat16).float().numpy()
    assert not np.array_equal(got, portable)                         # a different kernel produced the bits ...
    ok, ma, _ = U.rel_abs_ok(got, portable.astype(np.float64))
    assert ok, ma                                                     # ... of the same result


def test_config3_full_size_properties(dev):
    """BASELINE config 3 at its real sizes on one layer: a 65 536-token prefix (4 096 blocks) shared by 16
    copy-on-write branches with private tails of up to 4 096 tokens.  Properties that need no oracle at
    this size: every prefix block carries 17 references and the tables agree on them; the call that
    streams the prefix once equals the per-branch call; evicting down to 25 % free blocks frees private
    pages only -- the prefix keeps its references and its bytes (attention over it is unchanged)."""
    torch = _torch()
    from deusridet_amd import host
    L, KVH, QH, D, bs, B, P = 1, 8, 32, 128, 16, 16, 65536
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    cm = host.CacheManager()
    NBW = P // bs + B * (4096 // bs + 1) + 64
    assert cm.init(NBW * L * 2 * KVH * bs * D * 2, bs, None, 1 + B)
    NB, stride = cm.pool_max_blocks(), cm.table_stride()
    hl = host.lib()
    st = U.stream_ptr()
    gen = torch.Generator(device="cuda").manual_seed(3)

    def write(branch, pos0, n):
        k = (torch.randn(n, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        v = (torch.randn(n, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        hl.drkh_paged_kv_cache_write_batch(U.p(k), U.p(v), cm.pool_ptr(), cm.d_block_table(branch), 0, pos0, n, NB, bs, st)
        U.sync()

    assert cm.ensure_blocks_for_range(0, 0, P)
    cm.sync_block_table(st)
    for p0 in range(0, P, 8192):
        write(0, p0, 8192)
    cm.set_seq_len(0, P)
    rng = np.random.default_rng(3)
    priv = rng.integers(0, 4097, size=B)
    priv[0], priv[1] = 0, 4096
    kids = []
    for i in range(B):
        b = cm.fork_branch(0, P)
        assert b > 0
        kids.append(b)
    prefix = cm.h_block_table(0)[:P // bs].copy()
    assert all(cm.pool_refcount(int(x)) == 1 + B for x in prefix[[0, 1, 2047, 4095]])
    for i, b in enumerate(kids):
        n = int(priv[i])
        if n:
            assert cm.ensure_blocks_for_range(b, P, n)
    cm.sync_block_table(st)
    for i, b in enumerate(kids):
        if priv[i]:
            write(b, P, int(priv[i]))
        cm.set_seq_len(b, P + int(priv[i]))
        assert np.array_equal(cm.h_block_table(b)[:P // bs], prefix)           # the shared pages, not copies
    assert cm.common_prefix_tokens(kids) == P
    lens = (P + priv).astype(np.int32)
    mx = int(lens.max())
    tabs = np.stack([cm.h_block_table(b) for b in kids])
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    lib = cabi.lib()
    pool_ptr = C.c_void_p(cm.pool_ptr()) if not isinstance(cm.pool_ptr(), C.c_void_p) else cm.pool_ptr()
    q = (torch.randn(B, QH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
    dl, dt = U.dev_i32(lens), U.dev_i32(tabs)
    wsb = max(lib.drk_decode_shared_workspace_bytes(C.byref(g), B, mx, P), lib.drk_decode_workspace_bytes(C.byref(g), B, mx))
    ws = U.dev_zeros(wsb)
    scale = float(1 / np.sqrt(D))

    def attend(shared):
        out = torch.zeros_like(q)
        if shared:
            cabi.call("drk_paged_decode_attention_shared", C.byref(g), U.p(q), pool_ptr, U.p(dt), stride, U.p(dl), B, mx, P, U.p(out),
                      0, scale, cabi.BF16, U.p(ws), wsb, st)
        else:
            cabi.call("drk_paged_decode_attention_branches", C.byref(g), U.p(q), pool_ptr, U.p(dt), stride, U.p(dl), B, mx, U.p(out),
                      0, scale, cabi.BF16, 0, U.p(ws), wsb, st)
        U.sync()
        return out.float().cpu().numpy()

    once, per_branch = attend(True), attend(False)
    ok, ma, _ = U.rel_abs_ok(once, per_branch)
    assert ok, ma
    # torch fp32 attention over what the pool holds (prefix + private tail, gathered through the C ABI) for
    # three branches: no tail, the longest tail, the last one -- against both prefix kernels and the per-branch call
    lib.drk_debug_set_prefix_stream(0)
    try:
        once_staged = attend(True)
    finally:
        lib.drk_debug_set_prefix_stream(1)
    for i in (0, 1, B - 1):
        n = int(lens[i])
        flat = torch.empty(2 * n * KVH * D, dtype=torch.bfloat16, device="cuda")
        cabi.call("drk_kv_extract", C.byref(g), U.p(flat), None, pool_ptr, U.p(dt[i]), 0, n, 1, st)
        U.sync()
        kv = flat.view(2, n, KVH, D).float()
        s = torch.einsum("hgd,thd->hgt", q[i].float().view(KVH, QH // KVH, D), kv[0]) * scale
        want = torch.einsum("hgt,thd->hgd", torch.softmax(s, dim=-1), kv[1]).reshape(QH, D).cpu().numpy()
        for name, got in (("prefix once", once), ("prefix once, every wave stages", once_staged), ("per branch", per_branch)):
            ok, ma, _ = U.rel_abs_ok(got[i], want)
            assert ok, (name, i, ma)
    # make room for 500 more blocks: private pages go (oldest first), the prefix stays
    private_blocks = int(sum((int(n) + bs - 1) // bs for n in priv))
    assert private_blocks > 600
    free0 = cm.free_blocks()
    assert cm.ensure_free_blocks(free0 + 500) and cm.free_blocks() == free0 + 500
    assert not cm.ensure_free_blocks(NB - P // bs + 1)                          # more than everything unshared: refused ...
    assert cm.free_blocks() == NB - P // bs                                     # ... after every private page has gone
    assert all(cm.pool_refcount(int(x)) == 1 + B for x in prefix[[0, 1, 2047, 4095]])
    for b in kids:
        assert np.array_equal(cm.h_block_table(b)[:P // bs], prefix)
        assert (cm.h_block_table(b)[P // bs:] < 0).all()
    # attention over the prefix alone is what it was: same bytes, same tables
    cm.sync_block_table(st)
    dl2 = U.dev_i32(np.full(B, P, np.int32))
    dt2 = U.dev_i32(np.stack([cm.h_block_table(b) for b in kids]))
    out_a, out_b = torch.zeros_like(q), torch.zeros_like(q)
    cabi.call("drk_paged_decode_attention_shared", C.byref(g), U.p(q), pool_ptr, U.p(dt2), stride, U.p(dl2), B, P, P, U.p(out_a), 0,
              scale, cabi.BF16, U.p(ws), wsb, st)
    cabi.call("drk_paged_decode_attention_shared", C.byref(g), U.p(q), pool_ptr, U.p(dt), stride, U.p(dl2), B, P, P, U.p(out_b), 0,
              scale, cabi.BF16, U.p(ws), wsb, st)
    U.sync()
    assert torch.equal(out_a, out_b)


def test_config3_fork_tree_layer_in_one_call(dev):
    """Config 3 at its real sizes through the host classes: a 65 536-token prefix, 16 branches forked from it and from one
    another at random block boundaries (every fourth inside a block: copy-on-write), private tails of up to 4 096
    tokens.  Three decode steps, each as the caller runs it -- blocks for the new token (copies where a page is still
    shared), table upload, CacheManager::common_prefix_groups, the step's plan -- then the layer twice from the same
    pool bytes: append + planned attention as two calls, and drk_kv_append_decode_planned (the attention launch
    writes the new rows).  Same pool bytes, same output bits; the new token's page is the branch's own in every
    step."""
    torch = _torch()
    from deusridet_amd import host
    L, KVH, QH, D, bs, B, P = 1, 8, 32, 128, 16, 16, 65536
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    cm = host.CacheManager()
    rng = np.random.default_rng(12)
    private = rng.integers(0, 4097, size=B)
    NBW = P // bs + int(private.sum()) // bs + 8 * B + 64
    assert cm.init(NBW * L * 2 * KVH * bs * D * 2, bs, None, 1 + B)
    NB, stride = cm.pool_max_blocks(), cm.table_stride()
    st = U.stream_ptr()
    lib = cabi.lib()
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    pool_ptr = C.c_void_p(cm.pool_ptr())
    pool_bytes = lib.drk_kv_pool_bytes(C.byref(g))
    gen = torch.Generator(device="cuda").manual_seed(5)

    def bulk(branch, p0, m):
        assert cm.ensure_blocks_for_range(branch, p0, m)
        cm.sync_block_table(st)
        k = (torch.randn(L, m, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        v = (torch.randn(L, m, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        cabi.call("drk_kv_append_batch", C.byref(g), pool_ptr, C.c_void_p(cm.d_block_table(branch)), 0, L, p0, m, U.p(k), U.p(v),
                  cabi.BF16, st)
        U.sync()
        cm.set_seq_len(branch, p0 + m)

    for p0 in range(0, P, 8192):
        bulk(0, p0, 8192)
    parent = [-1] + [int(rng.integers(-1, i)) for i in range(1, B)]
    forks = []

    def grow(node, par_branch, fp):
        if node % 4 == 0:
            fp -= int(rng.integers(1, bs))
        b = cm.fork_branch(par_branch, fp)
        assert b > 0
        forks.append(b)
        for p0 in range(0, int(private[node]), 2048):
            bulk(b, fp + p0, min(2048, int(private[node]) - p0))
        descend(node, b)

    def descend(node, branch):
        held = cm.seq_len(branch)
        kids = [(P + bs * int(rng.integers(0, (held - P) // bs + 1)) if branch else P, c)
                for c in range(node + 1, B) if parent[c] == node]
        for fp, c in sorted(kids, key=lambda k: -k[0]):
            grow(c, branch, fp)

    descend(-1, 0)
    assert forks == list(range(forks[0], forks[0] + B))
    dtabs = C.c_void_p(cm.d_block_table(forks[0]))
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    before = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
    after_two = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
    after_one = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")

    def copy(dst, src):
        U.sync()
        assert hip.hipMemcpy(dst, src, pool_bytes, 3) == 0

    q = (torch.randn(B, QH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
    scale = float(1 / np.sqrt(D))
    n_with_groups = 0
    for step in range(3):
        lens = np.array([cm.seq_len(b) for b in forks], dtype=np.int32)
        for i, b in enumerate(forks):
            assert cm.ensure_blocks_for(b, int(lens[i]))                 # the new token's block; a copy where it is shared
        cm.sync_block_table(st)
        groups = cm.common_prefix_groups(forks, 64 // (QH // KVH), 256, cabi.MAX_PREFIX_GROUPS)
        n_with_groups += len(groups) >= 3
        arr = cabi.prefix_groups(groups)
        tabs = np.stack([cm.h_block_table(b) for b in forks])
        for i in range(B):                                               # nobody else maps the page the new token goes to
            blk = tabs[i, int(lens[i]) // bs]
            assert blk >= 0 and (tabs[:, :] == blk).sum() == 1
        mx = int(lens.max()) + 1
        dlen, dpos = U.dev_i32(lens + 1), U.dev_i32(lens)
        pb = lib.drk_decode_plan_bytes(C.byref(g), B, mx, len(groups))
        plan = U.dev_zeros(pb)
        cabi.call("drk_decode_plan_build", C.byref(g), dtabs, stride, U.p(dlen), B, mx, arr, len(groups), U.p(plan), pb, st)
        wsb = lib.drk_decode_grouped_workspace_bytes(C.byref(g), B, mx, arr, len(groups))
        ws = U.dev_zeros(wsb)
        nk = (torch.randn(B, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        nv = (torch.randn(B, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        out_two, out_one = torch.zeros_like(q), torch.zeros_like(q)
        copy(U.p(before), pool_ptr)
        cabi.call("drk_kv_append_branches", C.byref(g), pool_ptr, dtabs, stride, U.p(dpos), B, 0, 1, U.p(nk), U.p(nv), cabi.BF16, st)
        cabi.call("drk_paged_decode_attention_planned", C.byref(g), U.p(q), pool_ptr, dtabs, stride, U.p(dlen), B, mx, arr,
                  len(groups), U.p(plan), U.p(out_two), 0, scale, cabi.BF16, None, 0, U.p(ws), wsb, st)
        copy(U.p(after_two), pool_ptr)
        copy(pool_ptr, U.p(before))
        cabi.call("drk_kv_append_decode_planned", C.byref(g), pool_ptr, dtabs, stride, U.p(dlen), B, mx, arr, len(groups),
                  U.p(plan), U.p(nk), U.p(nv), cabi.BF16, U.p(q), U.p(out_one), 0, scale, cabi.BF16, None, 0, U.p(ws), wsb, st)
        copy(U.p(after_one), pool_ptr)
        assert torch.equal(after_one, after_two), step
        assert not torch.equal(after_one, before), step
        assert torch.equal(out_one, out_two), step
        assert bool(torch.isfinite(out_one.float()).all())
        for i, b in enumerate(forks):
            cm.set_seq_len(b, int(lens[i]) + 1)
    assert n_with_groups == 3


def test_config3_sustained_eviction(dev):
    """BASELINE config 3 run for 520 decode steps on two layers: a 65 536-token prefix shared by 16 copy-on-write
    branches with private tails of up to 4 096 tokens, every step appends one token per branch and layer and
    attends with the prefix streamed once; at steps 256 and 512 the pool is brought to 25 % free blocks.  After
    each eviction: the free count, the references on the prefix pages (parent + 16 forks), the prefix rows of
    every table and the bytes of the prefix are what they were; at the end two branches are checked against
    torch fp32 attention over the pages their tables still name."""
    torch = _torch()
    from deusridet_amd import host
    L, KVH, QH, D, bs, B, P = 2, 8, 32, 128, 16, 16, 65536
    steps, evict_at = 520, (256, 512)
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    rng = np.random.default_rng(33)
    priv = rng.integers(0, 4097, size=B)
    priv[0], priv[1] = 0, 4096
    cm = host.CacheManager()
    want_blocks = int((P // bs + int(priv.sum()) // bs + 4 * B + steps * B // bs) / 0.8)     # ~80 % full when everything is resident
    assert cm.init(want_blocks * L * 2 * KVH * bs * D * 2, bs, None, 1 + B)
    NB, stride = cm.pool_max_blocks(), cm.table_stride()
    st = U.stream_ptr()
    lib = cabi.lib()
    pool_ptr = C.c_void_p(cm.pool_ptr())
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    gen = torch.Generator(device="cuda").manual_seed(34)

    def bulk(branch, p0, m):
        assert cm.ensure_blocks_for_range(branch, p0, m)
        cm.sync_block_table(st)
        k = (torch.randn(L, m, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        v = (torch.randn(L, m, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
        cabi.call("drk_kv_append_batch", C.byref(g), pool_ptr, C.c_void_p(cm.d_block_table(branch)), 0, L, p0, m, U.p(k), U.p(v),
                  cabi.BF16, st)
        U.sync()
        cm.set_seq_len(branch, p0 + m)

    for p0 in range(0, P, 8192):
        bulk(0, p0, 8192)
    kids = [cm.fork_branch(0, P) for _ in range(B)]
    assert min(kids) > 0 and kids == list(range(kids[0], kids[0] + B))
    for b, n in zip(kids, priv):
        for p0 in range(0, int(n), 2048):
            bulk(b, P + p0, min(2048, int(n) - p0))
    prefix_blocks = cm.h_block_table(0)[:P // bs].copy()

    def prefix_bytes():
        flat = torch.empty(L * 2 * P * KVH * D, dtype=torch.bfloat16, device="cuda")
        cabi.call("drk_kv_extract", C.byref(g), U.p(flat), None, pool_ptr, C.c_void_p(cm.d_block_table(0)), 0, P, L, st)
        U.sync()
        return flat

    prefix0 = prefix_bytes()
    scale = float(1 / np.sqrt(D))
    q = (torch.randn(L, B, QH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
    nk = (torch.randn(L, B, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
    nv = (torch.randn(L, B, KVH, D, device="cuda", generator=gen) * 0.5).to(torch.bfloat16)
    out = torch.zeros(L, B, QH, D, device="cuda", dtype=torch.bfloat16)
    lens = np.array([cm.seq_len(b) for b in kids], dtype=np.int32)
    max_ctx = int(lens.max()) + steps + 1
    wsb = lib.drk_decode_shared_workspace_bytes(C.byref(g), B, max_ctx, P)
    ws = U.dev_zeros(wsb)
    dpos = torch.zeros(B, dtype=torch.int32, device="cuda")
    dlen = torch.zeros(B, dtype=torch.int32, device="cuda")
    dtabs = C.c_void_p(cm.d_block_table(kids[0]))
    qrow, krow = B * QH * D * 2, B * KVH * D * 2
    evictions = 0
    for s in range(1, steps + 1):
        for i, b in enumerate(kids):
            assert cm.ensure_blocks_for(b, int(lens[i]))
        if s in evict_at:
            before = cm.free_blocks()
            assert cm.ensure_free_blocks(NB // 4)
            assert cm.free_blocks() >= NB // 4 and cm.free_blocks() > before      # the pool was fuller than that: pages went
            evictions += 1
            assert all(cm.pool_refcount(int(x)) == 1 + B for x in prefix_blocks[[0, 1, 1000, 2047, 4095]])
            for b in kids:
                assert np.array_equal(cm.h_block_table(b)[:P // bs], prefix_blocks)
                assert cm.h_block_table(b)[int(lens[kids.index(b)]) // bs] >= 0    # the page this step writes stayed
            assert cm.common_prefix_tokens(kids) == P
        cm.sync_block_table(st)
        if s in evict_at:
            assert torch.equal(prefix_bytes(), prefix0)
        dpos.copy_(torch.from_numpy(lens))
        dlen.copy_(torch.from_numpy(lens + 1))
        for l in range(L):
            cabi.call("drk_kv_append_branches", C.byref(g), pool_ptr, dtabs, stride, U.p(dpos), B, l, 1,
                      C.c_void_p(nk.data_ptr() + l * krow), C.c_void_p(nv.data_ptr() + l * krow), cabi.BF16, st)
            cabi.call("drk_paged_decode_attention_shared", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow), pool_ptr, dtabs, stride,
                      U.p(dlen), B, max_ctx, P, C.c_void_p(out.data_ptr() + l * qrow), l, scale, cabi.BF16, U.p(ws), wsb, st)
        U.sync()                                                  # the device arrays are rewritten by the next step
        lens += 1
        for i, b in enumerate(kids):
            cm.set_seq_len(b, int(lens[i]))
    assert evictions == 2
    holes = sum(int((cm.h_block_table(b)[:(int(lens[i]) + bs - 1) // bs] < 0).sum()) for i, b in enumerate(kids))
    assert holes > 0                                              # private pages did go
    # the last step's output of layer 1 for two branches, against fp32 attention over the pages still present
    l = L - 1
    for i in (1, B - 1):
        n = int(lens[i])
        table = cm.h_block_table(kids[i])
        present = torch.from_numpy(np.repeat(table[:(n + bs - 1) // bs] >= 0, bs)[:n]).cuda()
        flat = torch.empty(L * 2 * n * KVH * D, dtype=torch.bfloat16, device="cuda")
        cabi.call("drk_kv_extract", C.byref(g), U.p(flat), None, pool_ptr, C.c_void_p(cm.d_block_table(kids[i])), 0, n, L, st)
        U.sync()
        kv = flat.view(L, 2, n, KVH, D)[l].float()
        sc = torch.einsum("hgd,thd->hgt", q[l, i].float().view(KVH, QH // KVH, D), kv[0]) * scale
        sc = sc.masked_fill(~present, float("-inf"))
        want = torch.einsum("hgt,thd->hgd", torch.softmax(sc, dim=-1), kv[1]).reshape(QH, D).cpu().numpy()
        ok, ma, _ = U.rel_abs_ok(out[l, i].float().cpu().numpy(), want)
        assert ok, (i, ma)
