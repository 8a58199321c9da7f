"""GPU: the per-step launch sequence (append one token per branch, attend) is
capturable in a HIP graph -- no entry point allocates, memsets or synchronises --
and every replay equals the eager run of the same step."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi
from tests import util as U

pytestmark = pytest.mark.gpu


def test_decode_step_graph_replays_match_eager(dev):
    import torch
    L, KVH, QH, D, bs, B, NB = 3, 8, 32, 128, 16, 4, 400
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    lib = cabi.lib()
    rng = np.random.default_rng(1)
    start = np.array([700, 64, 1023, 5], dtype=np.int32)
    steps = 6
    nblk = (int(start.max()) + 2 * steps + bs) // bs + 1
    perm = rng.permutation(NB).astype(np.int32)
    tables = torch.from_numpy(np.stack([perm[b * nblk:(b + 1) * nblk] for b in range(B)])).cuda()
    gen = torch.Generator(device="cuda").manual_seed(3)

    def fresh_pool():
        pool = torch.zeros(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
        g2 = torch.Generator(device="cuda").manual_seed(5)
        for b in range(B):
            n = int(start[b])
            k = torch.randn(L, n, KVH, D, device="cuda", generator=g2).to(torch.bfloat16)
            v = torch.randn(L, n, KVH, D, device="cuda", generator=g2).to(torch.bfloat16)
            cabi.call("drk_kv_append_batch", C.byref(g), U.p(pool), C.c_void_p(tables[b].data_ptr()), 0, L, 0, n,
                      U.p(k), U.p(v), cabi.BF16, U.stream_ptr())
        torch.cuda.synchronize()
        return pool

    q = torch.randn(L, B, QH, D, device="cuda", generator=gen).to(torch.bfloat16)
    nk = torch.randn(steps, L, B, KVH, D, device="cuda", generator=gen).to(torch.bfloat16)
    nv = torch.randn(steps, L, B, KVH, D, device="cuda", generator=gen).to(torch.bfloat16)
    max_ctx = int(start.max()) + steps + 1
    wsb = lib.drk_decode_workspace_bytes(C.byref(g), B, max_ctx)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    scale = 1 / np.sqrt(D)
    qrow, krow = B * QH * D * 2, B * KVH * D * 2

    def launch_step(pool, pos, lens, kbuf, vbuf, out):
        sp = U.stream_ptr()
        for l in range(L):
            cabi.call("drk_kv_append_branches", C.byref(g), U.p(pool), U.p(tables), nblk, U.p(pos), B, l, 1,
                      C.c_void_p(kbuf.data_ptr() + l * krow), C.c_void_p(vbuf.data_ptr() + l * krow), cabi.BF16, sp)
            cabi.call("drk_paged_decode_attention_branches", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow), U.p(pool),
                      U.p(tables), nblk, U.p(lens), B, max_ctx, C.c_void_p(out.data_ptr() + l * qrow), l, float(scale),
                      cabi.BF16, 0, U.p(ws), wsb, sp)

    # eager reference
    pool_e = fresh_pool()
    pos = torch.from_numpy(start.copy()).cuda()
    eager = []
    for s in range(steps):
        out = torch.zeros(L, B, QH, D, dtype=torch.bfloat16, device="cuda")
        launch_step(pool_e, pos, pos + 1, nk[s], nv[s], out)
        torch.cuda.synchronize()
        eager.append(out.clone())
        pos += 1

    # one captured step, replayed; inputs are refreshed by eager copies between replays
    pool_g = fresh_pool()
    pos_g = torch.from_numpy(start.copy()).cuda()
    lens_g = pos_g + 1
    kbuf, vbuf = nk[0].clone(), nv[0].clone()
    out_g = torch.zeros(L, B, QH, D, dtype=torch.bfloat16, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up on the capture stream
        launch_step(pool_g, pos_g, lens_g, kbuf, vbuf, out_g)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    pool_g = fresh_pool()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch_step(pool_g, pos_g, lens_g, kbuf, vbuf, out_g)
    for s in range(steps):
        kbuf.copy_(nk[s]); vbuf.copy_(nv[s])
        out_g.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, eager[s]), f"replay {s} differs from the eager step"
        pos_g += 1
        lens_g += 1
    assert torch.equal(pool_g, pool_e)
