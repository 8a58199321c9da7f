"""GPU: the drop-in boundary beyond single calls.

  - the reference's two layer wrappers, full_attention_forward_paged[_prefill]
    (src/machina/paged_attention.h:75-106, .cu:314-376, 563-638), with the projections served
    from buffers: pool bit for bit and gated attention within the attention tolerance against
    the oracle's composition of the reference's separate steps;
  - perception on one stream and decode on another over one pool (the reference's P/D split,
    docs/en/architecture/11-machina.md:22-31): each stream has split-K partials of its own;
  - a captured decode step that is replayed after a perception frame has run behind a long
    context (the frame needs more workspace than the step did: nothing the step captured may move);
  - the scorer a KvStream is given must cover every branch's table row, and a closed branch
    leaves no attention mass behind."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi, host
from oracle import binding as orc
from tests import test_gpu_stream as ts
from tests import util as U

pytestmark = pytest.mark.gpu


@pytest.fixture
def long_context():
    saved = (ts.NPOS, ts.POOL_BLOCKS)
    ts.NPOS, ts.POOL_BLOCKS = 2304, 170
    yield
    ts.NPOS, ts.POOL_BLOCKS = saved


def _inputs(rng, T):
    return tuple(U.normal_bits(rng, sh, ts.DT, m) for sh, m in (((T, ts.QH, 2 * ts.D), 1.0), ((T, ts.KVH, ts.D), 0.7),
                                                                  ((T, ts.KVH, ts.D), 0.5)))


def test_layer_wrappers_match_the_oracle(dev):
    import torch
    L, QH, KVH, D, BS = ts.L, ts.QH, ts.KVH, ts.D, ts.BS
    s = ts.Session(1)
    rng = np.random.default_rng(31)
    qw, kw = U.normal_bits(rng, (D,), ts.DT), U.normal_bits(rng, (D,), ts.DT)
    dqw, dkw = U.dev_bytes(qw), U.dev_bytes(kw)
    og = orc.layout(L, KVH, QH, D, BS, s.NB, ts.KVDT)
    opool = orc.new_pool(og)
    host.lib().drkh_set_rope_table(U.p(s.dtab), ts.NPOS)
    T = 64
    state = dict(q_buf=U.dev_zeros(T * QH * 2 * D * 2), kv_buf=U.dev_zeros(T * KVH * D * 2), dn_z=U.dev_zeros(T * 2 * KVH * D * 2),
                 dn_qkv=U.dev_zeros(T * QH * D * 2), attn_out=U.dev_zeros(T * QH * D * 2), norm_out=U.dev_zeros(T * QH * D * 2))
    bufs = (C.c_void_p * 6)(*[t.data_ptr() for t in state.values()])
    dpos = U.dev_i32(np.zeros(1, np.int32))
    st = U.stream_ptr()
    NB, pool_ptr = s.cm.pool_max_blocks(), s.cm.pool_ptr()
    pos0 = 0
    try:
        for M in (40, 7):                                              # two chunks through the prefill wrapper
            assert s.cm.ensure_blocks_for_range(0, pos0, M)
            s.cm.sync_block_table(st)
            table0 = s.cm.h_block_table(0).copy()
            for layer in range(L):
                qg, k, v = _inputs(rng, M)
                dqg, dk, dv = U.dev_bytes(qg), U.dev_bytes(k), U.dev_bytes(v)
                host.lib().drkh_full_attention_forward_paged_prefill(U.p(dqg), U.p(dk), U.p(dv), U.p(dqw), U.p(dkw), pool_ptr,
                                                                     s.cm.d_block_table(0), layer, pos0, M, pos0 + M, NB, BS, bufs, st)
                U.sync()
                got = U.host(state["norm_out"], np.uint16)[:M * QH * D].reshape(M, QH, D)
                pos = (pos0 + np.arange(M)).astype(np.int32)
                want = ts.oracle_layer(og, opool, [table0] * M, pos, layer, qg, k, v, qw, kw, s.tab)
                ok, mx, _ = U.rel_abs_ok(U.from_bits(got, ts.DT), want)
                assert ok, ("prefill", M, layer, mx)
            pos0 += M
            s.cm.set_seq_len(0, pos0)
        for step in range(3):                                          # single tokens through the decode wrapper
            assert s.cm.ensure_blocks_for(0, pos0)
            s.cm.sync_block_table(st)
            dpos.copy_(torch.tensor([pos0], dtype=torch.int32))
            table0 = s.cm.h_block_table(0).copy()
            for layer in range(L):
                qg, k, v = _inputs(rng, 1)
                dqg, dk, dv = U.dev_bytes(qg), U.dev_bytes(k), U.dev_bytes(v)
                host.lib().drkh_full_attention_forward_paged(U.p(dqg), U.p(dk), U.p(dv), U.p(dqw), U.p(dkw), pool_ptr,
                                                             s.cm.d_block_table(0), layer, pos0, pos0 + 1, NB, BS, bufs, U.p(dpos), st)
                U.sync()
                got = U.host(state["norm_out"], np.uint16)[:QH * D].reshape(1, QH, D)
                want = ts.oracle_layer(og, opool, [table0], np.array([pos0], np.int32), layer, qg, k, v, qw, kw, s.tab)
                ok, mx, _ = U.rel_abs_ok(U.from_bits(got, ts.DT), want)
                assert ok, ("decode", step, layer, mx)
            pos0 += 1
            s.cm.set_seq_len(0, pos0)
        assert np.array_equal(s.pool(), opool)                         # what the wrappers wrote: every byte
    finally:
        host.lib().drkh_set_rope_table(None, 0)


def test_prefill_and_decode_on_two_streams_over_one_pool(dev):
    """A short perception chunk behind 2 304 tokens of one sequence (context split over the chip: it keeps
    partials) on one stream, a decode step of six other sequences on another, both through the calls
    that take no workspace, launched back to back many times without waiting: the streams must not
    share partials.  Both results against the fp64 oracle."""
    import torch
    L, KVH, QH, D, bs, NB = 1, 8, 32, 128, 16, 900
    dt = cabi.BF16
    assert host.set_attention_geometry(L, QH, KVH, D, dt, dt)
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dt)
    rng = np.random.default_rng(77)
    perm = rng.permutation(NB).astype(np.int32)
    ctx, M = 2304, 24                                                  # the chunk is tokens 2280..2303
    lens = np.array([1500, 900, 2000, 640, 1111, 1800], np.int32)
    nblk = [(ctx + bs - 1) // bs] + [int(n + bs - 1) // bs for n in lens]
    stride = max(nblk) + 1
    tables = np.full((1 + len(lens), stride), -1, np.int32)
    o = 0
    for i, n in enumerate(nblk):
        tables[i, :n] = perm[o:o + n]
        o += n
    assert o <= NB
    opool = orc.new_pool(og)
    for i, n in enumerate([ctx] + lens.tolist()):
        k, v = U.normal_bits(rng, (n, KVH, D), dt, 0.7), U.normal_bits(rng, (n, KVH, D), dt, 0.5)
        orc.append_batch(og, opool, tables[i], 0, 0, k, v, dt)
    qp = U.normal_bits(rng, (M, QH, D), dt)
    qd = U.normal_bits(rng, (len(lens), QH, D), dt)
    scale = 1.0 / np.sqrt(D)
    want_p = np.stack([orc.decode_f64(og, qp[t], opool, tables[0], 0, ctx - M + t + 1, scale, dt) for t in range(M)])
    want_d = np.stack([orc.decode_f64(og, qd[b], opool, tables[1 + b], 0, int(lens[b]), scale, dt) for b in range(len(lens))])
    dpool, dtab = U.dev_bytes(opool), U.dev_i32(tables)
    dqp, dqd, dlens = U.dev_bytes(qp), U.dev_bytes(qd), U.dev_i32(lens)
    outp, outd = U.dev_zeros(M * QH * D * 2), U.dev_zeros(len(lens) * QH * D * 2)
    assert cabi.lib().drk_prefill_workspace_bytes(C.byref(g), ctx - M, M) > 0
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    p1, p2 = C.c_void_p(s1.cuda_stream), C.c_void_p(s2.cuda_stream)
    torch.cuda.synchronize()
    H = host.lib()
    try:
        for it in range(40):
            H.drkh_paged_prefill_attention(U.p(dqp), U.p(dpool), U.p(dtab), U.p(outp), 0, ctx - M, M, NB, bs, float(scale), p1)
            H.drkh_paged_gqa_decode_attention_branches(U.p(dqd), U.p(dpool), U.p(dtab[1:]), stride, U.p(dlens), len(lens),
                                                       int(lens.max()), U.p(outd), 0, NB, bs, float(scale), p2)
            if it % 8 == 7:
                torch.cuda.synchronize()
                for name, out, want, shape in (("prefill", outp, want_p, (M, QH, D)), ("decode", outd, want_d, (len(lens), QH, D))):
                    ok, mx, _ = U.rel_abs_ok(U.from_bits(U.host(out, np.uint16, shape), dt), want)
                    assert ok, (name, it, mx)
                outp.zero_(); outd.zero_()
                torch.cuda.synchronize()
    finally:
        torch.cuda.synchronize()
        H.drkh_paged_attention_release_workspace()


def test_captured_step_survives_a_perception_frame(dev, long_context):
    """Capture a decode step of two branches behind 2 112 tokens, replay it, let the stream perceive a
    17-token frame (behind 2 048+ tokens that takes the split path, whose partials need more room than
    the step's), replay again: every output against the oracle, the pool bit for bit."""
    import torch
    L, QH, KVH, D, BS = ts.L, ts.QH, ts.KVH, ts.D, ts.BS
    s = ts.Session(2)
    rng = np.random.default_rng(9)
    qw, kw = U.normal_bits(rng, (D,), ts.DT), U.normal_bits(rng, (D,), ts.DT)
    s.set_weights(qw, kw)
    st = U.stream_ptr()
    og = orc.layout(L, KVH, QH, D, BS, s.NB, ts.KVDT)
    opool = orc.new_pool(og)
    tables = {}

    def follow(ids):
        for b in ids:
            new = s.cm.h_block_table(b).copy()
            old = tables.get(b)
            if old is not None:
                for lb in np.nonzero((old >= 0) & (new >= 0) & (old != new))[0]:
                    orc.copy_block(og, opool, int(old[lb]), int(new[lb]))
            tables[b] = new

    def perceive(M, check):
        pos0 = s.ks.current_pos()
        assert s.ks.begin_prefill(M, st)
        follow([0])
        pos = (pos0 + np.arange(M)).astype(np.int32)
        for layer in range(L):
            qg, k, v = _inputs(rng, M)
            s.load(qg, k, v)
            s.ks.prefill_layer(layer, s.io(), M, st)
            if check:
                got = s.out(M)
                want = ts.oracle_layer(og, opool, [tables[0]] * M, pos, layer, qg, k, v, qw, kw, s.tab)
                ok, mx, _ = U.rel_abs_ok(U.from_bits(got, ts.DT), want)
                assert ok, ("frame", M, layer, mx)
            else:
                kr = orc.apply_rope(orc.head_norm(k, kw, ts.EPS, ts.DT).reshape(M, KVH, D), pos, s.tab, ts.RD, ts.DT)
                orc.append_batch(og, opool, tables[0], layer, pos0, kr, v, ts.DT)
        s.ks.end_prefill(M)

    for _ in range(33):
        perceive(64, False)
    assert s.ks.open_branches(2) == 2
    ids = [s.ks.branch_id(i) for i in range(2)]
    for b in ids:
        tables[b] = s.cm.h_block_table(b).copy()
    lay = [dict(qg=U.dev_zeros(2 * QH * 2 * D * 2), k=U.dev_zeros(2 * KVH * D * 2), v=U.dev_zeros(2 * KVH * D * 2),
                q=U.dev_zeros(2 * QH * D * 2), out=U.dev_zeros(2 * QH * D * 2)) for _ in range(L)]

    def layers(stream):
        for layer in range(L):
            b = lay[layer]
            s.ks.decode_layer(layer, (U.p(b["qg"]), U.p(b["k"]), U.p(b["v"]), U.p(s.dqw), U.p(s.dkw), U.p(b["q"]), U.p(b["out"])), stream)

    side = torch.cuda.Stream()
    sp = C.c_void_p(side.cuda_stream)
    assert s.ks.capture_decode_step(layers, sp)

    def replay():
        pos = np.array([s.ks.branch_pos(i) for i in range(2)], np.int32)
        ins = [_inputs(rng, 2) for _ in range(L)]
        for layer in range(L):
            for name, a in zip(("qg", "k", "v"), ins[layer]):
                lay[layer][name].copy_(torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)))
        torch.cuda.synchronize()
        assert s.ks.replay_decode_step(sp)
        side.synchronize()
        follow(ids)
        for layer in range(L):
            got = U.host(lay[layer]["out"], np.uint16).reshape(2, QH, D)
            want = ts.oracle_layer(og, opool, [tables[b] for b in ids], pos, layer, *ins[layer], qw, kw, s.tab)
            ok, mx, _ = U.rel_abs_ok(U.from_bits(got, ts.DT), want)
            assert ok, ("replay", layer, mx)

    replay()
    g = cabi.layout(L, KVH, QH, D, BS, s.NB, ts.KVDT)
    assert cabi.lib().drk_prefill_workspace_bytes(C.byref(g), s.ks.current_pos(), 17) > \
        cabi.lib().drk_decode_workspace_bytes(C.byref(g), 3, ts.NPOS)
    perceive(17, True)
    replay()
    perceive(5, True)
    replay()
    assert np.array_equal(s.pool(), opool)
    s.ks.close_branches()


def test_kvstream_checks_the_scorer_and_clears_closed_branches(dev):
    L, QH, KVH, D, BS = ts.L, ts.QH, ts.KVH, ts.D, ts.BS
    assert host.set_attention_geometry(L, QH, KVH, D, ts.KVDT, ts.DT)
    cm, small = host.CacheManager(), host.ImportanceScorer()
    assert cm.init(ts.POOL_BLOCKS * L * 2 * KVH * BS * D * 2, BS, small, 3)
    assert small.init(cm.table_stride())                               # one sequence's blocks, as the reference sizes it
    ks = host.KvStream()
    assert not ks.init(cm, ts.NPOS, small)                             # three table rows do not fit
    del ks, cm
    # a session with a scorer: after the branches close, their rows of the new-score buffer are zero
    rec, pool, s = ts.run_session(2, 2, "eager", seed=126, scorer=True)
    stride = s.cm.table_stride()
    new = ts.d2h(s.sc.d_new_scores(), 3 * stride * 4).view(np.float32).reshape(3, stride)
    assert new[1].sum() > 0 and new[2].sum() > 0 and new[0].sum() == 0
    s.ks.close_branches()
    new = ts.d2h(s.sc.d_new_scores(), 3 * stride * 4).view(np.float32).reshape(3, stride)
    assert not new.any()
