"""GPU: the KV side of the consciousness stream (conscientia/kv_stream.h, after
src/conscientia/stream.cpp:145-401): chunked perception into branch 0, decode branches forked
copy-on-write from it, one fused launch pair per layer, and a captured step replayed.

Checked against the oracle's composition of the reference's separate steps (split, head norm,
RoPE, page write, attention, gate): the pool bit for bit, the attention output within the
attention tolerance; and the replayed graph against the eager session bit for bit."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi, host
from oracle import binding as orc
from tests import util as U

pytestmark = pytest.mark.gpu

L, QH, KVH, D, BS, RD = 2, 32, 8, 128, 16, 32
EPS, THETA = 1e-6, 1.0e7
DT = cabi.BF16
KVDT = cabi.BF16          # storage type of the pages (DT: what the model hands over and gets back)
NPOS = 512
POOL_BLOCKS = 48


@pytest.fixture(params=[cabi.INT8, cabi.FP8_E4M3])
def eight_bit_pages(request):
    global KVDT
    KVDT = request.param
    yield
    KVDT = cabi.BF16


@pytest.fixture
def reference_model_shape():
    """24 Q / 4 KV heads x 256, 256-token blocks, 64 rotary dims, fp16: the reference's own model
    (model.h:39-42, block_pool.h:34-38) instead of the 8B-class shape of the other tests."""
    global QH, KVH, D, BS, RD, DT, KVDT, POOL_BLOCKS
    saved = (QH, KVH, D, BS, RD, DT, KVDT, POOL_BLOCKS)
    QH, KVH, D, BS, RD, DT, KVDT, POOL_BLOCKS = 24, 4, 256, 256, 64, cabi.F16, cabi.F16, 10
    yield
    QH, KVH, D, BS, RD, DT, KVDT, POOL_BLOCKS = saved


def d2h(ptr, nbytes):
    out = np.empty(nbytes, dtype=np.uint8)
    cabi.call("drk_memcpy_d2h", out.ctypes.data_as(C.c_void_p), C.c_void_p(ptr), nbytes, U.stream_ptr())
    return out


class Session:
    """One cache manager + stream driver + the device buffers a model would own."""

    def __init__(self, nbranch, scorer=False):
        import torch
        assert host.set_attention_geometry(L, QH, KVH, D, KVDT, DT)
        assert host.lib().drkh_set_rope(RD, THETA, EPS)
        self.cm = host.CacheManager()
        self.sc = host.ImportanceScorer() if scorer else None
        assert self.cm.init(POOL_BLOCKS * L * 2 * KVH * BS * D * 2, BS, self.sc, 1 + nbranch)
        if scorer:
            assert self.sc.init((1 + nbranch) * self.cm.table_stride(), 0.5)
        self.tab = orc.rope_table(NPOS, RD, THETA)
        self.dtab = torch.from_numpy(self.tab).cuda()
        self.ks = host.KvStream()
        assert self.ks.init(self.cm, NPOS, self.sc, U.p(self.dtab), NPOS)
        T = 64
        self.qw, self.kw = None, None
        self.bufs = dict(qg=U.dev_zeros(T * QH * 2 * D * 2), k=U.dev_zeros(T * KVH * D * 2), v=U.dev_zeros(T * KVH * D * 2),
                         q=U.dev_zeros(T * QH * D * 2), out=U.dev_zeros(T * QH * D * 2))
        self.NB = self.cm.pool_max_blocks()

    def set_weights(self, qw, kw):
        self.dqw, self.dkw = U.dev_bytes(qw), U.dev_bytes(kw)

    def load(self, qg, k, v):
        import torch
        for name, a in (("qg", qg), ("k", k), ("v", v)):
            t = torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1))
            self.bufs[name][:t.numel()].copy_(t)

    def io(self):
        b = self.bufs
        return (U.p(b["qg"]), U.p(b["k"]), U.p(b["v"]), U.p(self.dqw), U.p(self.dkw), U.p(b["q"]), U.p(b["out"]))

    def out(self, T):
        U.sync()
        return U.host(self.bufs["out"], np.uint16)[:T * QH * D].reshape(T, QH, D).copy()

    def pool(self):
        return d2h(self.cm.pool_ptr(), self.cm.pool_total_bytes())


def oracle_layer(og, opool, table_rows, pos, layer, qg, k, v, qw, kw, tab, prefill_start=None):
    """The reference's sequence for T tokens; table_rows[t] is the table token t writes through."""
    T = qg.shape[0]
    q0, gate = orc.split_q_gate(qg, T, QH, D)
    qr = orc.apply_rope(orc.head_norm(q0, qw, EPS, DT).reshape(T, QH, D), pos, tab, RD, DT)
    kr = orc.apply_rope(orc.head_norm(k, kw, EPS, DT).reshape(T, KVH, D), pos, tab, RD, DT)
    for t in range(T):
        orc.append_token(og, opool, table_rows[t], layer, int(pos[t]), kr[t], v[t], DT)
    want = np.empty((T, QH, D), np.float64)
    for t in range(T):
        want[t] = orc.decode_f64(og, qr[t], opool, table_rows[t], layer, int(pos[t]) + 1, 1 / np.sqrt(D), DT)
    g = U.from_bits(gate, DT).astype(np.float64)
    return want / (1.0 + np.exp(-g))


def run_session(nbranch, steps, mode, seed=120, scorer=False, shared_policy=None):
    """mode 'eager' or 'graph'.  Returns (prefill outs, per-step decode outs, final pool, session)."""
    s = Session(nbranch, scorer)
    if shared_policy:
        s.ks.set_shared_prefix_policy(*shared_policy)
    rng = np.random.default_rng(seed)
    qw, kw = U.normal_bits(rng, (D,), DT), U.normal_bits(rng, (D,), DT)
    s.set_weights(qw, kw)
    st = U.stream_ptr()
    og = orc.layout(L, KVH, QH, D, BS, s.NB, KVDT)
    opool = orc.new_pool(og)
    record = dict(prefill=[], decode=[], inputs=[])
    # ---- perception: 100 tokens in chunks of 64 + 36 ----
    for M in (64, 36):
        pos0 = s.ks.current_pos()
        assert s.ks.begin_prefill(M, st)
        table0 = s.cm.h_block_table(0).copy()
        for layer in range(L):
            qg, k, v = (U.normal_bits(rng, sh, DT, m) for sh, m in (((M, QH, 2 * D), 1.0), ((M, KVH, D), 0.7), ((M, KVH, D), 0.5)))
            s.load(qg, k, v)
            s.ks.prefill_layer(layer, s.io(), M, st)
            got = s.out(M)
            pos = (pos0 + np.arange(M)).astype(np.int32)
            want = oracle_layer(og, opool, [table0] * M, pos, layer, qg, k, v, qw, kw, s.tab)
            ok, mx, _ = U.rel_abs_ok(U.from_bits(got, DT), want)
            assert ok, (M, layer, mx)
            record["prefill"].append(got)
        s.ks.end_prefill(M, st)
    assert s.ks.current_pos() == 100 and s.cm.seq_len(0) == 100
    assert np.array_equal(s.pool(), opool)
    # ---- decode branches ----
    assert s.ks.open_branches(nbranch) == nbranch
    assert s.ks.shared_tokens() == 100 // BS * BS                      # the whole blocks of the 100-token prefix
    ids = [s.ks.branch_id(i) for i in range(nbranch)]
    assert ids == list(range(1, nbranch + 1)) and all(s.ks.branch_pos(i) == 100 for i in range(nbranch))
    step_inputs = [[tuple(U.normal_bits(rng, sh, DT, m) for sh, m in (((nbranch, QH, 2 * D), 1.0), ((nbranch, KVH, D), 0.7),
                                                                       ((nbranch, KVH, D), 0.5))) for _ in range(L)]
                   for _ in range(steps)]
    if mode == "graph":
        # the model's buffers are fixed; one set per layer so that a replay reads this step's inputs
        import torch
        lay_bufs = [dict(qg=U.dev_zeros(nbranch * QH * 2 * D * 2), k=U.dev_zeros(nbranch * KVH * D * 2), v=U.dev_zeros(nbranch * KVH * D * 2),
                         q=U.dev_zeros(nbranch * QH * D * 2), out=U.dev_zeros(nbranch * QH * D * 2)) for _ in range(L)]

        def layers(stream):
            for layer in range(L):
                b = lay_bufs[layer]
                s.ks.decode_layer(layer, (U.p(b["qg"]), U.p(b["k"]), U.p(b["v"]), U.p(s.dqw), U.p(s.dkw), U.p(b["q"]), U.p(b["out"])), stream)

        side = torch.cuda.Stream()
        sp = C.c_void_p(side.cuda_stream)
        assert s.ks.capture_decode_step(layers, sp)
    for step in range(steps):
        if mode == "eager":
            assert s.ks.begin_decode_step(st)
            tables = [s.cm.h_block_table(b).copy() for b in ids]
            outs = []
            for layer in range(L):
                qg, k, v = step_inputs[step][layer]
                s.load(qg, k, v)
                s.ks.decode_layer(layer, s.io(), st)
                got = s.out(nbranch)
                pos = np.full(nbranch, 100 + step, np.int32)
                if step == 0 and layer == 0:                         # first write into the shared tail block: copy-on-write
                    tail = 100 // BS
                    for b in range(nbranch):
                        for src_blk, dst_blk in [(s.cm.h_block_table(0)[tail], tables[b][tail])]:
                            assert src_blk != dst_blk
                            orc.copy_block(og, opool, int(src_blk), int(dst_blk))
                want = oracle_layer(og, opool, tables, pos, layer, qg, k, v, qw, kw, s.tab)
                ok, mx, _ = U.rel_abs_ok(U.from_bits(got, DT), want)
                assert ok, (step, layer, mx)
                outs.append(got)
            s.ks.end_decode_step(st)
            record["decode"].append(outs)
        else:
            import torch
            for layer in range(L):
                qg, k, v = step_inputs[step][layer]
                for name, a in (("qg", qg), ("k", k), ("v", v)):
                    lay_bufs[layer][name].copy_(torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)))
            torch.cuda.synchronize()
            assert s.ks.replay_decode_step(sp)
            side.synchronize()
            record["decode"].append([U.host(lay_bufs[layer]["out"], np.uint16).reshape(nbranch, QH, D).copy() for layer in range(L)])
        assert [s.ks.branch_pos(i) for i in range(nbranch)] == [101 + step] * nbranch
        assert [s.cm.seq_len(b) for b in ids] == [101 + step] * nbranch
    final_pool = s.pool()
    if mode == "eager":
        assert np.array_equal(final_pool, opool)                      # every byte, all branches, all layers
    return record, final_pool, s


def test_stream_session_matches_the_oracle_and_its_graph_replay(dev):
    rec_e, pool_e, s_e = run_session(3, 5, "eager")
    # the prefix blocks are shared: 6 whole blocks of branch 0 are referenced by all four tables
    shared = s_e.cm.h_block_table(0)[:6]
    for b in (1, 2, 3):
        assert np.array_equal(s_e.cm.h_block_table(b)[:6], shared) and s_e.cm.h_block_table(b)[6] != s_e.cm.h_block_table(0)[6]
    s_e.ks.close_branches()
    assert s_e.cm.gpu_blocks_used() == 7                               # only the stream's own blocks stay
    del s_e
    rec_g, pool_g, s_g = run_session(3, 5, "graph")
    for step in range(5):
        for layer in range(L):
            assert np.array_equal(rec_g["decode"][step][layer], rec_e["decode"][step][layer]), (step, layer)
    assert np.array_equal(pool_g, pool_e)
    s_g.ks.close_branches()


def test_stream_session_at_the_reference_models_shape(dev, reference_model_shape):
    """The whole KV path at 24 Q / 4 KV heads x 256 with 256-token blocks: fused norm + RoPE + page write
    at head_dim 256, MFMA prefill at head_dim 256 with 21 tokens x 6 heads per workgroup, decode
    with 6 heads per kv head, copy-on-write of a 256-token block, and the captured step."""
    rec_e, pool_e, s_e = run_session(2, 3, "eager", seed=124)
    s_e.ks.close_branches()
    assert s_e.cm.gpu_blocks_used() == 1
    del s_e
    rec_g, pool_g, s_g = run_session(2, 3, "graph", seed=124)
    for step in range(3):
        for layer in range(L):
            assert np.array_equal(rec_g["decode"][step][layer], rec_e["decode"][step][layer]), (step, layer)
    assert np.array_equal(pool_g, pool_e)
    s_g.ks.close_branches()


def test_stream_session_with_8bit_pages(dev, eight_bit_pages):
    """int8 (+ fp16 scales) and fp8 pages under the same session: K and V are quantised by the fused
    norm + RoPE + page write (codes and scales bit for bit the oracle's), prefill and decode dequantise
    inside attention, the copy-on-write copies carry the scales along, and the captured step replays."""
    rec_e, pool_e, s_e = run_session(3, 3, "eager", seed=125)
    s_e.ks.close_branches()
    del s_e
    rec_g, pool_g, s_g = run_session(3, 3, "graph", seed=125)
    for step in range(3):
        for layer in range(L):
            assert np.array_equal(rec_g["decode"][step][layer], rec_e["decode"][step][layer]), (step, layer)
    assert np.array_equal(pool_g, pool_e)
    s_g.ks.close_branches()


def test_stream_session_with_the_prefix_streamed_once(dev):
    """Same session, but the decode attention reads the branches' common prefix once for all of
    them (here from 64 shared tokens on; the default asks for 4096): still the oracle's results
    within the attention tolerance (checked inside run_session), the same pool bytes as the
    per-branch path, and the captured step replays to the eager bits."""
    rec_e, pool_e, s_e = run_session(4, 4, "eager", seed=122, shared_policy=(2, 64))
    s_e.ks.close_branches()
    del s_e
    rec_g, pool_g, s_g = run_session(4, 4, "graph", seed=122, shared_policy=(2, 64))
    for step in range(4):
        for layer in range(L):
            assert np.array_equal(rec_g["decode"][step][layer], rec_e["decode"][step][layer]), (step, layer)
    assert np.array_equal(pool_g, pool_e)
    s_g.ks.close_branches()
    del s_g
    rec_p, pool_p, s_p = run_session(4, 4, "eager", seed=122)           # per-branch path, same inputs
    assert np.array_equal(pool_p, pool_e)
    diff = max(np.abs(U.from_bits(rec_p["decode"][st][l], DT).astype(np.float64) - U.from_bits(rec_e["decode"][st][l], DT)).max()
               for st in range(4) for l in range(L))
    assert 0 < diff < 2e-2                                             # another summation order, not another result
    s_p.ks.close_branches()


def test_stream_session_feeds_the_scorer(dev):
    """With a scorer attached every decode step leaves the attention mass of the step in the
    scores (score = score * decay + mass, summed over the layers): a branch's blocks sum to
    L * QH per step."""
    rec, pool, s = run_session(2, 3, "eager", seed=121, scorer=True)
    s.sc.sync_to_host()
    stride = s.cm.table_stride()
    for b in (1, 2):
        tot = sum(s.sc.score(b * stride + lb) for lb in range(8))
        want = L * QH * (1 + 0.5 + 0.25)                               # three steps, decay 0.5
        assert abs(tot - want) < 0.05 * want, (b, tot, want)
    # branch 0 took no decode step: its row holds what the two perception frames (64 and 36 tokens) left, folded
    # once per frame and decayed by every fold since
    tot0 = sum(s.sc.score(lb) for lb in range(8))
    want0 = L * QH * (64 * 0.5 + 36) * 0.5 ** 3
    assert abs(tot0 - want0) < 0.02 * want0, (tot0, want0)
    s.ks.close_branches()


def test_perception_frames_feed_the_scorer(dev):
    """With a scorer attached every perception frame leaves, block by block, the attention mass its rows gave to the
    context (summed over the layers) in the stream's row of the scores -- against the fp64 oracle, frame after frame
    (score = score * decay + mass)."""
    s = Session(1, scorer=True)
    rng = np.random.default_rng(77)
    qw, kw = U.normal_bits(rng, (D,), DT), U.normal_bits(rng, (D,), DT)
    s.set_weights(qw, kw)
    st = U.stream_ptr()
    og = orc.layout(L, KVH, QH, D, BS, s.NB, KVDT)
    opool = orc.new_pool(og)
    stride = s.cm.table_stride()
    want = np.zeros(stride)
    for M in (64, 5, 36):
        pos0 = s.ks.current_pos()
        assert s.ks.begin_prefill(M, st)
        table0 = s.cm.h_block_table(0).copy()
        pos = (pos0 + np.arange(M)).astype(np.int32)
        frame = np.zeros(stride)
        for layer in range(L):
            qg, k, v = (U.normal_bits(rng, sh, DT, m) for sh, m in (((M, QH, 2 * D), 1.0), ((M, KVH, D), 0.7), ((M, KVH, D), 0.5)))
            s.load(qg, k, v)
            s.ks.prefill_layer(layer, s.io(), M, st)
            q0, _ = orc.split_q_gate(qg, M, QH, D)
            qr = orc.apply_rope(orc.head_norm(q0, qw, EPS, DT).reshape(M, QH, D), pos, s.tab, RD, DT)
            kr = orc.apply_rope(orc.head_norm(k, kw, EPS, DT).reshape(M, KVH, D), pos, s.tab, RD, DT)
            for tkn in range(M):
                orc.append_token(og, opool, table0, layer, int(pos[tkn]), kr[tkn], v[tkn], DT)
            tables = np.ascontiguousarray(np.broadcast_to(table0, (M, stride)))
            frame += orc.block_attention_mass(og, qr, opool, tables, (pos + 1).astype(np.int32), layer, 1 / np.sqrt(D), DT, stride).sum(axis=0)
        s.ks.end_prefill(M, st)
        want = 0.5 * want + frame
        U.sync()
        s.sc.sync_to_host()
        got = np.array([s.sc.score(lb) for lb in range(stride)])
        assert np.all(np.abs(got - want) <= 4e-3 * M + 3e-3 * np.abs(want)), (M, float(np.abs(got - want).max()))
        assert abs(frame.sum() - M * QH * L) < 1e-6 * M * QH * L
    assert np.array_equal(s.pool(), opool)


@pytest.mark.parametrize("mode", ["eager", "graph"])
def test_scorer_with_branches_open_across_perception_frames(dev, mode):
    """A frame folds its masses into the stream's own row only: the rows of open branches still hold their last
    step's masses, which that step folded in already -- a frame must neither count them again nor age them.
    Frames and decode steps run on two streams (the folds order themselves); in graph mode the step's fold is
    part of the replayed graph.  Per row, mass sums are known in closed form: a decode step gives every branch
    L * QH, a frame of M tokens gives the stream M * L * QH; every fold of a row halves what it held."""
    import torch
    nbranch = 2
    s = Session(nbranch, scorer=True)
    rng = np.random.default_rng(133)
    s.set_weights(U.normal_bits(rng, (D,), DT), U.normal_bits(rng, (D,), DT))
    frames, steps = torch.cuda.Stream(), torch.cuda.Stream()
    fp, sp = C.c_void_p(frames.cuda_stream), C.c_void_p(steps.cuda_stream)
    stride = s.cm.table_stride()
    LQ = L * QH

    def frame(M):
        assert s.ks.begin_prefill(M, fp)
        for layer in range(L):
            qg, k, v = (U.normal_bits(rng, sh, DT, m) for sh, m in (((M, QH, 2 * D), 1.0), ((M, KVH, D), 0.7), ((M, KVH, D), 0.5)))
            frames.synchronize()                           # the previous layer has read the buffers
            s.load(qg, k, v)
            torch.cuda.current_stream().synchronize()      # the copies ran on torch's stream; the step's stream is not waited for
            s.ks.prefill_layer(layer, s.io(), M, fp)
        s.ks.end_prefill(M)                                # no stream given: the fold follows the layers' stream

    lay_bufs = [dict(qg=U.dev_zeros(nbranch * QH * 2 * D * 2), k=U.dev_zeros(nbranch * KVH * D * 2), v=U.dev_zeros(nbranch * KVH * D * 2),
                     q=U.dev_zeros(nbranch * QH * D * 2), out=U.dev_zeros(nbranch * QH * D * 2)) for _ in range(L)]

    def layers(stream):
        for layer in range(L):
            b = lay_bufs[layer]
            s.ks.decode_layer(layer, (U.p(b["qg"]), U.p(b["k"]), U.p(b["v"]), U.p(s.dqw), U.p(s.dkw), U.p(b["q"]), U.p(b["out"])), stream)

    def step():
        steps.synchronize()                                # the previous step has read its inputs
        for layer in range(L):
            for name, sh, m in (("qg", (nbranch, QH, 2 * D), 1.0), ("k", (nbranch, KVH, D), 0.7), ("v", (nbranch, KVH, D), 0.5)):
                a = U.normal_bits(rng, sh, DT, m)
                lay_bufs[layer][name].copy_(torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)))
        torch.cuda.current_stream().synchronize()          # the frame's last layers and its fold may still be running
        if mode == "graph":
            assert s.ks.replay_decode_step(sp)
        else:
            assert s.ks.begin_decode_step(sp)
            layers(sp)
            s.ks.end_decode_step(sp)

    frame(40)
    assert s.ks.open_branches(nbranch) == nbranch
    if mode == "graph":
        assert s.ks.capture_decode_step(layers, sp)
    want0, wantb = 40.0 * LQ, 0.0
    for M in (20, 10, 33):
        step()                                             # folds every row
        want0, wantb = 0.5 * want0, 0.5 * wantb + LQ
        frame(M)                                           # folds the stream's row; not ordered against the step by the caller
        want0 = 0.5 * want0 + M * LQ
    step()
    want0, wantb = 0.5 * want0, 0.5 * wantb + LQ
    torch.cuda.synchronize()
    s.sc.sync_to_host()
    got0 = sum(s.sc.score(lb) for lb in range(stride))
    assert abs(got0 - want0) < 0.02 * want0, (got0, want0)
    for b in (1, 2):
        got = sum(s.sc.score(b * stride + lb) for lb in range(stride))
        assert abs(got - wantb) < 0.02 * wantb, (b, got, wantb)
    s.ks.close_branches()


def test_time_division_perception_between_decode_steps_and_a_changing_branch_count(dev):
    """The scheduler's regime (scheduler.h:8-24, 53-56): perception goes on while branches think, and
    the number of branches follows the wakefulness state.  The stream writes into a block it still
    shares with its branches (copy-on-write on the stream's side), two more branches fork later at
    another position, the youngest are closed again.  Every step against the oracle; the pool bit
    for bit at the end."""
    s = Session(4)
    rng = np.random.default_rng(123)
    qw, kw = U.normal_bits(rng, (D,), DT), U.normal_bits(rng, (D,), DT)
    s.set_weights(qw, kw)
    st = U.stream_ptr()
    og = orc.layout(L, KVH, QH, D, BS, s.NB, KVDT)
    opool = orc.new_pool(og)
    tables = {0: s.cm.h_block_table(0).copy()}

    def follow_tables(ids):
        """copy-on-write in the oracle: a table cell that moved to another block took the old block's bytes along"""
        for b in ids:
            new = s.cm.h_block_table(b).copy()
            old = tables.get(b)
            if old is not None:
                for lb in np.nonzero((old >= 0) & (new >= 0) & (old != new))[0]:
                    orc.copy_block(og, opool, int(old[lb]), int(new[lb]))
            tables[b] = new

    def perceive(M):
        pos0 = s.ks.current_pos()
        assert s.ks.begin_prefill(M, st)
        follow_tables([0])
        for layer in range(L):
            qg, k, v = (U.normal_bits(rng, sh, DT, m) for sh, m in (((M, QH, 2 * D), 1.0), ((M, KVH, D), 0.7), ((M, KVH, D), 0.5)))
            s.load(qg, k, v)
            s.ks.prefill_layer(layer, s.io(), M, st)
            got = s.out(M)
            pos = (pos0 + np.arange(M)).astype(np.int32)
            want = oracle_layer(og, opool, [tables[0]] * M, pos, layer, qg, k, v, qw, kw, s.tab)
            ok, mx, _ = U.rel_abs_ok(U.from_bits(got, DT), want)
            assert ok, ("prefill", M, layer, mx)
        s.ks.end_prefill(M)

    def think():
        n = s.ks.num_branches()
        ids = [s.ks.branch_id(i) for i in range(n)]
        pos = np.array([s.ks.branch_pos(i) for i in range(n)], np.int32)
        assert s.ks.begin_decode_step(st)
        follow_tables(ids)
        for layer in range(L):
            qg, k, v = (U.normal_bits(rng, sh, DT, m) for sh, m in (((n, QH, 2 * D), 1.0), ((n, KVH, D), 0.7), ((n, KVH, D), 0.5)))
            s.load(qg, k, v)
            s.ks.decode_layer(layer, s.io(), st)
            got = s.out(n)
            want = oracle_layer(og, opool, [tables[b] for b in ids], pos, layer, qg, k, v, qw, kw, s.tab)
            ok, mx, _ = U.rel_abs_ok(U.from_bits(got, DT), want)
            assert ok, ("decode", n, layer, mx)
        s.ks.end_decode_step(st)
        assert [s.ks.branch_pos(i) for i in range(n)] == (pos + 1).tolist()

    def fork_tables():
        for i in range(s.ks.num_branches()):
            b = s.ks.branch_id(i)
            if b not in tables:
                tables[b] = s.cm.h_block_table(b).copy()

    perceive(64)
    perceive(36)
    assert s.ks.set_branch_count(2) == 2                      # DAYDREAM: two branches at 100
    fork_tables()
    shared_tail = int(tables[0][6])
    perceive(12)                                              # ACTIVE again: the stream writes tokens 100..111 into block 6,
    assert int(tables[0][6]) != shared_tail                   # which its branches still share: the stream takes a copy
    assert [int(tables[b][6]) for b in (1, 2)] == [shared_tail] * 2
    think(); think()
    perceive(16)
    assert s.ks.current_pos() == 128
    think()
    assert s.ks.set_branch_count(4) == 4                      # DREAMING: two more, forked at 128
    fork_tables()
    assert [s.ks.branch_pos(i) for i in range(4)] == [103, 103, 128, 128]
    assert s.ks.shared_tokens() == 96
    think(); think()
    assert s.ks.set_branch_count(1) == 1 and s.ks.branch_id(0) == 1
    for b in (2, 3, 4):
        tables.pop(b)
    think()
    perceive(16)
    think()
    assert np.array_equal(s.pool(), opool)
    s.ks.close_branches()
    assert s.cm.gpu_blocks_used() == 9                        # 144 tokens of the stream


def test_perception_frames_behind_a_long_context(dev):
    """Frames of a few tokens after 2 112 tokens of context: prefill_layer then runs with the context
    split over the chip (rows = the frame's tokens) instead of the chunk kernel -- same pool bits, same
    outputs within the attention tolerance."""
    global NPOS, POOL_BLOCKS
    saved = (NPOS, POOL_BLOCKS)
    NPOS, POOL_BLOCKS = 2304, 160
    try:
        s = Session(1)
        rng = np.random.default_rng(7)
        qw, kw = U.normal_bits(rng, (D,), DT), U.normal_bits(rng, (D,), DT)
        s.set_weights(qw, kw)
        st = U.stream_ptr()
        og = orc.layout(L, KVH, QH, D, BS, s.NB, KVDT)
        opool = orc.new_pool(og)
        g = cabi.layout(L, KVH, QH, D, BS, s.NB, KVDT)
        for M, check in [(64, False)] * 33 + [(5, True), (17, True), (1, True)]:
            pos0 = s.ks.current_pos()
            # from 2 048 tokens on, frames take the split path: it is the one that asks for a workspace
            assert (cabi.lib().drk_prefill_workspace_bytes(C.byref(g), pos0, M) > 0) == (pos0 >= 2048)
            assert s.ks.begin_prefill(M, st)
            table0 = s.cm.h_block_table(0).copy()
            pos = (pos0 + np.arange(M)).astype(np.int32)
            for layer in range(L):
                qg, k, v = (U.normal_bits(rng, sh, DT, m) for sh, m in (((M, QH, 2 * D), 1.0), ((M, KVH, D), 0.7), ((M, KVH, D), 0.5)))
                s.load(qg, k, v)
                s.ks.prefill_layer(layer, s.io(), M, st)
                if check:
                    got = s.out(M)
                    want = oracle_layer(og, opool, [table0] * M, pos, layer, qg, k, v, qw, kw, s.tab)
                    ok, mx, _ = U.rel_abs_ok(U.from_bits(got, DT), want)
                    assert ok, (M, layer, mx)
                else:                                                  # the context itself: only the pages are mirrored
                    kr = orc.apply_rope(orc.head_norm(k, kw, EPS, DT).reshape(M, KVH, D), pos, s.tab, RD, DT)
                    orc.append_batch(og, opool, table0, layer, pos0, kr, v, DT)
            s.ks.end_prefill(M)
        assert s.ks.current_pos() == 33 * 64 + 23
        assert np.array_equal(s.pool(), opool)
    finally:
        NPOS, POOL_BLOCKS = saved
