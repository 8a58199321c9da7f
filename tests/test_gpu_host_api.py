"""GPU: the C++ host classes (CacheManager / BlockPool / ImportanceScorer) and the
reference-named launchers of machina/paged_attention.h, driven in the caller's
order (src/conscientia/stream.cpp:151-156, 297-305, 319-334: ensure blocks ->
sync table -> write K/V -> attend with seq_len = pos + 1)."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi, host
from oracle import binding as orc
from tests import util as U

pytestmark = pytest.mark.gpu


def d2h(ptr, nbytes):
    out = np.empty(nbytes, dtype=np.uint8)
    cabi.call("drk_memcpy_d2h", out.ctypes.data_as(C.c_void_p), C.c_void_p(ptr), nbytes, U.stream_ptr())
    return out


def test_config1_through_the_reference_interface(dev):
    L, KVH, QH, D, bs, T = 1, 4, 16, 128, 16, 512
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.F16)
    cm = host.CacheManager()
    block_bytes = L * 2 * KVH * bs * D * 2
    assert cm.init(256 * block_bytes, bs)
    NB = cm.pool_max_blocks()
    assert NB == 256 and cm.pool_total_bytes() == 256 * block_bytes and cm.free_blocks() == 256
    assert not d2h(cm.pool_ptr(), 4096).any()                     # zero-filled (block_pool.cpp:49)
    rng = np.random.default_rng(1)
    # a shuffled table: allocate all, free in random order, then let the sequence allocate
    ids = [cm.pool_alloc_block() for _ in range(NB)]
    for i in rng.permutation(NB):
        cm.pool_free_block(int(ids[i]))
    assert cm.ensure_blocks_for_range(0, 0, T)
    table = cm.h_block_table(0)
    assert sorted(table[:T // bs].tolist()) != table[:T // bs].tolist() and (table[T // bs:] == -1).all()
    cm.sync_block_table(U.stream_ptr())
    k, v, q = (U.normal_bits(rng, s, cabi.F16) for s in ((T, KVH, D), (T, KVH, D), (QH, D)))
    dk, dv, dq = U.dev_bytes(k), U.dev_bytes(v), U.dev_bytes(q)
    L_ = host.lib()
    L_.drkh_paged_kv_cache_write_batch(U.p(dk), U.p(dv), cm.pool_ptr(), cm.d_block_table(0), 0, 0, T, NB, bs,
                                       U.stream_ptr())
    cm.set_seq_len(0, T)
    assert cm.num_logical_blocks(0) == T // bs
    out = U.dev_zeros(QH * D * 2)
    scale = 1 / np.sqrt(D)
    L_.drkh_paged_gqa_decode_attention(U.p(dq), cm.pool_ptr(), cm.d_block_table(0), U.p(out), 0, T, NB, bs,
                                       float(scale), U.stream_ptr())
    flat = U.dev_zeros(2 * T * KVH * D * 2)
    L_.drkh_invoke_extract_kv_from_pages(U.p(flat), cm.pool_ptr(), cm.d_block_table(0), 0, T, 1, KVH, D, bs, NB,
                                         U.stream_ptr())
    U.sync()
    og = orc.layout(L, KVH, QH, D, bs, NB, orc.F16)
    opool = orc.new_pool(og)
    orc.append_batch(og, opool, table, 0, 0, k, v, orc.F16)
    assert np.array_equal(d2h(cm.pool_ptr(), cm.pool_total_bytes()), opool)
    got_flat = U.host(flat, np.uint16, (1, 2, T, KVH, D))
    assert np.array_equal(got_flat[0, 0], k) and np.array_equal(got_flat[0, 1], v)
    want = orc.decode_f64(og, q, opool, table, 0, T, scale, orc.F16)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(U.host(out, np.uint16, (QH, D)), cabi.F16), want)
    assert ok, ma


def test_decode_loop_protocol_with_eviction(dev):
    """One sequence decoding token by token in a pool that is too small: old pages
    are evicted (FIFO), the table keeps -1 holes, attention skips them."""
    L, KVH, QH, D, bs = 2, 4, 16, 128, 16
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    cm = host.CacheManager()
    NBw = 6
    assert cm.init(NBw * L * 2 * KVH * bs * D * 2, bs)
    NB = cm.pool_max_blocks()
    og = orc.layout(L, KVH, QH, D, bs, NB, orc.BF16)
    opool = orc.new_pool(og)
    oc = orc.CacheManager(NB, bs)
    rng = np.random.default_rng(12)
    steps = 8 * bs + 3
    lib = host.lib()
    dpos = U.dev_i32(np.zeros(1, dtype=np.int32))
    scale = 1 / np.sqrt(D)
    for pos in range(steps):
        assert cm.ensure_blocks_for(0, pos) and oc.ensure(0, pos)
        cm.sync_block_table(U.stream_ptr())
        dpos.fill_(pos)
        k, v = U.normal_bits(rng, (L, KVH, D), cabi.BF16), U.normal_bits(rng, (L, KVH, D), cabi.BF16)
        dk, dv = U.dev_bytes(k), U.dev_bytes(v)
        for l in range(L):
            lib.drkh_paged_kv_cache_write(C.c_void_p(dk.data_ptr() + l * KVH * D * 2),
                                          C.c_void_p(dv.data_ptr() + l * KVH * D * 2), cm.pool_ptr(),
                                          cm.d_block_table(0), l, U.p(dpos), NB, bs, U.stream_ptr())
            orc.append_token(og, opool, oc.table(0), l, pos, k[l], v[l], orc.BF16)
        cm.set_seq_len(0, pos + 1)
        if pos % 23 == 0 or pos == steps - 1:
            q = U.normal_bits(rng, (QH, D), cabi.BF16)
            dq, out = U.dev_bytes(q), U.dev_zeros(QH * D * 2)
            lib.drkh_paged_gqa_decode_attention(U.p(dq), cm.pool_ptr(), cm.d_block_table(0), U.p(out), L - 1,
                                                pos + 1, NB, bs, float(scale), U.stream_ptr())
            U.sync()
            want = orc.decode_f64(og, q, opool, oc.table(0), L - 1, pos + 1, scale, orc.BF16)
            ok, ma, _ = U.rel_abs_ok(U.from_bits(U.host(out, np.uint16, (QH, D)), cabi.BF16), want)
            assert ok, (pos, ma)
        U.sync()
    assert np.array_equal(cm.h_block_table(0), oc.table(0))
    assert (cm.h_block_table(0)[:3] == -1).all() and cm.gpu_blocks_used() == NB
    assert np.array_equal(d2h(cm.pool_ptr(), cm.pool_total_bytes()), opool)
    dtab = d2h(cm.d_block_table(0), cm.table_stride() * 4).view(np.int32)
    assert np.array_equal(dtab, cm.h_block_table(0))              # device mirror follows the host table


def test_shared_prefix_branches_copy_on_write(dev):
    """BASELINE config 3 in small: a persistent prefix shared by several branches
    that fork at block boundaries and inside a block, append privately, get evicted
    and released; every branch's gathered K/V and attention output must equal a
    model in which the branch owns a private copy."""
    L, KVH, QH, D, bs, branches = 2, 8, 32, 128, 16, 6
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    cm = host.CacheManager()
    assert cm.init(64 * L * 2 * KVH * bs * D * 2, bs, None, branches)
    NB = cm.pool_max_blocks()
    stride = cm.table_stride()
    og = orc.layout(L, KVH, QH, D, bs, NB, orc.BF16)
    rng = np.random.default_rng(33)
    lib = host.lib()
    model = {0: []}                                        # branch -> list of (k, v) [L, KVH, D]

    def append(bs_list):
        """one token for each listed branch, one launch per layer"""
        for b in bs_list:
            assert cm.ensure_blocks_for(b, len(model[b]))
        cm.sync_block_table(U.stream_ptr())               # issues the COW copies, uploads tables
        B = len(bs_list)
        k, v = U.normal_bits(rng, (L, B, KVH, D), cabi.BF16), U.normal_bits(rng, (L, B, KVH, D), cabi.BF16)
        pos = np.array([len(model[b]) for b in bs_list], dtype=np.int32)
        tabs = np.stack([cm.h_block_table(b) for b in bs_list])
        dk, dv, dpos, dtabs = U.dev_bytes(k), U.dev_bytes(v), U.dev_i32(pos), U.dev_i32(tabs)
        for l in range(L):
            lib.drkh_paged_kv_cache_write_branches(C.c_void_p(dk.data_ptr() + l * B * KVH * D * 2),
                                                   C.c_void_p(dv.data_ptr() + l * B * KVH * D * 2), cm.pool_ptr(),
                                                   U.p(dtabs), stride, U.p(dpos), B, l, NB, bs, U.stream_ptr())
        U.sync()
        for i, b in enumerate(bs_list):
            model[b].append((k[:, i].copy(), v[:, i].copy()))
            cm.set_seq_len(b, len(model[b]))

    for _ in range(5 * bs + 7):                            # the persistent prefix on branch 0
        append([0])
    kids = []
    for fork_pos in (5 * bs, 3 * bs, 5 * bs + 7, 2 * bs + 1):     # block boundaries and mid-block
        nb = cm.fork_branch(0, fork_pos)
        assert nb > 0
        model[nb] = list(model[0][:fork_pos])
        kids.append(nb)
    assert cm.pool_refcount(int(cm.h_block_table(0)[0])) == 5
    used_before = cm.gpu_blocks_used()
    for _ in range(2 * bs + 3):
        append(kids + [0])
    assert cm.gpu_blocks_used() > used_before
    cm.release_branch(kids[1])
    del model[kids[1]]
    assert cm.evict_blocks(3) == 3                          # private pages of someone, oldest first
    for _ in range(5):
        append([kids[0], kids[2]])

    pool_host = d2h(cm.pool_ptr(), cm.pool_total_bytes())
    scale = 1 / np.sqrt(D)
    alive = sorted(model)
    for b in alive:
        tab, n = cm.h_block_table(b), len(model[b])
        flat, _ = orc.extract(og, pool_host, tab, 0, n, L)
        for t in range(n):
            if tab[t // bs] < 0:
                assert not flat[:, :, t].any()
            else:
                k, v = model[b][t]
                assert np.array_equal(flat[:, 0, t], k) and np.array_equal(flat[:, 1, t], v), (b, t)
    # all branches attend in one launch; the oracle runs on the private-copy model
    B = len(alive)
    q = U.normal_bits(rng, (B, QH, D), cabi.BF16)
    lens = np.array([len(model[b]) for b in alive], dtype=np.int32)
    tabs = np.stack([cm.h_block_table(b) for b in alive])
    dq, dl, dt, out = U.dev_bytes(q), U.dev_i32(lens), U.dev_i32(tabs), U.dev_zeros(B * QH * D * 2)
    lib.drkh_paged_gqa_decode_attention_branches(U.p(dq), cm.pool_ptr(), U.p(dt), stride, U.p(dl), B,
                                                 int(lens.max()), U.p(out), 1, NB, bs, float(scale), U.stream_ptr())
    U.sync()
    got = U.from_bits(U.host(out, np.uint16, (B, QH, D)), cabi.BF16)
    for i, b in enumerate(alive):
        n = len(model[b])
        pg = orc.layout(L, KVH, QH, D, bs, (n + bs - 1) // bs, orc.BF16)
        ppool = orc.new_pool(pg)
        ptab = np.arange((n + bs - 1) // bs, dtype=np.int32)
        ptab[cm.h_block_table(b)[:len(ptab)] < 0] = -1     # evicted pages are holes in the model too
        kk = np.stack([m[0][1] for m in model[b]])
        vv = np.stack([m[1][1] for m in model[b]])
        orc.append_batch(pg, ppool, ptab, 1, 0, kk, vv, orc.BF16)
        want = orc.decode_f64(pg, q[i], ppool, ptab, 1, n, scale, orc.BF16)
        ok, ma, _ = U.rel_abs_ok(got[i], want)
        assert ok, (b, ma)


def test_fork_tree_through_the_host_classes(dev):
    """Branches that fork from one another at different block boundaries (and once inside a block): the groups
    CacheManager::common_prefix_groups finds, handed to the grouped decode call, against the fp64 oracle on a
    model in which every branch owns a private copy of its context."""
    L, KVH, QH, D, bs = 2, 8, 32, 128, 16
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    lib = host.lib()
    assert lib.drkh_paged_gqa_decode_grouped_supported(bs)
    cm = host.CacheManager()
    assert cm.init(160 * L * 2 * KVH * bs * D * 2, bs, None, 8)
    NB, stride = cm.pool_max_blocks(), cm.table_stride()
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    rng = np.random.default_rng(71)
    model = {0: (np.zeros((L, 0, KVH, D), np.uint16), np.zeros((L, 0, KVH, D), np.uint16))}

    def bulk(b, m):
        p0 = cm.seq_len(b)
        assert model[b][0].shape[1] == p0 and cm.ensure_blocks_for_range(b, p0, m)
        cm.sync_block_table(U.stream_ptr())               # copy-on-write copies, table upload
        k, v = U.normal_bits(rng, (L, m, KVH, D), cabi.BF16), U.normal_bits(rng, (L, m, KVH, D), cabi.BF16)
        dk, dv = U.dev_bytes(k), U.dev_bytes(v)
        cabi.call("drk_kv_append_batch", C.byref(g), C.c_void_p(cm.pool_ptr()), C.c_void_p(cm.d_block_table(b)), 0, L, p0, m,
                  U.p(dk), U.p(dv), cabi.BF16, U.stream_ptr())
        U.sync()
        model[b] = (np.concatenate([model[b][0], k], axis=1), np.concatenate([model[b][1], v], axis=1))
        cm.set_seq_len(b, p0 + m)

    def fork(parent, pos):
        b = cm.fork_branch(parent, pos)
        assert b > 0
        model[b] = (model[parent][0][:, :pos].copy(), model[parent][1][:, :pos].copy())
        return b

    bulk(0, 20 * bs + 5)                                   # the persistent context: 325 tokens
    b1 = fork(0, 20 * bs)                                  # at a block boundary
    bulk(b1, 9 * bs + 3)
    b2 = fork(b1, 28 * bs)                                 # 8 blocks into what b1 wrote
    bulk(b2, 6 * bs)
    b3 = fork(b2, 32 * bs)                                 # 4 blocks into what b2 wrote
    bulk(b3, 2 * bs + 9)
    b4 = fork(b1, 24 * bs + 7)                             # inside a block of b1: shares 24 whole blocks with it
    bulk(b4, 3 * bs)
    bulk(b2, 11)                                           # the parents go on after their children left
    bulk(0, 2 * bs)
    branches = [0, b1, b2, b3, b4]
    assert branches == list(range(5))
    groups = cm.common_prefix_groups(branches, 64 // (QH // KVH), 4 * bs)
    assert groups == [(0, 5, 0, 20 * bs), (1, 4, 20 * bs, 24 * bs), (1, 3, 24 * bs, 28 * bs), (2, 2, 28 * bs, 32 * bs)]

    B = len(branches)
    lens = np.array([cm.seq_len(b) for b in branches], dtype=np.int32)
    q = U.normal_bits(rng, (B, QH, D), cabi.BF16)
    dq, dl = U.dev_bytes(q), U.dev_i32(lens)
    scale = 1 / np.sqrt(D)
    cm.sync_block_table(U.stream_ptr())
    garr = np.array(groups, dtype=np.int32)
    outs = []
    for n_groups in (len(groups), 2, 0):                   # the whole tree, its first two levels, no sharing at all
        out = U.dev_zeros(B * QH * D * 2)
        lib.drkh_paged_gqa_decode_attention_grouped(U.p(dq), cm.pool_ptr(), cm.d_block_table(0), stride, U.p(dl), B,
                                                    int(lens.max()), garr.ctypes.data_as(C.c_void_p), n_groups, U.p(out), 1,
                                                    NB, bs, float(scale), U.stream_ptr())
        U.sync()
        outs.append(U.from_bits(U.host(out, np.uint16, (B, QH, D)), cabi.BF16))
    for i, b in enumerate(branches):
        n = int(lens[i])
        pg = orc.layout(L, KVH, QH, D, bs, (n + bs - 1) // bs, orc.BF16)
        ppool = orc.new_pool(pg)
        ptab = np.arange((n + bs - 1) // bs, dtype=np.int32)
        orc.append_batch(pg, ppool, ptab, 1, 0, model[b][0][1], model[b][1][1], orc.BF16)
        want = orc.decode_f64(pg, q[i], ppool, ptab, 1, n, scale, orc.BF16)
        for got in outs:
            ok, ma, _ = U.rel_abs_ok(got[i], want)
            assert ok, (b, ma)


def test_importance_scorer_on_device(dev):
    sc = host.ImportanceScorer()
    assert sc.init(64, 0.5)
    new = np.arange(64, dtype=np.float32)
    dn = U.dev_bytes(new)
    for _ in range(3):
        sc.update(U.p(dn), 64)
    sc.sync_to_host()
    want = new * (1 + 0.5 + 0.25)
    assert [sc.score(i) for i in range(64)] == want.tolist()
    assert sc.least_important([9, 3, 7]) == 3


@pytest.mark.parametrize("geom", [(24, 4, 256, 64, cabi.F16), (32, 8, 128, 32, cabi.BF16)])
def test_layer_steps_in_the_wrappers_order_fused_and_separate(dev, geom):
    """full_attention_forward_paged's steps 1b-7 (paged_attention.cu:331-370) for 3 decode branches:
    once as the reference's separate calls (split, head_norm x2, apply_rope, write, attend,
    sigmoid_gate; layer.h:77-79, 124-140), once as the two fused launches.  Same bits."""
    QH, KVH, D, rd, dt = geom
    L, bs, B = 2, 16, 3
    assert host.set_attention_geometry(L, QH, KVH, D, dt)
    assert host.lib().drkh_set_rope(rd, 1.0e7, 1e-6)
    assert not host.lib().drkh_set_rope(48, 1.0e7, 1e-6)             # 48 / 16 is no power of two: refused, nothing changes
    L_ = host.lib()
    rng = np.random.default_rng(90)
    outs = []
    for fused in (False, True):
        cm = host.CacheManager()
        assert cm.init(64 * L * 2 * KVH * bs * D * 2, bs, None, B)
        NB = cm.pool_max_blocks()
        ctx = [40, 17, 33]
        rs = np.random.default_rng(91)                                # the same inputs in both passes
        # prior context: plain appends into three independent branches (forks at position 0 share nothing)
        assert [cm.fork_branch(0, 0) for _ in range(B - 1)] == [1, 2]
        for b in range(B):
            assert cm.ensure_blocks_for_range(b, 0, ctx[b] + 1)
        cm.sync_block_table(U.stream_ptr())
        keep = []
        for b in range(B):
            k0, v0 = U.normal_bits(rs, (ctx[b], KVH, D), dt, 0.5), U.normal_bits(rs, (ctx[b], KVH, D), dt, 0.5)
            dk0, dv0 = U.dev_bytes(k0), U.dev_bytes(v0)
            keep += [dk0, dv0]
            L_.drkh_paged_kv_cache_write_batch(U.p(dk0), U.p(dv0), cm.pool_ptr(), cm.d_block_table(b), 1, 0, ctx[b], NB, bs,
                                               U.stream_ptr())
        qg = U.normal_bits(rs, (B, QH, 2 * D), dt, 1.5)
        k, v = U.normal_bits(rs, (B, KVH, D), dt), U.normal_bits(rs, (B, KVH, D), dt)
        qw, kw = U.normal_bits(rs, (D,), dt), U.normal_bits(rs, (D,), dt)
        dqg, dk, dv, dqw, dkw = (U.dev_bytes(a) for a in (qg, k, v, qw, kw))
        dpos, dlens = U.dev_i32(np.array(ctx)), U.dev_i32(np.array(ctx) + 1)
        dq, dgate, out = U.dev_zeros(B * QH * D * 2), U.dev_zeros(B * QH * D * 2), U.dev_zeros(B * QH * D * 2)
        scale, st = float(1 / np.sqrt(D)), U.stream_ptr()
        if fused:
            L_.drkh_paged_qk_norm_rope_write_branches(U.p(dqg), U.p(dk), U.p(dv), U.p(dqw), U.p(dkw), U.p(dq), cm.pool_ptr(),
                                                      cm.d_block_table(0), cm.table_stride(), U.p(dpos), B, 1, NB, bs, None, 0, st)
            L_.drkh_paged_gqa_decode_attention_gated_branches(U.p(dq), cm.pool_ptr(), cm.d_block_table(0), cm.table_stride(),
                                                              U.p(dlens), B, max(ctx) + 1, C.c_void_p(dqg.data_ptr() + D * 2), 2 * D,
                                                              U.p(out), 1, NB, bs, scale, st)
        else:
            cabi.call("drk_split_q_gate", U.p(dqg), U.p(dq), U.p(dgate), B, QH, D, st)
            L_.drkh_head_norm(U.p(dq), U.p(dqw), U.p(dq), B * QH, D, 1e-6, st)
            L_.drkh_head_norm(U.p(dk), U.p(dkw), U.p(dk), B * KVH, D, 1e-6, st)
            for b in range(B):                                        # one token per call, as the reference does
                L_.drkh_apply_rope(C.c_void_p(dq.data_ptr() + b * QH * D * 2), C.c_void_p(dk.data_ptr() + b * KVH * D * 2), QH, KVH, D,
                                   rd, C.c_void_p(dpos.data_ptr() + 4 * b), 1.0e7, st)
            L_.drkh_paged_kv_cache_write_branches(U.p(dk), U.p(dv), cm.pool_ptr(), cm.d_block_table(0), cm.table_stride(), U.p(dpos),
                                                  B, 1, NB, bs, st)
            L_.drkh_paged_gqa_decode_attention_branches(U.p(dq), cm.pool_ptr(), cm.d_block_table(0), cm.table_stride(), U.p(dlens), B,
                                                        max(ctx) + 1, U.p(out), 1, NB, bs, scale, st)
            L_.drkh_sigmoid_gate(U.p(out), U.p(dgate), U.p(out), B * QH * D, st)
        U.sync()
        outs.append((U.host(out, np.uint16).copy(), d2h(cm.pool_ptr(), cm.pool_total_bytes()), U.host(dq, np.uint16).copy()))
        del cm
    assert np.array_equal(outs[0][2], outs[1][2])          # Q after norm + rope
    assert np.array_equal(outs[0][1], outs[1][1])          # every byte of the pool
    assert np.array_equal(outs[0][0], outs[1][0])          # gated attention output
    assert outs[0][0].any()


def test_eviction_guided_by_measured_attention_mass(dev):
    """The loop the reference describes but never wires (docs/en/architecture/02-memoria.md:40-44,
    importance_scorer.h:7-14): attention reports the weight each block received, summed over the
    full-attention layers; the scorer folds it in; the next eviction takes the least attended
    block of any branch."""
    L, QH, KVH, D, bs, B = 2, 32, 8, 128, 16, 2
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    cm, sc = host.CacheManager(), host.ImportanceScorer()
    NBLK = 40
    assert cm.init(NBLK * L * 2 * KVH * bs * D * 2, bs, sc, B)
    stride = cm.table_stride()
    assert sc.init(B * stride, 0.5)
    NB = cm.pool_max_blocks()
    assert cm.fork_branch(0, 0) == 1
    ctx = [10 * bs, 7 * bs]                         # whole blocks: a short last block would trivially weigh least
    rng = np.random.default_rng(92)
    q = rng.standard_normal((L, B, QH, D)).astype(np.float32) * 0.5
    og = orc.layout(L, KVH, QH, D, bs, NB, orc.BF16)
    keep = []
    for b in range(B):
        assert cm.ensure_blocks_for_range(b, 0, ctx[b])
    cm.sync_block_table(U.stream_ptr())
    L_ = host.lib()
    cold = (1, 4)                                   # branch 1, logical block 4: keys opposed to every query of its group
    kv_host = []
    for b in range(B):
        k = rng.standard_normal((L, ctx[b], KVH, D)).astype(np.float32) * 0.5
        if b == cold[0]:
            for l in range(L):
                for h in range(KVH):
                    k[l, cold[1] * bs:(cold[1] + 1) * bs, h] = -2.0 * q[l, b, 4 * h:4 * h + 4].mean(axis=0)
        v = rng.standard_normal((L, ctx[b], KVH, D)).astype(np.float32) * 0.5
        kb, vb = U.to_bits(k, cabi.BF16), U.to_bits(v, cabi.BF16)
        kv_host.append((kb, vb))
        for l in range(L):
            dk, dv = U.dev_bytes(kb[l]), U.dev_bytes(vb[l])
            keep += [dk, dv]
            L_.drkh_paged_kv_cache_write_batch(U.p(dk), U.p(dv), cm.pool_ptr(), cm.d_block_table(b), l, 0, ctx[b], NB, bs,
                                               U.stream_ptr())
    qb = U.to_bits(q, cabi.BF16)
    dq, dlens, out = U.dev_bytes(qb), U.dev_i32(np.array(ctx)), U.dev_zeros(L * B * QH * D * 2)
    scale = float(1 / np.sqrt(D))
    for l in range(L):
        L_.drkh_paged_gqa_decode_attention_branches_scored(
            C.c_void_p(dq.data_ptr() + l * B * QH * D * 2), cm.pool_ptr(), cm.d_block_table(0), stride, U.p(dlens), B, max(ctx),
            C.c_void_p(out.data_ptr() + l * B * QH * D * 2), l, NB, bs, scale, sc.d_new_scores(), 1 if l > 0 else 0,
            U.stream_ptr())
    sc.apply_new_scores(U.stream_ptr())
    sc.sync_to_host()
    # the oracle's masses on the same pool contents
    tables = np.stack([cm.h_block_table(b) for b in range(B)])
    opool = orc.new_pool(og)
    for b in range(B):
        for l in range(L):
            orc.append_batch(og, opool, tables[b], l, 0, kv_host[b][0][l], kv_host[b][1][l], orc.BF16)
    want = sum(orc.block_attention_mass(og, qb[l], opool, tables, np.array(ctx, np.int32), l, scale, orc.BF16, stride)
               for l in range(L))
    got = np.array([[sc.score(b * stride + lb) for lb in range(stride)] for b in range(B)])
    assert np.all(np.abs(got - want) <= 4e-3 + 2e-3 * np.abs(want)), float(np.abs(got - want).max())
    assert np.allclose(got.sum(axis=1), L * QH, atol=5e-2)
    live = [(b, lb) for b in range(B) for lb in range((ctx[b] + bs - 1) // bs)]
    assert min(live, key=lambda c: want[c]) == cold and want[cold] < 0.5 * sorted(want[c] for c in live)[1]
    # the next eviction takes exactly that block
    before = tables.copy()
    assert cm.evict_blocks(1) == 1
    after = np.stack([cm.h_block_table(b) for b in range(B)])
    changed = np.argwhere(before != after)
    assert changed.tolist() == [list(cold)] and after[cold] == -1
    assert cm.block_location(*cold) == host.CacheManager.INVALID


def test_prefill_as_the_first_call_without_a_reserved_workspace(dev):
    """The usual order of a session is prefill first.  A long chunk on the MFMA kernel needs no workspace: the
    wrapper must launch it also when nothing has been reserved or allocated yet (it once returned silently)."""
    L, KVH, QH, D, bs, M = 1, 4, 16, 128, 16, 40
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.F16)
    cm = host.CacheManager()
    assert cm.init(16 * L * 2 * KVH * bs * D * 2, bs)
    NB = cm.pool_max_blocks()
    assert cm.ensure_blocks_for_range(0, 0, M)
    cm.sync_block_table(U.stream_ptr())
    rng = np.random.default_rng(5)
    k, v, q = (U.normal_bits(rng, s, cabi.F16) for s in ((M, KVH, D), (M, KVH, D), (M, QH, D)))
    dk, dv, dq = U.dev_bytes(k), U.dev_bytes(v), U.dev_bytes(q)
    L_ = host.lib()
    L_.drkh_paged_kv_cache_write_batch(U.p(dk), U.p(dv), cm.pool_ptr(), cm.d_block_table(0), 0, 0, M, NB, bs, U.stream_ptr())
    out = U.dev_bytes(np.full(M * QH * D * 2, 0x7B, np.uint8))
    U.sync()
    L_.drkh_paged_attention_release_workspace()
    scale = 1 / np.sqrt(D)
    L_.drkh_paged_prefill_attention(U.p(dq), cm.pool_ptr(), cm.d_block_table(0), U.p(out), 0, 0, M, NB, bs, float(scale),
                                    U.stream_ptr())
    U.sync()
    og = orc.layout(L, KVH, QH, D, bs, NB, orc.F16)
    opool = orc.new_pool(og)
    orc.append_batch(og, opool, cm.h_block_table(0), 0, 0, k, v, orc.F16)
    want = orc.prefill_f64(og, q, opool, cm.h_block_table(0), 0, 0, scale, orc.F16)
    ok, ma, _ = U.rel_abs_ok(U.from_bits(U.host(out, np.uint16, (M, QH, D)), cabi.F16), want)
    assert ok, ma
