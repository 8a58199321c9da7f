"""Host bookkeeping without a GPU: BlockPool / CacheManager (detached mode, i.e.
the same allocator and tables with no device memory) against closed forms, the
oracle's restatement of the reference (block_pool.cpp:51-75,
cache_manager.cpp:73-164, 185-205, 294-326) on random traces, and a naive
simulator in which every branch owns a private copy of its tokens."""
import numpy as np
import pytest

from deusridet_amd import cabi, host
from oracle import binding as orc
from tests import util as U


def make(NB, bs, branches=1, scorer=None):
    assert host.set_attention_geometry(2, 4, 2, 16, cabi.F16)
    cm = host.CacheManager()
    assert cm.init_detached(NB, bs, scorer, branches)
    return cm


# ---------------------------------------------------------------- closed forms
def test_free_stack_closed_form():
    for sut in (make(6, 4), orc.CacheManager(6, 4)):
        alloc = sut.pool_alloc_block if hasattr(sut, "pool_alloc_block") else sut.alloc_block
        free = sut.pool_free_block if hasattr(sut, "pool_free_block") else sut.free_block
        count = sut.pool_free_count if hasattr(sut, "pool_free_count") else sut.free_count
        assert [alloc() for _ in range(6)] == [0, 1, 2, 3, 4, 5]       # fresh pool yields 0,1,2,...
        assert alloc() == -1 and count() == 0                            # exhausted
        free(2); free(4)
        assert count() == 2
        assert [alloc(), alloc()] == [4, 2]                              # last in, first out
        assert alloc() == -1


def test_pool_offsets_match_the_layout_contract():
    assert host.set_attention_geometry(3, 8, 4, 32, cabi.BF16)
    cm = host.CacheManager()
    assert cm.init_detached(10, 16, None, 1)
    plane = 4 * 16 * 32 * 2
    for l, b in [(0, 0), (0, 3), (2, 9), (1, 5)]:
        k = l * 10 * 2 * plane + b * 2 * plane
        assert cm.pool_k_offset(l, b) == k and cm.pool_v_offset(l, b) == k + plane
    assert cm.pool_total_bytes() == 3 * 10 * 2 * plane
    assert cm.table_stride() == 20                                        # 2x physical (cache_manager.cpp:39)


def test_single_sequence_fifo_eviction():
    """Without a scorer the victim is the oldest allocation (cache_manager.cpp:203-204)."""
    for sut in (make(4, 4), orc.CacheManager(4, 4)):
        ens = (lambda p: sut.ensure_blocks_for(0, p)) if isinstance(sut, host.CacheManager) else (lambda p: sut.ensure(0, p))
        table = (lambda: sut.h_block_table(0)) if isinstance(sut, host.CacheManager) else (lambda: sut.table(0))
        for pos in range(0, 16):
            assert ens(pos)
        assert table()[:4].tolist() == [0, 1, 2, 3] and sut.gpu_blocks_used() == 4
        assert ens(16)                                    # pool full: logical 0 is evicted, its block reused
        assert table()[:5].tolist() == [-1, 1, 2, 3, 0]
        assert ens(20)
        assert table()[:6].tolist() == [-1, -1, 2, 3, 0, 1]
        assert ens(0)                                     # an evicted block comes back as a fresh allocation
        assert table()[:6].tolist() == [2, -1, -1, 3, 0, 1]
        assert sut.evict_blocks(2) == 2
        assert table()[:6].tolist() == [2, -1, -1, -1, -1, 1]
        assert not ens(4 * 2 * 4)                         # beyond max_logical = 2*NB blocks
        assert sut.ensure_free_blocks(4) and sut.gpu_blocks_used() == 0
        assert not sut.ensure_free_blocks(5)              # nothing left to evict


def test_scorer_guided_eviction_takes_first_minimum():
    scores = np.array([5, 1, 3, 1, 0.5, 9, 9, 9], dtype=np.float32)
    sc = host.ImportanceScorer()
    assert sc.init_detached(8)
    sc.load_host_scores(scores)
    cm = make(4, 4, 1, sc)
    oc = orc.CacheManager(4, 4)
    oc.set_scores(scores)
    for pos in (0, 4, 8, 12):
        assert cm.ensure_blocks_for(0, pos) and oc.ensure(0, pos)
    assert cm.evict_blocks(1) == 1 and oc.evict_blocks(1) == 1
    assert cm.h_block_table(0)[:4].tolist() == [0, -1, 2, 3] == oc.table(0)[:4].tolist()    # logical 1: first of the two 1.0
    assert cm.ensure_blocks_for(0, 16) and oc.ensure(0, 16)                                  # logical 4, score 0.5
    assert cm.evict_blocks(1) == 1 and oc.evict_blocks(1) == 1
    assert cm.h_block_table(0)[:5].tolist() == [0, -1, 2, 3, -1] == oc.table(0)[:5].tolist()
    assert sc.least_important([4, 2, 7, 1]) == 4 and sc.least_important([]) == -1


def test_fork_shares_and_write_copies():
    cm = make(8, 4, branches=3)
    assert cm.ensure_blocks_for_range(0, 0, 10)                  # logical 0,1,2 -> phys 0,1,2
    b = cm.fork_branch(0, 10)
    assert b == 1 and cm.seq_len(1) == 10
    assert cm.h_block_table(1)[:3].tolist() == [0, 1, 2]
    assert [cm.pool_refcount(i) for i in range(3)] == [2, 2, 2] and cm.gpu_blocks_used() == 3
    assert cm.ensure_blocks_for(1, 10)                           # write into the shared, partly filled block
    assert cm.take_pending_copies() == [(2, 3)]
    assert cm.h_block_table(1)[:3].tolist() == [0, 1, 3] and cm.h_block_table(0)[:3].tolist() == [0, 1, 2]
    assert [cm.pool_refcount(i) for i in range(4)] == [2, 2, 1, 1]
    assert cm.ensure_blocks_for(1, 11) and cm.take_pending_copies() == []     # now private: no second copy
    assert cm.ensure_blocks_for(0, 10) and cm.take_pending_copies() == []     # parent's block is private again
    # shared blocks are pinned: only the two private ones can go
    assert cm.evict_blocks(10) == 2
    assert cm.h_block_table(0)[:3].tolist() == [0, 1, -1] and cm.h_block_table(1)[:3].tolist() == [0, 1, -1]
    assert not cm.ensure_free_blocks(7)
    cm.release_branch(1)
    assert [cm.pool_refcount(i) for i in range(2)] == [1, 1]
    assert cm.ensure_free_blocks(8) and cm.gpu_blocks_used() == 0
    assert cm.fork_branch(0, 0) == 1                             # the id is free again
    assert cm.fork_branch(5, 0) == -1 and cm.fork_branch(2, 0) == -1     # bad / dead parent


def test_a_step_never_loses_the_blocks_it_is_about_to_write():
    """Several branches forked at a position that is not block-aligned share their tail block; the
    first write of each takes a private copy.  With fewer free blocks than branches the later
    allocations must find their victims elsewhere: a block made resident in this step (the target
    of a copy that is still queued, or another branch's write block) is never taken, and when
    nothing else is left the call fails instead of leaving a hole behind."""
    for mk in ("lib", "oracle"):
        def fresh(NB):
            return make(NB, 4, branches=6) if mk == "lib" else orc.CacheManager(NB, 4, 6)
        ens = lambda m, b, p: m.ensure_blocks_for(b, p) if mk == "lib" else m.ensure(b, p)
        fork = lambda m, b, p: m.fork_branch(b, p) if mk == "lib" else m.fork(b, p)
        tab = lambda m, b: m.h_block_table(b) if mk == "lib" else m.table(b)
        drain = lambda m: m.take_pending_copies() if mk == "lib" else m.drain_copies()
        # 10 tokens: blocks 0, 1 full, block 2 half; 4 branches share all three; the pool has 2 free blocks
        m = fresh(5)
        for pos in range(10):
            assert ens(m, 0, pos)
        drain(m)
        kids = [fork(m, 0, 10) for _ in range(4)]
        assert kids == [1, 2, 3, 4]
        got = [ens(m, b, 10) for b in kids]
        # two private copies fit; the third and fourth find only pinned (shared) and protected cells
        assert got == [True, True, False, False], (mk, got)
        for b in kids[:2]:
            assert tab(m, b)[2] >= 0 and tab(m, b)[2] != tab(m, 0)[2], (mk, b)     # no hole where the step writes
        assert sorted(drain(m)) == [(2, 3), (2, 4)]
        # the same with an old private block around: that one is the victim, not a block of the step
        m = fresh(6)
        for pos in range(10):
            assert ens(m, 0, pos)
        drain(m)
        kids = [fork(m, 0, 10) for _ in range(4)]
        assert ens(m, 0, 10) and drain(m) == [(2, 3)]           # the stream's own copy: block 3 is private, unprotected now
        got = [ens(m, b, 10) for b in kids]
        assert got == [True, True, True, True], (mk, got)       # 2 free blocks, the stream's private block 3, and the
        assert tab(m, 0)[2] == -1                               # last sharer keeps block 2; block 3 was the victim
        assert [int(tab(m, b)[2]) for b in kids] == [4, 5, 3, 2], mk
        assert drain(m) == [(2, 4), (2, 5), (2, 3)]


def test_a_queued_copy_keeps_its_source_block():
    """The source of a queued copy is not handed out again before the copy has been issued, even when
    its last table entry goes away in between."""
    for mk in ("lib", "oracle"):
        m = make(4, 4, branches=3) if mk == "lib" else orc.CacheManager(4, 4, 3)
        ens = (lambda b, p: m.ensure_blocks_for(b, p)) if mk == "lib" else (lambda b, p: m.ensure(b, p))
        drain = (lambda: m.take_pending_copies()) if mk == "lib" else (lambda: m.drain_copies())
        stack = (lambda: m.pool_free_stack().tolist()) if mk == "lib" else (lambda: m.free_stack().tolist())
        refc = (lambda i: m.pool_refcount(i)) if mk == "lib" else (lambda i: m.refcount(i))
        assert ens(0, 0) and ens(0, 1)
        drain()
        kid = m.fork_branch(0, 2) if mk == "lib" else m.fork(0, 2)
        assert ens(kid, 2)                                     # copy 0 -> 1 queued
        (m.release_branch if mk == "lib" else m.release)(0)    # the source's last table entry goes
        assert 0 not in stack() and refc(0) == 1, mk           # ... but the block is not free yet
        assert ens(kid, 4)                                     # a new block: 2, not the copy's source
        t = (m.h_block_table(kid) if mk == "lib" else m.table(kid))[:2].tolist()
        assert t == [1, 2], (mk, t)
        assert drain() == [(0, 1)]
        assert 0 in stack() and refc(0) == 0, mk


def test_touch_makes_it_lru():
    for sut in (make(4, 4), orc.CacheManager(4, 4)):
        is_p = isinstance(sut, host.CacheManager)
        for pos in (0, 4, 8, 12):
            assert sut.ensure_blocks_for(0, pos) if is_p else sut.ensure(0, pos)
        (sut.touch_block if is_p else sut.touch)(0, 0)
        assert sut.evict_blocks(1) == 1
        t = sut.h_block_table(0) if is_p else sut.table(0)
        assert t[:4].tolist() == [0, -1, 2, 3]
        order = sut.lru_snapshot() if is_p else sut.lru()
        assert order == [(0, 2), (0, 3), (0, 0)]


# ---------------------------------------------------------------- random traces
def _state(cm, oc, branches):
    assert cm.pool_free_stack().tolist() == oc.free_stack().tolist()
    assert cm.lru_snapshot() == oc.lru()
    assert cm.gpu_blocks_used() == oc.gpu_blocks_used()
    for b in range(branches):
        assert np.array_equal(cm.h_block_table(b), oc.table(b)), b
        assert cm.seq_len(b) == oc.seq_len(b)
    NB = cm.pool_max_blocks()
    refs = [cm.pool_refcount(i) for i in range(NB)]
    assert refs == [oc.refcount(i) for i in range(NB)]
    # invariants: refcount == number of table entries naming the block; free blocks have none
    counts = np.zeros(NB, dtype=np.int64)
    for b in range(branches):
        t = cm.h_block_table(b)
        np.add.at(counts, t[t >= 0], 1)
    assert counts.tolist() == refs
    free = set(cm.pool_free_stack().tolist())
    assert all(refs[i] == 0 for i in free) and len(free) + int((counts > 0).sum()) == NB


@pytest.mark.parametrize("seed", range(6))
def test_random_trace_matches_oracle(seed):
    rng = np.random.default_rng(seed)
    NB, bs, branches = int(rng.integers(6, 24)), int(rng.choice([2, 4, 16])), 4
    use_scores = seed % 2 == 1
    sc = None
    cm_scorer = None
    if use_scores:
        # one score per table cell (branch, logical block); ties on purpose
        scores = rng.random(branches * 2 * NB).astype(np.float32).round(1)
        cm_scorer = host.ImportanceScorer()
        assert cm_scorer.init_detached(branches * 2 * NB)
        cm_scorer.load_host_scores(scores)
        sc = scores
    cm = make(NB, bs, branches, cm_scorer)
    oc = orc.CacheManager(NB, bs, branches)
    oc.set_scores(sc)
    alive = {0}
    for step in range(400):
        op = rng.choice(["ensure", "ensure", "ensure", "range", "fork", "release", "evict", "free", "touch", "len"])
        b = int(rng.choice(sorted(alive)))
        if op == "ensure":
            pos = int(rng.integers(0, 2 * NB * bs + 3))
            assert cm.ensure_blocks_for(b, pos) == oc.ensure(b, pos), (step, op)
        elif op == "range":
            pos, M = int(rng.integers(0, NB * bs)), int(rng.integers(1, 3 * bs))
            assert cm.ensure_blocks_for_range(b, pos, M) == oc.ensure_range(b, pos, M), (step, op)
        elif op == "fork":
            pos = int(rng.integers(0, NB * bs))
            r1, r2 = cm.fork_branch(b, pos), oc.fork(b, pos)
            assert r1 == r2, (step, op)
            if r1 >= 0:
                alive.add(r1)
        elif op == "release":
            cm.release_branch(b); oc.release(b)
            if b != 0:
                alive.discard(b)
        elif op == "evict":
            n = int(rng.integers(0, 4))
            assert cm.evict_blocks(n) == oc.evict_blocks(n), (step, op)
        elif op == "free":
            n = int(rng.integers(0, NB + 2))
            assert cm.ensure_free_blocks(n) == oc.ensure_free_blocks(n), (step, op)
        elif op == "touch":
            l = int(rng.integers(0, 2 * NB))
            cm.touch_block(b, l); oc.touch(b, l)
        else:
            n = int(rng.integers(0, NB * bs))
            cm.set_seq_len(b, n); oc.set_seq_len(b, n)
        # usually every operation is its own step (copies issued right away); sometimes several
        # operations share a step, and the cells they made resident stay protected across them
        if rng.random() < 0.7:
            assert cm.take_pending_copies() == oc.drain_copies(), (step, op)
            if step % 20 == 0:
                _state(cm, oc, branches)
    assert cm.take_pending_copies() == oc.drain_copies()
    _state(cm, oc, branches)


# ---------------------------------------------------------------- model-based check
@pytest.mark.parametrize("seed", range(4))
def test_branches_equal_private_copies(seed):
    """After any sequence of append / fork / evict / release, what each branch can
    gather equals a naive model where every branch holds its own list of tokens
    (evicted pages read back as zeros).  Data moves use the oracle's CPU pool."""
    rng = np.random.default_rng(100 + seed)
    L, KVH, QH, D, bs, NB, branches = 2, 2, 4, 16, 4, 24, 4
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.F16)
    cm = host.CacheManager()
    assert cm.init_detached(NB, bs, None, branches)
    og = orc.layout(L, KVH, QH, D, bs, NB, orc.F16)
    pool = orc.new_pool(og)
    model = {0: []}                       # branch -> list of (k, v) rows [L, KVH, D], None where evicted
    tok_id = 0
    for step in range(300):
        alive = sorted(model)
        b = int(rng.choice(alive))
        op = rng.choice(["append"] * 6 + ["fork", "fork", "release", "evict"])
        before = {x: cm.h_block_table(x).copy() for x in alive}
        if op == "append":
            pos = len(model[b])
            if pos >= 2 * NB * bs:
                continue
            ok = cm.ensure_blocks_for(b, pos)
            for s, d in cm.take_pending_copies():
                orc.copy_block(og, pool, s, d)
            if ok:
                k = rng.integers(1, 65536, (L, KVH, D)).astype(np.uint16)
                v = rng.integers(1, 65536, (L, KVH, D)).astype(np.uint16)
                tab = cm.h_block_table(b)
                for l in range(L):
                    orc.append_token(og, pool, tab, l, pos, k[l], v[l], orc.F16)
                model[b].append((k, v))
                cm.set_seq_len(b, pos + 1)
                tok_id += 1
        elif op == "fork":
            pos = int(rng.integers(0, len(model[b]) + 1))
            nb = cm.fork_branch(b, pos)
            if nb >= 0:
                model[nb] = list(model[b][:pos])
        elif op == "release" and b != 0:
            cm.release_branch(b)
            del model[b]
        elif op == "evict":
            cm.evict_blocks(int(rng.integers(1, 3)))
        # eviction (explicit or inside ensure) turns whole pages of some branch into holes
        for x in sorted(model):
            now = cm.h_block_table(x)
            gone = np.nonzero((before.get(x, now) >= 0) & (now < 0))[0]
            for lb in gone:
                for t in range(lb * bs, min((lb + 1) * bs, len(model[x]))):
                    model[x][t] = None
        if step % 10 == 0 or step == 299:
            for x in sorted(model):
                n = len(model[x])
                if n == 0:
                    continue
                flat, _ = orc.extract(og, pool, cm.h_block_table(x), 0, n, L)
                tab = cm.h_block_table(x)
                for t in range(n):
                    if tab[t // bs] < 0:
                        assert not flat[:, :, t].any()
                        continue
                    if model[x][t] is None:
                        continue          # its page was evicted and later re-allocated: contents undefined
                    k, v = model[x][t]
                    assert np.array_equal(flat[:, 0, t], k) and np.array_equal(flat[:, 1, t], v), (step, x, t)
    # no block with references sits in the free stack
    free = set(cm.pool_free_stack().tolist())
    for x in sorted(model):
        t = cm.h_block_table(x)
        assert not (set(t[t >= 0].tolist()) & free)
