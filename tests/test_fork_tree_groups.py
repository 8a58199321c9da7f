"""CacheManager::common_prefix_groups on the CPU (detached manager: bookkeeping only): the shared ranges it
reports for fork trees must be true (same physical blocks in every member over the whole range), must form the
chains drk_paged_decode_attention_grouped accepts (for every branch its ranges follow one another from token 0),
and must find the sharing a brute-force look at the tables finds between neighbours."""
import numpy as np
import pytest

from deusridet_amd import host


def grow(cm, branch, n):
    """append n tokens to a branch the way the decode protocol does (ensure, then the length moves on)"""
    p = cm.seq_len(branch)
    for t in range(n):
        assert cm.ensure_blocks_for(branch, p + t)
    cm.take_pending_copies()
    cm.set_seq_len(branch, p + n)


def check(cm, branches, groups, bs, max_group_branches=16, min_tokens=64):
    tabs = [np.array(cm.h_block_table(b)) for b in branches]
    lens = [cm.seq_len(b) for b in branches]
    covered = [0] * len(branches)
    for (f, c, t0, t1) in groups:                              # parents come first: each extends its members' chains
        assert 0 <= f and c >= 2 and f + c <= len(branches) and c <= max_group_branches
        assert t0 % bs == 0 and t1 % bs == 0 and t1 - t0 >= min_tokens
        for i in range(f, f + c):
            assert lens[i] >= t1
            assert covered[i] == t0, "ranges of a branch must follow one another from token 0"
            covered[i] = t1
            assert np.array_equal(tabs[i][t0 // bs:t1 // bs], tabs[f][t0 // bs:t1 // bs])
        assert np.all(tabs[f][t0 // bs:t1 // bs] >= 0)
    return covered


def test_single_prefix():
    bs = 16
    cm = host.CacheManager()
    assert cm.init_detached(4096, bs, None, 17)
    grow(cm, 0, 1000)
    kids = [cm.fork_branch(0, 1000) for _ in range(8)]
    for i, b in enumerate(kids):
        grow(cm, b, 5 + 40 * i)
    groups = cm.common_prefix_groups(kids)
    assert groups == [(0, 8, 0, 992)]                          # whole blocks of the 1000 tokens
    check(cm, kids, groups, bs)
    assert cm.common_prefix_groups(kids[:1]) == []
    assert cm.common_prefix_groups(kids, min_tokens=2048) == []


def test_forks_at_several_moments_and_forks_of_forks():
    bs = 16
    cm = host.CacheManager()
    assert cm.init_detached(8192, bs, None, 32)
    grow(cm, 0, 2048)
    old = [cm.fork_branch(0, 2048) for _ in range(3)]          # ids 1, 2, 3
    grow(cm, 0, 1024)                                          # perception goes on
    young = [cm.fork_branch(0, 3072) for _ in range(4)]        # ids 4..7: share 3072 tokens among themselves
    for b in old + young:
        grow(cm, b, 100)
    sub = [cm.fork_branch(young[-1], cm.seq_len(young[-1])) for _ in range(2)]   # ids 8, 9: forks of a fork
    for b in sub:
        grow(cm, b, 70)
    branches = old + young + sub
    assert branches == list(range(1, 10))
    groups = cm.common_prefix_groups(branches)
    covered = check(cm, branches, groups, bs)
    assert groups[0] == (0, 9, 0, 2048)
    assert (3, 6, 2048, 3072) in groups                        # the young ones and the forks of one of them
    assert (6, 3, 3072, 3168) in groups                        # branch 7 and its two forks: 3172 tokens, whole blocks
    assert covered == [2048] * 3 + [3072] * 3 + [3168] * 3
    # cut short, the list is still a tree
    for k in range(len(groups)):
        check(cm, branches, cm.common_prefix_groups(branches, max_groups=k + 1), bs)
    # a wide set is cut into groups of at most max_group_branches over the same range
    g4 = cm.common_prefix_groups(branches, max_group_branches=4)
    check(cm, branches, g4, bs, max_group_branches=4)
    assert [x for x in g4 if x[2] == 0] == [(0, 4, 0, 2048), (4, 4, 0, 2048)]      # the ninth branch reads the range in its tail


@pytest.mark.parametrize("seed", range(12))
def test_random_fork_trees_against_the_tables(seed):
    rng = np.random.default_rng(seed)
    bs = 16
    cm = host.CacheManager()
    assert cm.init_detached(20000, bs, None, 24)
    grow(cm, 0, int(rng.integers(200, 3000)))
    alive = []
    for step in range(int(rng.integers(4, 14))):
        if alive and rng.random() < 0.4:
            parent = int(rng.choice(alive))
            pos = cm.seq_len(parent) if rng.random() < 0.5 else int(rng.integers(1, cm.seq_len(parent) + 1))
        else:
            parent, pos = 0, cm.seq_len(0) if rng.random() < 0.7 else int(rng.integers(1, cm.seq_len(0) + 1))
        b = cm.fork_branch(parent, pos)
        if b < 0:
            break
        alive.append(b)
        for x in alive:
            grow(cm, x, int(rng.integers(0, 300)))
        if rng.random() < 0.5:
            grow(cm, 0, int(rng.integers(1, 500)))
    branches = sorted(alive)
    if branches != list(range(branches[0], branches[0] + len(branches))):
        pytest.skip("ids not consecutive in this draw")
    for cap, mt in ((16, 64), (3, 64), (16, 256)):
        groups = cm.common_prefix_groups(branches, max_group_branches=cap, min_tokens=mt)
        covered = check(cm, branches, groups, bs, cap, mt)
        # nothing big is missed: what neighbours share beyond what is covered is either short of min_tokens per
        # level or lost to a cut of a wide set
        tabs = [np.array(cm.h_block_table(b)) for b in branches]
        if cap == 16:
            for i in range(len(branches) - 1):
                n = min(cm.seq_len(branches[i]), cm.seq_len(branches[i + 1])) // bs
                k = 0
                while k < n and tabs[i][k] >= 0 and tabs[i][k] == tabs[i + 1][k]:
                    k += 1
                depth = sum(1 for g in groups if g[0] <= i < g[0] + g[1])
                assert min(covered[i], covered[i + 1]) >= k * bs - (depth + 2) * max(mt, bs), (i, k * bs, covered, groups)


def test_the_grid_is_dealt_so_that_every_unit_has_a_workgroup_and_no_run_outgrows_the_table():
    """The fork-tree kernel's grid goes to runs of units of the shared ranges and runs of units of the tails
    (region_split in drk_decode_group.hip, the same arithmetic in kernel and merge).  Whatever the shape -- no
    shared range, no tail, thousands of one-tile tails behind a short range, the host's upper bound above the
    lengths on the device -- every unit must belong to a workgroup's run and no run may be longer than the
    kernel's descriptor table.  CPU only: the library's own arithmetic through its debug entry points."""
    import ctypes as C
    from deusridet_amd import cabi
    lib = cabi.lib()
    rng = np.random.default_rng(20)
    out = (C.c_int * 3)()
    for table in (64, 128):                                    # the 16-bit tile kernel's table and the general kernel's
        for _ in range(20000):
            kvh = int(rng.choice([1, 2, 4, 8]))
            B = int(rng.integers(1, 65))
            gu = kvh * int(rng.choice([0, rng.integers(0, 50), rng.integers(0, 5000)]))
            tails = [int(rng.choice([0, 1, rng.integers(0, 9), rng.integers(0, 3000)])) for _ in range(B)]
            upper = [t + int(rng.integers(0, 4)) for t in tails]
            tu, tr = kvh * sum(tails), kvh * sum(1 for t in tails if t > 0)
            if gu + kvh * sum(upper) == 0:
                continue
            grid = lib.drk_debug_grouped_grid(kvh, gu, kvh * sum(upper), table)
            assert grid >= 1
            lib.drk_debug_grouped_region_split(gu, tu, tr, grid, table, out)
            gs, us, ut = out[0], out[1], out[2]
            assert 0 <= gs <= grid and 1 <= us <= table and 1 <= ut <= table, (kvh, gu, tu, tr, grid, gs, us, ut)
            if gu > 0:
                assert gs >= 1 and gs * us >= gu, (kvh, gu, tu, tr, grid, gs, us, ut)
            if tu > 0:
                assert grid - gs >= 1 and (grid - gs) * ut >= tu, (kvh, gu, tu, tr, grid, gs, us, ut)
    # right after a fork: 128 one-tile tails behind 8 192 shared tiles get enough workgroups not to be the last to finish
    lib.drk_debug_grouped_region_split(8192, 128, 128, 512, 64, out)
    assert 512 - out[0] >= 16 and out[2] <= 8
