"""Decode over branches that share pages as a tree (drk_paged_decode_attention_grouped):
one launch streams every shared range once for all its branches and every private tail
once.  Checked per branch against the fp64 oracle (tolerance 1e-2 relative / 2e-2
absolute, the attention bar) and against the plain per-branch call."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi
from oracle import binding as orc
from tests import util as U

pytestmark = pytest.mark.gpu
REL, ABS = 1e-2, 2e-2


@pytest.fixture(scope="module")
def dev():
    import torch
    assert torch.cuda.is_available()
    return torch.device("cuda:0")


class Tree:
    """B branches whose tables share physical blocks as `groups` say: (first, count, begin, end) in
    tokens, multiples of the block size, a fork tree.  K/V of a shared range are written once."""

    def __init__(self, heads, dtype, groups, lens, seed, bs=16, holes=()):
        KVH, QH, D = heads
        self.io = dtype if dtype in (cabi.F16, cabi.BF16) else cabi.BF16
        self.groups, self.lens = list(groups), np.asarray(lens, dtype=np.int32)
        B = len(lens)
        rng = np.random.default_rng(seed)
        nblk = [(int(l) + bs - 1) // bs for l in lens]
        self.stride = max(nblk) + 3
        shared_blocks = sum((e - b) // bs for (_, _, b, e) in groups)
        start = np.zeros(B, dtype=np.int64)
        for (f, c, b, e) in groups:
            assert b % bs == 0 and e % bs == 0
            start[f:f + c] = np.maximum(start[f:f + c], e)
        priv = [nblk[i] - int(start[i]) // bs for i in range(B)]
        assert min(priv) >= 0
        NB = shared_blocks + sum(priv) + 9
        self.g, self.og = U.both_layouts(1, KVH, QH, D, bs, NB, dtype)
        perm = rng.permutation(NB).astype(np.int32)
        self.tables = np.full((B, self.stride), -1, dtype=np.int32)
        self.opool = orc.new_pool(self.og)
        self.opool[:] = 0x5A if dtype in (cabi.F16, cabi.BF16) else 0        # stale bytes behind every row's end
        o = 0

        def fill(b, p0, n):
            k = U.normal_bits(rng, (n, KVH, D), self.io, 0.7)
            v = U.normal_bits(rng, (n, KVH, D), self.io, 0.7)
            orc.append_batch(self.og, self.opool, self.tables[b], 0, p0, k, v, self.io)

        for (f, c, b, e) in sorted(groups, key=lambda t: t[2]):
            n = (e - b) // bs
            self.tables[f:f + c, b // bs:e // bs] = perm[o:o + n]
            o += n
            fill(f, b, e - b)
        for i in range(B):
            s = int(start[i]) // bs
            self.tables[i, s:s + priv[i]] = perm[o:o + priv[i]]
            o += priv[i]
            if int(lens[i]) > int(start[i]):
                fill(i, int(start[i]), int(lens[i]) - int(start[i]))
        for (b, lb) in holes:
            self.tables[b, lb] = -1
        self.q = U.normal_bits(rng, (B, QH, D), self.io, 0.7)
        self.scale = 1.0 / np.sqrt(D)
        self.B, self.QH, self.D = B, QH, D
        self.dq, self.dpool = U.dev_bytes(self.q), U.dev_bytes(self.opool)
        self.dtab, self.dl = U.dev_i32(self.tables), U.dev_i32(self.lens)

    def want(self):
        return np.stack([orc.decode_f64(self.og, self.q[b], self.opool, self.tables[b], 0, int(self.lens[b]),
                                        self.scale, self.io) for b in range(self.B)])

    def run_grouped(self, groups=None, gate=None, fill=0x7B, ws_max_depth=None):
        lib = cabi.lib()
        groups = self.groups if groups is None else groups
        arr = cabi.prefix_groups(groups)
        mx = int(self.lens.max())
        if ws_max_depth is None:
            wsb = lib.drk_decode_grouped_workspace_bytes(C.byref(self.g), self.B, mx, arr, len(groups))
        else:
            wsb = lib.drk_decode_grouped_workspace_bytes_max(C.byref(self.g), self.B, mx, ws_max_depth)
        assert wsb > 0
        ws = U.dev_bytes(np.full(wsb, 0xFF, dtype=np.uint8))          # NaN patterns: a slot read before it is written shows
        out = U.dev_bytes(np.full(self.B * self.QH * self.D * 2, fill, dtype=np.uint8))
        cabi.call("drk_paged_decode_attention_grouped", C.byref(self.g), U.p(self.dq), U.p(self.dpool), U.p(self.dtab),
                  self.stride, U.p(self.dl), self.B, mx, arr, len(groups), U.p(out), 0, float(self.scale), self.io,
                  U.p(gate) if gate is not None else None, 2 * self.D if gate is not None else 0, U.p(ws), wsb,
                  U.stream_ptr())
        U.sync()
        return U.host(out, np.uint16, (self.B, self.QH, self.D))

    def run_plain(self):
        lib = cabi.lib()
        mx = int(self.lens.max())
        wsb = lib.drk_decode_workspace_bytes(C.byref(self.g), self.B, mx)
        ws, out = U.dev_zeros(wsb), U.dev_zeros(self.B * self.QH * self.D * 2)
        cabi.call("drk_paged_decode_attention_branches", C.byref(self.g), U.p(self.dq), U.p(self.dpool), U.p(self.dtab),
                  self.stride, U.p(self.dl), self.B, mx, U.p(out), 0, float(self.scale), self.io, 0, U.p(ws), wsb,
                  U.stream_ptr())
        U.sync()
        return U.host(out, np.uint16, (self.B, self.QH, self.D))


TREE8 = ([(0, 8, 0, 1040), (0, 4, 1040, 2000), (4, 4, 1040, 1216), (0, 2, 2000, 2512)],
         [2512 + 300, 2512, 2000 + 5, 2000 + 700, 1216 + 64, 1216 + 1, 1216 + 1000, 1216 + 130])
# the same tree with every branch's last token behind the ranges it shares (branch 1 above ends with its range)
TREE8_OWN_LAST = (TREE8[0], [2512 + 300, 2512 + 1, 2000 + 5, 2000 + 700, 1216 + 64, 1216 + 1, 1216 + 1000, 1216 + 130])
# forks spread over a prefix: every branch leaves the common context somewhere else
SPREAD = ([(0, 6, 0, 512), (1, 5, 512, 1024), (2, 4, 1024, 2048), (3, 3, 2048, 2560), (4, 2, 2560, 4096)],
          [512 + 77, 1024 + 1, 2048 + 300, 2560 + 64, 4096 + 5, 4096 + 640])
ONE = ([(0, 16, 0, 8192 + 64)], [8192 + 64 + (37 * i) % 900 for i in range(16)])
TWO_ROOTS = ([(0, 3, 0, 640), (3, 2, 0, 1280), (3, 1, 1280, 1344)], [640 + 9, 640, 640 + 200, 1344 + 3, 1280 + 65])


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
@pytest.mark.parametrize("tree,heads", [(TREE8, (8, 32, 128)), (SPREAD, (8, 32, 128)), (ONE, (8, 32, 128)),
                                        (TWO_ROOTS, (2, 16, 128)), (TREE8, (4, 4, 128)), (SPREAD, (1, 10, 128))])
def test_fork_tree_decode(dev, dtype, tree, heads):
    """every branch of a fork tree against fp64 attention over its own table, and against the per-branch call"""
    groups, lens = tree
    t = Tree(heads, dtype, groups, lens, seed=len(lens) * 7 + heads[1])
    got = U.from_bits(t.run_grouped(), t.io)
    want = t.want()
    ok, ma, _ = U.rel_abs_ok(got, want, REL, ABS)
    assert ok, ma
    ok, ma, _ = U.rel_abs_ok(got, U.from_bits(t.run_plain(), t.io).astype(np.float64), REL, ABS)
    assert ok, ma
    # fewer groups than the tables would allow is still right (the tails read what no group covers)
    got2 = U.from_bits(t.run_grouped(groups=groups[:1], ws_max_depth=1), t.io)
    ok, ma, _ = U.rel_abs_ok(got2, want, REL, ABS)
    assert ok, ma
    # a workspace sized for any tree of this depth serves the call too
    got3 = t.run_grouped(ws_max_depth=len(groups))
    assert np.array_equal(got3, U.to_bits(got, t.io))


def test_fork_tree_with_missing_pages(dev):
    """evicted pages (table entry -1) inside shared ranges and tails take no part, for every branch that shared them"""
    groups, lens = TREE8
    t = Tree((8, 32, 128), cabi.BF16, groups, lens, seed=5,
             holes=[(b, 3) for b in range(8)] + [(b, 70) for b in range(4)] + [(0, 2512 // 16 + 2), (6, 1216 // 16 + 9)])
    got = U.from_bits(t.run_grouped(), t.io)
    ok, ma, _ = U.rel_abs_ok(got, t.want(), REL, ABS)
    assert ok, ma


def test_fork_tree_gated_and_rows_without_tokens(dev):
    """the gate in the merge's epilogue; a branch of length 0 keeps what out held (gated when a gate is given)"""
    groups = [(0, 3, 0, 256)]
    t = Tree((8, 32, 128), cabi.F16, groups, [256 + 40, 256, 256 + 129, 0], seed=11)
    rng = np.random.default_rng(3)
    gate = U.normal_bits(rng, (t.B, t.QH, 2 * t.D), t.io)          # rows 2 * head_dim apart, as the Q|gate projection leaves them
    dg = U.dev_bytes(gate)
    plain = t.run_grouped()
    got = t.run_grouped(gate=dg)
    fill = np.frombuffer(np.full(2, 0x7B, dtype=np.uint8).tobytes(), dtype=np.uint16)[0]
    assert np.all(plain[3] == fill)
    x = plain.copy()
    x[3] = fill
    want = orc.sigmoid_gate(x.reshape(-1, t.D), np.ascontiguousarray(gate[:, :, :t.D]).reshape(-1, t.D), t.io).reshape(t.B, t.QH, t.D)
    assert np.array_equal(got, want)


def test_groups_that_are_no_tree_are_refused(dev):
    groups, lens = TREE8
    t = Tree((8, 32, 128), cabi.BF16, groups, lens, seed=2)
    lib = cabi.lib()
    mx = int(t.lens.max())
    ws = U.dev_zeros(64 << 20)
    out = U.dev_zeros(t.B * t.QH * t.D * 2)

    def rc(gr, B=t.B):
        arr = cabi.prefix_groups(gr)
        return lib.drk_paged_decode_attention_grouped(C.byref(t.g), U.p(t.dq), U.p(t.dpool), U.p(t.dtab), t.stride, U.p(t.dl),
                                                      B, mx, arr, len(gr), U.p(out), 0, float(t.scale), t.io, None, 0,
                                                      U.p(ws), 64 << 20, U.stream_ptr())

    assert rc([(0, 8, 64, 1024)]) == cabi.ERR_INVALID                       # does not start at token 0
    assert rc([(0, 8, 0, 1024), (0, 4, 1088, 2000)]) == cabi.ERR_INVALID    # a gap
    assert rc([(0, 8, 0, 1024), (0, 4, 512, 2000)]) == cabi.ERR_INVALID     # overlap
    assert rc([(0, 4, 0, 1024), (2, 4, 0, 1024)]) == cabi.ERR_INVALID       # branches 2, 3 in two roots
    assert rc([(0, 9, 0, 1024)]) == cabi.ERR_INVALID                        # more branches than the call has
    assert rc([(0, 8, 0, mx + 64)]) == cabi.ERR_INVALID                     # beyond max_seq_len
    assert rc([(0, 1, 0, 64)] * 17) == cabi.ERR_INVALID                     # more groups than DRK_MAX_PREFIX_GROUPS
    assert rc([(0, 8, 0, 1024)]) == cabi.OK
    U.sync()
    arr = cabi.prefix_groups(groups)
    assert lib.drk_decode_grouped_workspace_bytes(C.byref(t.g), t.B, mx, arr, len(groups)) > 4096
    r = lib.drk_paged_decode_attention_grouped(C.byref(t.g), U.p(t.dq), U.p(t.dpool), U.p(t.dtab), t.stride, U.p(t.dl), t.B, mx,
                                               arr, len(groups), U.p(out), 0, float(t.scale), t.io, None, 0, U.p(ws), 4096,
                                               U.stream_ptr())
    assert r == cabi.ERR_WORKSPACE


def test_more_rows_than_one_group_takes_is_refused(dev):
    t = Tree((2, 32, 128), cabi.BF16, [(0, 5, 0, 128)], [130] * 5, seed=1)      # 5 branches x 16 heads per kv head = 80 rows
    lib = cabi.lib()
    ws, out = U.dev_zeros(8 << 20), U.dev_zeros(t.B * t.QH * t.D * 2)
    arr = cabi.prefix_groups(t.groups)
    r = lib.drk_paged_decode_attention_grouped(C.byref(t.g), U.p(t.dq), U.p(t.dpool), U.p(t.dtab), t.stride, U.p(t.dl), t.B, 130,
                                               arr, 1, U.p(out), 0, float(t.scale), t.io, None, 0, U.p(ws), 8 << 20, U.stream_ptr())
    assert r == cabi.ERR_UNSUPPORTED
    # split in two it runs: the range is then read twice
    t.groups = [(0, 4, 0, 128)]
    ok, ma, _ = U.rel_abs_ok(U.from_bits(t.run_grouped(), t.io), t.want(), REL, ABS)
    assert ok, ma


@pytest.mark.parametrize("dtype", [cabi.BF16, cabi.INT8])
@pytest.mark.parametrize("tree,heads", [(TREE8, (8, 32, 128)), (ONE, (8, 32, 128)), (SPREAD, (1, 10, 128)), (([], TREE8[1]), (8, 32, 128)),
                                        (([], SPREAD[1]), (4, 24, 256))])
def test_unit_descriptors_built_once_for_the_layers_of_a_step(dev, dtype, tree, heads):
    """drk_decode_plan_build + drk_paged_decode_attention_planned against the unplanned calls: the same bits, with
    and without groups (no groups: the plain tiled kernel, also at head_dim 256), with the plan reused by a second
    call and a gate."""
    if heads[2] == 256:
        dtype = cabi.F16 if dtype == cabi.BF16 else dtype
    t = Tree(heads, dtype, tree[0], tree[1], seed=31, holes=() if tree[0] else ((1, 5),))     # a missing page where nothing is shared
    lib = cabi.lib()
    arr = cabi.prefix_groups(t.groups)
    n_groups = len(t.groups)
    mx = int(t.lens.max())
    pb = lib.drk_decode_plan_bytes(C.byref(t.g), t.B, mx, n_groups)
    assert pb > 0
    plan = U.dev_bytes(np.full(pb, 0xEE, dtype=np.uint8))
    cabi.call("drk_decode_plan_build", C.byref(t.g), U.p(t.dtab), t.stride, U.p(t.dl), t.B, mx, arr, n_groups, U.p(plan), pb,
              U.stream_ptr())
    wsb = lib.drk_decode_grouped_workspace_bytes(C.byref(t.g), t.B, mx, arr, n_groups)
    rng = np.random.default_rng(5)
    gate = U.normal_bits(rng, (t.B, t.QH, 2 * t.D), t.io)
    dgate = U.dev_bytes(gate)
    for use_gate in ((False, True, False) if t.D == 128 else (False, False)):
        ws = U.dev_bytes(np.full(wsb, 0xFF, dtype=np.uint8))
        outs = []
        for planned in (True, False):
            out = U.dev_bytes(np.full(t.B * t.QH * t.D * 2, 0x7B, dtype=np.uint8))
            tail = (U.p(out), 0, float(t.scale), t.io, U.p(dgate) if use_gate else None, 2 * t.D if use_gate else 0, U.p(ws), wsb,
                    U.stream_ptr())
            if planned:
                cabi.call("drk_paged_decode_attention_planned", C.byref(t.g), U.p(t.dq), U.p(t.dpool), U.p(t.dtab), t.stride,
                          U.p(t.dl), t.B, mx, arr, n_groups, U.p(plan), *tail)
            elif t.D == 128:
                cabi.call("drk_paged_decode_attention_grouped", C.byref(t.g), U.p(t.dq), U.p(t.dpool), U.p(t.dtab), t.stride,
                          U.p(t.dl), t.B, mx, arr, n_groups, *tail)
            else:                                              # the grouped entry point is for head_dim 128
                cabi.call("drk_paged_decode_attention_branches", C.byref(t.g), U.p(t.dq), U.p(t.dpool), U.p(t.dtab), t.stride,
                          U.p(t.dl), t.B, mx, U.p(out), 0, float(t.scale), t.io, 0, U.p(ws), wsb, U.stream_ptr())
            U.sync()
            outs.append(U.host(out, np.uint16, (t.B, t.QH, t.D)))
        assert np.array_equal(outs[0], outs[1]), "the planned call differs from the unplanned one"
    got = U.from_bits(outs[0], t.io)
    ok, ma, _ = U.rel_abs_ok(got, t.want())
    assert ok, ma


def test_plan_argument_errors(dev):
    g = cabi.layout(1, 8, 32, 128, 16, 64, cabi.BF16)
    lib = cabi.lib()
    assert lib.drk_decode_plan_bytes(C.byref(g), 65, 1000, 0) == 0                 # more than 64 branches
    g64 = cabi.layout(1, 4, 16, 64, 16, 64, cabi.F16)                              # a geometry of the portable kernel
    assert lib.drk_decode_plan_bytes(C.byref(g64), 4, 1000, 0) == 0
    x = U.dev_zeros(1 << 16)
    rc = lib.drk_decode_plan_build(C.byref(g), U.p(x), 8, U.p(x), 4, 1000, None, 0, U.p(x), 64, U.stream_ptr())
    assert rc == cabi.ERR_WORKSPACE
    rc = lib.drk_decode_plan_build(C.byref(g64), U.p(x), 8, U.p(x), 4, 1000, None, 0, U.p(x), 1 << 16, U.stream_ptr())
    assert rc == cabi.ERR_UNSUPPORTED


@pytest.mark.parametrize("dtype,heads,tree", [(cabi.BF16, (8, 32, 128), ([], TREE8[1])), (cabi.F16, (4, 24, 256), ([], SPREAD[1])),
                                              (cabi.INT8, (8, 32, 128), ([], TREE8[1])), (cabi.BF16, (8, 32, 128), TREE8_OWN_LAST),
                                              (cabi.F16, (8, 32, 128), SPREAD), (cabi.FP8_E4M3, (8, 32, 128), TREE8_OWN_LAST),
                                              (cabi.F16, (2, 16, 128), ([], [1, 64, 65, 128, 1000]))])
def test_append_and_attention_of_a_layer_in_one_call(dev, dtype, heads, tree):
    """drk_kv_append_decode_planned against drk_kv_append_branches + drk_paged_decode_attention_planned: the same bytes
    in the pool and the same output bits -- in one launch for 16-bit pages (the workgroup that owns a branch's last
    tile writes the new rows; with fork trees that is a unit of the branch's private tail), in two for 8-bit pages; a
    branch whose last page is missing keeps it missing.  Every branch's new token lies in a page of its own, as
    copy-on-write leaves it: a branch that ends where a shared range ends would write into the other branches'
    context."""
    import torch
    holes = () if tree[0] else ((1, (int(tree[1][1]) - 1) // 16),)
    t = Tree(heads, dtype, tree[0], tree[1], seed=47, holes=holes)
    lib = cabi.lib()
    arr = cabi.prefix_groups(t.groups)
    n_groups = len(t.groups)
    mx = int(t.lens.max())
    KVH = heads[0]
    pb = lib.drk_decode_plan_bytes(C.byref(t.g), t.B, mx, n_groups)
    plan = U.dev_zeros(pb)
    cabi.call("drk_decode_plan_build", C.byref(t.g), U.p(t.dtab), t.stride, U.p(t.dl), t.B, mx, arr, n_groups, U.p(plan), pb,
              U.stream_ptr())
    wsb = lib.drk_decode_grouped_workspace_bytes(C.byref(t.g), t.B, mx, arr, n_groups)
    rng = np.random.default_rng(9)
    nk, nv = U.normal_bits(rng, (t.B, KVH, t.D), t.io, 0.7), U.normal_bits(rng, (t.B, KVH, t.D), t.io, 0.7)
    dnk, dnv = U.dev_bytes(nk), U.dev_bytes(nv)
    dpos = U.dev_i32(t.lens - 1)
    results = []
    for fused in (False, True):
        pool = U.dev_bytes(t.opool)
        ws = U.dev_bytes(np.full(wsb, 0xFF, dtype=np.uint8))
        out = U.dev_bytes(np.full(t.B * t.QH * t.D * 2, 0x7B, dtype=np.uint8))
        if fused:
            cabi.call("drk_kv_append_decode_planned", C.byref(t.g), U.p(pool), U.p(t.dtab), t.stride, U.p(t.dl), t.B, mx, arr,
                      n_groups, U.p(plan), U.p(dnk), U.p(dnv), t.io, U.p(t.dq), U.p(out), 0, float(t.scale), t.io, None, 0,
                      U.p(ws), wsb, U.stream_ptr())
        else:
            cabi.call("drk_kv_append_branches", C.byref(t.g), U.p(pool), U.p(t.dtab), t.stride, U.p(dpos), t.B, 0, 1, U.p(dnk),
                      U.p(dnv), t.io, U.stream_ptr())
            cabi.call("drk_paged_decode_attention_planned", C.byref(t.g), U.p(t.dq), U.p(pool), U.p(t.dtab), t.stride, U.p(t.dl),
                      t.B, mx, arr, n_groups, U.p(plan), U.p(out), 0, float(t.scale), t.io, None, 0, U.p(ws), wsb, U.stream_ptr())
        U.sync()
        results.append((U.host(out, np.uint16, (t.B, t.QH, t.D)).copy(), U.host(pool, np.uint8).copy()))
    assert np.array_equal(results[0][1], results[1][1]), "the pools differ"
    assert not np.array_equal(results[0][1], t.opool), "nothing was appended"
    assert np.array_equal(results[0][0], results[1][0]), "the outputs differ"
