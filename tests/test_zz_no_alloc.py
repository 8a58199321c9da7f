"""GPU parity of drk_paged_decode_attention_branches_static, the decode entry point that
allocates nothing and takes no workspace (its split-K partials live in a file-scope
device array), against drk_paged_decode_attention_branches with a caller workspace:
same kernels, same split, so the two must agree bit for bit -- on two calls in a row,
the second with a smaller input, so that whatever the first call left in the array is
seen not to matter.  Both are also held to the fp64 oracle at the attention tolerance."""
import ctypes as C

import numpy as np
import pytest

from deusridet_amd import cabi
from tests import util as U
from tests.test_gpu_decode import ABS, REL, Case

pytestmark = pytest.mark.gpu


def _static(case, fill=0x7B):
    B = len(case.seq_lens)
    QH, D = case.geom[2], case.geom[3]
    out = U.dev_bytes(np.full(B * QH * D * 2, fill, dtype=np.uint8))
    cabi.call("drk_paged_decode_attention_branches_static", C.byref(case.g), U.p(case.dq), U.p(case.dpool),
              U.p(case.dtab), case.stride, U.p(case.dlens), B, int(case.seq_lens.max()), U.p(out), case.layer,
              float(case.scale), case.io, U.stream_ptr())
    U.sync()
    return U.host(out, np.uint16, (B, QH, D))


@pytest.mark.parametrize("dtype", [cabi.BF16, cabi.INT8])
def test_static_scratch_decode_two_calls(dev, dtype):
    geom = (2, 8, 32, 128, 16, 1400)
    big = Case(geom, dtype, [4096, 1000, 2500, 3333, 17, 4000], seed=71)
    small = Case(geom, dtype, [300, 64, 1], seed=72)
    for case in (big, small, big):                      # larger, smaller, larger again: one scratch array
        got = _static(case)
        want = case.run_branches()
        assert np.array_equal(got, want), "static-scratch call differs from the workspace call"
        ok, max_abs, max_rel = U.rel_abs_ok(U.from_bits(got, case.io), case.want_f64(), REL, ABS)
        assert ok, f"max abs err {max_abs:.4g}, max rel err {max_rel:.4g}"


def test_static_scratch_rejects_what_does_not_fit(dev):
    """Sizes whose partials exceed the static array are refused before anything is launched."""
    g = cabi.layout(1, 8, 32, 128, 16, 64, cabi.BF16)
    B, mx = 64, 32768
    assert cabi.lib().drk_decode_workspace_bytes(C.byref(g), B, mx) > cabi.STATIC_SCRATCH_BYTES
    buf = U.dev_zeros(B * 32 * 128 * 2)
    lens = U.dev_i32(np.full(B, 16, dtype=np.int32))
    tab = U.dev_i32(np.zeros((B, 4), dtype=np.int32))
    pool = U.dev_zeros(cabi.lib().drk_kv_pool_bytes(C.byref(g)))
    rc = cabi.lib().drk_paged_decode_attention_branches_static(C.byref(g), U.p(buf), U.p(pool), U.p(tab), 4, U.p(lens),
                                                               B, mx, U.p(buf), 0, 0.1, cabi.BF16, U.stream_ptr())
    assert rc == cabi.ERR_WORKSPACE
    assert b"static scratch" in cabi.lib().drk_last_error()


def test_static_scratch_decode_under_graph_capture(dev):
    """What the entry point is for: a caller that may not allocate.  One warm call outside any capture (it looks
    the scratch array's address up), then the call is recorded into a graph and replayed: every replay equals the
    workspace call, with other launches that use the scratch array in between."""
    import torch
    geom = (2, 8, 32, 128, 16, 900)
    case = Case(geom, cabi.BF16, [2000, 777, 64, 1301], seed=73)
    other = Case(geom, cabi.BF16, [500, 3000], seed=74)
    want = case.run_branches()
    assert np.array_equal(_static(case), want)                 # the warm call
    B = len(case.seq_lens)
    QH, D = case.geom[2], case.geom[3]
    out = U.dev_bytes(np.full(B * QH * D * 2, 0x7B, dtype=np.uint8))
    side = torch.cuda.Stream()
    sp = C.c_void_p(side.cuda_stream)
    cabi.call("drk_graph_begin_capture", sp)
    cabi.call("drk_paged_decode_attention_branches_static", C.byref(case.g), U.p(case.dq), U.p(case.dpool), U.p(case.dtab),
              case.stride, U.p(case.dlens), B, int(case.seq_lens.max()), U.p(out), case.layer, float(case.scale), case.io, sp)
    graph = C.c_void_p()
    cabi.call("drk_graph_end_capture", sp, C.byref(graph))
    try:
        for replay in range(3):
            out.fill_(0x7B)
            torch.cuda.synchronize()
            cabi.call("drk_graph_launch", graph, sp)
            side.synchronize()
            assert np.array_equal(U.host(out, np.uint16, (B, QH, D)), want), f"replay {replay}"
            assert np.array_equal(_static(other), other.run_branches())     # eager work on the same scratch array
    finally:
        cabi.call("drk_graph_destroy", graph)
