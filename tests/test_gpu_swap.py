"""GPU: the overflow tier -- one block, all layers, between the pool and a host image / a
.kv file (KVSwapper, src/memoria/kv_swapper.cpp:154-300) and the CacheManager paths that use it
(src/memoria/cache_manager.cpp:118-156, 207-292).  Byte work: everything is bit-exact."""
import ctypes as C
import os

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


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.BF16, cabi.INT8, cabi.FP8_E4M3])
def test_block_image_round_trip_through_pinned_memory(dev, dtype):
    L, KVH, QH, D, bs, NB = 5, 4, 16, 128, 16, 9
    g, og = U.both_layouts(L, KVH, QH, D, bs, NB, dtype)
    rng = np.random.default_rng(110)
    pool = rng.integers(0, 256, size=orc.pool_bytes(og)).astype(np.uint8)
    dpool = U.dev_bytes(pool)
    n = cabi.lib().drk_kv_block_total_bytes(C.byref(g))
    assert n == L * cabi.lib().drk_kv_block_stride_bytes(C.byref(g))
    hp = C.c_void_p()
    cabi.call("drk_host_malloc", C.byref(hp), n)
    try:
        img = np.ctypeslib.as_array(C.cast(hp, C.POINTER(C.c_uint8)), shape=(n,))
        cabi.call("drk_kv_block_to_host", C.byref(g), U.p(dpool), 6, hp, U.stream_ptr())
        U.sync()
        assert np.array_equal(img, orc.block_image(og, pool, 6))
        cabi.call("drk_kv_block_from_host", C.byref(g), U.p(dpool), 2, hp, U.stream_ptr())
        U.sync()
        want = pool.copy()
        orc.block_from_image(og, want, 2, orc.block_image(og, pool, 6))
        assert np.array_equal(U.host(dpool, np.uint8), want)
        with pytest.raises(cabi.DrkError):
            cabi.call("drk_kv_block_to_host", C.byref(g), U.p(dpool), NB, hp, U.stream_ptr())
    finally:
        cabi.call("drk_host_free", hp)


@pytest.mark.parametrize("dtype", [cabi.F16, cabi.INT8])
def test_swapper_file_image_swap_in_and_prefetch(dev, dtype, tmp_path):
    L, KVH, QH, D, bs = 3, 4, 16, 128, 16
    assert host.set_attention_geometry(L, QH, KVH, D, dtype)
    cm, sw = host.CacheManager(), host.KVSwapper()
    og1 = orc.layout(L, KVH, QH, D, bs, 1, dtype)
    block_bytes = L * orc.lib().orc_block_stride_bytes(C.byref(og1))
    assert cm.init_ssd(8 * block_bytes, tmp_path / "kv", bs, sw)
    assert sw.init(cm, tmp_path / "kv", 2) and sw.block_bytes() == block_bytes
    try:
        NB = cm.pool_max_blocks()
        og = orc.layout(L, KVH, QH, D, bs, NB, dtype)
        rng = np.random.default_rng(111)
        pool = rng.integers(0, 256, size=cm.pool_total_bytes()).astype(np.uint8)
        cabi.call("drk_memcpy_h2d_async", C.c_void_p(cm.pool_ptr()), pool.ctypes.data_as(C.c_void_p), pool.size, U.stream_ptr())
        U.sync()
        path = tmp_path / "kv" / "block_5.kv"
        assert sw.swap_out(5, 3, path) and sw.pending() == 0
        img = orc.block_image(og, pool, 3)
        assert np.array_equal(np.fromfile(path, dtype=np.uint8), img)          # the reference's .kv layout
        assert sw.swap_in(5, 6, path)
        want = pool.copy()
        orc.block_from_image(og, want, 6, img)
        assert np.array_equal(d2h(cm.pool_ptr(), pool.size), want)
        # prefetch: file -> host cache; the swap-in that follows does not need the file any more
        sw.prefetch(5, path)
        sw.drain()
        assert sw.is_prefetched(5)
        os.unlink(path)
        assert sw.swap_in(5, 1, path) and not sw.is_prefetched(5)
        orc.block_from_image(og, want, 1, img)
        assert np.array_equal(d2h(cm.pool_ptr(), pool.size), want)
        assert not sw.swap_in(5, 1, path)                                          # cache used up, file gone: reported
    finally:
        sw.shutdown()


def test_swapper_calls_back_in_submission_order_and_refuses_work_after_shutdown(dev, tmp_path):
    """Requests that have no device phase (a prefetch) or whose first phase fails (a swap-in of a missing file)
    complete at once -- but not before the copies submitted ahead of them; after shutdown() a request fails
    immediately and leaves nothing pending."""
    L, KVH, QH, D, bs = 3, 4, 16, 128, 16
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.F16)
    cm, sw = host.CacheManager(), host.KVSwapper()
    og1 = orc.layout(L, KVH, QH, D, bs, 1, cabi.F16)
    block_bytes = L * orc.lib().orc_block_stride_bytes(C.byref(og1))
    assert cm.init_ssd(8 * block_bytes, tmp_path / "kv", bs, sw)
    assert sw.init(cm, tmp_path / "kv", 3)
    try:
        d = tmp_path / "kv"
        assert sw.swap_out(9, 0, d / "seed.kv")
        reqs = [(0, 0, 0, d / "a.kv"), (0, 1, 1, d / "b.kv"), (1, 7, 2, d / "missing.kv"), (0, 2, 3, d / "c.kv"),
                (1, 9, -1, d / "seed.kv"), (0, 3, 4, d / "d.kv"), (1, 8, -1, d / "missing2.kv")]
        order, ok = sw.swap_many(reqs)
        assert order == list(range(len(reqs)))
        assert ok == [True, True, False, True, True, True, False]
        assert sw.pending() == 0
        sw.remove_writer_stream(U.stream_ptr())
        assert sw.swap_out(4, 5, d / "e.kv")
    finally:
        sw.shutdown()
    assert not sw.swap_out(5, 5, tmp_path / "kv" / "late.kv") and sw.pending() == 0


def test_cache_manager_spills_to_the_overflow_tier_and_brings_blocks_back(dev, tmp_path):
    """A sequence twice the size of the pool: the oldest blocks go to <dir>/block_<i>.kv
    (cache_manager.cpp:132-141, 207-243), come back on demand into other physical blocks
    (245-292), and every token reads back bit for bit."""
    L, KVH, QH, D, bs = 2, 4, 16, 128, 16
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    cm, sw = host.CacheManager(), host.KVSwapper()
    block_bytes = L * 2 * KVH * bs * D * 2
    NBLK = 6
    assert cm.init_ssd(NBLK * block_bytes, tmp_path / "spill", bs, sw)
    assert sw.init(cm, tmp_path / "spill")
    L_ = host.lib()
    try:
        NB = cm.pool_max_blocks()
        assert NB == NBLK
        T = 2 * NBLK * bs
        rng = np.random.default_rng(112)
        k = U.normal_bits(rng, (L, T, KVH, D), cabi.BF16)
        v = U.normal_bits(rng, (L, T, KVH, D), cabi.BF16)
        keep = []
        for blk in range(T // bs):                                   # append block by block, as a prefill in chunks would
            assert cm.ensure_blocks_for_range(0, blk * bs, bs)
            cm.sync_block_table(U.stream_ptr())
            for l in range(L):
                dk, dv = U.dev_bytes(k[l, blk * bs:(blk + 1) * bs]), U.dev_bytes(v[l, blk * bs:(blk + 1) * bs])
                keep += [dk, dv]
                L_.drkh_paged_kv_cache_write_batch(U.p(dk), U.p(dv), cm.pool_ptr(), cm.d_block_table(0), l, blk * bs, bs, NB, bs,
                                                   U.stream_ptr())
        cm.set_seq_len(0, T)
        assert cm.ssd_blocks_used() == NBLK and cm.gpu_blocks_used() == NBLK and cm.free_blocks() == 0
        assert [cm.block_location(0, i) for i in range(2 * NBLK)] == [host.CacheManager.SSD] * NBLK + [host.CacheManager.GPU] * NBLK
        assert sorted(os.listdir(tmp_path / "spill")) == sorted("block_%d.kv" % i for i in range(NBLK))
        table = cm.h_block_table(0)
        assert (table[:NBLK] == -1).all() and sorted(table[NBLK:2 * NBLK].tolist()) == list(range(NBLK))

        def resident_tokens_match():
            cm.sync_block_table(U.stream_ptr())
            flat = U.dev_zeros(L * 2 * T * KVH * D * 2)
            L_.drkh_invoke_extract_kv_from_pages(U.p(flat), cm.pool_ptr(), cm.d_block_table(0), 0, T, L, KVH, D, bs, NB, U.stream_ptr())
            U.sync()
            got = U.host(flat, np.uint16, (L, 2, T, KVH, D))
            tab = cm.h_block_table(0)
            n = 0
            for blk in range(T // bs):
                sl = slice(blk * bs, (blk + 1) * bs)
                if tab[blk] >= 0:
                    assert np.array_equal(got[:, 0, sl], k[:, sl]) and np.array_equal(got[:, 1, sl], v[:, sl]), blk
                    n += 1
                else:
                    assert not got[:, :, sl].any()                       # a swapped-out block gathers as zeros
            return n

        assert resident_tokens_match() == NBLK
        # bring the first three back (with a prefetch for one of them); three resident ones make room
        cm.prefetch_block(0, 1)
        sw.drain()
        assert sw.is_prefetched(1)
        for blk in (0, 1, 2):
            assert cm.ensure_blocks_for(0, blk * bs)
        assert [cm.block_location(0, i) for i in (0, 1, 2)] == [host.CacheManager.GPU] * 3
        assert cm.ssd_blocks_used() == NBLK and not sw.is_prefetched(1)
        assert [cm.block_location(0, i) for i in (NBLK, NBLK + 1, NBLK + 2)] == [host.CacheManager.SSD] * 3   # oldest resident went out
        assert resident_tokens_match() == NBLK
        # and the rest, one after the other: every block survives any number of trips
        for blk in range(2 * NBLK):
            assert cm.ensure_blocks_for(0, blk * bs)
            cm.sync_block_table(U.stream_ptr())
        assert resident_tokens_match() == NBLK
    finally:
        sw.shutdown()


def test_without_a_swapper_eviction_discards(dev, tmp_path):
    """cache_manager.cpp:143-147: no swapper, or a swapper that was never initialised."""
    L, KVH, QH, D, bs = 1, 4, 16, 128, 16
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.F16)
    cm, sw = host.CacheManager(), host.KVSwapper()
    assert cm.init_ssd(4 * L * 2 * KVH * bs * D * 2, tmp_path / "x", bs, sw)       # swapper not initialised
    for blk in range(6):
        assert cm.ensure_blocks_for(0, blk * bs)
    assert cm.ssd_blocks_used() == 0
    assert [cm.block_location(0, i) for i in range(6)] == [host.CacheManager.INVALID] * 2 + [host.CacheManager.GPU] * 4


def test_batch_eviction_pipelines_behind_the_writers_stream(dev, tmp_path):
    """ensure_free_blocks() under the overflow tier: every victim's swap-out is queued at once and the
    swapper overlaps one block's copy with its neighbour's file write.  The blocks are written by a
    kernel on a stream of its own right before the request, with no wait in between: the copies order
    themselves behind that stream (it was announced by sync_block_table) instead of stalling the device.
    Every file holds its block's image; every block comes back bit for bit."""
    import torch
    L, KVH, QH, D, bs = 4, 8, 32, 128, 16
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    cm, sw = host.CacheManager(), host.KVSwapper()
    block_bytes = L * 2 * KVH * bs * D * 2
    NBLK = 24
    assert cm.init_ssd(NBLK * block_bytes, tmp_path / "batch", bs, sw)
    assert sw.init(cm, tmp_path / "batch", 3)
    L_ = host.lib()
    side = torch.cuda.Stream()
    sp = C.c_void_p(side.cuda_stream)
    try:
        NB = cm.pool_max_blocks()
        og = orc.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
        T = NBLK * bs
        rng = np.random.default_rng(113)
        k = U.normal_bits(rng, (L, T, KVH, D), cabi.BF16)
        v = U.normal_bits(rng, (L, T, KVH, D), cabi.BF16)
        dk, dv = [U.dev_bytes(k[l]) for l in range(L)], [U.dev_bytes(v[l]) for l in range(L)]
        torch.cuda.synchronize()
        assert cm.ensure_blocks_for_range(0, 0, T)
        cm.sync_block_table(sp)
        table = cm.h_block_table(0).copy()
        for l in range(L):
            L_.drkh_paged_kv_cache_write_batch(U.p(dk[l]), U.p(dv[l]), cm.pool_ptr(), cm.d_block_table(0), l, 0, T, NB, bs, sp)
        cm.set_seq_len(0, T)
        assert cm.ensure_free_blocks(NBLK)                               # all 24 go out in one batch, no sync before
        assert cm.ssd_blocks_used() == NBLK and cm.free_blocks() == NBLK and sw.pending() == 0
        opool = orc.new_pool(og)
        for l in range(L):
            orc.append_batch(og, opool, table, l, 0, k[l], v[l], cabi.BF16)
        for blk in range(NBLK):
            img = np.fromfile(tmp_path / "batch" / ("block_%d.kv" % blk), dtype=np.uint8)
            assert np.array_equal(img, orc.block_image(og, opool, int(table[blk]))), blk
        # ... and back, into whatever blocks are free
        for blk in range(NBLK):
            assert cm.ensure_blocks_for(0, blk * bs)
        cm.sync_block_table(sp)
        flat = U.dev_zeros(L * 2 * T * KVH * D * 2)
        L_.drkh_invoke_extract_kv_from_pages(U.p(flat), cm.pool_ptr(), cm.d_block_table(0), 0, T, L, KVH, D, bs, NB, sp)
        side.synchronize()
        got = U.host(flat, np.uint16, (L, 2, T, KVH, D))
        assert np.array_equal(got[:, 0], k) and np.array_equal(got[:, 1], v)
    finally:
        sw.shutdown()
