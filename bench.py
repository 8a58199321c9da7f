#!/usr/bin/env python3
"""Benchmark of the paged-KV hot path on one MI355X.

Workload (BASELINE config 2): 36 layers, 32 Q / 8 KV heads x 128, bf16 KV in
16-token pages shuffled across a 40 GB pool, 8 decode branches at 32k context.
One step = for every layer: append one token per branch, then paged GQA decode
attention over all branches.  Prints ONE JSON line.

Torch is used for device memory, streams and events only; every kernel is
reached through the C ABI in include/drk_kv.h.
"""
import argparse
import ctypes as C
import gc
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the decode kernel come from the counter runs recorded in this
# profile summary (two `rocprofv3 --pmc` runs of this script: FETCH_SIZE, then WRITE_SIZE).
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "decode_stream_bf16_config2_8x32k.md")


def measured_traffic(launch_bytes):
    """(bytes per launch, source) from the profile summary, when it was taken on a launch of
    exactly these algorithmic bytes; (None, reason) otherwise.  The summary carries two lines,
    `algorithmic_bytes_per_launch: N` and `traffic_bytes_per_launch: N`."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, "no profile summary"
    alg = re.search(r"^algorithmic_bytes_per_launch:\s*(\d+)", text, re.M)
    tr = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", text, re.M)
    if not alg or not tr:
        return None, "profile summary carries no traffic figure"
    if int(alg.group(1)) != launch_bytes:
        return None, "profile summary was taken on another launch size"
    return int(tr.group(1)), os.path.relpath(TRAFFIC_PROFILE, ROOT)


def bf16_bits(rng, shape, mul):
    """N(0,1) * mul as bf16 bit patterns (round to nearest even), for the CPU sample."""
    u = (rng.standard_normal(shape).astype(np.float32) * np.float32(mul)).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--layers", type=int, default=36)
    ap.add_argument("--branches", type=int, default=8)
    ap.add_argument("--ctx", type=int, default=32768, help="context length of every branch at the last timed step")
    ap.add_argument("--ctx-mode", choices=["fixed", "uniform"], default="fixed",
                    help="fixed: every branch at --ctx (the 70%% target point); uniform: U{1024..ctx}")
    ap.add_argument("--pool-gb", type=float, default=40.0)
    ap.add_argument("--split", type=int, default=0, help="tokens per split-K workgroup (0 = library default)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the kernel measurements of configs 3, 4 and 5 that the default line carries")
    ap.add_argument("--no-ragged", action="store_true", help="skip the side measurements that launch the headline kernel on other shapes (profiling: one shape per kernel name)")
    ap.add_argument("--cpu-sample-tokens", type=int, default=0, help="context per branch for the CPU sample (0 = auto)")
    ap.add_argument("--bulk-append-tokens", type=int, default=2048)
    ap.add_argument("--seed", type=int, default=2)
    ap.add_argument("--config", type=int, default=2, choices=[2, 3, 4, 5, 6, 7],
                    help="BASELINE config: 2 (default, the headline) | 3 shared prefix + COW + eviction | "
                         "4 int8/fp8 pages at 128k | 5 chunked MFMA prefill interleaved with decode | "
                         "6 config 3's shape through the stream driver (whole layer path, captured step) | "
                         "7 config 2's workload at the reference's own model shape (24 Q / 4 KV x 256, block 256)")
    ap.add_argument("--kv-dtype", choices=["bf16", "int8", "fp8"], default=None,
                    help="storage type of the pages: config 4 int8 (default) | fp8; config 5 bf16 (default) | int8 | fp8")
    ap.add_argument("--no-graph", action="store_true", help="launch every kernel of a step from the host instead of "
                                                            "replaying one captured HIP graph per step")
    ap.add_argument("--no-fused-append", action="store_true", help="launch the one-token append of every layer by itself instead of "
                                                                   "letting the attention launch write the new rows")
    ap.add_argument("--no-plan", action="store_true", help="build the decode kernel's unit descriptors in every layer's launch "
                                                           "instead of once per step (drk_decode_plan_build)")
    ap.add_argument("--no-cascade", action="store_true", help="config 3: read the shared prefix once per branch")
    ap.add_argument("--forks", choices=["tree", "prefix"], default="tree",
                    help="config 3: branches fork from the prefix or from one another at random block boundaries (tree), "
                         "or all from the prefix's end (prefix)")
    ap.add_argument("--shared-kernel", choices=["auto", "pair"], default="auto",
                    help="config 3: how shared pages are read: auto = one launch over shared and private tiles where the "
                         "geometry allows; pair = always the prefix pass followed by the tail kernel")
    ap.add_argument("--d256-waves", type=int, choices=[0, 1], default=None,
                    help="head_dim 256 chunk kernel: 0 = four waves that do both products, 1 = score waves and value waves "
                         "(default: the library's choice)")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (nothing here shards across GPUs)", file=sys.stderr)
        sys.exit(2)
    import torch
    from deusridet_amd import cabi

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    # The interpreter's cycle collector stays off while anything is timed: a full collection over torch's and numpy's
    # objects takes tens of milliseconds, and the workloads that launch every kernel from Python (config 3: some 110
    # calls a step) reach its threshold in the middle of their timed steps.
    gc.collect()
    gc.disable()
    cabi.lib().drk_debug_set_grouped_decode(1 if args.shared_kernel == "pair" else 0)
    if args.d256_waves is not None:
        cabi.lib().drk_debug_set_prefill_d256_waves(args.d256_waves)
    if args.config != 2:
        import bench_extra
        print(json.dumps(bench_extra.run(args)))
        return
    lib = cabi.lib()
    torch.cuda.set_device(0)
    rng = np.random.default_rng(args.seed)

    L, KVH, QH, D, bs = args.layers, 8, 32, 128, 16
    B, W, K = args.branches, args.warmup, args.steps
    probe = cabi.layout(L, KVH, QH, D, bs, 1, cabi.BF16)
    NB = lib.drk_kv_max_blocks_for_budget(C.byref(probe), int(args.pool_gb * 1e9))
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    pool_bytes = lib.drk_kv_pool_bytes(C.byref(g))

    # context lengths at the START of the run; every step appends one token
    if args.ctx_mode == "fixed":
        final = np.full(B, args.ctx, dtype=np.int64)
    else:
        final = rng.integers(1024, args.ctx + 1, size=B)
    start = np.maximum(final - (W + K), 1).astype(np.int32)
    nblk = [(int(s) + W + K + bs - 1) // bs for s in start]
    assert sum(nblk) <= NB, f"pool of {NB} blocks too small for {sum(nblk)}"
    stride = max(nblk) + 1
    perm = rng.permutation(NB).astype(np.int32)           # physical blocks shuffled over the whole pool
    tables = np.full((B, stride), -1, dtype=np.int32)
    o = 0
    for b in range(B):
        tables[b, :nblk[b]] = perm[o:o + nblk[b]]
        o += nblk[b]

    stream = torch.cuda.current_stream()
    sp = C.c_void_p(stream.cuda_stream)
    pool = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
    pool.zero_()
    dtab = torch.from_numpy(tables).cuda()

    # fill the pages through the append path itself, N(0,1)*0.5 -> bf16
    chunk = 2048
    t_fill = time.time()
    for b in range(B):
        n = int(start[b])
        for p0 in range(0, n, chunk):
            m = min(chunk, n - p0)
            k = (torch.randn(L, m, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
            v = (torch.randn(L, m, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
            cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(pool), C.c_void_p(dtab[b].data_ptr()), 0, L, p0, m,
                      cabi.p(k), cabi.p(v), cabi.BF16, sp)
            del k, v
    torch.cuda.synchronize()
    t_fill = time.time() - t_fill

    scale = 1.0 / np.sqrt(D)
    q = (torch.randn(L, B, QH, D, device="cuda") * 0.5).to(torch.bfloat16)
    newk = (torch.randn(L, B, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
    newv = (torch.randn(L, B, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
    out = torch.zeros(L, B, QH, D, device="cuda", dtype=torch.bfloat16)
    max_ctx = int(final.max())
    split = args.split          # 0: the library's own choice (persistent workgroups, equal tiles each)
    wsb = (lib.drk_decode_workspace_bytes_for_split(C.byref(g), B, max_ctx, split) if split
           else lib.drk_decode_workspace_bytes(C.byref(g), B, max_ctx))
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    # device arrays of positions / lengths for every step, prepared up front so the
    # timed loop does no host->device traffic
    pos_steps = torch.from_numpy(np.stack([start + s for s in range(W + K)]).astype(np.int32)).cuda()
    len_steps = pos_steps + 1                                 # write-then-attend: the new token is visible
    qrow, krow = B * QH * D * 2, B * KVH * D * 2
    # The layers of a step read the same tables and lengths: the decode kernel's unit descriptors are built once per
    # step (one small launch) and read by the 36 attention launches.
    plan_bytes = 0 if (split or args.no_plan) else lib.drk_decode_plan_bytes(C.byref(g), B, max_ctx, 0)
    plan = torch.empty(max(plan_bytes, 16), dtype=torch.uint8, device="cuda")

    def build_plan(dlen, spx):
        if plan_bytes:
            cabi.call("drk_decode_plan_build", C.byref(g), cabi.p(dtab), stride, dlen, B, max_ctx, None, 0, cabi.p(plan), plan_bytes, spx)

    def attend(l, dlen, spx):
        if plan_bytes:
            cabi.call("drk_paged_decode_attention_planned", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow), cabi.p(pool),
                      cabi.p(dtab), stride, dlen, B, max_ctx, None, 0, cabi.p(plan), C.c_void_p(out.data_ptr() + l * qrow), l,
                      float(scale), cabi.BF16, None, 0, cabi.p(ws), wsb, spx)
        else:
            cabi.call("drk_paged_decode_attention_branches", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow),
                      cabi.p(pool), cabi.p(dtab), stride, dlen, B, max_ctx, C.c_void_p(out.data_ptr() + l * qrow), l,
                      float(scale), cabi.BF16, split, cabi.p(ws), wsb, spx)

    fused_append = bool(plan_bytes) and not args.no_fused_append

    def layer_step(l, dpos, dlen, spx):
        """append one token per branch, then attend: one call (one launch for these bf16 pages) or two"""
        if fused_append:
            cabi.call("drk_kv_append_decode_planned", C.byref(g), cabi.p(pool), cabi.p(dtab), stride, dlen, B, max_ctx, None, 0,
                      cabi.p(plan), C.c_void_p(newk.data_ptr() + l * krow), C.c_void_p(newv.data_ptr() + l * krow), cabi.BF16,
                      C.c_void_p(q.data_ptr() + l * qrow), C.c_void_p(out.data_ptr() + l * qrow), l, float(scale), cabi.BF16,
                      None, 0, cabi.p(ws), wsb, spx)
        else:
            cabi.call("drk_kv_append_branches", C.byref(g), cabi.p(pool), cabi.p(dtab), stride, dpos, B, l, 1,
                      C.c_void_p(newk.data_ptr() + l * krow), C.c_void_p(newv.data_ptr() + l * krow), cabi.BF16, spx)
            attend(l, dlen, spx)

    def step(s):
        dpos = C.c_void_p(pos_steps[s].data_ptr())
        dlen = C.c_void_p(len_steps[s].data_ptr())
        build_plan(dlen, sp)
        for l in range(L):
            layer_step(l, dpos, dlen, sp)

    use_graph = not args.no_graph
    if use_graph:
        # one step captured once: positions / lengths live in device buffers that the
        # graph itself advances, so a replay is the whole step with no host work
        pos_cur, len_cur = pos_steps[0].clone(), len_steps[0].clone()

        def graph_step():
            dpos, dlen = C.c_void_p(pos_cur.data_ptr()), C.c_void_p(len_cur.data_ptr())
            gsp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
            build_plan(dlen, gsp)
            for l in range(L):
                layer_step(l, dpos, dlen, gsp)
            pos_cur.add_(1)
            len_cur.add_(1)

        side = torch.cuda.Stream()
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            graph_step()                                   # step 0, eager, on the capture stream
        stream.wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            graph_step()                                   # step 1 (captured; runs on first replay)
        for s in range(1, W):
            graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for s in range(W, W + K):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
        assert int(pos_cur[0]) == int(start[0]) + W + K, "graph replays did not advance the positions"
    else:
        for s in range(W):
            step(s)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for s in range(W, W + K):
            step(s)
        e1.record(stream)
        torch.cuda.synchronize()
    total_ms = e0.elapsed_time(e1)
    ms_per_step = total_ms / K

    ctx_sum_steps = [int((start + s + 1).sum()) for s in range(W, W + K)]       # tokens attended per layer
    kv_bytes_per_token = 2 * KVH * D * 2                                          # K + V, all kv heads, bf16
    attn_bytes = sum(ctx_sum_steps) * kv_bytes_per_token * L
    value_gbps = attn_bytes / (total_ms * 1e-3) / 1e9

    # ---- dominant kernel alone: the split-K partial kernel of one layer -------
    # timed back to back (queue busy) with one event pair per launch around the
    # partial kernel only; the merge kernel sits between the pairs
    last = W + K - 1
    dlen = C.c_void_p(len_steps[last].data_ptr())
    n_timed = max(2 * L, 40)

    def attn_only(n):
        for it in range(n):
            l = it % L
            cabi.call("drk_paged_decode_attention_branches", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow), cabi.p(pool),
                      cabi.p(dtab), stride, dlen, B, max_ctx, C.c_void_p(out.data_ptr() + l * qrow), l, float(scale),
                      cabi.BF16, split, cabi.p(ws), wsb, sp)

    # (event pairs recorded here, around calls that leave the merge kernel out: cabi.time_partial_kernels)
    planned_for = [None]

    def attn_one(it, lens=dlen):
        if planned_for[0] != lens.value:                     # the timed launches read the plan of their lengths
            build_plan(lens, sp)
            planned_for[0] = lens.value
        attend(it % L, lens, sp)

    ker_avg_ms = cabi.time_partial_kernels(attn_one, n_timed, warm=8)
    launch_bytes = int((start + last + 1).sum()) * kv_bytes_per_token               # one layer, one launch
    achieved = launch_bytes / (ker_avg_ms * 1e-3) / 1e9

    # ---- the same kernel on config 2's context distribution, U{1024..32768} per branch (same pool and
    # tables; only the lengths change), when the headline run is the fixed 32k point
    ragged = None
    if args.ctx_mode == "fixed" and not args.no_ragged:
        rl = np.random.default_rng(args.seed + 1).integers(1024, min(args.ctx, max_ctx) + 1, size=B).astype(np.int32)
        rlen = torch.from_numpy(rl).cuda()

        def ragged_only(n):
            for it in range(n):
                l = it % L
                cabi.call("drk_paged_decode_attention_branches", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow), cabi.p(pool),
                          cabi.p(dtab), stride, cabi.p(rlen), B, max_ctx, C.c_void_p(out.data_ptr() + l * qrow), l, float(scale),
                          cabi.BF16, split, cabi.p(ws), wsb, sp)

        r_ms = cabi.time_partial_kernels(lambda it: attn_one(it, cabi.p(rlen)), n_timed, warm=8)
        r_bytes = int(rl.sum()) * kv_bytes_per_token
        # what a launch pays before its first tile: the same launches with the kernel leaving once the branch
        # lengths are scanned and the workgroup's unit descriptors (one table read per 16-token run) are built
        lib.drk_debug_set_stream_descriptors_only(1)
        ragged_pro_ms = cabi.time_partial_kernels(lambda it: attn_one(it, cabi.p(rlen)), n_timed, warm=8)
        fixed_pro_ms = cabi.time_partial_kernels(attn_one, n_timed, warm=8)
        lib.drk_debug_set_stream_descriptors_only(0)
        planned_for[0] = None
        attn_only(2)                                                 # leave real results behind
        ragged = {"ctx": [int(x) for x in rl], "kernel_us": round(r_ms * 1e3, 2), "bytes_per_launch": r_bytes,
                  "GBps": round(r_bytes / (r_ms * 1e-3) / 1e9, 1), "hbm_frac": round(r_bytes / (r_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                  "prologue_only_us": round(ragged_pro_ms * 1e3, 2),
                  "streaming_GBps": round(r_bytes / ((r_ms - ragged_pro_ms) * 1e-3) / 1e9, 1),
                  "headline_prologue_only_us": round(fixed_pro_ms * 1e3, 2),
                  "headline_streaming_GBps": round(launch_bytes / ((ker_avg_ms - fixed_pro_ms) * 1e-3) / 1e9, 1),
                  "what": "prologue_only = the launch with the kernel leaving after its prologue (launch, scan of the lengths, "
                          "unit descriptors); streaming = bytes over the rest of the launch"}

    # ---- achievable ceiling on this box: plain 128-bit streaming read of the pool
    probe_bytes = min(pool_bytes, 32 << 30)
    sink = torch.zeros(16, dtype=torch.uint8, device="cuda")
    gb = C.c_float(0)
    torch.cuda.synchronize()
    cabi.call("drk_probe_read_bandwidth", cabi.p(pool), probe_bytes, 5, cabi.p(sink), C.byref(gb))
    read_probe_gbps = float(gb.value)
    # ... and the decode kernels' own access pattern: 4 KiB granules in a scattered order
    cabi.call("drk_probe_read_bandwidth_permuted", cabi.p(pool), probe_bytes, 4096, 5, cabi.p(sink), C.byref(gb))
    permuted_probe_gbps = float(gb.value)
    # the dense bf16 rate the matrix cores sustain with no memory traffic at all
    cabi.call("drk_probe_mfma_rate", 20, cabi.p(sink), C.byref(gb))
    mfma_probe_tflops = float(gb.value)
    # ... and how much of a wave's matrix products hides another wave's vector work on the same SIMD
    t_m, t_v, t_b = C.c_float(0), C.c_float(0), C.c_float(0)
    cabi.call("drk_probe_mfma_valu_coexec", 3, cabi.p(sink), C.byref(t_m), C.byref(t_v), C.byref(t_b))
    coexec = {"mfma_waves_ms": round(t_m.value, 3), "vector_waves_ms": round(t_v.value, 3), "both_ms": round(t_b.value, 3),
              "hidden_share_of_mfma_time": round((t_m.value + t_v.value - t_b.value) / t_m.value, 3),
              "what": "one workgroup of 8 waves per CU: waves 4-7 issue 32x32x16 bf16 products, waves 0-3 exp / fma / max3 / pack; "
                      "perfect overlap gives both = max(alone), none gives the sum"}

    # ... and the same for two waves that take turns between barriers (the two-phase prefill kernels), one kind of
    # vector instruction at a time: the share of the vector turns' time that the other wave's products hide
    phase = {}
    for op, name in enumerate(("v_exp_f32", "v_fma_f32", "v_dot2_f32_bf16", "v_cvt_pk_bf16_f32", "v_max3_f32", "v_cmp_gt_f32",
                               "v_permlane32_swap_b32", "s_nop 3")):
        cabi.call("drk_probe_phase_coexec", op, 2, cabi.p(sink), C.byref(t_m), C.byref(t_v), C.byref(t_b))
        phase[name] = round(1.0 - (t_b.value - t_m.value) / t_v.value, 2)
    coexec["hidden_share_by_instruction_in_turns"] = phase

    # ---- bulk append bandwidth (read source + write pages), all layers in one launch
    m = args.bulk_append_tokens
    scratch_tab = torch.from_numpy(perm[o:o + (m + bs - 1) // bs].copy()).cuda() if o + (m + bs - 1) // bs <= NB else None
    append_gbps = None
    if scratch_tab is not None:
        k = (torch.randn(L, m, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
        v = (torch.randn(L, m, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
        for _ in range(3):
            cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(pool), cabi.p(scratch_tab), 0, L, 0, m, cabi.p(k), cabi.p(v),
                      cabi.BF16, sp)
        a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a0.record(stream)
        reps = 10
        for _ in range(reps):
            cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(pool), cabi.p(scratch_tab), 0, L, 0, m, cabi.p(k), cabi.p(v),
                      cabi.BF16, sp)
        a1.record(stream)
        torch.cuda.synchronize()
        ab = 2 * (2 * L * m * KVH * D * 2)                                          # K,V read + written
        append_gbps = ab * reps / (a0.elapsed_time(a1) * 1e-3) / 1e9

    # ---- bulk gather (extract) and scatter (inject) of the same tokens, all layers, read + write
    gather_gbps = scatter_gbps = None
    if scratch_tab is not None:
        flat = torch.empty(L * 2 * m * KVH * D * 2, dtype=torch.uint8, device="cuda")
        for name in ("drk_kv_extract", "drk_kv_inject"):
            def go():
                if name == "drk_kv_extract":
                    cabi.call(name, C.byref(g), cabi.p(flat), None, cabi.p(pool), cabi.p(scratch_tab), 0, m, L, sp)
                else:
                    cabi.call(name, C.byref(g), cabi.p(pool), cabi.p(flat), None, cabi.p(scratch_tab), 0, m, L, sp)
            for _ in range(3):
                go()
            a0.record(stream)
            for _ in range(reps):
                go()
            a1.record(stream)
            torch.cuda.synchronize()
            gbps = 2 * flat.numel() * reps / (a0.elapsed_time(a1) * 1e-3) / 1e9
            if name == "drk_kv_extract":
                gather_gbps = gbps
            else:
                scatter_gbps = gbps

    # ---- the whole attention block of a layer, raw projections in, gated output out:
    # the reference's sequence of separate launches (split, head_norm x2, rope, page write,
    # attention, sigmoid gate: paged_attention.cu:331-370) against the two fused launches
    layer_steps = None
    if use_graph:
        rd, theta, eps = D // 4, 1.0e7, 1e-6
        qg = (torch.randn(L, B, QH, 2 * D, device="cuda") * 0.5).to(torch.bfloat16)
        qw = torch.randn(D, device="cuda").to(torch.bfloat16)
        kw = torch.randn(D, device="cuda").to(torch.bfloat16)
        qsep, gsep = torch.empty_like(q), torch.empty_like(q)
        ktmp = torch.empty_like(newk)
        npos = max_ctx + 1
        rtab = torch.empty(npos * (rd // 2) * 2, dtype=torch.float32, device="cuda")
        cabi.call("drk_rope_table_fill", cabi.p(rtab), npos, rd, theta, sp)
        dpos_l, dlen_l = C.c_void_p(pos_steps[last].data_ptr()), C.c_void_p(len_steps[last].data_ptr())
        qgrow = B * QH * 2 * D * 2
        wsb_g = lib.drk_decode_workspace_bytes(C.byref(g), B, max_ctx)
        ws_g = torch.empty(wsb_g, dtype=torch.uint8, device="cuda")

        def separate(gsp):
            for l in range(L):
                qp, gp, op = (C.c_void_p(t.data_ptr() + l * qrow) for t in (qsep, gsep, out))
                kp = C.c_void_p(ktmp.data_ptr() + l * krow)
                cabi.call("drk_split_q_gate", C.c_void_p(qg.data_ptr() + l * qgrow), qp, gp, B, QH, D, gsp)
                cabi.call("drk_head_norm", qp, cabi.p(qw), qp, B * QH, D, eps, cabi.BF16, gsp)
                cabi.call("drk_head_norm", C.c_void_p(newk.data_ptr() + l * krow), cabi.p(kw), kp, B * KVH, D, eps, cabi.BF16, gsp)
                cabi.call("drk_apply_rope", qp, kp, B, QH, KVH, D, rd, dpos_l, 0, theta, cabi.p(rtab), npos, cabi.BF16, gsp)
                cabi.call("drk_kv_append_branches", C.byref(g), cabi.p(pool), cabi.p(dtab), stride, dpos_l, B, l, 1, kp,
                          C.c_void_p(newv.data_ptr() + l * krow), cabi.BF16, gsp)
                cabi.call("drk_paged_decode_attention_branches", C.byref(g), qp, cabi.p(pool), cabi.p(dtab), stride, dlen_l, B,
                          max_ctx, op, l, float(scale), cabi.BF16, split, cabi.p(ws), wsb, gsp)
                cabi.call("drk_sigmoid_gate", op, gp, op, B * QH, D, D, cabi.BF16, gsp)

        def fused(gsp):
            for l in range(L):
                qp, op = (C.c_void_p(t.data_ptr() + l * qrow) for t in (qsep, out))
                qgp = qg.data_ptr() + l * qgrow
                cabi.call("drk_qk_norm_rope_append", C.byref(g), cabi.p(pool), cabi.p(dtab), stride, dpos_l, 0, B, l,
                          C.c_void_p(qgp), C.c_void_p(newk.data_ptr() + l * krow), C.c_void_p(newv.data_ptr() + l * krow),
                          cabi.p(qw), cabi.p(kw), eps, rd, theta, cabi.p(rtab), npos, qp, cabi.BF16, gsp)
                cabi.call("drk_paged_decode_attention_gated", C.byref(g), qp, cabi.p(pool), cabi.p(dtab), stride, dlen_l, B, max_ctx,
                          op, l, float(scale), cabi.BF16, C.c_void_p(qgp + D * 2), 2 * D, cabi.p(ws_g), wsb_g, gsp)

        res = {}
        for name, fn in (("separate", separate), ("fused", fused)):
            sd = torch.cuda.Stream()
            sd.wait_stream(stream)
            with torch.cuda.stream(sd):
                fn(C.c_void_p(sd.cuda_stream))
            stream.wait_stream(sd)
            torch.cuda.synchronize()
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=sd):
                fn(C.c_void_p(torch.cuda.current_stream().cuda_stream))
            gr.replay()
            torch.cuda.synchronize()
            a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a0.record(stream)
            for _ in range(5):
                gr.replay()
            a1.record(stream)
            torch.cuda.synchronize()
            res[name] = a0.elapsed_time(a1) / 5 * 1e3
            res[name + "_out"] = out.clone()
        layer_steps = {
            "what": "per layer: Q|gate split, head RMSNorm of Q and K, partial RoPE (rotary_dim %d), page write, "
                    "decode attention, sigmoid gate; one captured graph per step" % rd,
            "separate_us_per_step": round(res["separate"], 1), "separate_launches_per_layer": 8,
            "fused_us_per_step": round(res["fused"], 1), "fused_launches_per_layer": 3,
            "same_output_bits": bool(torch.equal(res["separate_out"], res["fused_out"])),
        }

    # ---- decode attention that also reports the attention mass per block (importance scores)
    mass_wsb = lib.drk_decode_mass_workspace_bytes(C.byref(g), B, max_ctx)
    attention_mass = None
    if mass_wsb:
        mws = torch.empty(mass_wsb, dtype=torch.uint8, device="cuda")
        mstride = (max_ctx + bs - 1) // bs
        mass = torch.zeros(B * mstride, dtype=torch.float32, device="cuda")
        tm = {}
        for name in ("plain", "with_mass"):
            def go(n):
                for it in range(n):
                    l = it % L
                    qp, op = C.c_void_p(q.data_ptr() + l * qrow), C.c_void_p(out.data_ptr() + l * qrow)
                    if name == "plain":
                        cabi.call("drk_paged_decode_attention_branches", C.byref(g), qp, cabi.p(pool), cabi.p(dtab), stride, dlen, B,
                                  max_ctx, op, l, float(scale), cabi.BF16, 0, cabi.p(mws), mass_wsb, sp)
                    else:
                        cabi.call("drk_paged_decode_attention_mass", C.byref(g), qp, cabi.p(pool), cabi.p(dtab), stride, dlen, B,
                                  max_ctx, op, l, float(scale), cabi.BF16, cabi.p(mass), mstride, 1 if l else 0, cabi.p(mws),
                                  mass_wsb, sp)
            go(4)
            a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a0.record(stream)
            go(2 * L)
            a1.record(stream)
            torch.cuda.synchronize()
            tm[name] = a0.elapsed_time(a1) / (2 * L) * 1e3
        attention_mass = {"plain_us_per_layer": round(tm["plain"], 2), "with_mass_us_per_layer": round(tm["with_mass"], 2),
                          "mass_sum_branch0": round(float(mass[:mstride].sum()), 2), "expected_sum": L * QH}

    # ---- overflow tier: one block (all layers) per strided 2-D copy to / from pinned host memory
    overflow = None
    blk_bytes = lib.drk_kv_block_total_bytes(C.byref(g))
    hp = C.c_void_p()
    nswap = 64
    if cabi.lib().drk_host_malloc(C.byref(hp), blk_bytes * 4) == 0:
        res = {}
        for name in ("drk_kv_block_to_host", "drk_kv_block_from_host"):
            def go(n):
                for i in range(n):
                    cabi.call(name, C.byref(g), cabi.p(pool), int(perm[i % NB]), C.c_void_p(hp.value + (i % 4) * blk_bytes), sp)
            go(4)
            torch.cuda.synchronize()
            t0 = time.time()
            go(nswap)
            torch.cuda.synchronize()
            res[name] = blk_bytes * nswap / (time.time() - t0) / 1e9
        cabi.call("drk_host_free", hp)
        overflow = {"block_MiB": round(blk_bytes / 2**20, 2), "to_host_GBps": round(res["drk_kv_block_to_host"], 1),
                    "from_host_GBps": round(res["drk_kv_block_from_host"], 1),
                    "what": "%d blocks of %d layers each way, one strided copy per block, pinned host memory" % (nswap, L)}

    # ---- CPU baseline: the oracle's restatement of the reference loop, OpenMP ----
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import binding as orc
        cores = min(os.cpu_count() or 1, 16)
        n_cpu = args.cpu_sample_tokens or 4096
        og = orc.layout(1, KVH, QH, D, bs, B * (n_cpu // bs + 1), orc.BF16)
        hp = orc.new_pool(og)
        nb1 = n_cpu // bs + 1
        htab = np.arange(B * nb1, dtype=np.int32).reshape(B, nb1)
        crng = np.random.default_rng(7)
        for b in range(B):
            kk = bf16_bits(crng, (n_cpu, KVH, D), 0.5)
            vv = bf16_bits(crng, (n_cpu, KVH, D), 0.5)
            orc.append_batch(og, hp, htab[b], 0, 0, kk, vv, orc.BF16)
        hq = bf16_bits(crng, (B, QH, D), 0.5)
        lens = np.full(B, n_cpu, dtype=np.int32)
        t0 = time.time()
        reps = 0
        while time.time() - t0 < 10.0:
            orc.decode_branches(og, hq, hp, htab, lens, 0, float(scale), orc.BF16, threads=cores)
            reps += 1
        dt = time.time() - t0
        cpu_bytes = reps * B * n_cpu * kv_bytes_per_token
        # the same loop on one thread, a shorter sample
        t1 = time.time()
        reps1 = 0
        while time.time() - t1 < 4.0:
            orc.decode_branches(og, hq, hp, htab, lens, 0, float(scale), orc.BF16, threads=1)
            reps1 += 1
        dt1 = time.time() - t1
        cpu = {"value": cpu_bytes / dt / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": f"{reps} x (1 layer, {B} branches x {n_cpu} tokens) of the same decode attention, "
                         f"oracle's reference-order loop, OpenMP over (branch, q head)",
               "single_thread_value": reps1 * B * n_cpu * kv_bytes_per_token / dt1 / 1e9}

    # ---- the dominant kernels of configs 3, 4 and 5 on their own shapes, in the same buffer
    other = None
    if not args.no_other_configs:
        import bench_extra
        del ws
        other = bench_extra.kernel_fractions(pool)

    tokens_per_s = B * K / (total_ms * 1e-3)
    traffic, traffic_source = measured_traffic(launch_bytes)
    line = {
        "metric": "paged_decode_attention_GBps",
        "value": round(value_gbps, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"config 2: {L} layers, 32 Q / 8 KV heads x 128, bf16 KV, 16-token pages shuffled over a "
                        f"{args.pool_gb:g} GB pool ({NB} blocks), {B} branches, ctx {args.ctx_mode} "
                        f"{int(final.min())}..{int(final.max())}; step = per layer: append 1 token/branch + paged decode attention",
            "branches": B, "layers": L, "ctx_final": [int(x) for x in final],
            "launch": "one captured HIP graph per step" if use_graph else "host launches",
            "unit_descriptors": "built once per step" if plan_bytes else "built by every launch",
            "append": "written by the attention launch" if fused_append else "a launch of its own",
        },
        "hbm_frac_step": round(value_gbps / HBM_PEAK_GBPS, 4),
        "us_per_step": round(ms_per_step * 1e3, 1),
        "tokens_per_s": round(tokens_per_s, 1),
        "bulk_append_GBps": None if append_gbps is None else round(append_gbps, 1),
        "bulk_append_hbm_frac": None if append_gbps is None else round(append_gbps / HBM_PEAK_GBPS, 4),
        "bulk_gather_GBps": None if gather_gbps is None else round(gather_gbps, 1),
        "bulk_scatter_GBps": None if scatter_gbps is None else round(scatter_gbps, 1),
        "hbm_read_probe_GBps": round(read_probe_gbps, 1),
        "hbm_read_probe_permuted_4KiB_GBps": round(permuted_probe_gbps, 1),
        "mfma_bf16_probe_TFLOPs": round(mfma_probe_tflops, 1),
        "mfma_valu_coexec_probe": coexec,
        "other_configs": other,
        "ragged_ctx_decode": ragged,
        "fill_seconds": round(t_fill, 2),
        "layer_steps": layer_steps,
        "attention_mass": attention_mass,
        "overflow_tier": overflow,
        "roofline": {
            "kernel": "decode_stream_kernel<bf16>", "bound": "hbm", "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic, "traffic_source": traffic_source, "avg_launch_us": round(ker_avg_ms * 1e3, 2), "bytes_per_launch": launch_bytes,
        },
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
