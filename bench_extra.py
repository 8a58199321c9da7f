"""bench.py --config 3|4|5: the other BASELINE configurations, same JSON shape.

Not the headline line (that is config 2, bench.py's default); these runs put
measured numbers beside the parity tests of the same shapes.  Torch is plumbing
for memory, streams and events; kernels go through the C ABI, block tables of
config 3 through the C++ CacheManager.
"""
import ctypes as C
import sys
import time

import numpy as np

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def _common(args):
    import torch
    from deusridet_amd import cabi
    lib = cabi.lib()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream()
    return torch, cabi, None, lib, stream, C.c_void_p(stream.cuda_stream)


def _timed_decode(lib, cabi, call, n):
    """average duration (ms) of the kernels that read the pages over n back-to-back calls, merge left out;
    call(i) makes the i-th call"""
    return cabi.time_partial_kernels(call, n)


def config4(args):
    """4 branches x 128k tokens, 8 KV heads x 128, int8 (+fp16 scale per token and
    head) or fp8-e4m3 pages quantised on append, dequantised inside attention."""
    torch, cabi, U, lib, stream, sp = _common(args)
    kv_name = args.kv_dtype if args.kv_dtype in ("int8", "fp8") else "int8"
    dt = cabi.INT8 if kv_name == "int8" else cabi.FP8_E4M3
    L, KVH, QH, D, bs, B, ctx = args.layers, 8, 32, 128, 16, 4, 131072
    W, K = args.warmup, args.steps
    probe = cabi.layout(L, KVH, QH, D, bs, 1, dt)
    NB = lib.drk_kv_max_blocks_for_budget(C.byref(probe), int(args.pool_gb * 1e9))
    g = cabi.layout(L, KVH, QH, D, bs, NB, dt)
    rng = np.random.default_rng(4)
    start = ctx - (W + K)
    nblk = ctx // bs + 1
    assert B * nblk <= NB, "pool too small"
    perm = rng.permutation(NB).astype(np.int32)
    tables = np.stack([perm[b * nblk:(b + 1) * nblk] for b in range(B)])
    pool = torch.zeros(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
    dtab = torch.from_numpy(tables).cuda()
    # fill through the quantising append: N(0,1) with 1 % outliers x20; time it as the bulk append figure
    chunk = 2048
    a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    append_ms, append_tokens = 0.0, 0
    for b in range(B):
        for p0 in range(0, start, chunk):
            m = min(chunk, start - p0)
            k = torch.randn(L, m, KVH, D, device="cuda")
            k = torch.where(torch.rand_like(k) < 0.01, k * 20, k).to(torch.bfloat16)
            v = torch.randn(L, m, KVH, D, device="cuda")
            v = torch.where(torch.rand_like(v) < 0.01, v * 20, v).to(torch.bfloat16)
            a0.record(stream)
            cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(pool), C.c_void_p(dtab[b].data_ptr()), 0, L, p0, m,
                      cabi.p(k), cabi.p(v), cabi.BF16, sp)
            a1.record(stream)
            torch.cuda.synchronize()
            if m == chunk and p0 > 0:
                append_ms += a0.elapsed_time(a1)
                append_tokens += m
    code_bytes = 2 * KVH * D + (2 * KVH * 2 if dt == cabi.INT8 else 0)      # per token and layer
    append_gbps = append_tokens * L * (2 * KVH * D * 2 + code_bytes) / (append_ms * 1e-3) / 1e9
    scale = 1.0 / np.sqrt(D)
    q = torch.randn(L, B, QH, D, device="cuda").to(torch.bfloat16)
    nk = torch.randn(L, B, KVH, D, device="cuda").to(torch.bfloat16)
    nv = torch.randn(L, B, KVH, D, device="cuda").to(torch.bfloat16)
    out = torch.zeros(L, B, QH, D, device="cuda", dtype=torch.bfloat16)
    wsb = lib.drk_decode_workspace_bytes(C.byref(g), B, ctx)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    pos_steps = torch.from_numpy(np.stack([np.full(B, start + s, dtype=np.int32) for s in range(W + K)])).cuda()
    len_steps = pos_steps + 1
    qrow, krow = B * QH * D * 2, B * KVH * D * 2

    def attn(l, dlen):
        cabi.call("drk_paged_decode_attention_branches", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow), cabi.p(pool),
                  cabi.p(dtab), nblk, dlen, B, ctx, C.c_void_p(out.data_ptr() + l * qrow), l, float(scale), cabi.BF16, 0,
                  cabi.p(ws), wsb, sp)

    def step(s):
        dpos, dlen = C.c_void_p(pos_steps[s].data_ptr()), C.c_void_p(len_steps[s].data_ptr())
        for l in range(L):
            cabi.call("drk_kv_append_branches", C.byref(g), cabi.p(pool), cabi.p(dtab), nblk, dpos, B, l, 1,
                      C.c_void_p(nk.data_ptr() + l * krow), C.c_void_p(nv.data_ptr() + l * krow), cabi.BF16, sp)
            attn(l, dlen)

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
    toks = sum(B * (start + s + 1) for s in range(W, W + K))
    value = toks * code_bytes * L / (total_ms * 1e-3) / 1e9
    dlen = C.c_void_p(len_steps[W + K - 1].data_ptr())
    ker_ms = _timed_decode(lib, cabi, lambda i: attn(i % L, dlen), 60)
    launch_bytes = B * ctx * code_bytes
    ach = launch_bytes / (ker_ms * 1e-3) / 1e9
    return {
        "metric": "paged_decode_attention_GBps", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": K,
        "warmup": W, "ms_per_step": round(total_ms / K, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8" if dt == cabi.INT8 else "fp8", "data": "synthetic",
        "config": {"workload": f"config 4: {L} layers, 32 Q / 8 KV heads x 128, {kv_name} pages "
                               f"({code_bytes} B per token and layer), 4 branches x 131072 tokens, K/V N(0,1) with 1 % x20 "
                               f"outliers quantised on append; step = per layer: append 1 token/branch + decode attention",
                   "branches": B, "layers": L, "ctx_final": [ctx] * B},
        "tokens_per_s": round(B * K / (total_ms * 1e-3), 1), "us_per_step": round(total_ms / K * 1e3, 1),
        "quantising_append_GBps": round(append_gbps, 1),
        "quantising_append_hbm_frac": round(append_gbps / HBM_PEAK_GBPS, 4),
        "roofline": {"kernel": f"decode_stream_kernel<{kv_name}>", "bound": "hbm", "achieved": round(ach, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": None,
                     "avg_launch_us": round(ker_ms * 1e3, 2), "bytes_per_launch": launch_bytes},
        "cpu_baseline": None,
    }


def config3(args):
    """One persistent 64k-token prefix shared by 16 branches (copy-on-write forks,
    refcounts), 0-4k private tokens each, eviction down to 25 % free."""
    torch, cabi, U, lib, stream, sp = _common(args)
    from deusridet_amd import host
    L, KVH, QH, D, bs, NBR = args.layers, 8, 32, 128, 16, 16
    W, K = args.warmup, args.steps
    prefix = 65536
    rng = np.random.default_rng(3)
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    cm = host.CacheManager()
    private = rng.integers(0, 4097, size=NBR)
    # a pool that is ~80 % full once everything is resident, so that "free 25 %" has to evict
    want_blocks = int((prefix // bs + int(private.sum()) // bs + 4 * NBR) / 0.8)
    budget = min(int(args.pool_gb * 1e9), want_blocks * L * 2 * KVH * bs * D * 2)
    assert cm.init(budget, bs, None, NBR + 1), "CacheManager.init failed"
    NB, stride = cm.pool_max_blocks(), cm.table_stride()
    hl = host.lib()
    pool_ptr = C.c_void_p(cm.pool_ptr())
    chunk = 2048

    def bulk(branch, p0, m):
        assert cm.ensure_blocks_for_range(branch, p0, m)
        cm.sync_block_table(sp)
        k = (torch.randn(L, m, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
        v = (torch.randn(L, m, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
        g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
        cabi.call("drk_kv_append_batch", C.byref(g), pool_ptr, C.c_void_p(cm.d_block_table(branch)), 0, L, p0, m,
                  cabi.p(k), cabi.p(v), cabi.BF16, sp)
        torch.cuda.synchronize()
        cm.set_seq_len(branch, p0 + m)

    for p0 in range(0, prefix, chunk):
        bulk(0, p0, chunk)
    # The fork tree.  "prefix": every branch forks from the prefix's end.  "tree": a branch forks from the prefix or
    # from an earlier branch, at a random block boundary of what that branch holds beyond the prefix, so the 16
    # branches share the prefix and subsets of them share what they wrote before they split again.  Every fourth
    # fork lands inside a block instead (forces a copy-on-write).  Branches are created parents first, then their
    # children from the latest fork point to the earliest, so that branches which share pages are neighbours in the
    # table.
    tree = getattr(args, "forks", "tree") == "tree"
    parent = [-1] + [int(rng.integers(-1, i)) if tree else -1 for i in range(1, NBR)]
    forks, fork_points, order, fork_s = [], [], [], 0.0

    def grow(node, par_branch, fp):
        nonlocal fork_s
        if node % 4 == 0:
            fp -= int(rng.integers(1, bs))
        t0 = time.perf_counter()
        b = cm.fork_branch(par_branch, fp)
        fork_s += time.perf_counter() - t0
        assert b > 0
        forks.append(b)
        fork_points.append(fp)
        order.append(node)
        for p0 in range(0, int(private[node]), chunk):
            bulk(b, fp + p0, min(chunk, int(private[node]) - p0))
        descend(node, b)

    def descend(node, branch):
        held = cm.seq_len(branch)
        kids = [(prefix + bs * int(rng.integers(0, (held - prefix) // bs + 1)) if branch else prefix, c)
                for c in range(node + 1, NBR) if parent[c] == node]
        for fp, c in sorted(kids, key=lambda k: -k[0]):           # the latest fork first
            grow(c, branch, fp)

    descend(-1, 0)
    fork_ns = fork_s / NBR * 1e9
    parent = [-1 if parent[n] < 0 else order.index(parent[n]) for n in order]          # in table-row numbering
    lens0 = np.array([cm.seq_len(b) for b in forks], dtype=np.int32)
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    B = NBR
    scale = 1.0 / np.sqrt(D)
    q = (torch.randn(L, B, QH, D, device="cuda") * 0.5).to(torch.bfloat16)
    nk = (torch.randn(L, B, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
    nv = (torch.randn(L, B, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
    out = torch.zeros(L, B, QH, D, device="cuda", dtype=torch.bfloat16)
    max_ctx = int(lens0.max()) + W + K + 1
    cascade = not getattr(args, "no_cascade", False)
    grouped = cascade and getattr(args, "shared_kernel", "auto") != "pair"       # else: the common prefix alone, as a kernel pair
    wsb = max(lib.drk_decode_shared_workspace_bytes(C.byref(g), B, max_ctx, prefix),
              lib.drk_decode_grouped_workspace_bytes_max(C.byref(g), B, max_ctx, cabi.MAX_PREFIX_GROUPS) if grouped else 0)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    shared_now, groups_now = [0], [[], cabi.prefix_groups([])]
    # the unit descriptors of the grouped kernel, built once per step for the 36 layers
    plan_bytes = lib.drk_decode_plan_bytes(C.byref(g), B, max_ctx, cabi.MAX_PREFIX_GROUPS) if grouped and not getattr(args, "no_plan", False) else 0
    fused_append = bool(plan_bytes) and not getattr(args, "no_fused_append", False)
    plan = torch.empty(max(plan_bytes, 16), dtype=torch.uint8, device="cuda")
    dpos = torch.zeros(B, dtype=torch.int32, device="cuda")
    dlen = torch.zeros(B, dtype=torch.int32, device="cuda")
    # the forked branches' rows are consecutive in the device table: branch ids forks[0]..forks[-1]
    assert forks == list(range(forks[0], forks[0] + B))
    dtabs = C.c_void_p(cm.d_block_table(forks[0]))
    qrow, krow = B * QH * D * 2, B * KVH * D * 2
    ensure_ns, evicted, evict_ns = [], 0, 0.0

    def attend(l, dl):
        if plan_bytes:
            cabi.call("drk_paged_decode_attention_planned", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow), pool_ptr,
                      dtabs, stride, dl, B, max_ctx, groups_now[1], len(groups_now[0]), cabi.p(plan),
                      C.c_void_p(out.data_ptr() + l * qrow), l, float(scale), cabi.BF16, None, 0, cabi.p(ws), wsb, sp)
        elif grouped:
            cabi.call("drk_paged_decode_attention_grouped", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow), pool_ptr,
                      dtabs, stride, dl, B, max_ctx, groups_now[1], len(groups_now[0]), C.c_void_p(out.data_ptr() + l * qrow),
                      l, float(scale), cabi.BF16, None, 0, cabi.p(ws), wsb, sp)
        else:
            cabi.call("drk_paged_decode_attention_shared", C.byref(g), C.c_void_p(q.data_ptr() + l * qrow), pool_ptr,
                      dtabs, stride, dl, B, max_ctx, shared_now[0], C.c_void_p(out.data_ptr() + l * qrow), l,
                      float(scale), cabi.BF16, cabi.p(ws), wsb, sp)

    def step(s, lens):
        nonlocal evicted, evict_ns
        t = time.perf_counter()
        for i, b in enumerate(forks):
            assert cm.ensure_blocks_for(b, int(lens[i]))
        ensure_ns.append((time.perf_counter() - t) / B * 1e9)
        # pressure: free 25 % of the pool, oldest private pages first -- every 256 steps, as the configuration says,
        # and once in the middle of a timed region too short to reach step 256
        if s >= W and ((s - W) % 256 == 255 or (K < 256 and s == W + K // 2)):
            t = time.perf_counter()
            before = cm.free_blocks()
            cm.ensure_free_blocks(NB // 4)
            evicted += cm.free_blocks() - before
            evict_ns += (time.perf_counter() - t) * 1e9
        cm.sync_block_table(sp)                               # COW copies, then table deltas
        shared_now[0] = cm.common_prefix_tokens(forks) if cascade else 0
        if grouped:
            groups_now[0] = cm.common_prefix_groups(forks, 64 // (QH // KVH), 256, cabi.MAX_PREFIX_GROUPS)
            groups_now[1] = cabi.prefix_groups(groups_now[0])
        dpos.copy_(torch.from_numpy(lens))
        dlen.copy_(torch.from_numpy(lens + 1))
        if plan_bytes:
            cabi.call("drk_decode_plan_build", C.byref(g), dtabs, stride, cabi.p(dlen), B, max_ctx, groups_now[1],
                      len(groups_now[0]), cabi.p(plan), plan_bytes, sp)
        for l in range(L):
            if fused_append:                                      # the attention launch writes the new rows itself
                cabi.call("drk_kv_append_decode_planned", C.byref(g), pool_ptr, dtabs, stride, cabi.p(dlen), B, max_ctx,
                          groups_now[1], len(groups_now[0]), cabi.p(plan), C.c_void_p(nk.data_ptr() + l * krow),
                          C.c_void_p(nv.data_ptr() + l * krow), cabi.BF16, C.c_void_p(q.data_ptr() + l * qrow),
                          C.c_void_p(out.data_ptr() + l * qrow), l, float(scale), cabi.BF16, None, 0, cabi.p(ws), wsb, sp)
                continue
            cabi.call("drk_kv_append_branches", C.byref(g), pool_ptr, dtabs, stride, cabi.p(dpos), B, l, 1,
                      C.c_void_p(nk.data_ptr() + l * krow), C.c_void_p(nv.data_ptr() + l * krow), cabi.BF16, sp)
            attend(l, cabi.p(dlen))
        for i, b in enumerate(forks):
            cm.set_seq_len(b, int(lens[i]) + 1)

    per_tok = 2 * KVH * D * 2

    def distinct_bytes(lens_now):
        """bytes a launch must fetch: every physical page some branch reads, once, up to the last token read in it"""
        held = {}
        for b, n in zip(forks, lens_now):
            tab = cm.h_block_table(b)
            for k in range((int(n) + bs - 1) // bs):
                if tab[k] >= 0:
                    held[int(tab[k])] = max(held.get(int(tab[k]), 0), min(bs, int(n) - k * bs))
        return sum(held.values()) * per_tok

    lens = lens0.copy()
    for s in range(W):
        step(s, lens); lens += 1
    torch.cuda.synchronize()
    # the launch as the warm-up left it: every page resident (the timed steps evict)
    full_ms = _timed_decode(lib, cabi, lambda i: attend(i % L, cabi.p(dlen)), 60)
    full_bytes = distinct_bytes(lens)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    logical = 0
    for s in range(W, W + K):
        step(s, lens); lens += 1
        logical += int(lens.sum())
    e1.record(stream)
    torch.cuda.synchronize()
    total_ms = e0.elapsed_time(e1)
    unique_tokens = cm.gpu_blocks_used() * bs
    value = logical * per_tok * L / (total_ms * 1e-3) / 1e9
    dl = cabi.p(dlen)
    ker_ms = _timed_decode(lib, cabi, lambda i: attend(i % L, dl), 60)
    launch_logical = int(lens.sum()) * per_tok
    launch_unique = distinct_bytes(lens)
    # what the launch streams once: the ranges it was given as groups, and every branch's remainder
    in_groups = sum((e - b0) // 64 * 64 * (nb - 1) for _, nb, b0, e in groups_now[0]) if grouped else shared_now[0] // 64 * 64 * (B - 1)
    launch_streamed = launch_logical - in_groups * per_tok
    ach = launch_unique / (ker_ms * 1e-3) / 1e9
    value_unique = value * launch_unique / launch_logical
    return {
        "metric": "paged_decode_attention_GBps", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": K,
        "warmup": W, "ms_per_step": round(total_ms / K, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"config 3: {L} layers, 8 KV heads x 128 bf16, 65536-token prefix shared by 16 copy-on-write "
                               f"branches (+0..4096 private tokens), eviction to 25 % free every 256 steps (once, mid-way, when fewer steps are timed); "
                               f"value counts LOGICAL bytes (every branch's whole context); shared pages streamed "
                               f"{'once for all branches' if cascade else 'once per branch'}",
                   "branches": B, "layers": L, "ctx_final": [int(x) for x in lens], "shared_tokens": int(shared_now[0]),
                   "forks": "tree" if tree else "prefix", "fork_parent": parent, "fork_points": fork_points,
                   "shared_ranges": [list(x) for x in groups_now[0]] if grouped else [[0, B, 0, int(shared_now[0])]],
                   "pool_blocks": NB,
                   "unit_descriptors": "built once per step" if plan_bytes else "built by every launch",
                   "append": "written by the attention launch" if fused_append else "a launch of its own"},
        "logical_GB_per_layer_step": round(launch_logical / 1e9, 3),
        "unique_GB_per_layer_step": round(launch_unique / 1e9, 3),
        "resident_GB_per_layer": round(unique_tokens * per_tok / 1e9, 3),
        "value_unique_bytes_GBps": round(value_unique, 2),
        "us_per_step": round(total_ms / K * 1e3, 1), "tokens_per_s": round(B * K / (total_ms * 1e-3), 1),
        "host_ns": {"fork_branch": round(fork_ns), "ensure_blocks_for": round(float(np.mean(ensure_ns))),
                    "evict_per_block": round(evict_ns / max(evicted, 1)), "blocks_evicted": int(evicted)},
        "roofline": {"kernel": "decode_group16_kernel<bf16>" if grouped else
                               "prefix_stream_kernel<bf16> + decode_stream_kernel<bf16>", "bound": "hbm",
                     "achieved": round(ach, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": None,
                     "avg_launch_us": round(ker_ms * 1e3, 2), "bytes_per_launch": launch_unique,
                     "streamed_bytes_per_launch": launch_streamed,
                     "all_pages_resident": {"avg_launch_us": round(full_ms * 1e3, 2), "bytes_per_launch": full_bytes,
                                            "frac": round(full_bytes / (full_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                            "what": "the same launch after the warm-up steps, before the timed steps evicted "
                                                    "%d blocks (an evicted page is a hole the kernel skips: its tile still "
                                                    "takes a turn, its bytes are not counted)" % evicted},
                     "note": "DISTINCT bytes: every physical page some branch reads, counted once.  streamed_bytes is what "
                             "the launch reads given the shared ranges it was handed (ranges under 256 tokens and what "
                             "rounding to 64-token tiles cuts off are read once per branch).  The merge is not in "
                             "avg_launch_us" + ("" if grouped else "; the prefix pass and the tail kernel are timed as one unit")},
        "cpu_baseline": None,
    }


def config5(args):
    """Chunked prefill to 32k in 2048-token chunks (append into pages, then causal
    MFMA attention over all prior pages plus the chunk) with 4 decode branches at
    8k interleaved on the same pool."""
    torch, cabi, U, lib, stream, sp = _common(args)
    L, KVH, QH, D, bs = min(args.layers, 4), 8, 32, 128, 16
    chunk, total, DB, dctx = 2048, 32768, 4, 8192
    NB = (total + DB * (dctx + 64)) // bs + 64
    kv_name = args.kv_dtype or "bf16"
    g = cabi.layout(L, KVH, QH, D, bs, NB, {"bf16": cabi.BF16, "int8": cabi.INT8, "fp8": cabi.FP8_E4M3}[kv_name])
    rng = np.random.default_rng(5)
    perm = rng.permutation(NB).astype(np.int32)
    nb_seq, nb_dec = total // bs, dctx // bs + 4
    tab_seq = torch.from_numpy(perm[:nb_seq].copy()).cuda()
    tab_dec = torch.from_numpy(np.stack([perm[nb_seq + b * nb_dec: nb_seq + (b + 1) * nb_dec] for b in range(DB)])).cuda()
    pool = torch.zeros(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
    scale = 1.0 / np.sqrt(D)
    for b in range(DB):
        for p0 in range(0, dctx, chunk):
            k = torch.randn(L, chunk, KVH, D, device="cuda").to(torch.bfloat16)
            v = torch.randn(L, chunk, KVH, D, device="cuda").to(torch.bfloat16)
            cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(pool), C.c_void_p(tab_dec[b].data_ptr()), 0, L, p0, chunk,
                      cabi.p(k), cabi.p(v), cabi.BF16, sp)
            torch.cuda.synchronize()
    qd = torch.randn(L, DB, QH, D, device="cuda").to(torch.bfloat16)
    od = torch.zeros_like(qd)
    nk = torch.randn(L, DB, KVH, D, device="cuda").to(torch.bfloat16)
    nv = torch.randn(L, DB, KVH, D, device="cuda").to(torch.bfloat16)
    wsb = lib.drk_decode_workspace_bytes(C.byref(g), DB, dctx + 64)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    dpos = torch.full((DB,), dctx, dtype=torch.int32, device="cuda")
    dlen = dpos + 1
    qrow, krow = DB * QH * D * 2, DB * KVH * D * 2
    pf_ms, pf_flops, ap_ms, dec_ms = 0.0, 0.0, 0.0, []
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    passes = max(1, args.steps // 16) + 1                        # first pass warms up
    for ps in range(passes):
        for c in range(total // chunk):
            k = torch.randn(L, chunk, KVH, D, device="cuda").to(torch.bfloat16)
            v = torch.randn(L, chunk, KVH, D, device="cuda").to(torch.bfloat16)
            q = torch.randn(L, chunk, QH, D, device="cuda").to(torch.bfloat16)
            o = torch.empty_like(q)
            ev[0].record(stream)
            cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(pool), cabi.p(tab_seq), 0, L, c * chunk, chunk, cabi.p(k), cabi.p(v),
                      cabi.BF16, sp)
            ev[1].record(stream)
            for l in range(L):
                cabi.call("drk_paged_prefill_attention", C.byref(g), C.c_void_p(q.data_ptr() + l * chunk * QH * D * 2),
                          cabi.p(pool), cabi.p(tab_seq), C.c_void_p(o.data_ptr() + l * chunk * QH * D * 2), l, c * chunk, chunk,
                          float(scale), cabi.BF16, None, 0, sp)
            ev[2].record(stream)
            for l in range(L):                                   # one interleaved decode step of the 4 branches
                cabi.call("drk_kv_append_branches", C.byref(g), cabi.p(pool), cabi.p(tab_dec), nb_dec, cabi.p(dpos), DB, l, 1,
                          C.c_void_p(nk.data_ptr() + l * krow), C.c_void_p(nv.data_ptr() + l * krow), cabi.BF16, sp)
                cabi.call("drk_paged_decode_attention_branches", C.byref(g), C.c_void_p(qd.data_ptr() + l * qrow),
                          cabi.p(pool), cabi.p(tab_dec), nb_dec, cabi.p(dlen), DB, dctx + 64, C.c_void_p(od.data_ptr() + l * qrow),
                          l, float(scale), cabi.BF16, 0, cabi.p(ws), wsb, sp)
            ev[3].record(stream)
            torch.cuda.synchronize()
            if ps > 0:
                ap_ms += ev[0].elapsed_time(ev[1])
                pf_ms += ev[1].elapsed_time(ev[2])
                pf_flops += L * 4.0 * chunk * (c * chunk + (chunk + 1) / 2.0) * D * QH
                dec_ms.append(ev[2].elapsed_time(ev[3]))
    tfl = pf_flops / (pf_ms * 1e-3) / 1e12
    nchunks = (passes - 1) * (total // chunk)
    ap_gbps = nchunks * L * chunk * 2 * (2 * KVH * D * 2) / (ap_ms * 1e-3) / 1e9
    # a short chunk at the end of the same context (a perception frame of a few tokens): the chunk kernel
    # against the path that splits the context over the chip
    short = {}
    for rows in (() if getattr(args, "no_ragged", False) else (16, 64)):
        pos = total - rows
        qs = torch.randn(rows, QH, D, device="cuda").to(torch.bfloat16)
        os_ = torch.empty_like(qs)
        us = []
        for mode in (0, -1):
            lib.drk_debug_set_prefill_split(mode)
            wsb_s = lib.drk_prefill_workspace_bytes(C.byref(g), pos, rows)
            ws_s = torch.empty(max(wsb_s, 256), dtype=torch.uint8, device="cuda")

            def go(n):
                for i in range(n):
                    cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(qs), cabi.p(pool), cabi.p(tab_seq), cabi.p(os_), i % L, pos, rows,
                              float(scale), cabi.BF16, cabi.p(ws_s), wsb_s, sp)
            go(3)
            ev[0].record(stream)
            go(20)
            ev[1].record(stream)
            torch.cuda.synchronize()
            us.append(ev[0].elapsed_time(ev[1]) / 20 * 1e3)
        lib.drk_debug_set_prefill_split(-1)
        short[f"{rows}_rows_at_{pos}"] = {"chunk_kernel_us": round(us[0], 1), "context_split_us": round(us[1], 1)}
    return {
        "metric": "chunked_prefill_attention_TFLOPs", "value": round(tfl, 1), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": nchunks, "warmup": total // chunk, "ms_per_step": round(pf_ms / nchunks / L, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if kv_name == "bf16" else "f16",
        "data": "synthetic",
        "config": {"workload": f"config 5: one sequence prefilled to 32768 in 2048-token chunks, 32 Q / 8 KV heads x 128 "
                               f"bf16 in, {kv_name} 16-token pages, {L} layers; per chunk: append, causal attention over all pages so far "
                               f"(MFMA), then one decode step of 4 branches at 8192 on the same pool; a step here is one "
                               f"(chunk, layer) attention launch", "layers": L},
        "chunk_append_GBps": round(ap_gbps, 1),
        "interleaved_decode_us_per_layer": round(float(np.mean(dec_ms)) / L * 1e3, 1),
        "short_chunk_attention": short,
        "roofline": {"kernel": f"prefill_mfma_kernel<{kv_name}>", "bound": "mfma", "achieved": round(tfl, 1),
                     "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tfl / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": None},
        "cpu_baseline": None,
    }


def config6(args):
    """The caller protocol at config 3's shape: one perception stream takes a 64k-token prefix in
    2048-token chunks through the whole layer path (fused split + norm + RoPE + page write, then
    MFMA prefill attention with the gate), 16 decode branches fork from it copy-on-write and step
    together -- from the host layer by layer, and as one captured step replayed."""
    torch, cabi, U, lib, _, _ = _common(args)
    from deusridet_amd import host
    stream = torch.cuda.Stream()                     # the default stream cannot be captured
    sp = C.c_void_p(stream.cuda_stream)
    L, KVH, QH, D, bs, NBR = args.layers, 8, 32, 128, 16, 16
    W, K = args.warmup, args.steps
    prefix, chunk, RD, THETA = 65536, 2048, 32, 1.0e7
    max_ctx = prefix + 2 * (W + K) + 64
    assert host.set_attention_geometry(L, QH, KVH, D, cabi.BF16)
    assert host.lib().drkh_set_rope(RD, THETA, 1e-6)
    cm = host.CacheManager()
    blocks = prefix // bs + NBR * ((2 * (W + K)) // bs + 3) + 64
    assert cm.init(blocks * L * 2 * KVH * bs * D * 2, bs, None, NBR + 1), "CacheManager.init failed"
    table = torch.empty(max_ctx * RD, dtype=torch.float32, device="cuda")
    cabi.call("drk_rope_table_fill", cabi.p(table), max_ctx, RD, THETA, sp)
    ks = host.KvStream()
    assert ks.init(cm, max_ctx, None, cabi.p(table), max_ctx)
    bf = torch.bfloat16
    qw = (1 + 0.1 * torch.randn(D, device="cuda")).to(bf)
    kw = (1 + 0.1 * torch.randn(D, device="cuda")).to(bf)
    # ---- perception ----
    qg = (torch.randn(chunk, QH, 2 * D, device="cuda")).to(bf)
    k = (torch.randn(chunk, KVH, D, device="cuda") * 0.7).to(bf)
    v = (torch.randn(chunk, KVH, D, device="cuda") * 0.5).to(bf)
    qs, ao = torch.empty(chunk, QH, D, device="cuda", dtype=bf), torch.empty(chunk, QH, D, device="cuda", dtype=bf)
    io = (cabi.p(qg), cabi.p(k), cabi.p(v), cabi.p(qw), cabi.p(kw), cabi.p(qs), cabi.p(ao))
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for p0 in range(0, prefix, chunk):
        assert ks.begin_prefill(chunk, sp)
        for l in range(L):
            ks.prefill_layer(l, io, chunk, sp)
        ks.end_prefill(chunk)
    e1.record(stream)
    torch.cuda.synchronize()
    prefill_ms = e0.elapsed_time(e1)
    prefill_flops = 4.0 * QH * D * L * sum((p0 + (chunk + 1) / 2.0) * chunk for p0 in range(0, prefix, chunk))
    # ---- decode branches ----
    assert ks.open_branches(NBR) == NBR and ks.shared_tokens() == prefix
    B = NBR
    lay = [dict(qg=torch.randn(B, QH, 2 * D, device="cuda").to(bf), k=(torch.randn(B, KVH, D, device="cuda") * 0.7).to(bf),
                v=(torch.randn(B, KVH, D, device="cuda") * 0.5).to(bf), q=torch.empty(B, QH, D, device="cuda", dtype=bf),
                out=torch.empty(B, QH, D, device="cuda", dtype=bf)) for _ in range(L)]

    torch.cuda.synchronize()

    def layers(st):
        for l in range(L):
            b = lay[l]
            ks.decode_layer(l, (cabi.p(b["qg"]), cabi.p(b["k"]), cabi.p(b["v"]), cabi.p(qw), cabi.p(kw), cabi.p(b["q"]), cabi.p(b["out"])), st)

    per_tok = 2 * KVH * D * 2

    def timed(step_fn):
        for _ in range(W):
            step_fn()
        torch.cuda.synchronize()
        host_s, logical = 0.0, 0
        e0.record(stream)
        for _ in range(K):
            t = time.perf_counter()
            step_fn()
            host_s += time.perf_counter() - t
            logical += sum(ks.branch_pos(i) for i in range(B))
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / K, host_s / K * 1e3, logical

    def eager():
        assert ks.begin_decode_step(sp)
        layers(sp)
        ks.end_decode_step(sp)

    eager_ms, eager_host_ms, _ = timed(eager)
    assert ks.capture_decode_step(layers, sp)
    graph_ms, graph_host_ms, logical = timed(lambda: ks.replay_decode_step(sp) or (_ for _ in ()).throw(RuntimeError("replay failed")))
    value = logical * per_tok * L / (graph_ms * K * 1e-3) / 1e9
    launch_unique = (prefix + sum(ks.branch_pos(i) - prefix for i in range(B))) * per_tok
    ks.close_branches()
    return {
        "metric": "paged_decode_attention_GBps", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": K,
        "warmup": W, "ms_per_step": round(graph_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"config 3's shape through the stream driver: {L} layers, 32 Q / 8 KV heads x 128 bf16, a "
                               f"{prefix}-token prefix taken in {chunk}-token chunks (whole layer path), then {B} copy-on-write "
                               f"branches decoding together, one captured step replayed; value counts LOGICAL bytes",
                   "branches": B, "layers": L, "shared_tokens": prefix},
        "decode_step_ms": {"graph_replay": round(graph_ms, 4), "host_launched": round(eager_ms, 4),
                           "host_time_graph_replay": round(graph_host_ms, 4), "host_time_host_launched": round(eager_host_ms, 4)},
        "unique_GBps": round(launch_unique * L / (graph_ms * 1e-3) / 1e9, 1),
        "prefill": {"tokens_per_s": round(prefix / (prefill_ms * 1e-3), 1), "ms": round(prefill_ms, 1),
                    "attention_TFLOPs_over_whole_path_time": round(prefill_flops / (prefill_ms * 1e-3) / 1e12, 1)},
        "roofline": None, "cpu_baseline": None,
    }


def config7(args):
    """The reference's own model shape (24 Q / 4 KV heads x 256, 256-token blocks, fp16, 16 full-attention
    layers; model.h:39-42, block_pool.h:34-38) on config 2's workload: 8 branches x 32k tokens; step = per
    layer the fused split + norm + RoPE + page write, then decode attention with the gate."""
    torch, cabi, U, lib, stream, sp = _common(args)
    L, KVH, QH, D, bs, B, ctx, RD = min(args.layers, 16), 4, 24, 256, 256, 8, 32768, 64
    W, K = args.warmup, args.steps
    nblk = ctx // bs + 1
    NB = B * nblk + 8
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.F16)
    rng = np.random.default_rng(7)
    perm = rng.permutation(NB).astype(np.int32)
    tables = np.stack([perm[b * nblk:(b + 1) * nblk] for b in range(B)])
    dtab = torch.from_numpy(tables).cuda()
    pool = torch.empty(lib.drk_kv_pool_bytes(C.byref(g)), dtype=torch.uint8, device="cuda")
    pool.view(torch.float16).normal_(0, 0.5)
    start = ctx - (W + K)
    pos_steps = torch.from_numpy(np.stack([np.full(B, start + s, dtype=np.int32) for s in range(W + K)])).cuda()
    len_steps = pos_steps + 1
    h = torch.float16
    qg = (torch.randn(L, B, QH, 2 * D, device="cuda") * 0.5).to(h)
    k = (torch.randn(L, B, KVH, D, device="cuda") * 0.5).to(h)
    v = (torch.randn(L, B, KVH, D, device="cuda") * 0.5).to(h)
    qn = (1 + 0.1 * torch.randn(D, device="cuda")).to(h)
    kn = (1 + 0.1 * torch.randn(D, device="cuda")).to(h)
    qs = torch.empty(L, B, QH, D, device="cuda", dtype=h)
    out = torch.empty(L, B, QH, D, device="cuda", dtype=h)
    table = torch.empty(ctx * RD, dtype=torch.float32, device="cuda")
    cabi.call("drk_rope_table_fill", cabi.p(table), ctx, RD, 1.0e7, sp)
    wsb = lib.drk_decode_workspace_bytes(C.byref(g), B, ctx)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    scale = 1.0 / np.sqrt(D)
    qgrow, krow, qrow = B * QH * 2 * D * 2, B * KVH * D * 2, B * QH * D * 2

    def attn(l, dlen):
        cabi.call("drk_paged_decode_attention_gated", C.byref(g), C.c_void_p(qs.data_ptr() + l * qrow), cabi.p(pool), cabi.p(dtab),
                  nblk, dlen, B, ctx, C.c_void_p(out.data_ptr() + l * qrow), l, float(scale), cabi.F16,
                  C.c_void_p(qg.data_ptr() + l * qgrow + D * 2), 2 * D, cabi.p(ws), wsb, sp)

    def step(s):
        dpos, dlen = C.c_void_p(pos_steps[s].data_ptr()), C.c_void_p(len_steps[s].data_ptr())
        for l in range(L):
            cabi.call("drk_qk_norm_rope_append", C.byref(g), cabi.p(pool), cabi.p(dtab), nblk, dpos, 0, B, l,
                      C.c_void_p(qg.data_ptr() + l * qgrow), C.c_void_p(k.data_ptr() + l * krow),
                      C.c_void_p(v.data_ptr() + l * krow), cabi.p(qn), cabi.p(kn), 1e-6, RD, 1.0e7, cabi.p(table), ctx,
                      C.c_void_p(qs.data_ptr() + l * qrow), cabi.F16, sp)
            attn(l, dlen)

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
    per_tok = 2 * KVH * D * 2
    toks = sum(B * (start + s + 1) for s in range(W, W + K))
    value = toks * per_tok * L / (total_ms * 1e-3) / 1e9
    dlen = C.c_void_p(len_steps[W + K - 1].data_ptr())
    ker_ms = _timed_decode(lib, cabi, lambda i: attn(i % L, dlen), 60)
    launch_bytes = B * ctx * per_tok
    ach = launch_bytes / (ker_ms * 1e-3) / 1e9
    # the same shape's chunked prefill: 2 048-token chunks at positions 0, 6 144 and 30 720 of branch 0's pages
    M = 2048
    qc = (torch.randn(M, QH, D, device="cuda") * 0.5).to(h)
    oc = torch.empty_like(qc)
    pwsb = lib.drk_prefill_workspace_bytes_max(C.byref(g), ctx, M)
    pws = torch.empty(max(pwsb, 16), dtype=torch.uint8, device="cuda")
    prefill = {}
    for pos in (0, 3 * M, 15 * M):
        for _ in range(2):
            cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(qc), cabi.p(pool), cabi.p(dtab), cabi.p(oc), 0, pos, M,
                      float(scale), cabi.F16, cabi.p(pws), pwsb, sp)
        a0, a1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a0.record(stream)
        for _ in range(4):
            cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(qc), cabi.p(pool), cabi.p(dtab), cabi.p(oc), 0, pos, M,
                      float(scale), cabi.F16, cabi.p(pws), pwsb, sp)
        a1.record(stream)
        torch.cuda.synchronize()
        ms = a0.elapsed_time(a1) / 4
        fl = 4.0 * M * (pos + (M + 1) / 2.0) * D * QH
        prefill["pos_%d" % pos] = {"us": round(ms * 1e3, 1), "TFLOPs": round(fl / (ms * 1e-3) / 1e12, 1),
                                   "frac": round(fl / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
    return {
        "prefill_chunks_2048": {"kernel": "prefill_d256w_kernel<f16>" if getattr(args, "d256_waves", None) != 0 else "prefill_d256_kernel<f16>", "bound": "mfma", "peak": MFMA_BF16_PEAK_TFLOPS, **prefill},
        "metric": "paged_decode_attention_GBps", "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": K,
        "warmup": W, "ms_per_step": round(total_ms / K, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"the reference's model shape: {L} full-attention layers, 24 Q / 4 KV heads x 256, fp16, 256-token "
                               f"blocks, 64 rotary dims, 8 branches x 32768 tokens; step = per layer: fused split + head norm + "
                               f"RoPE + page write, decode attention with the sigmoid gate; kernels launched from the host",
                   "branches": B, "layers": L, "ctx_final": [ctx] * B},
        "tokens_per_s": round(B * K / (total_ms * 1e-3), 1), "us_per_step": round(total_ms / K * 1e3, 1),
        "roofline": {"kernel": "decode_stream_kernel<f16, 256>", "bound": "hbm", "achieved": round(ach, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": None,
                     "avg_launch_us": round(ker_ms * 1e3, 2), "bytes_per_launch": launch_bytes},
        "cpu_baseline": None,
    }


def run(args):
    return {3: config3, 4: config4, 5: config5, 6: config6, 7: config7}[args.config](args)


# ---------------------------------------------------------------------------------------------
# Short kernel measurements of configs 3, 4 and 5 for bench.py's default line: the dominant kernel
# of each configuration on its real shape, in a pool carved out of the device buffer the headline
# run leaves behind.  Every figure is algorithmic bytes (or flops) per launch over the average
# launch duration from HIP events recorded on the launch stream.
# ---------------------------------------------------------------------------------------------
def _entry(kernel, bound, per_launch, ms, what, extra=None):
    peak = HBM_PEAK_GBPS if bound == "hbm" else MFMA_BF16_PEAK_TFLOPS
    ach = per_launch / (ms * 1e-3) / (1e9 if bound == "hbm" else 1e12)
    e = {"kernel": kernel, "bound": bound, "avg_launch_us": round(ms * 1e3, 2),
         ("bytes_per_launch" if bound == "hbm" else "flops_per_launch"): int(per_launch),
         "achieved": round(ach, 1), "peak": peak, "unit": "GB/s" if bound == "hbm" else "TFLOP/s",
         "frac": round(ach / peak, 4), "workload": what}
    if extra:
        e.update(extra)
    return e


def _shuffled_rows(rng, NB, nblk_per_row):
    perm = rng.permutation(NB).astype(np.int32)
    stride = max(nblk_per_row) + 1
    tab = np.full((len(nblk_per_row), stride), -1, dtype=np.int32)
    o = 0
    for i, n in enumerate(nblk_per_row):
        tab[i, :n] = perm[o:o + n]
        o += n
    return tab, stride, perm[o:]


def _fork_tree(rng, n_blocks, prefix, private, bs, tree, per_group):
    """Block tables of len(private) branches over one prefix, built by a bookkeeping-only CacheManager (forks and the
    shared ranges are the host classes' own), with the page ids sent through a random permutation of the pool.
    Returns (tables [B, stride], lengths, fork points, parents, shared ranges)."""
    from deusridet_amd import cabi, host
    B = len(private)
    cm = host.CacheManager()
    assert cm.init_detached(n_blocks, bs, None, B + 1), "CacheManager.init_detached failed"
    assert cm.ensure_blocks_for_range(0, 0, prefix)
    cm.set_seq_len(0, prefix)
    parent = [-1] + [int(rng.integers(-1, i)) if tree else -1 for i in range(1, B)]
    ids, points, order = [], [], []

    def grow(node, par_branch, fp):
        b = cm.fork_branch(par_branch, fp)
        assert b > 0
        if private[node]:
            assert cm.ensure_blocks_for_range(b, fp, int(private[node]))
        cm.set_seq_len(b, fp + int(private[node]))
        ids.append(b)
        points.append(fp)
        order.append(node)
        descend(node, b)

    def descend(node, branch):
        # the children of a node, the latest fork first: then branches that share pages are neighbours in the table
        held = cm.seq_len(branch)
        kids = [(prefix + bs * int(rng.integers(0, (held - prefix) // bs + 1)) if branch else prefix, c)
                for c in range(node + 1, B) if parent[c] == node]
        for fp, c in sorted(kids, key=lambda k: -k[0]):
            grow(c, branch, fp)

    descend(-1, 0)
    perm = rng.permutation(n_blocks).astype(np.int32)
    lens = np.array([cm.seq_len(b) for b in ids], dtype=np.int32)
    stride = (int(lens.max()) + bs - 1) // bs + 1
    tab = np.full((B, stride), -1, dtype=np.int32)
    for i, b in enumerate(ids):
        row = cm.h_block_table(b)[:stride]
        tab[i, :len(row)] = np.where(row >= 0, perm[np.maximum(row, 0)], -1)
    groups = cm.common_prefix_groups(ids, per_group, 256, cabi.MAX_PREFIX_GROUPS)
    parent_row = [-1 if parent[n] < 0 else order.index(parent[n]) for n in order]      # in table-row numbering
    return tab, lens, points, parent_row, groups


def kernel_fractions(buf, seed=11):
    """buf: a torch uint8 device tensor of at least 16 GiB that may be overwritten."""
    import torch
    from deusridet_amd import cabi
    lib = cabi.lib()
    stream = torch.cuda.current_stream()
    sp = C.c_void_p(stream.cuda_stream)
    KVH, QH, D, bs = 8, 32, 128, 16
    scale = float(1.0 / np.sqrt(D))
    rng = np.random.default_rng(seed)
    res = {}
    ev = lambda: torch.cuda.Event(enable_timing=True)

    def fit_blocks(L, dt, want):
        probe = cabi.layout(L, KVH, QH, D, bs, 1, dt)
        nb = lib.drk_kv_max_blocks_for_budget(C.byref(probe), buf.numel())
        return min(nb, want)

    def fill(g, table_row_ptr, n_tokens, L, outliers, timed=None, chunk=8192):
        """append n_tokens N(0,1) tokens (x20 outliers on 1 % of the elements if asked) to one table row"""
        for p0 in range(0, n_tokens, chunk):
            m = min(chunk, n_tokens - p0)
            k = torch.randn(L, m, KVH, D, device="cuda")
            v = torch.randn(L, m, KVH, D, device="cuda")
            if outliers:
                k = torch.where(torch.rand_like(k) < 0.01, k * 20, k)
                v = torch.where(torch.rand_like(v) < 0.01, v * 20, v)
            k, v = k.to(torch.bfloat16), v.to(torch.bfloat16)
            a0, a1 = ev(), ev()
            a0.record(stream)
            cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(buf), table_row_ptr, 0, L, p0, m, cabi.p(k), cabi.p(v),
                      cabi.BF16, sp)
            a1.record(stream)
            torch.cuda.synchronize()
            if timed is not None and m == chunk and p0 > 0:
                timed.append((a0.elapsed_time(a1), m))

    # ---- config 4: 4 branches x 131 072 tokens of int8 (+ fp16 scales) / fp8 pages ---------------------
    for name, dt in (("int8", cabi.INT8), ("fp8", cabi.FP8_E4M3)):
        L, B, ctx = 2, 4, 131072
        NB = fit_blocks(L, dt, 200000)
        g = cabi.layout(L, KVH, QH, D, bs, NB, dt)
        tab, stride, _ = _shuffled_rows(rng, NB, [ctx // bs] * B)
        dtab = torch.from_numpy(tab).cuda()
        for b in range(B):
            fill(g, C.c_void_p(dtab[b].data_ptr()), ctx, L, True)
        code = 2 * KVH * D + (2 * KVH * 2 if dt == cabi.INT8 else 0)              # bytes per token and layer
        q = torch.randn(L, B, QH, D, device="cuda").to(torch.bfloat16)
        out = torch.zeros_like(q)
        wsb = lib.drk_decode_workspace_bytes(C.byref(g), B, ctx)
        ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
        dlen = torch.full((B,), ctx, dtype=torch.int32, device="cuda")
        row = B * QH * D * 2
        ms = _timed_decode(lib, cabi, lambda i: cabi.call(
            "drk_paged_decode_attention_branches", C.byref(g), C.c_void_p(q.data_ptr() + (i % L) * row), cabi.p(buf),
            cabi.p(dtab), stride, cabi.p(dlen), B, ctx, C.c_void_p(out.data_ptr() + (i % L) * row), i % L, scale, cabi.BF16, 0,
            cabi.p(ws), wsb, sp), 40)
        res["config4_%s" % name] = _entry(
            "decode_stream_kernel<%s>" % name, "hbm", B * ctx * code, ms,
            "config 4: 4 branches x 131072 tokens, %s pages (%d B per token and layer), K/V N(0,1) with 1 %% x20 outliers "
            "quantised on append, pages shuffled over %d blocks" % (name, code, NB))
        del q, out, ws, dtab

    # ---- config 4's append: the quantising bulk append on a prefill chunk's shape -------------------------
    # 2048 tokens x 36 layers of bf16 K and V per launch, four source sets in rotation (1.2 GB, so no launch
    # finds its source in a cache), written to 16 successive positions of a shuffled table.
    L, m, NSRC = 36, 2048, 4
    srcs = []
    for _ in range(NSRC):
        kv = []
        for _ in range(2):
            x = torch.randn(L, m, KVH, D, device="cuda")
            kv.append(torch.where(torch.rand_like(x) < 0.01, x * 20, x).to(torch.bfloat16))
            del x
        srcs.append(kv)
    for name, dt in (("int8", cabi.INT8), ("fp8", cabi.FP8_E4M3)):
        NB = fit_blocks(L, dt, 16 * m // bs + 8)
        g = cabi.layout(L, KVH, QH, D, bs, NB, dt)
        npos = min(16, (NB - 8) * bs // m)
        tab = torch.from_numpy(rng.permutation(NB).astype(np.int32)).cuda()
        code = 2 * KVH * D + (2 * KVH * 2 if dt == cabi.INT8 else 0)

        def launches(n):
            for it in range(n):
                k, v = srcs[it % NSRC]
                cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(buf), cabi.p(tab), 0, L, (it % npos) * m, m, cabi.p(k), cabi.p(v),
                          cabi.BF16, sp)
        launches(4)
        a0, a1 = ev(), ev()
        torch.cuda.synchronize()
        a0.record(stream)
        launches(32)
        a1.record(stream)
        torch.cuda.synchronize()
        res["config4_%s_append" % name] = _entry(
            "append_quant_kernel<%s>" % name, "hbm", m * L * (2 * KVH * D * 2 + code), a0.elapsed_time(a1) / 32,
            "quantising bulk append: %d tokens x %d layers per launch, reads 4096 B bf16 and writes %d B per token and layer; "
            "four source sets in rotation" % (m, L, code))
    del srcs

    # ---- config 3: 65 536-token prefix shared by 16 branches + private tokens U{0..4096}, 36 layers of pages ----
    # Two draws of the fork points: every branch from the prefix's end, and a tree (a branch forks from the prefix or
    # from an earlier branch at a random block boundary of what that branch wrote).
    L, B, prefix = 36, 16, 65536
    NB = fit_blocks(L, cabi.BF16, 200000)
    g = cabi.layout(L, KVH, QH, D, bs, NB, cabi.BF16)
    per_tok = 2 * KVH * D * 2
    for key, tree in (("config3_shared_prefix", False), ("config3_fork_tree", True)):
        private = rng.integers(0, 4097, size=B)
        tab, lens, points, parent, groups = _fork_tree(rng, NB, prefix, private, bs, tree, 64 // (QH // KVH))
        stride = tab.shape[1]
        dtab = torch.from_numpy(tab).cuda()
        fill(g, C.c_void_p(dtab[0].data_ptr()), prefix, L, False, chunk=4096)
        for b in range(B):                                                        # private tokens, through the branch's own row
            n = int(lens[b]) - points[b]
            if n:
                k = (torch.randn(L, n, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
                v = (torch.randn(L, n, KVH, D, device="cuda") * 0.5).to(torch.bfloat16)
                cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(buf), C.c_void_p(dtab[b].data_ptr()), 0, L, points[b], n,
                          cabi.p(k), cabi.p(v), cabi.BF16, sp)
                torch.cuda.synchronize()
        dlen = torch.from_numpy(lens).cuda()
        max_ctx = int(lens.max())
        q = (torch.randn(L, B, QH, D, device="cuda") * 0.5).to(torch.bfloat16)
        out = torch.zeros_like(q)
        wsb = max(lib.drk_decode_shared_workspace_bytes(C.byref(g), B, max_ctx, prefix),
                  lib.drk_decode_grouped_workspace_bytes_max(C.byref(g), B, max_ctx, cabi.MAX_PREFIX_GROUPS))
        ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
        row = B * QH * D * 2
        garr = cabi.prefix_groups(groups)

        def shared_one(i):
            l = i % L
            if tree:
                cabi.call("drk_paged_decode_attention_grouped", C.byref(g), C.c_void_p(q.data_ptr() + l * row), cabi.p(buf),
                          cabi.p(dtab), stride, cabi.p(dlen), B, max_ctx, garr, len(groups), C.c_void_p(out.data_ptr() + l * row),
                          l, scale, cabi.BF16, None, 0, cabi.p(ws), wsb, sp)
            else:
                cabi.call("drk_paged_decode_attention_shared", C.byref(g), C.c_void_p(q.data_ptr() + l * row), cabi.p(buf),
                          cabi.p(dtab), stride, cabi.p(dlen), B, max_ctx, prefix, C.c_void_p(out.data_ptr() + l * row), l, scale,
                          cabi.BF16, cabi.p(ws), wsb, sp)

        ker_ms = _timed_decode(lib, cabi, shared_one, 72)                         # without the merge
        for i in range(6):
            shared_one(i)
        a0, a1 = ev(), ev()
        a0.record(stream)
        for i in range(72):
            shared_one(i)
        a1.record(stream)
        torch.cuda.synchronize()
        call_ms = a0.elapsed_time(a1) / 72
        distinct = (prefix + int(private.sum())) * per_tok
        in_groups = sum((e - b0) // 64 * 64 * (nb - 1) for _, nb, b0, e in groups)
        res[key] = _entry(
            "decode_group16_kernel<bf16>", "hbm", distinct, ker_ms,
            "config 3: 65536-token prefix shared by 16 branches + private tokens U{0..4096} (sum %d), bf16, %d layers of pages "
            "in the pool; %s; DISTINCT bytes (a page that several branches read is counted once)"
            % (int(private.sum()), L, "a branch forks from the prefix or from an earlier branch at a random block boundary"
               if tree else "every branch forks at the prefix's end"),
            {"with_merge_us": round(call_ms * 1e3, 2), "with_merge_frac": round(distinct / (call_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
             "logical_bytes_per_launch": int(lens.sum()) * per_tok,
             "streamed_bytes_per_launch": (int(lens.sum()) - in_groups) * per_tok,
             "fork_parent": parent, "fork_points": points, "shared_ranges": [list(x) for x in groups]})
        del q, out, ws, dtab

    # ---- config 5: chunked causal prefill to 32 768 tokens in 2 048-token chunks -------------------------
    L, chunk, total = 1, 2048, 32768

    def chunk_flops(pos, m, qh, d):
        return 4.0 * m * (pos + (m + 1) / 2.0) * d * qh

    def prefill_entry(key, kernel, per_chunk, what, extra=None):
        tot_ms, tot_fl = sum(t for t, _ in per_chunk), sum(f for _, f in per_chunk)
        e = {"last_chunk_us": round(per_chunk[-1][0] * 1e3, 1),
             "last_chunk_TFLOPs": round(per_chunk[-1][1] / (per_chunk[-1][0] * 1e-3) / 1e12, 1),
             "last_chunk_frac": round(per_chunk[-1][1] / (per_chunk[-1][0] * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
             "first_chunk_TFLOPs": round(per_chunk[0][1] / (per_chunk[0][0] * 1e-3) / 1e12, 1)}
        e.update(extra or {})
        res[key] = _entry(kernel, "mfma", tot_fl / len(per_chunk), tot_ms / len(per_chunk), what +
                          "; average over the 16 launches (flops = 4 M (pos_start + (M+1)/2) D QH per chunk)", e)

    for key, name, dt in (("config5_prefill_int8", "int8", cabi.INT8), ("config5_prefill_fp8", "fp8", cabi.FP8_E4M3),
                          ("config5_prefill", "bf16", cabi.BF16)):
        NB = fit_blocks(L, dt, 65536)
        g = cabi.layout(L, KVH, QH, D, bs, NB, dt)
        tab, stride, _ = _shuffled_rows(rng, NB, [total // bs])
        dtab = torch.from_numpy(tab).cuda()
        per_chunk = []
        for ps in range(2):                                                       # the first pass warms up
            per_chunk = []
            for c in range(total // chunk):
                k = torch.randn(L, chunk, KVH, D, device="cuda").to(torch.bfloat16)
                v = torch.randn(L, chunk, KVH, D, device="cuda").to(torch.bfloat16)
                q = torch.randn(chunk, QH, D, device="cuda").to(torch.bfloat16)
                o = torch.empty_like(q)
                cabi.call("drk_kv_append_batch", C.byref(g), cabi.p(buf), cabi.p(dtab), 0, L, c * chunk, chunk, cabi.p(k), cabi.p(v),
                          cabi.BF16, sp)
                a0, a1 = ev(), ev()
                a0.record(stream)
                cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), cabi.p(o), 0, c * chunk, chunk,
                          scale, cabi.BF16, None, 0, sp)
                a1.record(stream)
                torch.cuda.synchronize()
                per_chunk.append((a0.elapsed_time(a1), chunk_flops(c * chunk, chunk, QH, D)))
        if dt != cabi.BF16:
            # the last chunk as a perception frame: attention that leaves the rows' log-sum-exps, then the one-walk mass pass
            pos8 = total - chunk
            lse8 = torch.empty(chunk * QH, dtype=torch.float32, device="cuda")
            mass8 = torch.zeros(total // bs, dtype=torch.float32, device="cuda")

            def frame8(with_mass):
                cabi.call("drk_paged_prefill_attention_lse", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), cabi.p(o), 0, pos8, chunk,
                          scale, cabi.BF16, None, 0, cabi.p(lse8), None, 0, sp)
                if with_mass:
                    cabi.call("drk_paged_prefill_attention_mass_lse", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), 0, pos8, chunk,
                              scale, cabi.BF16, cabi.p(lse8), cabi.p(mass8), total // bs, 1, sp)

            frame_us = []
            for with_mass in (False, True):
                frame8(with_mass)
                a0, a1 = ev(), ev()
                a0.record(stream)
                for _ in range(4):
                    frame8(with_mass)
                a1.record(stream)
                torch.cuda.synchronize()
                frame_us.append(round(a0.elapsed_time(a1) / 4 * 1e3, 1))
            prefill_entry(key, "prefill_pp_kernel<%s>" % name, per_chunk,
                          "config 5 over %s pages: causal prefill of 32768 tokens in 16 chunks of 2048 over 16-token pages, 32 Q / 8 KV "
                          "x 128, bf16 queries, codes turned into 16-bit MFMA operands on the way into LDS" % name,
                          {"last_chunk_as_frame": {"attention_us": frame_us[0], "with_one_walk_mass_us": frame_us[1]}})
            del lse8, mass8
    # the same kernel at position 30 720 with fewer workgroups (shorter chunks): microseconds per 64-token tile of the
    # longest walk.  One workgroup per CU either way -- what changes is how much of the chip draws power.
    by_wgs = {}
    for m in (64, 512, 1024, 2048):
        q = torch.randn(m, QH, D, device="cuda").to(torch.bfloat16)
        o = torch.empty_like(q)
        pos = total - chunk
        lib.drk_debug_set_prefill_two_phase(2)                                    # also where the rule would pick the four-wave kernel
        for _ in range(2):
            cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), cabi.p(o), 0, pos, m, scale,
                      cabi.BF16, None, 0, sp)
        a0, a1 = ev(), ev()
        a0.record(stream)
        for _ in range(4):
            cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), cabi.p(o), 0, pos, m, scale,
                      cabi.BF16, None, 0, sp)
        a1.record(stream)
        torch.cuda.synchronize()
        lib.drk_debug_set_prefill_two_phase(1)
        by_wgs[str(m // 64 * KVH)] = round(a0.elapsed_time(a1) / 4 * 1e3 / ((pos + m + 63) // 64), 3)
    # ---- the attention mass of a perception frame: the last chunk (2 048 rows at 30 720) with and without it ----
    q = torch.randn(chunk, QH, D, device="cuda").to(torch.bfloat16)
    o = torch.empty_like(q)
    lse = torch.empty(chunk * QH, dtype=torch.float32, device="cuda")
    mass = torch.zeros(total // bs, dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    ssp = C.c_void_p(side.cuda_stream)
    pos = total - chunk
    ev_a, ev_m = C.c_void_p(), C.c_void_p()
    cabi.call("drk_event_create", C.byref(ev_a))
    cabi.call("drk_event_create", C.byref(ev_m))

    def attn_plain():
        cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), cabi.p(o), 0, pos, chunk, scale,
                  cabi.BF16, None, 0, sp)

    def attn_two_walks():
        attn_plain()
        cabi.call("drk_paged_prefill_attention_mass", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), 0, pos, chunk, scale, cabi.BF16,
                  cabi.p(mass), total // bs, 1, sp)

    def attn_lse(mass_stream):
        if mass_stream is not sp:
            cabi.call("drk_stream_wait_event", sp, ev_m)                           # the pass before still reads q
        cabi.call("drk_paged_prefill_attention_lse", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), cabi.p(o), 0, pos, chunk, scale,
                  cabi.BF16, None, 0, cabi.p(lse), None, 0, sp)
        if mass_stream is not sp:
            cabi.call("drk_event_record", ev_a, sp)
            cabi.call("drk_stream_wait_event", mass_stream, ev_a)
        cabi.call("drk_paged_prefill_attention_mass_lse", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), 0, pos, chunk, scale,
                  cabi.BF16, cabi.p(lse), cabi.p(mass), total // bs, 1, mass_stream)
        if mass_stream is not sp:
            cabi.call("drk_event_record", ev_m, mass_stream)

    def timed(fn, n=6):
        cabi.call("drk_event_record", ev_m, ssp)
        fn(); fn()
        torch.cuda.synchronize()
        a0, a1 = ev(), ev()
        a0.record(stream)
        for _ in range(n):
            fn()
        cabi.call("drk_stream_wait_event", sp, ev_m)
        a1.record(stream)
        torch.cuda.synchronize()
        return round(a0.elapsed_time(a1) / n * 1e3, 1)

    frame_mass = {"attention_us": timed(attn_plain), "with_two_walk_mass_us": timed(attn_two_walks),
                  "with_one_walk_mass_same_stream_us": timed(lambda: attn_lse(sp)),
                  "with_one_walk_mass_second_stream_us": timed(lambda: attn_lse(ssp)),
                  "what": "config 5's last chunk (2048 rows behind 30720 tokens, 32 Q / 8 KV x 128 bf16), per layer: the chunk's "
                          "attention alone; followed by the mass pass that walks the keys twice; by the pass that takes the rows' "
                          "log-sum-exps from the attention call and walks once; and with that pass on a second stream behind an "
                          "event, back to back launches (the next attention call waits for the pass, which reads its Q)"}
    # a short frame behind the same context: 64 rows at 32 704 (the split path for the attention, the mass pass with its
    # walks in parts)
    big = (q, o, lse, chunk, pos)
    chunk = 64
    pos = total - chunk
    q = torch.randn(chunk, QH, D, device="cuda").to(torch.bfloat16)
    o = torch.empty_like(q)
    lse = torch.empty(chunk * QH, dtype=torch.float32, device="cuda")
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos, chunk)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")

    def short_attn():
        cabi.call("drk_paged_prefill_attention_lse", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), cabi.p(o), 0, pos, chunk, scale,
                  cabi.BF16, None, 0, cabi.p(lse), cabi.p(ws), wsb, sp)

    def short_both():
        short_attn()
        cabi.call("drk_paged_prefill_attention_mass_lse", C.byref(g), cabi.p(q), cabi.p(buf), cabi.p(dtab), 0, pos, chunk, scale,
                  cabi.BF16, cabi.p(lse), cabi.p(mass), total // bs, 1, sp)

    frame_mass["short_frame_64_rows"] = {"attention_us": timed(short_attn), "with_one_walk_mass_us": timed(short_both)}
    # ... and 16 rows at 32 752: 64 of a workgroup's 256 rows exist, the other six waves only move tiles
    chunk = 16
    pos = total - chunk
    q = torch.randn(chunk, QH, D, device="cuda").to(torch.bfloat16)
    o = torch.empty_like(q)
    lse = torch.empty(chunk * QH, dtype=torch.float32, device="cuda")
    wsb = lib.drk_prefill_workspace_bytes(C.byref(g), pos, chunk)
    ws = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")
    frame_mass["short_frame_16_rows"] = {"attention_us": timed(short_attn), "with_one_walk_mass_us": timed(short_both)}
    q, o, lse, chunk, pos = big
    # the last chunk's launch once more on constant data (every K and V element 0.5, every Q element 0.25): the same
    # instructions on the same addresses -- what differs is how many bits toggle, i.e. the clock the part holds
    buf[:lib.drk_kv_pool_bytes(C.byref(g))].view(torch.bfloat16).fill_(0.5)
    qc = torch.full_like(q, 0.25)

    def attn_const():
        cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(qc), cabi.p(buf), cabi.p(dtab), cabi.p(o), 0, pos, chunk, scale,
                  cabi.BF16, None, 0, sp)

    const_us = timed(attn_const)
    last_fl = chunk_flops(pos, chunk, QH, D)
    on_const = {"random_data_us": frame_mass["attention_us"], "constant_data_us": const_us,
                "random_data_frac": round(last_fl / (frame_mass["attention_us"] * 1e-6) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                "constant_data_frac": round(last_fl / (const_us * 1e-6) / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                "what": "the last chunk's launch six times back to back, on the pages of the run and on pages and queries that "
                        "hold one constant: same kernel, same addresses, same instruction stream"}
    del qc
    cabi.call("drk_event_destroy", ev_a)
    cabi.call("drk_event_destroy", ev_m)
    res["frame_mass"] = frame_mass
    prefill_entry("config5_prefill", "prefill_ppd_kernel<bf16>", per_chunk,
                  "config 5: causal prefill of 32768 tokens in 16 chunks of 2048 over 16-token pages, 32 Q / 8 KV x 128 bf16",
                  {"us_per_tile_by_workgroups_at_30720": by_wgs, "last_chunk_by_data": on_const})
    del dtab

    # ---- the reference's model shape: 24 Q / 4 KV heads x 256, fp16, 256-token blocks, 16 layers --------------
    L7, KVH7, QH7, D7, bs7, B7, ctx7 = 16, 4, 24, 256, 256, 8, 32768
    nblk = ctx7 // bs7 + 1
    NB7 = B7 * nblk + 8
    g = cabi.layout(L7, KVH7, QH7, D7, bs7, NB7, cabi.F16)
    pool_bytes = lib.drk_kv_pool_bytes(C.byref(g))
    assert pool_bytes <= buf.numel()
    buf[:pool_bytes].view(torch.float16).normal_(0, 0.5)
    dtab = torch.from_numpy(np.stack(np.split(rng.permutation(NB7).astype(np.int32)[:B7 * nblk], B7))).cuda()
    h = torch.float16
    q = (torch.randn(L7, B7, QH7, D7, device="cuda") * 0.5).to(h)
    gate = (torch.randn(L7, B7, QH7, D7, device="cuda") * 0.5).to(h)
    out = torch.empty_like(q)
    dlen = torch.full((B7,), ctx7, dtype=torch.int32, device="cuda")
    wsb = lib.drk_decode_workspace_bytes(C.byref(g), B7, ctx7)
    ws = torch.empty(wsb, dtype=torch.uint8, device="cuda")
    scale7 = float(1.0 / np.sqrt(D7))
    row = B7 * QH7 * D7 * 2
    ms = _timed_decode(lib, cabi, lambda i: cabi.call(
        "drk_paged_decode_attention_gated", C.byref(g), C.c_void_p(q.data_ptr() + (i % L7) * row), cabi.p(buf), cabi.p(dtab), nblk,
        cabi.p(dlen), B7, ctx7, C.c_void_p(out.data_ptr() + (i % L7) * row), i % L7, scale7, cabi.F16,
        C.c_void_p(gate.data_ptr() + (i % L7) * row), D7, cabi.p(ws), wsb, sp), 48)
    res["config7_decode_d256"] = _entry(
        "decode_stream_kernel<f16, 256>", "hbm", B7 * ctx7 * 2 * KVH7 * D7 * 2, ms,
        "the reference's model shape: 24 Q / 4 KV heads x 256, fp16, 256-token blocks shuffled over %d, %d layers of pages; decode "
        "attention of 8 branches x 32768 tokens with the sigmoid gate (applied in the merge, not in this kernel)" % (NB7, L7))
    qc = (torch.randn(chunk, QH7, D7, device="cuda") * 0.5).to(h)
    oc = torch.empty_like(qc)
    pwsb = lib.drk_prefill_workspace_bytes_max(C.byref(g), total, chunk)          # the pieces of the last round's walks
    pws = torch.empty(max(pwsb, 16), dtype=torch.uint8, device="cuda")
    per_chunk = []
    for ps in range(2):
        per_chunk = []
        for c in range(total // chunk):
            a0, a1 = ev(), ev()
            a0.record(stream)
            cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(qc), cabi.p(buf), cabi.p(dtab), cabi.p(oc), c % L7, c * chunk, chunk,
                      scale7, cabi.F16, cabi.p(pws), pwsb, sp)
            a1.record(stream)
            torch.cuda.synchronize()
            per_chunk.append((a0.elapsed_time(a1), chunk_flops(c * chunk, chunk, QH7, D7)))
    whole = []
    lib.drk_debug_set_prefill_pieces(0)
    for c in (0, total // chunk - 1):
        for _ in range(2):
            a0, a1 = ev(), ev()
            a0.record(stream)
            cabi.call("drk_paged_prefill_attention", C.byref(g), cabi.p(qc), cabi.p(buf), cabi.p(dtab), cabi.p(oc), 0, c * chunk, chunk,
                      scale7, cabi.F16, cabi.p(pws), pwsb, sp)
            a1.record(stream)
            torch.cuda.synchronize()
        whole.append(round(a0.elapsed_time(a1) * 1e3, 1))
    lib.drk_debug_set_prefill_pieces(1)
    # the attention mass of a perception frame at this shape: the last chunk, and a 64-row frame behind 32 704 tokens
    # (table of branch 0; the attention call leaves the rows' log-sum-exps, the pass walks the keys once)
    fm7 = {}
    mass7 = torch.zeros(nblk, dtype=torch.float32, device="cuda")
    for rows7 in (chunk, 64):
        pos7 = total - rows7
        q7 = (torch.randn(rows7, QH7, D7, device="cuda") * 0.5).to(h)
        o7 = torch.empty_like(q7)
        lse7 = torch.empty(rows7 * QH7, dtype=torch.float32, device="cuda")

        def attn7():
            cabi.call("drk_paged_prefill_attention_lse", C.byref(g), cabi.p(q7), cabi.p(buf), cabi.p(dtab), cabi.p(o7), 0, pos7, rows7,
                      scale7, cabi.F16, None, 0, cabi.p(lse7), cabi.p(pws), pwsb, sp)

        def both7():
            attn7()
            cabi.call("drk_paged_prefill_attention_mass_lse", C.byref(g), cabi.p(q7), cabi.p(buf), cabi.p(dtab), 0, pos7, rows7,
                      scale7, cabi.F16, cabi.p(lse7), cabi.p(mass7), nblk, 1, sp)

        t = []
        for fn in (attn7, both7):
            fn(); fn()
            a0, a1 = ev(), ev()
            a0.record(stream)
            for _ in range(4):
                fn()
            a1.record(stream)
            torch.cuda.synchronize()
            t.append(round(a0.elapsed_time(a1) / 4 * 1e3, 1))
        fm7["%d_rows" % rows7] = {"attention_us": t[0], "with_one_walk_mass_us": t[1]}
    prefill_entry("config7_prefill_d256", "prefill_d256w_kernel<f16> + prefill_piece_merge_kernel", per_chunk,
                  "the reference's model shape: causal prefill of 32768 tokens in 16 chunks of 2048 over 256-token blocks, 24 Q / 4 KV "
                  "heads x 256, fp16 (the pages hold N(0, 0.5), written beforehand); 384 walks of 128 rows: 256 whole, the last 128 "
                  "in two pieces each and a merge of their rows, timed together",
                  {"first_and_last_chunk_us_with_whole_walks": whole, "frame_mass_behind_32768_tokens": fm7})
    return res
