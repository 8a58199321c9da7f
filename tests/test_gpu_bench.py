"""GPU: every workload of bench.py runs to its one JSON line on a reduced number of layers and steps --
the entry points are used there the way a caller would (workspaces sized once for the largest case, one
captured graph per step), which is how a change of a size contract shows."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
KEYS = {"metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
        "dtype", "data", "config", "roofline", "cpu_baseline"}


@pytest.mark.parametrize("extra", [[], ["--ctx-mode", "uniform", "--no-other-configs"], ["--no-plan", "--no-other-configs"],
                                   ["--no-fused-append", "--no-graph", "--no-other-configs"], ["--config", "3"], ["--config", "3", "--forks", "prefix"],
                                   ["--config", "3", "--shared-kernel", "pair"], ["--config", "4"], ["--config", "4", "--kv-dtype", "fp8"],
                                   ["--config", "5"], ["--config", "5", "--kv-dtype", "int8"], ["--config", "6"], ["--config", "7"]],
                         ids=lambda e: "-".join(x.strip("-") for x in e) or "default")
def test_bench_workload_runs(dev, extra):
    cmd = [sys.executable, os.path.join(ROOT, "bench.py"), "--layers", "2", "--steps", "2", "--warmup", "1", "--no-cpu-baseline"] + extra
    r = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    j = json.loads(lines[0])
    assert KEYS <= set(j) and j["n_gpus"] == 1 and j["value"] > 0 and "workload" in j["config"]
    if not extra:
        # the default line carries the dominant kernel of every other configuration, each with its own roofline entry
        other = j["other_configs"]
        assert set(other) == {"config3_shared_prefix", "config3_fork_tree", "config4_int8", "config4_fp8", "config4_int8_append",
                              "config4_fp8_append", "config5_prefill", "config5_prefill_int8", "config5_prefill_fp8",
                              "config7_decode_d256", "config7_prefill_d256", "frame_mass"}
        assert len(other["config3_fork_tree"]["shared_ranges"]) >= 3
        fm = other.pop("frame_mass")
        assert fm["attention_us"] < fm["with_one_walk_mass_same_stream_us"] < fm["with_two_walk_mass_us"]
        for rows in ("short_frame_64_rows", "short_frame_16_rows"):
            assert 0 < fm[rows]["attention_us"] < fm[rows]["with_one_walk_mass_us"] < 3 * fm[rows]["attention_us"]
        by_data = other["config5_prefill"]["last_chunk_by_data"]                   # the same launch on constant data is not slower
        assert 0 < by_data["constant_data_us"] <= by_data["random_data_us"] * 1.05
        for name, e in other.items():
            assert 0 < e["frac"] < 1 and e["avg_launch_us"] > 0 and e["peak"] in (8000.0, 2500.0), name
        assert j["hbm_read_probe_permuted_4KiB_GBps"] > 1000 and j["mfma_bf16_probe_TFLOPs"] > 500


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], cwd=ROOT, capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "ONE GPU" in (r.stdout + r.stderr)
