"""The bench's own line, run the way the driver runs it (a child process, default flags
but for fewer steps), checked for the contract's keys and for the stated targets:
bit-exact migration at >= 75 % of the 8 TB/s HBM peak at the LLaMA-2-7B shape, and a
bit-exact swap round trip at >= 80 % of the host link measured in the same run.  Collected
last: it needs most of the GPU's memory, so the tests before it must have let go of theirs."""
import json
import os
import subprocess
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*flags, timeout=300):
    # the child needs most of the GPU and 36 GiB of pinned host memory: hand back what this
    # process's allocators still cache from the tests before
    import gc
    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    release_pinned = getattr(torch._C, "_host_emptyCache", None)
    if release_pinned is not None:
        release_pinned()
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], cwd=ROOT,
                         capture_output=True, text=True, timeout=timeout)
    if out.returncode != 0:
        print(out.stderr[-6000:])
    assert out.returncode == 0, f"bench.py {' '.join(flags)} exited with {out.returncode}"
    lines = [ln for ln in out.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, f"bench.py must print exactly one line, got {len(lines)}"
    return json.loads(lines[0])


def test_migration_line_meets_the_contract_and_the_target():
    line = run_bench("--steps", "10", "--warmup", "3", timeout=600)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 10 and line["warmup"] == 3
    assert line["unit"] == "GB/s" and line["dtype"] == "u8" and line["vs_baseline"] is None
    assert "cfg2" in line["config"]["workload"] and "model" not in line["config"]
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    # the kernel's average launch and the whole timed region must tell the same story
    assert abs(roof["achieved"] - line["value"]) / line["value"] < 0.03
    assert line["bit_exact"] is True
    cpu = line["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["unit"] == "GB/s" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    assert roof["frac"] >= 0.75, f"migration at {roof['frac']:.3f} of the HBM peak"
    assert "traffic_source" in roof and "profiles/" in roof["traffic_source"]
    assert 0 < line["host_call_us"] < 100                     # one call on an idle stream: microseconds
    # every other configuration rides along in the same line
    configs = line["configs"]
    assert sorted(configs) == ["cfg1", "cfg2_batched", "cfg3", "cfg3_batched", "cfg4", "cfg4_batched", "cfg5"]
    for name in ("cfg1", "cfg2_batched", "cfg3", "cfg3_batched", "cfg4", "cfg4_batched"):
        c = configs[name]
        assert c["bit_exact"] is True, name
        for key in ("GBps", "frac", "us_per_request", "blocks_per_s", "pattern", "kernel"):
            assert key in c, (name, key)
        assert abs(c["frac"] - c["GBps"] / 8000.0) < 1e-3
    assert configs["cfg1"].get("cache_resident") is True and "cache_resident" not in configs["cfg3"]
    assert configs["cfg3"]["frac"] >= 0.75 and configs["cfg4"]["frac"] >= 0.70
    swap = configs["cfg5"]
    assert swap["bit_exact"] is True
    for phase in ("alone", "beside_8_requests", "beside_continuous_migration"):
        assert swap[phase]["swap_out_frac_of_link"] >= 0.80 and swap[phase]["swap_in_frac_of_link"] >= 0.80, (phase, swap)
    assert swap["host_enqueue_us"]["swap_out_beside_8_requests"] <= 1000


def test_swap_line_meets_the_target():
    line = run_bench("--config", "5", "--no-cpu-baseline")
    assert line["unit"] == "GB/s" and line["roofline"]["bound"] == "host link"
    taken = line["default_swap_mode"]["variant"]
    rows = line["swap"][taken]
    assert all(r["round_trip_bit_exact"] for rows_ in line["swap"].values() for r in rows_)
    overlapped = [r for r in rows if r["overlapped_with_migration"]][0]
    assert overlapped["swap_out_frac_of_link"] >= 0.80 and overlapped["swap_in_frac_of_link"] >= 0.80, overlapped
    # the migration beside the swap is not starved by it
    alone = overlapped["migration_ms_alone"]
    beside = sorted(overlapped["migration_ms_beside_swap_out"] + overlapped["migration_ms_beside_swap_in"])
    assert beside[len(beside) // 2] <= 1.25 * alone, overlapped
