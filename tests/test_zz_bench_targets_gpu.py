"""The bench's own line, run the way the driver runs it (a child process, default flags
but for fewer steps), checked for the contract's keys and for the stated targets:
bit-exact migration at >= 75 % of the 8 TB/s HBM peak at the LLaMA-2-7B shape, and a
bit-exact swap round trip at >= 80 % of the host link measured in the same run.  Collected
last: it needs most of the GPU's memory, so the tests before it must have let go of theirs."""
import functools
import json
import os
import re
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


@functools.lru_cache(maxsize=None)
def default_line():
    return run_bench("--steps", "10", "--warmup", "3", timeout=600)


def probe_rows(section: int):
    """Rows of one section of the stand-alone ceiling probe, split into their columns."""
    exe = os.path.join(ROOT, "tests", "hbm_probe", "hbm_probe")
    assert os.path.exists(exe), "tests/hbm_probe/hbm_probe is not built: make -C tests/hbm_probe"
    out = subprocess.run([exe, "--section", str(section)], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr[-2000:]
    rows = [re.split(r"\s{2,}", ln.strip()) for ln in out.stdout.splitlines()]
    return [r for r in rows if len(r) >= 6 and re.fullmatch(r"[0-9.]+", r[-1]) and re.fullmatch(r"[0-9.]+", r[-2])]


def test_migration_line_meets_the_contract_and_the_target():
    line = default_line()
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
    assert sorted(configs) == ["cfg1", "cfg2_batched", "cfg2_handoff", "cfg2_ipc", "cfg3", "cfg3_batched", "cfg4",
                               "cfg4_batched", "cfg5"]
    hand = configs["cfg2_handoff"]
    assert hand["bit_exact"] is True and hand["block_tables_equal_workload"] is True and hand["frac_of_hbm_peak"] >= 0.70
    assert hand["transmission_us_per_request"] > hand["transmission_us_per_request_stamped_at_enqueue"] > 0
    by_size = hand["by_request_blocks"]
    assert sorted(by_size) == ["1", "16", "4"], by_size
    for n, r in by_size.items():
        assert r["bit_exact"] is True and r["prompt_tokens"] == 16 * int(n), (n, r)
        assert 0 < r["host_us_per_request"] <= r["us_per_request"], (n, r)
    assert by_size["16"]["longer_leg"] == "gpu" and by_size["16"]["host_us_per_request"] < 30, \
        f"performance, not correctness: {by_size['16']}"
    assert configs["cfg2_ipc"].get("bit_exact") is True, configs["cfg2_ipc"]
    assert configs["cfg2_ipc"]["other_over_this_process"] >= 0.85, \
        f"performance, not correctness: pools of another process at {configs['cfg2_ipc']}"
    for name in ("cfg1", "cfg2_batched", "cfg3", "cfg3_batched", "cfg4", "cfg4_batched"):
        c = configs[name]
        assert c["bit_exact"] is True, name
        for key in ("GBps", "frac", "us_per_request", "blocks_per_s", "pattern", "ms_per_step", "ms_per_step_median",
                    "ms_per_step_min", "roofline", "cpu_baseline"):
            assert key in c, (name, key)
        assert abs(c["frac"] - c["GBps"] / 8000.0) < 1e-3
        assert c["ms_per_step_min"] <= c["ms_per_step_median"]
        # every configuration's own roofline record and its own CPU figure from this run
        r = c["roofline"]
        for key in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "launches_per_step", "avg_launch_us",
                    "algorithmic_bytes_per_launch"):
            assert key in r, (name, key)
        assert r["bound"] == "hbm" and r["peak"] == 8000.0 and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
        assert abs(r["achieved"] - r["algorithmic_bytes_per_launch"] / r["avg_launch_us"] / 1e3) / r["achieved"] < 1e-3
        cpu = c["cpu_baseline"]
        assert cpu["kind"] == "port" and cpu["unit"] == "GB/s" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    # counted traffic comes from the committed counter summary of the very kernel that ran, or not at all
    for name in ("cfg3", "cfg4"):
        r = configs[name]["roofline"]
        assert r["traffic"] is None or (r["kernel"] in open(os.path.join(
            ROOT, r["traffic_source"].split(":")[0])).read()), (name, r)
    assert configs["cfg1"].get("cache_resident") is True and "cache_resident" not in configs["cfg3"]
    # measured 0.81-0.84 and 0.73-0.77 over a dozen boxes; the bounds leave room for a slower one
    assert configs["cfg3"]["frac"] >= 0.75 and configs["cfg4"]["frac"] >= 0.67, \
        f"performance, not correctness: cfg3 {configs['cfg3']['frac']}, cfg4 {configs['cfg4']['frac']}"
    swap = configs["cfg5"]
    assert swap["bit_exact"] is True
    assert swap["roofline"]["bound"] == "host link" and swap["roofline"]["frac"] >= 0.80
    assert swap["cpu_baseline"]["kind"] == "port" and swap["cpu_baseline"]["value"] > 0
    # swap-out and swap-in in flight together, each against the link measured both ways at once
    # (the denominators are two large copies in flight both ways, which the copy engines split unevenly and not the
    # same way on every box: 49-52 GB/s down, 30-57 up; the swap's own rates are steadier than what they are read against)
    duplex = swap["duplex"]
    assert duplex["round_trip_bit_exact"] is True
    assert duplex["swap_out_frac_of_duplex_link"] >= 0.70 and duplex["swap_in_frac_of_duplex_link"] >= 0.70, \
        f"performance, not correctness: {duplex}"
    assert duplex["swap_out_GBps"] >= 40 and duplex["swap_in_GBps"] >= 40, f"performance, not correctness: {duplex}"
    # the migration beside a swap loses a few percent, not more
    mig = swap["migration_ms"]
    beside = sorted(mig["beside_swap_out"] + mig["beside_swap_in"])
    assert beside[len(beside) // 2] <= 1.08 * mig["alone"], f"performance, not correctness: {mig}"
    for phase in ("alone", "beside_8_requests", "beside_continuous_migration"):
        assert swap[phase]["swap_out_frac_of_link"] >= 0.80 and swap[phase]["swap_in_frac_of_link"] >= 0.80, (phase, swap)
    assert swap["host_enqueue_us"]["swap_out_beside_8_requests"] <= 1000


def test_configurations_3_and_4_reach_what_the_plainest_kernel_reaches_on_their_geometry():
    """The probe's block-table kernel has no segments, no index search and no division by a
    run-time value: what it reaches on configuration 4's geometry (8 KiB of every 16 KiB from
    two pools, blocks placed at random on both sides) is what the memory system gives that
    access pattern.  The migration kernel, with all its generality, must be within a few
    percent of it on the same box."""
    table = probe_rows(3)
    rows = [r for r in table if r[0] == "70B 8 KiB of 16 KiB" and r[1] == "random" and r[2] == "random"]
    per_request = [float(r[-1]) for r in rows if r[3] == "272"]
    long_launch = [float(r[-1]) for r in rows if r[3] == "1024"]
    assert len(per_request) >= 3 and len(long_launch) == 3, rows      # three workgroup orders each (272 blocks: twice)
    assert all(3000 < v < 8000 for v in per_request + long_launch), rows
    configs = default_line()["configs"]
    note = "performance, not correctness (bit-exactness is asserted elsewhere): "
    assert configs["cfg4"]["GBps"] >= 0.85 * max(per_request), note + f"cfg4 {configs['cfg4']['GBps']} vs probe {per_request}"
    assert configs["cfg4_batched"]["GBps"] >= 0.85 * max(long_launch), \
        note + f"cfg4 merged {configs['cfg4_batched']['GBps']} vs probe {long_launch}"
    # configuration 3's geometry: whole blocks, 80 KiB pieces of two pools side by side
    rows = [r for r in table if r[0] == "13B 2 x 80 KiB" and r[1] == "random" and r[2] == "random"]
    per_request = [float(r[-1]) for r in rows if r[3] == "72"]
    assert len(per_request) == 3, rows
    assert configs["cfg3"]["GBps"] >= 0.85 * max(per_request), note + f"cfg3 {configs['cfg3']['GBps']} vs probe {per_request}"


def test_swap_line_meets_the_target():
    line = run_bench("--config", "5", "--no-cpu-baseline")
    assert line["unit"] == "GB/s" and line["roofline"]["bound"] == "host link"
    for name, d in line["swap_duplex"].items():
        assert d["round_trip_bit_exact"] is True, name
    d = line["swap_duplex"][line["default_swap_mode"]["variant"]]
    assert d["swap_out_frac_of_duplex_link"] >= 0.70 and d["swap_in_frac_of_duplex_link"] >= 0.70, \
        f"performance, not correctness: {d}"
    taken = line["default_swap_mode"]["variant"]
    rows = line["swap"][taken]
    assert all(r["round_trip_bit_exact"] for rows_ in line["swap"].values() for r in rows_)
    overlapped = [r for r in rows if r["overlapped_with_migration"]][0]
    assert overlapped["swap_out_frac_of_link"] >= 0.80 and overlapped["swap_in_frac_of_link"] >= 0.80, overlapped
    # the migration beside the swap is not starved by it
    alone = overlapped["migration_ms_alone"]
    beside = sorted(overlapped["migration_ms_beside_swap_out"] + overlapped["migration_ms_beside_swap_in"])
    assert beside[len(beside) // 2] <= 1.10 * alone, f"performance, not correctness: {overlapped}"


@pytest.mark.parametrize("pattern", ["handoff", "scheduler", "scheduler-batched"])
def test_hand_off_lines_are_bit_exact_and_keep_the_workloads_tables(pattern):
    """The whole hand-off (block allocation, the torch op, release of the context blocks), alone
    or driven by the decoding scheduler: same bytes, same block tables, and the host work per
    request stays a fraction of the copy."""
    line = run_bench("--config", "2", "--pattern", pattern, "--steps", "5", "--warmup", "2")
    assert line["bit_exact"] is True and line["block_tables_equal_workload"] is True
    assert line["unit"] == "GB/s" and line["frac_of_hbm_peak"] >= 0.70, line["frac_of_hbm_peak"]
    assert 0 < line["host_us_per_request"] < line["us_per_request"]
    # the end stamped after the copy covers it; stamped at the return of the calls it does not
    assert line["transmission_us_per_request"] > line["transmission_us_per_request_stamped_at_enqueue"]
    if pattern.startswith("scheduler"):
        assert "post_process" in line["config"]["pattern"]


def test_hand_off_by_request_size_shows_where_the_host_is_the_longer_leg():
    """`--request-blocks N ...`: the hand-off over requests of one size each.  The host's share per
    request does not depend on the size; the copy's does, so short prompts are host-bound and the
    record says from where on they are not."""
    line = run_bench("--pattern", "handoff", "--request-blocks", "2", "16", "64", "--steps", "5", "--warmup", "2")
    rows = line["by_request_blocks"]
    assert sorted(rows) == ["16", "2", "64"]
    for n, r in rows.items():
        assert r["bit_exact"] is True and r["block_tables_equal_workload"] is True, n
        assert r["prompt_tokens"] == int(n) * 16 and 0 < r["host_us_per_request"] <= r["us_per_request"]
        assert set(r["host_us_per_request_by_step"]) == {"allocate", "migrate_call", "release"}
    assert rows["64"]["copy_alone_us_per_request"] > 4 * rows["16"]["copy_alone_us_per_request"] / 2
    assert rows["64"]["longer_leg"] == "gpu", f"performance, not correctness: {rows['64']}"
    # the host's share is a per-request constant: within a factor of two from 2 to 64 blocks
    assert rows["64"]["host_us_per_request"] <= 2 * rows["2"]["host_us_per_request"], \
        f"performance, not correctness: {rows}"


def test_migration_out_of_another_process_runs_at_the_speed_of_local_pools():
    """`--pattern ipc`: the context pools live in a child process and are read through their
    hipIpc mapping; the same calls out of identical local pools are timed beside them."""
    line = run_bench("--pattern", "ipc", "--steps", "10", "--warmup", "2", timeout=600)
    assert line["bit_exact"] is True and line["bit_exact_by_source"] == {"other_process": True, "this_process": True}
    assert line["context_process_pid"] != line["this_pid"] and line["mappings_opened"] == 2
    assert line["frac_of_hbm_peak"] >= 0.70
    assert line["other_over_this_process"] >= 0.85, f"performance, not correctness: {line}"
