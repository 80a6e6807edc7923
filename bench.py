#!/usr/bin/env python3
"""Benchmark of the KV-block migration path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--pattern request|batch]

A *step* is one pass of the hot path over one batch: every request of the configuration
is migrated from the context pools to the decoding pools.  ``--pattern request`` (the
default) issues one ``kvm_migrate`` call per request, as the reference engine does
(distserve/single_stage_engine.py:524-529); ``--pattern batch`` issues one call for the
whole batch.  Pools are resident in HBM before the timed region; timing uses HIP events on
the stream the kernels are launched on.  Prints ONE JSON line.

The default run launches nothing but the migration kernel of the timed workload (warm-up
steps included), so a ``rocprofv3 --kernel-trace --stats`` of the same command shows that
kernel's average duration over the same population of launches.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0   # MI355X published HBM3E bandwidth


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=2, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--pattern", default="request", choices=["request", "batch"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--opt", action="append", default=[], help="kvmove tuning option name=value")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also time the plain contiguous copy kernel (adds launches to a profile)")
    ap.add_argument("--plain-copy-only", type=int, default=0, metavar="MiB",
                    help="launch nothing but plain contiguous copies of this size (counter calibration)")
    return ap.parse_args()


def measured_traffic(config: int, algorithmic_bytes_per_launch: float):
    """HBM bytes per launch from the committed hardware-counter summary of this configuration
    (two rocprofv3 --pmc runs, FETCH_SIZE and WRITE_SIZE, each scaled by a plain copy of
    known size), or None when no summary has been committed for it."""
    import re

    path = os.path.join(ROOT, "profiles", f"kvm_copy_kernel_cfg{config}_pmc.txt")
    if not os.path.exists(path):
        return None
    m = re.search(r"TRAFFIC_PER_ALGORITHMIC_BYTE read=([0-9.]+) write=([0-9.]+)", open(path).read())
    if not m:
        return None
    # algorithmic bytes are half reads and half writes
    return round(algorithmic_bytes_per_launch * (float(m.group(1)) + float(m.group(2))) / 2)


def make_calls(w, pattern):
    if pattern == "request" or w.recycles_blocks:
        return [(c.ctx_idx, c.dec_idx) for c in w.calls]
    return [([b for c in w.calls for b in c.ctx_idx], [b for c in w.calls for b in c.dec_idx])]


def cpu_baseline(w, budget_s=12.0):
    """Reference semantics on the host: torch index_select / cat / narrow / index_copy_ over
    the same block tables (oracle.migrate_cat), on pools compacted to the touched blocks of
    a sample of the requests (bytes moved per request unchanged)."""
    import torch

    import oracle
    from distserve_amd import workloads

    sh = w.shape
    g = oracle.Geom(sh.num_layers, sh.num_kv_heads, sh.block_size, sh.head_dim, sh.dtype_bytes,
                    w.ctx_pp, w.ctx_tp, w.dec_pp, w.dec_tp, w.dec_pp_rank, w.dec_tp_rank)
    sample, blocks = [], 0
    for c in w.calls:
        if blocks + len(c.ctx_idx) > 192 and sample:
            break
        sample.append(c)
        blocks += len(c.ctx_idx)
    # compact: context block j of the sample lives at j, decoding block j at a shuffled slot
    gen = torch.Generator().manual_seed(w.seed)
    perm_src = torch.randperm(blocks, generator=gen).tolist()
    perm_dst = torch.randperm(blocks, generator=gen).tolist()
    calls, at = [], 0
    for c in sample:
        n = len(c.ctx_idx)
        calls.append((perm_src[at:at + n], perm_dst[at:at + n]))
        at += n
    shape_src = w.shape.pool_shape(blocks, w.ctx_pp, w.ctx_tp)
    shape_dst = w.shape.pool_shape(blocks, w.dec_pp, w.dec_tp)
    src_k = [[workloads.fill_uniform(shape_src, w.seed + 10 * p + t) for t in range(w.ctx_tp)] for p in range(w.ctx_pp)]
    src_v = [[workloads.fill_uniform(shape_src, w.seed + 500 + 10 * p + t) for t in range(w.ctx_tp)]
             for p in range(w.ctx_pp)]
    dst_k, dst_v = workloads.fill_canary(shape_dst), workloads.fill_canary(shape_dst)

    def one_pass():
        for ci, di in calls:
            oracle.migrate_cat(g, src_k, ci, di, dst_k)
            oracle.migrate_cat(g, src_v, ci, di, dst_v)

    one_pass()
    t0 = time.perf_counter()
    passes = 0
    while True:
        one_pass()
        passes += 1
        if time.perf_counter() - t0 > budget_s or passes >= 50:
            break
    dt = time.perf_counter() - t0
    payload = blocks * w.payload_bytes_per_block * passes
    return {
        "value": round(2 * payload / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": (f"oracle.migrate_cat (torch index_select/cat/narrow/index_copy_ on CPU tensors), first "
                   f"{len(sample)} of {len(w.calls)} requests = {blocks} blocks, pools compacted to the touched "
                   f"blocks, {passes} passes in {dt:.1f} s; GB/s counts read+write bytes like the GPU figure"),
        "payload_GBps": round(payload / dt / 1e9, 3),
        "us_per_request": round(dt / (passes * len(sample)) * 1e6, 1),
        "host_cpu_count": os.cpu_count(),
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (source and destination pools share one HBM; "
              "there is no sharding or collective on this path); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the KV movement path has no CPU fallback", file=sys.stderr)
        sys.exit(3)

    from distserve_amd import cabi, workloads

    for kv in args.opt:
        name, value = kv.split("=")
        cabi.set_option(name, int(value))

    if args.plain_copy_only:
        torch.cuda.set_device(0)
        nbytes = args.plain_copy_only << 20
        gbps = time_plain_copy(cabi, torch.cuda.current_stream(), nbytes=nbytes, reps=args.steps, warm=args.warmup)
        print(json.dumps({"metric": "plain contiguous copy", "value": gbps, "unit": "GB/s",
                          "bytes_copied_per_call": nbytes, "hbm_bytes_per_call": 2 * nbytes,
                          "launches_per_call": -(-(nbytes // (8 << 20)) // 440), "steps": args.steps}))
        return

    if args.config == 5:
        from bench_swap import run_swap_bench

        print(json.dumps(run_swap_bench(args)))
        return

    w = {1: workloads.config1, 2: workloads.config2, 3: workloads.config3, 4: workloads.config4}[args.config]()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream()
    s = w.shape
    geom = cabi.geom(s.num_layers, s.num_kv_heads, s.block_size, s.head_dim, s.dtype_bytes,
                     w.ctx_pp, w.ctx_tp, w.dec_pp, w.dec_tp, w.dec_pp_rank, w.dec_tp_rank)

    # pools, resident in HBM before anything is timed
    cabi.reset()
    src_k = [[workloads.fill_uniform(w.src_pool_shape(), w.seed + 10 * p + t, "cuda") for t in range(w.ctx_tp)]
             for p in range(w.ctx_pp)]
    src_v = [[workloads.fill_uniform(w.src_pool_shape(), w.seed + 500 + 10 * p + t, "cuda") for t in range(w.ctx_tp)]
             for p in range(w.ctx_pp)]
    dst_k = workloads.fill_canary(w.dst_pool_shape(), "cuda")
    dst_v = workloads.fill_canary(w.dst_pool_shape(), "cuda")
    for p in range(w.ctx_pp):
        for t in range(w.ctx_tp):
            cabi.register_source(w.ctx_pp, w.ctx_tp, p, t, s.num_layers, s.num_kv_heads,
                                 src_k[p][t].data_ptr(), src_v[p][t].data_ptr(),
                                 src_k[p][t].numel() * s.dtype_bytes)
    calls = [(cabi.index_array(ci), cabi.index_array(di)) for ci, di in make_calls(w, args.pattern)]
    plan = cabi.migrate_plan(geom, max(len(c[0]) for c in calls), dst_k.data_ptr(), dst_v.data_ptr())
    launches_per_step = 0
    for ci, _ in calls:
        launches_per_step += cabi.migrate_plan(geom, len(ci), dst_k.data_ptr(), dst_v.data_ptr())["launches"]

    def step():
        for ci, di in calls:
            cabi.migrate(geom, ci, di, dst_k.data_ptr(), dst_v.data_ptr(), w.dst_blocks, stream.cuda_stream)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t_host0 = time.perf_counter()
    start.record(stream)
    for _ in range(args.steps):
        step()
    stop.record(stream)
    t_host_enqueued = time.perf_counter()
    torch.cuda.synchronize()
    elapsed_ms = start.elapsed_time(stop)
    ms_per_step = elapsed_ms / args.steps

    payload = w.payload_bytes                       # bytes the decoding rank receives per step
    hbm_bytes = 2 * payload                         # each byte read once and written once
    hbm_gbps = hbm_bytes / (ms_per_step * 1e-3) / 1e9
    launch_us = elapsed_ms * 1e3 / (args.steps * launches_per_step)
    bytes_per_launch = hbm_bytes / launches_per_step

    bit_exact = None
    if not args.no_verify:
        bit_exact = verify(w, src_k, src_v, dst_k, dst_v)

    copy_ceiling = None
    if args.calibrate_copy:
        copy_ceiling = time_plain_copy(cabi, stream)

    out = {
        "metric": "KV migration GB/s (% of HBM peak) + us/request at LLaMA-2-7B shape" if args.config == 2
                  else f"KV migration GB/s (% of HBM peak) + us/request, {w.name}",
        "value": round(hbm_gbps, 2), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {
            "workload": (f"{w.name}: {len(w.calls)} requests, {w.total_blocks} blocks of "
                         f"{w.payload_bytes_per_block} B (K+V, decoding rank's share), context pp{w.ctx_pp}/tp{w.ctx_tp}"
                         f" -> decoding pp{w.dec_pp}/tp{w.dec_tp} rank ({w.dec_pp_rank},{w.dec_tp_rank}), "
                         f"pools {w.src_blocks}/{w.dst_blocks} blocks, seed {w.seed}"),
            "pattern": "one call per request" if len(calls) > 1 else "one call per batch",
            "value_counts": "HBM bytes read + written (2 x payload) per second",
            "tuning": {k: cabi.get_option(k) for k in ("tile_bytes", "threads", "unroll", "nt_load", "nt_store")},
        },
        "payload_GBps": round(payload / (ms_per_step * 1e-3) / 1e9, 2),
        "frac_of_hbm_peak": round(hbm_gbps / HBM_PEAK_GBPS, 4),
        "us_per_request": round(ms_per_step * 1e3 / len(w.calls), 2),
        "blocks_per_s": round(w.total_blocks / (ms_per_step * 1e-3), 1),
        "host_enqueue_us_per_call": round((t_host_enqueued - t_host0) * 1e6 / (args.steps * len(calls)), 2),
        "bit_exact": bit_exact,
        "roofline": {
            "bound": "hbm", "achieved": round(bytes_per_launch / (launch_us * 1e-6) / 1e9, 2), "peak": HBM_PEAK_GBPS,
            "unit": "GB/s", "frac": round(bytes_per_launch / (launch_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic(args.config, bytes_per_launch),
            "kernel": "kvm_copy_kernel<u32x4>", "launches_per_step": launches_per_step,
            "avg_launch_us": round(launch_us, 2), "algorithmic_bytes_per_launch": round(bytes_per_launch),
            "workgroups_per_block": plan["workgroups_per_block"], "workgroup_size": plan["threads"],
        },
    }
    if copy_ceiling is not None:
        out["plain_copy_GBps"] = copy_ceiling
    if not args.no_cpu_baseline:
        del src_k, src_v, dst_k, dst_v
        torch.cuda.empty_cache()
        out["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(out))


def verify(w, src_k, src_v, dst_k, dst_v) -> bool:
    """Every migrated block equals its source rectangle (torch gather on the GPU, an
    implementation independent of the kernel); for recycled tables only the blocks whose
    last writer is known are checked."""
    import torch

    last_writer = {}
    for c in w.calls:
        for a, b in zip(c.ctx_idx, c.dec_idx):
            last_writer[b] = a
    # a context block overwritten later by another request's prefill does not occur here:
    # sources are never written by this benchmark
    dec = torch.tensor(list(last_writer.keys()), device="cuda")
    ctx = torch.tensor(list(last_writer.values()), device="cuda")
    L_d, H_d = w.shape.num_layers // w.dec_pp, w.shape.num_kv_heads // w.dec_tp
    L_c, H_c = w.shape.num_layers // w.ctx_pp, w.shape.num_kv_heads // w.ctx_tp
    l0, h0 = w.dec_pp_rank * L_d, w.dec_tp_rank * H_d
    ok = True
    for src, dst in ((src_k, dst_k), (src_v, dst_v)):
        for i0 in range(0, dec.numel(), 64):
            d = dst.view(torch.int16)[dec[i0:i0 + 64]]
            for p in range(w.ctx_pp):
                for t in range(w.ctx_tp):
                    la, lb = max(l0, p * L_c), min(l0 + L_d, (p + 1) * L_c)
                    ha, hb = max(h0, t * H_c), min(h0 + H_d, (t + 1) * H_c)
                    if la >= lb or ha >= hb:
                        continue
                    got = d[:, la - l0:lb - l0, ha - h0:hb - h0]
                    want = src[p][t].view(torch.int16)[ctx[i0:i0 + 64], la - p * L_c:lb - p * L_c,
                                                       ha - t * H_c:hb - t * H_c]
                    ok = ok and bool(torch.equal(got, want))
    return ok


def time_plain_copy(cabi, stream, nbytes=4 << 30, reps=10, warm=2):
    import torch

    a = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    b = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    a.fill_(3)
    for _ in range(warm):
        cabi.copy_plain(b.data_ptr(), a.data_ptr(), nbytes, stream.cuda_stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        cabi.copy_plain(b.data_ptr(), a.data_ptr(), nbytes, stream.cuda_stream)
    e1.record(stream)
    torch.cuda.synchronize()
    return round(2 * nbytes * reps / (e0.elapsed_time(e1) * 1e-3) / 1e9, 2)


if __name__ == "__main__":
    main()
