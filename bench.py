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
INFINITY_CACHE_BYTES = 256 << 20   # MI355X last-level cache in front of HBM


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=0, choices=[0, 1, 2, 3, 4, 5],
                    help="one configuration only (its full record, nothing else launched); default 0: configuration 2 "
                         "as the headline and every other configuration after it, in one line")
    ap.add_argument("--ctx-tp", type=int, default=0,
                    help="configuration 4 only: context tensor-parallel size. 2 is the configuration itself (8 KiB runs "
                         "at a 16 KiB source stride); 4 moves the same bytes from dense source pools, for comparison")
    ap.add_argument("--fresh-pools", action="store_true",
                    help="configurations 2-4, a comparison: block managers that have just started (free lists "
                         "0..n-1, a request's blocks are neighbours) instead of pools in service (shuffled lists)")
    ap.add_argument("--pattern", default="request",
                    choices=["request", "batch", "handoff", "handoff-batched", "scheduler", "scheduler-batched", "ipc"],
                    help="handoff*: the same requests through Worker / BlockManager / the migration handoff "
                         "(torch ops, block allocation and release included), one call per request or one per batch; "
                         "scheduler*: the same, with the decoding scheduler's post_process deciding acceptance "
                         "(bridge queue -> scheduler -> engine -> op), batch_migrations off or on; "
                         "ipc: configuration 2's shape with the context pools in ANOTHER process (memory handles "
                         "over a pipe, hipIpc mapping), against the same pools in this process")
    ap.add_argument("--request-blocks", type=int, nargs="*", default=None, metavar="N",
                    help="handoff*/scheduler* patterns: instead of a configuration, 48 requests of N blocks each at the "
                         "LLaMA-2-7B shape, one record per N (what the hand-off costs by prompt length)")
    ap.add_argument("--ipc-child", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-verify", action="store_true")
    ap.add_argument("--kernel-digest", action="store_true",
                    help="print the digest of the kernels' source (what a counter summary under profiles/ records) and exit")
    ap.add_argument("--opt", action="append", default=[], help="kvmove tuning option name=value")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also time the plain contiguous copy kernel (adds launches to a profile)")
    ap.add_argument("--swap-blocks", type=int, default=0, help="config 5: blocks to swap (default 2048)")
    ap.add_argument("--swap-shape", type=str, default="", metavar="L,H,D",
                    help="config 5: local layers, KV heads and head_dim of the pools instead of the LLaMA-2-7B "
                         "shape, e.g. 12,12,64 (288 KiB slabs) or 80,2,128 (640 KiB slabs)")
    ap.add_argument("--swap-wgs", type=str, nargs="*", default=None, metavar="N or OUT:IN",
                    help="config 5: workgroup counts to try for the swap kernel beside the library's own, one number "
                         "for both directions or swap-out:swap-in")
    ap.add_argument("--swap-kernel-only", action="store_true",
                    help="config 5: time the copy kernel's variants only, not the copy engines'")
    ap.add_argument("--plain-copy-only", type=int, default=0, metavar="MiB",
                    help="launch nothing but plain contiguous copies of this size (counter calibration)")
    return ap.parse_args()


def kernel_source_digest() -> str:
    """First 16 hex digits of the SHA-256 of the kernels' source: the text of kvmove.hip from
    the kernel-argument layout to the end of the device code (host-side edits do not change
    it).  A counter summary under profiles/ carries the digest of the source it was taken
    with (``KERNEL_SOURCE_DIGEST``; ``python3 bench.py --kernel-digest`` prints it)."""
    import hashlib

    text = open(os.path.join(ROOT, "distserve_amd", "csrc", "kvmove.hip")).read()
    begin = text.index("// ------------------------------------------------------------------ kernel argument")
    end = text.index("// --------------------------------------------------------------------------- host")
    return hashlib.sha256(text[begin:end].encode()).hexdigest()[:16]


def measured_traffic(config: int, kernel: str, algorithmic_bytes_per_launch: float):
    """(HBM bytes per launch, where the figure comes from).  Hardware counters cannot be read
    inside this run: the ratio of counted to algorithmic bytes is taken from the committed
    counter summary of this configuration's kernel (two rocprofv3 --pmc runs, FETCH_SIZE and
    WRITE_SIZE, each scaled by a plain copy of known size) and applied to this run's
    algorithmic bytes.  The summary names the kernel it was taken with (a line
    ``KERNEL_OF_RECORD <name>``) and the digest of the kernel source it was built from
    (``KERNEL_SOURCE_DIGEST``); (None, why) when no summary has been committed for the
    configuration, when it is of another kernel than this run's, or when the kernels' source
    has changed since."""
    import re

    name = f"profiles/kvm_copy_kernel_cfg{config}_pmc.txt"
    path = os.path.join(ROOT, name)
    if not os.path.exists(path):
        return None, None
    text = open(path).read()
    of_record = re.search(r"^KERNEL_OF_RECORD (.+)$", text, flags=re.M)
    if not of_record or of_record.group(1).strip() != kernel:
        return None, (f"{name} was taken with {of_record.group(1).strip() if of_record else 'an unnamed kernel'}, "
                      f"this run used {kernel}: not applied")
    digest = re.search(r"^KERNEL_SOURCE_DIGEST ([0-9a-f]+)$", text, flags=re.M)
    if not digest or digest.group(1) != kernel_source_digest():
        return None, (f"{name} was taken with kernel source {digest.group(1) if digest else '(no digest)'}, "
                      f"this tree's is {kernel_source_digest()}: not applied")
    m = re.search(r"TRAFFIC_PER_ALGORITHMIC_BYTE read=([0-9.]+) write=([0-9.]+)", text)
    if not m:
        return None, None
    # algorithmic bytes are half reads and half writes
    ratio = (float(m.group(1)) + float(m.group(2))) / 2
    return round(algorithmic_bytes_per_launch * ratio), (
        f"{name}: counted / algorithmic bytes = {ratio:.5f}, from the committed rocprofv3 counter runs of this "
        "kernel, not from this run")


def make_calls(w, pattern):
    """Index lists of the calls of one step.  "request": one call per request.  "batch": one
    call for everything; where the requests recycle block ids (configuration 4) that is not
    possible, and consecutive requests are merged for as long as no block id, on either
    side, occurs twice in the call -- what a decoding scheduler that batches its accepted
    requests can do between two releases of context blocks."""
    if pattern == "request":
        return [(c.ctx_idx, c.dec_idx) for c in w.calls]
    if not w.recycles_blocks:
        return [([b for c in w.calls for b in c.ctx_idx], [b for c in w.calls for b in c.dec_idx])]
    groups, ctx_seen, dec_seen = [], set(), set()
    for c in w.calls:
        if not groups or ctx_seen & set(c.ctx_idx) or dec_seen & set(c.dec_idx):
            groups.append(([], []))
            ctx_seen, dec_seen = set(), set()
        groups[-1][0].extend(c.ctx_idx)
        groups[-1][1].extend(c.dec_idx)
        ctx_seen |= set(c.ctx_idx)
        dec_seen |= set(c.dec_idx)
    return groups


def cpu_baseline(w, budget_s=12.0, max_blocks=192, max_payload_bytes=2 << 30):
    """Reference semantics on the host: torch index_select / cat / narrow / index_copy_ over
    the same block tables (oracle.migrate_cat), on pools compacted to the touched blocks of
    a sample of the requests (bytes moved per request unchanged).  The sample is the first
    requests up to `max_blocks` blocks and `max_payload_bytes` of payload (at least one
    request), timed for about `budget_s` seconds."""
    import torch

    import oracle
    from distserve_amd import workloads

    sh = w.shape
    g = oracle.Geom(sh.num_layers, sh.num_kv_heads, sh.block_size, sh.head_dim, sh.dtype_bytes,
                    w.ctx_pp, w.ctx_tp, w.dec_pp, w.dec_tp, w.dec_pp_rank, w.dec_tp_rank)
    sample, blocks = [], 0
    max_blocks = max(1, min(max_blocks, max_payload_bytes // w.payload_bytes_per_block))
    for c in w.calls:
        if blocks + len(c.ctx_idx) > max_blocks and sample:
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


def load_workload(config: int, ctx_tp=None, fresh_pools=False):
    from distserve_amd import workloads

    if config == 4 and (ctx_tp or fresh_pools):
        return workloads.config4(ctx_tp=ctx_tp or 2, fresh_pools=fresh_pools)
    if config in (2, 3) and fresh_pools:
        return {2: workloads.config2, 3: workloads.config3}[config](fresh_pools=True)
    return {1: workloads.config1, 2: workloads.config2, 3: workloads.config3, 4: workloads.config4}[config]()


def host_call_cost_us(cabi, geom, w, dst_k, dst_v, stream, calls=64):
    """Host time of one kvm_migrate call with nothing queued behind it: one-block calls, each
    issued on an idle stream and timed up to its return (validation, argument build and the
    launch), the GPU drained before the next.  Median and best of `calls`."""
    import torch

    first = w.calls[0]
    ci, di = cabi.index_array(first.ctx_idx[:1]), cabi.index_array(first.dec_idx[:1])
    costs = []
    for _ in range(calls + 8):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cabi.migrate(geom, ci, di, dst_k.data_ptr(), dst_v.data_ptr(), w.dst_blocks, stream.cuda_stream)
        costs.append((time.perf_counter() - t0) * 1e6)
    torch.cuda.synchronize()
    costs = sorted(costs[8:])
    return round(costs[len(costs) // 2], 2), round(costs[0], 2)


def bench_migrate(config: int, patterns, steps: int, warmup: int, verify_result: bool = True,
                  calibrate_copy: bool = False, ctx_tp=None, fresh_pools=False):
    """Times one migration workload under every call pattern of `patterns` ("request", "batch"),
    all on ONE set of pools (two patterns of a configuration are then compared on the same
    memory); returns (records in the order of `patterns`, workload).  Pools are made, timed
    and freed inside."""
    import gc

    import torch

    from distserve_amd import cabi, workloads

    w = load_workload(config, ctx_tp, fresh_pools)
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
    payload = w.payload_bytes                       # bytes the decoding rank receives per step
    hbm_bytes = 2 * payload                         # each byte read once and written once
    cache_resident = 2 * hbm_bytes <= INFINITY_CACHE_BYTES
    records = []
    for pattern in patterns:
        if records:
            # the next pattern must write every block itself
            dst_k.view(torch.int16).fill_(workloads.CANARY_BITS)
            dst_v.view(torch.int16).fill_(workloads.CANARY_BITS)
        calls = [(cabi.index_array(ci), cabi.index_array(di)) for ci, di in make_calls(w, pattern)]
        plan = cabi.migrate_plan(geom, max(len(c[0]) for c in calls), dst_k.data_ptr(), dst_v.data_ptr(), w.dst_blocks)
        launches_per_step = 0
        for ci, _ in calls:
            launches_per_step += cabi.migrate_plan(geom, len(ci), dst_k.data_ptr(), dst_v.data_ptr(),
                                                   w.dst_blocks)["launches"]

        def step():
            for ci, di in calls:
                cabi.migrate(geom, ci, di, dst_k.data_ptr(), dst_v.data_ptr(), w.dst_blocks, stream.cuda_stream)

        for _ in range(warmup):
            step()
        # no collector pass inside the timed region (a full one over torch's modules takes 35 ms)
        gc.collect()
        gc.freeze()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(steps):
            step()
        stop.record(stream)
        torch.cuda.synchronize()
        elapsed_ms = start.elapsed_time(stop)
        ms_per_step = elapsed_ms / steps

        # a second pass with an event between steps, for the spread (median and best step)
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        marks[0].record(stream)
        for i in range(steps):
            step()
            marks[i + 1].record(stream)
        torch.cuda.synchronize()
        per_step_ms = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(steps))

        hbm_gbps = hbm_bytes / (ms_per_step * 1e-3) / 1e9
        launch_us = elapsed_ms * 1e3 / (steps * launches_per_step)
        bytes_per_launch = hbm_bytes / launches_per_step

        bit_exact = verify(w, src_k, src_v, dst_k, dst_v) if verify_result else None
        host_call_us, host_call_us_min = host_call_cost_us(cabi, geom, w, dst_k, dst_v, stream)

        tuning = {"threads": plan["threads"], "vectors_per_lane": plan["vectors_per_lane"],
                  "pairs_per_launch": plan["pairs_per_launch"],
                  **{k: cabi.get_option(k) for k in ("xcd_map", "sort_pairs")}}
        # the name the kernel trace shows, shortened: vector type, lanes, vectors per lane, index-table form
        kernel = (("kvm_copy_simple_kernel" if plan["simple_kernel"] else "kvm_copy_kernel")
                  + f"<u32x{plan['vector_bytes'] // 4}, {plan['threads']}, {plan['vectors_per_lane']}, "
                  + ("packed" if plan["pairs_per_launch"] > 432 else "wide") + ">")
        traffic, traffic_source = measured_traffic(
            config if not (ctx_tp or fresh_pools) and pattern == "request" else 0, kernel, bytes_per_launch)
        out = {
            "metric": "KV migration GB/s (% of HBM peak) + us/request at LLaMA-2-7B shape" if config == 2
                      else f"KV migration GB/s (% of HBM peak) + us/request, {w.name}",
            "value": round(hbm_gbps, 2), "unit": "GB/s",
            "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {
                "workload": (f"{w.name}: {len(w.calls)} requests, {w.total_blocks} blocks of "
                             f"{w.payload_bytes_per_block} B (K+V, decoding rank's share), context pp{w.ctx_pp}/tp{w.ctx_tp}"
                             f" -> decoding pp{w.dec_pp}/tp{w.dec_tp} rank ({w.dec_pp_rank},{w.dec_tp_rank}), "
                             f"pools {w.src_blocks}/{w.dst_blocks} blocks, seed {w.seed}"),
                "pattern": ("one call per request" if pattern == "request" else
                            f"{len(calls)} calls per batch (requests merged until a block id recurs)" if len(calls) > 1
                            else "one call per batch"),
                "value_counts": "HBM bytes read + written (2 x payload) per second",
                "tuning": tuning,
            },
            "ms_per_step_median": round(per_step_ms[len(per_step_ms) // 2], 4),
            "ms_per_step_min": round(per_step_ms[0], 4),
            "payload_GBps": round(payload / (ms_per_step * 1e-3) / 1e9, 2),
            "frac_of_hbm_peak": round(hbm_gbps / HBM_PEAK_GBPS, 4),
            "us_per_request": round(ms_per_step * 1e3 / len(w.calls), 2),
            "blocks_per_s": round(w.total_blocks / (ms_per_step * 1e-3), 1),
            "host_call_us": host_call_us, "host_call_us_min": host_call_us_min,
            "bit_exact": bit_exact,
            "roofline": {
                "bound": "hbm", "achieved": round(bytes_per_launch / (launch_us * 1e-6) / 1e9, 2), "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "frac": round(bytes_per_launch / (launch_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                "traffic": traffic, "traffic_source": traffic_source,
                "kernel": kernel,
                "launches_per_step": launches_per_step,
                "avg_launch_us": round(launch_us, 2), "algorithmic_bytes_per_launch": round(bytes_per_launch),
                "workgroups_per_block": plan["workgroups_per_block"], "workgroup_size": plan["threads"],
            },
        }
        if cache_resident:
            # a step's reads and writes fit the 256 MB last-level cache and the steps repeat them:
            # the figure is a cache and launch-latency figure, not an HBM one
            out["cache_resident"] = True
        records.append(out)
    if calibrate_copy:
        records[0]["plain_copy_GBps"] = time_plain_copy(cabi, stream)
    del src_k, src_v, dst_k, dst_v
    cabi.reset()
    gc.unfreeze()
    torch.cuda.empty_cache()
    return records, w


def compact(d: dict) -> dict:
    """The figures of one configuration as they ride along in the headline line."""
    keys = ("value", "frac_of_hbm_peak", "us_per_request", "blocks_per_s", "payload_GBps", "ms_per_step",
            "ms_per_step_median", "ms_per_step_min", "host_call_us", "bit_exact", "cache_resident")
    out = {("GBps" if k == "value" else "frac" if k == "frac_of_hbm_peak" else k): d[k] for k in keys if k in d}
    out["pattern"] = d["config"]["pattern"]
    out["roofline"] = d["roofline"]
    if "cpu_baseline" in d:
        out["cpu_baseline"] = d["cpu_baseline"]
    return out


def main():
    args = parse_args()
    if args.kernel_digest:
        print(kernel_source_digest())
        return
    if args.ipc_child:
        run_ipc_child()
        return
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (source and destination pools share one HBM; "
              "there is no sharding or collective on this path); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.pattern == "ipc":
        print(json.dumps(run_ipc_bench(args)))    # starts its child before this process touches the GPU
        return

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the KV movement path has no CPU fallback", file=sys.stderr)
        sys.exit(3)

    from distserve_amd import cabi

    for kv in args.opt:
        name, value = kv.split("=")
        cabi.set_option(name, int(value))

    if args.plain_copy_only:
        torch.cuda.set_device(0)
        nbytes = args.plain_copy_only << 20
        gbps = time_plain_copy(cabi, torch.cuda.current_stream(), nbytes=nbytes, reps=args.steps, warm=args.warmup)
        print(json.dumps({"metric": "plain contiguous copy", "value": gbps, "unit": "GB/s",
                          "bytes_copied_per_call": nbytes, "hbm_bytes_per_call": 2 * nbytes,
                          "launches_per_call": -(-(nbytes // (8 << 20)) // 864), "steps": args.steps}))
        return

    if args.config == 5:
        print(json.dumps(run_swap_bench(args)))
        return

    if args.pattern.startswith(("handoff", "scheduler")):
        if args.request_blocks:
            print(json.dumps(run_handoff_by_size(args)))
            return
        print(json.dumps(run_handoff_bench(args, load_workload(args.config or 2))))
        return

    verify_result = not args.no_verify
    if args.config:
        # one configuration, nothing else launched: the command the kernel profiles are taken with
        (out,), w = bench_migrate(args.config, [args.pattern], args.steps, args.warmup, verify_result,
                                  args.calibrate_copy, args.ctx_tp, args.fresh_pools)
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_baseline(w)
        print(json.dumps(out))
        return

    # The default run: configuration 2, one call per request, is the headline; its batched form
    # (same pools) and every other configuration (own pools, both call patterns on them) ride
    # along in "configs".  An entry that fails says so in its place and costs neither the
    # headline nor the entries after it.
    def failed(e):
        import torch as _torch

        _torch.cuda.empty_cache()
        return {"error": f"{type(e).__name__}: {e}"}

    configs, cpu_of = {}, {}
    (out, batched2), w2 = bench_migrate(2, ["request", "batch"], args.steps, args.warmup, verify_result, args.calibrate_copy)
    configs["cfg2_batched"] = batched2
    for cfg, patterns in ((1, ["request"]), (3, ["request", "batch"]), (4, ["request", "batch"])):
        keys = [f"cfg{cfg}" if pattern == "request" else f"cfg{cfg}_batched" for pattern in patterns]
        try:
            records, w = bench_migrate(cfg, patterns, args.steps, args.warmup, verify_result)
            if not args.no_cpu_baseline:
                # every configuration's own CPU figure, on a sample that a few seconds cover; the
                # two patterns of a configuration move the same bytes on the host and share it
                cpu_of[cfg] = cpu_baseline(w, budget_s=2.5, max_blocks=64, max_payload_bytes=256 << 20)
            for key, d in zip(keys, records):
                if cfg in cpu_of:
                    d["cpu_baseline"] = cpu_of[cfg]
                configs[key] = compact(d)
        except Exception as e:      # noqa: BLE001
            for key in keys:
                configs[key] = failed(e)
    try:
        configs["cfg5"] = run_swap_bench(args, default_only=True)
    except Exception as e:          # noqa: BLE001
        configs["cfg5"] = failed(e)
    # configuration 2's shape out of pools that a child process holds
    try:
        ipc = run_ipc_bench(args)
        configs["cfg2_ipc"] = {"GBps": ipc["value"], "frac": ipc["frac_of_hbm_peak"],
                               "this_process_GBps": ipc["this_process_GBps"],
                               "other_over_this_process": ipc["other_over_this_process"],
                               "us_per_call": ipc["us_per_call"]["other_process"], "bit_exact": ipc["bit_exact"],
                               "pattern": "64-block calls out of 1.75 GiB pools held by a child process (hipIpc mapping)"}
    except Exception as e:      # noqa: BLE001
        configs["cfg2_ipc"] = failed(e)
    # the whole hand-off at configuration 2 (block allocation, the torch op, release of the context
    # blocks), driven by the decoding scheduler, with the transmission time the lifetime events give
    import copy

    hand = copy.copy(args)
    hand.pattern, hand.no_verify = "scheduler", not verify_result
    try:
        h = run_handoff_bench(hand, load_workload(2))
        configs["cfg2_handoff"] = {k: h[k] for k in (
            "us_per_request", "host_us_per_request", "transmission_us_per_request",
            "transmission_us_per_request_stamped_at_enqueue", "frac_of_hbm_peak", "block_tables_equal_workload",
            "bit_exact")}
        configs["cfg2_handoff"].update(GBps=h["value"], pattern=h["config"]["pattern"])
    except Exception as e:      # noqa: BLE001
        configs["cfg2_handoff"] = failed(e)
    # ... and by request size: below which prompt length the host, not the GPU, is the longer leg
    try:
        hand.pattern, hand.request_blocks = "handoff", [1, 4, 16]
        rows = run_handoff_by_size(hand)["by_request_blocks"]
        configs["cfg2_handoff"]["by_request_blocks"] = {
            n: {k: r[k] for k in ("prompt_tokens", "us_per_request", "host_us_per_request", "copy_alone_us_per_request",
                                  "longer_leg", "bit_exact")} for n, r in rows.items()}
    except Exception as e:      # noqa: BLE001
        configs["cfg2_handoff"]["by_request_blocks"] = failed(e)
    out["configs"] = configs
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w2)
        configs["cfg2_batched"]["cpu_baseline"] = out["cpu_baseline"]
    configs["cfg2_batched"] = compact(configs["cfg2_batched"])
    print(json.dumps(out))


def run_swap_bench(args, default_only: bool = False):
    """Configuration 5: swap 2048 blocks (16 GiB) from HBM to a pinned host pool and back into
    other GPU slots, on side streams, while an 8-request migration runs on the main stream.
    The denominator is the host link measured in the same run with one large pinned copy per
    direction.  A step is one swap-out plus one swap-in of the whole block list.  Every
    implementation is timed three times: alone, beside the 8-request migration (the headline
    row), and beside migrations issued back to back for as long as both swaps take.
    ``default_only``: only the implementation the library's default takes, reported compactly."""
    import torch

    from distserve_amd import cabi, workloads
    from distserve_amd.streams import side_streams

    torch.cuda.set_device(0)
    kw = {}
    if args.swap_blocks:
        kw["swap_blocks"] = args.swap_blocks
    if args.swap_shape:
        layers, heads, head_dim = (int(x) for x in args.swap_shape.split(","))
        kw["shape"] = workloads.KvShape(layers, heads, head_dim)
    w = workloads.config5(**kw)
    shape = w.shape
    main = torch.cuda.current_stream()
    out_stream, in_stream = side_streams(2)            # two that do not share a hardware queue

    k_gpu = workloads.fill_uniform(shape.pool_shape(w.gpu_blocks), w.seed, "cuda")
    v_gpu = workloads.fill_uniform(shape.pool_shape(w.gpu_blocks), w.seed + 500, "cuda")
    k_ref, v_ref = k_gpu.clone(), v_gpu.clone()            # what the round trip must reproduce
    t0 = time.perf_counter()
    k_host = torch.empty(shape.pool_shape(w.host_blocks), dtype=shape.dtype, pin_memory=True)
    v_host = torch.empty(shape.pool_shape(w.host_blocks), dtype=shape.dtype, pin_memory=True)
    pin_s = time.perf_counter() - t0
    mig = w.migrate
    src_k = workloads.fill_uniform(mig.src_pool_shape(), 77, "cuda")
    src_v = workloads.fill_uniform(mig.src_pool_shape(), 78, "cuda")
    cabi.reset()
    cabi.register_source(1, 1, 0, 0, shape.num_layers, shape.num_kv_heads, src_k.data_ptr(), src_v.data_ptr(),
                         src_k.numel() * shape.dtype_bytes)
    geom = cabi.geom(shape.num_layers, shape.num_kv_heads, shape.block_size, shape.head_dim, shape.dtype_bytes)
    mig_calls = [(cabi.index_array(c.ctx_idx), cabi.index_array(c.dec_idx)) for c in mig.calls]
    slab = w.slab_bytes
    ptrs = (k_gpu.data_ptr(), v_gpu.data_ptr(), k_host.data_ptr(), v_host.data_ptr())
    out_src, out_dst = cabi.index_array(w.out_gpu_ids), cabi.index_array(w.out_host_ids)
    in_dst = cabi.index_array(w.in_gpu_ids)

    # ---- the link itself: one large pinned copy per direction
    link_bytes = 4 << 30
    big_host = torch.empty(link_bytes, dtype=torch.uint8, pin_memory=True)
    big_gpu = torch.empty(link_bytes, dtype=torch.uint8, device="cuda")

    def timed(fn, stream):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3

    link = {}
    for name, fn in (("d2h", lambda: big_host.copy_(big_gpu, non_blocking=True)),
                     ("h2d", lambda: big_gpu.copy_(big_host, non_blocking=True))):
        fn()
        torch.cuda.synchronize()
        link[name] = link_bytes / min(timed(fn, main) for _ in range(3)) / 1e9

    # ... and both directions at once: the first halves of the two buffers go down while the
    # second halves come up, on the two side streams; the best of three for each direction
    half = link_bytes // 2

    def both_ways(down, up):
        """Runs `down` on the swap-out stream and `up` on the swap-in stream from a common start;
        returns the seconds each took."""
        e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        torch.cuda.synchronize()
        e[0].record(out_stream)
        e[2].record(in_stream)
        with torch.cuda.stream(out_stream):
            down()
        e[1].record(out_stream)
        with torch.cuda.stream(in_stream):
            up()
        e[3].record(in_stream)
        torch.cuda.synchronize()
        return e[0].elapsed_time(e[1]) * 1e-3, e[2].elapsed_time(e[3]) * 1e-3

    runs = [both_ways(lambda: big_host[:half].copy_(big_gpu[:half], non_blocking=True),
                      lambda: big_gpu[half:].copy_(big_host[half:], non_blocking=True)) for _ in range(4)][1:]
    link_duplex = {"d2h": half / min(r[0] for r in runs) / 1e9, "h2d": half / min(r[1] for r in runs) / 1e9}
    del big_host, big_gpu

    def migrate_once():
        for ci, di in mig_calls:
            cabi.migrate(geom, ci, di, k_gpu.data_ptr(), v_gpu.data_ptr(), w.gpu_blocks, main.cuda_stream)

    modes = [cabi.get_option("swap_mode")] * 2      # the implementation for swap-outs and for swap-ins

    def swap_out():
        cabi.set_option("swap_mode", modes[0])
        cabi.swap(out_src, out_dst, False, *ptrs, slab, w.gpu_blocks, w.host_blocks, out_stream.cuda_stream)

    def swap_in():
        cabi.set_option("swap_mode", modes[1])
        cabi.swap(out_dst, in_dst, True, *ptrs, slab, w.gpu_blocks, w.host_blocks, in_stream.cuda_stream)

    # the duplex phase: the first half of the block list is on the host already and comes back in
    # while the second half goes out -- what one pass of the decoding scheduler issues when it
    # swaps one request out and another in (distserve/decoding_stage_scheduler.py:190-215)
    # The two copies in flight together must not touch each other's blocks (the configuration's
    # own swap-in list reuses slots its swap-out frees, which is why that swap-in waits for
    # the whole swap-out): the first half comes back into slots no swap-out reads, the second
    # half, afterwards and untimed, into the slots the first half left.
    n_half = len(w.out_gpu_ids) // 2
    leaving = set(w.out_gpu_ids)
    untouched = [b for b in w.in_gpu_ids if b not in leaving][:n_half]
    assert len(untouched) == n_half, "not enough GPU slots outside the swap-out list for the duplex phase"
    first = [cabi.index_array(x) for x in (w.out_gpu_ids[:n_half], w.out_host_ids[:n_half], untouched)]
    second = [cabi.index_array(x) for x in (w.out_gpu_ids[n_half:2 * n_half], w.out_host_ids[n_half:2 * n_half],
                                            w.out_gpu_ids[:n_half])]

    def swap_part(part, is_swap_in, stream):
        src, dst = (part[1], part[2]) if is_swap_in else (part[0], part[1])
        cabi.set_option("swap_mode", modes[1 if is_swap_in else 0])
        cabi.swap(src, dst, is_swap_in, *ptrs, slab, w.gpu_blocks, w.host_blocks, stream.cuda_stream)

    def duplex_ok():
        ok = True
        for ref, pool in ((k_ref, k_gpu), (v_ref, v_gpu)):
            for came_from, now_at in ((w.out_gpu_ids[:n_half], untouched),
                                      (w.out_gpu_ids[n_half:2 * n_half], w.out_gpu_ids[:n_half])):
                for i0 in range(0, n_half, 256):
                    a = torch.tensor(came_from[i0:i0 + 256], device="cuda")
                    b = torch.tensor(now_at[i0:i0 + 256], device="cuda")
                    ok = ok and bool(torch.equal(pool.view(torch.int16)[b], ref.view(torch.int16)[a]))
        return ok

    def round_trip_ok():
        ok = True
        for ref, pool in ((k_ref, k_gpu), (v_ref, v_gpu)):
            for i0 in range(0, len(w.out_gpu_ids), 256):
                a = torch.tensor(w.out_gpu_ids[i0:i0 + 256], device="cuda")
                b = torch.tensor(w.in_gpu_ids[i0:i0 + 256], device="cuda")
                ok = ok and bool(torch.equal(pool.view(torch.int16)[b], ref.view(torch.int16)[a]))
        return ok

    results, duplex = {}, {}
    bytes_dir = w.bytes_per_direction
    option_mode = cabi.get_option("swap_mode")
    default_wgs = (cabi.get_option("swap_wgs"), cabi.get_option("swap_wgs_in"))     # swap-out, swap-in
    # --swap-wgs N gives both directions N workgroups; the library's own pair is always measured
    wgs_list = [tuple(int(x) for x in (g.split(":") if ":" in g else (g, g))) for g in (args.swap_wgs or [])]
    # what the library's default takes for this block list (mode 3 decides per call)
    default_mode = cabi.swap_plan(w.out_gpu_ids, w.out_host_ids, slab, False, w.gpu_blocks, w.host_blocks)["mode"]
    if default_mode == 1 and default_wgs not in wgs_list:
        wgs_list.append(default_wgs)

    def migrate_timed():
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(main)
        migrate_once()
        e1.record(main)
        return e0, e1

    # touch every page of the pinned pools and warm both directions before anything is timed
    swap_out()
    in_stream.wait_stream(out_stream)
    swap_in()
    migrate_once()
    torch.cuda.synchronize()
    alone_ms = []
    for _ in range(7):                       # the median of seven: every "beside" figure is read against it
        e0, e1 = migrate_timed()
        torch.cuda.synchronize()
        alone_ms.append(e0.elapsed_time(e1))
    migrate_alone_ms = sorted(alone_ms)[len(alone_ms) // 2]

    variants = [("hipMemcpyAsync per block", 0, None), ("hipMemcpyAsync per block, V on a forked stream", 2, None),
                ("hipMemcpyAsync per block, V on a forked stream for swap-in only", (0, 2), None)]
    variants += [(f"copy kernel over pinned memory, {g[0]} (out) / {g[1]} (in) workgroups per pool kind", 1, g)
                 for g in wgs_list]
    if args.swap_kernel_only:
        variants = [v for v in variants if v[1] == 1]
    if default_only:
        variants = [v for v in variants if v[1] == default_mode and (v[2] is None or v[2] == default_wgs)]
    for mode_name, mode, wgs in variants:
        modes[:] = list(mode) if isinstance(mode, tuple) else [mode, mode]
        if wgs:
            cabi.set_option("swap_wgs", wgs[0])
            cabi.set_option("swap_wgs_in", wgs[1])
        rows = []
        for phase in ("alone", "overlapped", "busy"):
            overlapped = phase != "alone"
            k_gpu.copy_(k_ref)
            v_gpu.copy_(v_ref)
            torch.cuda.synchronize()
            t_host = time.perf_counter()
            e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
            e[0].record(out_stream)
            swap_out()
            e[1].record(out_stream)
            host_out_us = (time.perf_counter() - t_host) * 1e6
            mig_ms = []
            if phase == "overlapped":
                m = [migrate_timed() for _ in range(3)]     # while the swap-out is in flight
            in_stream.wait_event(e[1])        # swap-in reuses slots the swap-out frees
            e[2].record(in_stream)
            swap_in()
            e[3].record(in_stream)
            if phase == "overlapped":
                main.wait_event(e[2])                       # start beside the swap-in
                m += [migrate_timed() for _ in range(3)]
            if phase == "busy":
                # migrations back to back on the main stream for longer than both swaps take:
                # the swap competes with kernels that saturate HBM for all of its duration
                n_busy = int(1.15 * (rows[0]["swap_out_ms"] + rows[0]["swap_in_ms"]) / migrate_alone_ms) + 1
                b0, b1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                b0.record(main)
                for _ in range(n_busy):
                    migrate_once()
                b1.record(main)
            torch.cuda.synchronize()
            if phase == "overlapped":
                mig_ms = [round(a.elapsed_time(b), 3) for a, b in m]
            t_out, t_in = e[0].elapsed_time(e[1]) * 1e-3, e[2].elapsed_time(e[3]) * 1e-3
            ok = round_trip_ok()
            if overlapped:
                for c in mig.calls:
                    a = torch.tensor(c.ctx_idx, device="cuda")
                    b = torch.tensor(c.dec_idx, device="cuda")
                    ok = ok and bool(torch.equal(k_gpu.view(torch.int16)[b], src_k.view(torch.int16)[a]))
                    ok = ok and bool(torch.equal(v_gpu.view(torch.int16)[b], src_v.view(torch.int16)[a]))
            row = {"overlapped_with_migration": overlapped,
                   "swap_out_GBps": round(bytes_dir / t_out / 1e9, 2),
                   "swap_in_GBps": round(bytes_dir / t_in / 1e9, 2),
                   "swap_out_frac_of_link": round(bytes_dir / t_out / 1e9 / link["d2h"], 4),
                   "swap_in_frac_of_link": round(bytes_dir / t_in / 1e9 / link["h2d"], 4),
                   "swap_out_ms": round(t_out * 1e3, 2), "swap_in_ms": round(t_in * 1e3, 2),
                   "host_enqueue_swap_out_us": round(host_out_us, 1), "round_trip_bit_exact": ok}
            if phase == "overlapped":
                row["migration_ms_beside_swap_out"] = mig_ms[:3]
                row["migration_ms_beside_swap_in"] = mig_ms[3:]
                row["migration_ms_alone"] = round(migrate_alone_ms, 3)
            if phase == "busy":
                row["continuous_migration"] = True
                row["migration_ms_avg_of_continuous"] = round(b0.elapsed_time(b1) / n_busy, 3)
                row["migration_ms_alone"] = round(migrate_alone_ms, 3)
            rows.append(row)
        results[mode_name] = rows
        # duplex: first half out (untimed), then second half out WHILE the first half comes back in
        k_gpu.copy_(k_ref)
        v_gpu.copy_(v_ref)
        torch.cuda.synchronize()
        swap_part(first, False, out_stream)
        t_out, t_in = both_ways(lambda: swap_part(second, False, out_stream), lambda: swap_part(first, True, in_stream))
        swap_part(second, True, in_stream)
        torch.cuda.synchronize()
        half_bytes = n_half * 2 * slab
        duplex[mode_name] = {
            "blocks_each_way": n_half,
            "swap_out_GBps": round(half_bytes / t_out / 1e9, 2), "swap_in_GBps": round(half_bytes / t_in / 1e9, 2),
            "swap_out_frac_of_duplex_link": round(half_bytes / t_out / 1e9 / link_duplex["d2h"], 4),
            "swap_in_frac_of_duplex_link": round(half_bytes / t_in / 1e9 / link_duplex["h2d"], 4),
            "both_ways_GBps": round(2 * half_bytes / max(t_out, t_in) / 1e9, 2),
            "round_trip_bit_exact": duplex_ok()}
    cabi.set_option("swap_mode", option_mode)
    cabi.set_option("swap_wgs", default_wgs[0])
    cabi.set_option("swap_wgs_in", default_wgs[1])
    cpu = None
    if not args.no_cpu_baseline:
        del k_ref, v_ref, src_k, src_v
        cpu = swap_cpu_baseline(w, 64, 2.5) if default_only else swap_cpu_baseline(w)
    default_name = [n for n, m, g in variants if m == default_mode and (g is None or g == default_wgs)]
    best = results[default_name[0] if default_name else variants[0][0]][1]
    total_s = best["swap_out_ms"] * 1e-3 + best["swap_in_ms"] * 1e-3
    cabi.reset()
    link_mean = (link["d2h"] + link["h2d"]) / 2
    roofline = {"bound": "host link", "achieved": round(2 * bytes_dir / total_s / 1e9, 2), "peak": round(link_mean, 2),
                "unit": "GB/s", "frac": round(2 * bytes_dir / total_s / 1e9 / link_mean, 4), "traffic": None,
                "peak_source": "measured in this run: one 4 GiB pinned copy per direction, mean of the two",
                "kernel": "kvm_walk_kernel<u32x4, packed>" if default_mode == 1 else "hipMemcpyAsync",
                "algorithmic_bytes_per_step": 2 * bytes_dir}
    if default_only:
        alone, beside, busy = results[default_name[0]]
        pick = ("swap_out_frac_of_link", "swap_in_frac_of_link", "swap_out_GBps", "swap_in_GBps")
        return {
            "roofline": roofline, "cpu_baseline": cpu,
            "duplex": dict(duplex[default_name[0]], link_duplex_GBps={k: round(v, 2) for k, v in link_duplex.items()}),
            "workload": (f"{w.name}: {len(w.out_gpu_ids)} blocks x {2 * slab} B (K+V) out to a pinned pool and back "
                         f"into other slots, beside a migration of {len(mig.calls)} requests on another stream"),
            "swap_implementation": default_name[0],
            "GBps": round(2 * bytes_dir / total_s / 1e9, 2),
            "link_GBps": {k: round(v, 2) for k, v in link.items()},
            "frac_of_link": round(2 * bytes_dir / total_s / 1e9 / ((link["d2h"] + link["h2d"]) / 2), 4),
            "alone": {k: alone[k] for k in pick},
            "beside_8_requests": {k: beside[k] for k in pick},
            "beside_continuous_migration": {k: busy[k] for k in pick},
            "host_enqueue_us": {"swap_out_alone": alone["host_enqueue_swap_out_us"],
                                "swap_out_beside_8_requests": beside["host_enqueue_swap_out_us"]},
            "migration_ms": {"alone": beside["migration_ms_alone"],
                             "beside_swap_out": beside["migration_ms_beside_swap_out"],
                             "beside_swap_in": beside["migration_ms_beside_swap_in"],
                             "continuous_avg": busy["migration_ms_avg_of_continuous"]},
            "blocks_per_s": round(2 * len(w.out_gpu_ids) / total_s, 1),
            "bit_exact": bool(alone["round_trip_bit_exact"] and beside["round_trip_bit_exact"]
                              and busy["round_trip_bit_exact"] and duplex[default_name[0]]["round_trip_bit_exact"]),
        }
    return {
        "metric": ("KV swap GB/s (fraction of measured host link), "
                   + (f"pools of {args.swap_shape} layers,heads,head_dim" if args.swap_shape else "LLaMA-2-7B shape")
                   + ", overlapped with an 8-request migration"),
        "value": round(2 * bytes_dir / total_s / 1e9, 2), "unit": "GB/s", "n_gpus": 1, "steps": 1, "warmup": 1,
        "ms_per_step": round(total_s * 1e3, 2), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": (f"{w.name}: {len(w.out_gpu_ids)} blocks x {2 * slab} B (K+V) out to a pinned pool of "
                                f"{w.host_blocks} blocks and back into other slots of a {w.gpu_blocks}-block GPU pool; "
                                f"concurrent migration of {len(mig.calls)} requests ({mig.total_blocks} blocks), seed {w.seed}"),
                   "value_counts": "bytes over the host link, swap-out plus swap-in, default swap mode, overlapped run"},
        "link_GBps": {k: round(v, 2) for k, v in link.items()},
        "pin_host_pools_s": round(pin_s, 2),
        "default_swap_mode": {"option": option_mode, "taken_for_this_workload": default_mode,
                              "variant": default_name[0] if default_name else None},
        "link_duplex_GBps": {k: round(v, 2) for k, v in link_duplex.items()},
        "swap": results,
        "swap_duplex": duplex,
        "cpu_baseline": cpu,
        "roofline": roofline,
    }


def swap_cpu_baseline(w, sample_blocks=256, budget_s=10.0):
    """Reference semantics of the swap on the host: index_copy_(index_select) between two CPU
    pools (oracle.swap_lib), out and back, on a sample of the block list with the pools
    compacted to the sample (bytes per block unchanged)."""
    import torch

    import oracle
    from distserve_amd import workloads

    n = min(sample_blocks, len(w.out_gpu_ids))
    gen = torch.Generator().manual_seed(w.seed)
    a, b, c = (torch.randperm(n, generator=gen).tolist() for _ in range(3))
    gpu_k = workloads.fill_uniform(w.shape.pool_shape(n), w.seed)
    gpu_v = workloads.fill_uniform(w.shape.pool_shape(n), w.seed + 1)
    host_k, host_v = workloads.fill_canary(w.shape.pool_shape(n)), workloads.fill_canary(w.shape.pool_shape(n))

    def one_pass():
        oracle.swap_lib(a, b, gpu_k, host_k)
        oracle.swap_lib(a, b, gpu_v, host_v)
        oracle.swap_lib(b, c, host_k, gpu_k)
        oracle.swap_lib(b, c, host_v, gpu_v)

    one_pass()
    t0, passes = time.perf_counter(), 0
    while time.perf_counter() - t0 < budget_s and passes < 50:
        one_pass()
        passes += 1
    dt = time.perf_counter() - t0
    moved = 2 * n * 2 * w.slab_bytes * passes            # out + in, K + V
    return {"value": round(moved / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": (f"oracle.swap_lib (torch index_select/index_copy_ between CPU pools), {n} of "
                       f"{len(w.out_gpu_ids)} blocks out and back, pools compacted to the sample, {passes} passes in "
                       f"{dt:.1f} s; GB/s counts bytes copied, like the link figure"),
            "host_cpu_count": os.cpu_count()}


IPC_POOL_BLOCKS = 448    # 1.75 GiB per pool at the LLaMA-2-7B shape: pools that cross a process boundary stay under 2 GiB
IPC_SEED = 77


def run_ipc_child():
    """The context instance of `--pattern ipc`, in a process of its own: makes the K and V
    pools the first line on stdin describes, prints its pid and their memory handles as one
    JSON line, and keeps the pools alive until stdin says anything more or closes."""
    spec = json.loads(sys.stdin.readline())
    import torch

    from distserve_amd import cabi, workloads

    torch.cuda.set_device(0)
    k = workloads.fill_uniform(tuple(spec["shape"]), spec["seed"], "cuda")
    v = workloads.fill_uniform(tuple(spec["shape"]), spec["seed"] + 500, "cuda")
    torch.cuda.synchronize()
    nbytes = k.numel() * k.element_size()
    print(json.dumps({"pid": os.getpid(), "k": cabi.get_mem_handle(k.data_ptr(), nbytes),
                      "v": cabi.get_mem_handle(v.data_ptr(), nbytes)}), flush=True)
    sys.stdin.readline()


def run_ipc_bench(args):
    """Migration out of pools that another process owns.  The child (this file again; when the
    pattern runs alone it is started before this process touches the GPU) holds the context
    pools and sends their handles; this process binds them as context instance 1 and, for
    comparison, identical pools of its own as instance 2, then times the same 7 calls of 64
    blocks out of each, alternating."""
    import subprocess
    import threading

    child = subprocess.Popen([sys.executable, "-u", os.path.abspath(__file__), "--ipc-child"], stdin=subprocess.PIPE,
                             stdout=subprocess.PIPE, text=True, cwd=os.path.dirname(os.path.abspath(__file__)))
    try:
        from distserve_amd import workloads as wl

        s = wl.config2().shape
        shape = (IPC_POOL_BLOCKS, s.num_layers, s.num_kv_heads, s.block_size, s.head_dim)
        child.stdin.write(json.dumps({"shape": shape, "seed": IPC_SEED}) + "\n")
        child.stdin.flush()
        answer = {}
        reader = threading.Thread(target=lambda: answer.update(line=child.stdout.readline()), daemon=True)
        reader.start()
        reader.join(timeout=240)          # the child's first import of torch can take minutes on a fresh box
        if not answer.get("line"):
            raise RuntimeError("the context process did not send its handles")
        hello = json.loads(answer["line"])

        import torch

        from distserve_amd import cabi

        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible; the KV movement path has no CPU fallback")
        for kv in args.opt:
            name, value = kv.split("=")
            cabi.set_option(name, int(value))
        torch.cuda.set_device(0)
        stream = torch.cuda.current_stream()
        cabi.reset()
        pc = [1, 0, 1, 0]
        cabi.register_mem_handle(hello["k"], hello["v"], s.num_layers, s.num_kv_heads, pc, pc, ctx_instance=1)
        opened = cabi.opened_handles()
        own_k = wl.fill_uniform(shape, IPC_SEED, "cuda")
        own_v = wl.fill_uniform(shape, IPC_SEED + 500, "cuda")
        nbytes = own_k.numel() * own_k.element_size()
        cabi.register_source(1, 1, 0, 0, s.num_layers, s.num_kv_heads, own_k.data_ptr(), own_v.data_ptr(), nbytes,
                             ctx_instance=2)
        dst_k, dst_v = wl.fill_canary(shape, "cuda"), wl.fill_canary(shape, "cuda")
        g = torch.Generator().manual_seed(IPC_SEED)
        src_order = torch.randperm(IPC_POOL_BLOCKS, generator=g).tolist()
        dst_order = torch.randperm(IPC_POOL_BLOCKS, generator=g).tolist()
        calls = [(cabi.index_array(src_order[i:i + 64]), cabi.index_array(dst_order[i:i + 64]))
                 for i in range(0, IPC_POOL_BLOCKS, 64)]
        geoms = {name: cabi.geom(s.num_layers, s.num_kv_heads, s.block_size, s.head_dim, s.dtype_bytes, ctx_instance=inst)
                 for name, inst in (("other_process", 1), ("this_process", 2))}

        def step(geom):
            for ci, di in calls:
                cabi.migrate(geom, ci, di, dst_k.data_ptr(), dst_v.data_ptr(), IPC_POOL_BLOCKS, stream.cuda_stream)

        def timed(geom, steps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(stream)
            for _ in range(steps):
                step(geom)
            b.record(stream)
            torch.cuda.synchronize()
            return a.elapsed_time(b) / steps

        exact = {}
        for name, geom in geoms.items():
            dst_k.view(torch.int16).fill_(0x7C01)
            dst_v.view(torch.int16).fill_(0x7C01)
            for _ in range(args.warmup):
                step(geom)
            torch.cuda.synchronize()
            # every block of the pools is a destination once: the whole pools must be the gather
            si, di = torch.tensor(src_order, device="cuda"), torch.tensor(dst_order, device="cuda")
            exact[name] = bool(torch.equal(dst_k[di].view(torch.int16), own_k[si].view(torch.int16))
                               and torch.equal(dst_v[di].view(torch.int16), own_v[si].view(torch.int16)))
        ms = {name: [] for name in geoms}
        for _ in range(5):                       # alternating, so that drift hits both alike
            for name, geom in geoms.items():
                ms[name].append(timed(geom, max(1, args.steps // 5)))
        hbm_bytes = 4 * nbytes                   # both pools, read once and written once
        med = {name: sorted(v)[len(v) // 2] for name, v in ms.items()}
        gbps = {name: hbm_bytes / (m * 1e-3) / 1e9 for name, m in med.items()}
        cabi.reset()
        return {
            "metric": "KV migration GB/s out of another process's pools (hipIpc mapping), LLaMA-2-7B shape",
            "value": round(gbps["other_process"], 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(med["other_process"], 4), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": f"cfg2 shape, {IPC_POOL_BLOCKS}-block pools ({nbytes >> 20} MiB each, below the 2 GiB "
                                   f"export limit), {len(calls)} calls of 64 blocks, every block moved once, seed {IPC_SEED}",
                       "pattern": "context pools in a child process, handles over a pipe; the same calls out of "
                                  "identical pools of this process, alternating, median of 5 rounds each"},
            "frac_of_hbm_peak": round(gbps["other_process"] / HBM_PEAK_GBPS, 4),
            "this_process_GBps": round(gbps["this_process"], 2),
            "other_over_this_process": round(gbps["other_process"] / gbps["this_process"], 4),
            "us_per_call": {name: round(m * 1e3 / len(calls), 2) for name, m in med.items()},
            "context_process_pid": hello["pid"], "this_pid": os.getpid(), "mappings_opened": opened,
            "bit_exact": all(exact.values()), "bit_exact_by_source": exact,
        }
    finally:
        try:
            child.stdin.write("\n")
            child.stdin.flush()
            child.wait(timeout=60)
        except Exception:
            child.kill()


def run_handoff_bench(args, w):
    """The whole hand-off, not only the op: for every request allocate decoding blocks in the
    BlockManager, call Worker.migrate_blocks (torch op -> C ABI -> kernel) on the decoding
    worker, release the context blocks.  The free lists start in the workload's seeded order,
    so the block tables are the same non-contiguous ones the default pattern uses.  Wall
    clock from the first allocation to the GPU having finished the last copy."""
    import torch

    from distserve_amd import (CacheConfig, ContextStageLLMEngine, DecodingStageFCFSScheduler,
                               DecodingStageLLMEngine, DecodingStageSchedConfig, ModelConfig, ParallelConfig, cabi,
                               create_request, workloads)

    assert not w.recycles_blocks and w.dec_pp == 1 and w.dec_tp == 1, "handoff patterns run configurations 1-3"
    s = w.shape
    model = ModelConfig.from_kv_shape(s.num_layers, s.num_kv_heads, s.head_dim, num_kv_heads=s.num_kv_heads)
    cache = CacheConfig(s.block_size, 4096)
    cabi.reset()
    ctx = ContextStageLLMEngine(model, ParallelConfig(w.ctx_tp, 0, w.ctx_pp, 0), cache)
    dec = DecodingStageLLMEngine(model, ParallelConfig(1, 0, 1, 0), cache,
                                 clear_migrated_blocks_callback=ctx.clear_migrated_blocks_callback)
    ctx._init_kvcache(w.src_blocks, 0)
    dec._init_kvcache(w.dst_blocks, 0)
    dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    for i, worker in enumerate(x for row in ctx.workers for x in row):
        worker.k_cache.copy_(workloads.fill_uniform(worker.k_cache.shape, w.seed + i, "cuda"))
        worker.v_cache.copy_(workloads.fill_uniform(worker.v_cache.shape, w.seed + 500 + i, "cuda"))
    batched = args.pattern in ("handoff-batched", "scheduler-batched")
    sched = None
    if args.pattern.startswith("scheduler"):
        # every request of the step is acceptable: the threshold on waiting prompts is off and
        # the pool holds them all, so the scheduler's work is its decisions, not a refusal
        sched = DecodingStageFCFSScheduler(
            DecodingStageSchedConfig("fcfs", len(w.calls), 1 << 30, waiting_block_prop_threshold=1.0),
            dec.parallel_config, dec.block_manager, dec._migrate_blocks,
            engine_migrate_blocks_batched_callback=dec._migrate_blocks_batched, batch_migrations=batched)

    # where the host time of a hand-off goes: the three steps of _migrate_blocks, timed apart
    spent = {"allocate": 0.0, "migrate_call": 0.0, "release": 0.0}

    def timed_step(name, fn):
        def wrapper(*a, **kw):
            t = time.perf_counter()
            try:
                return fn(*a, **kw)
            finally:
                spent[name] += time.perf_counter() - t
        return wrapper

    dec._allocate_for_migration = timed_step("allocate", dec._allocate_for_migration)
    dec._call_migrate = timed_step("migrate_call", dec._call_migrate)
    dec._release_source_blocks = timed_step("release", dec._release_source_blocks)

    def seeded_free_lists():
        used_src = [b for c in w.calls for b in c.ctx_idx]
        used_dst = [b for c in w.calls for b in c.dec_idx]
        ctx.block_manager.free_gpu_blocks_list[:] = used_src + sorted(set(range(w.src_blocks)) - set(used_src))
        dec.block_manager.free_gpu_blocks_list[:] = used_dst + sorted(set(range(w.dst_blocks)) - set(used_dst))

    def one_step(step):
        seeded_free_lists()
        migrating = []
        for c in w.calls:
            req = create_request(c.prompt_len, step * 1000 + c.request_id)
            ctx.block_manager.allocate_blocks(req)
            req.add_generated_token("t", 1)
            migrating.append(ctx.on_prefill_finished(req))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if sched is not None:
            for m in migrating:
                sched.add_request(m)
            sched.post_process()
            assert not sched.unaccepted_queue and len(sched.waiting_queue) == len(migrating)
            sched.waiting_queue.clear()
        elif batched:
            dec._migrate_blocks_batched(migrating)
        else:
            for m in migrating:
                dec._migrate_blocks(m)
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        tables = [(list(m.block_indexes), list(dec.block_manager.get_block_table(m.req.request_id))) for m in migrating]
        for m in migrating:
            dec.block_manager.free_blocks(m.req.request_id)
        return t1 - t0, t2 - t0, tables

    for i in range(args.warmup):
        one_step(i)
    # Everything allocated so far (torch's modules, the workload's tables) goes to the
    # collector's permanent generation, as a serving process does after start-up: a full
    # collection over them takes about 35 ms and would otherwise land, once, inside a timed
    # hand-off (the loop allocates request objects, which is what triggers collections).
    import gc

    gc.collect()
    gc.freeze()
    host_s, total_s, tables = 0.0, 0.0, None
    for k in spent:
        spent[k] = 0.0
    for i in range(args.steps):
        h, t, tables = one_step(args.warmup + i)
        host_s += h
        total_s += t
    host_breakdown = {k: round(v / args.steps / len(w.calls) * 1e6, 2) for k, v in spent.items()}
    # "Transmission" as the reference's plots derive it from the lifetime events
    # (migration_end - migration_begin): once as the reference stamps it, when the asynchronous
    # calls have returned, and once with the end stamped after the copy has finished on the GPU
    from distserve_amd.lifetime import transmission_seconds

    transmission_us = {}
    for name, wait in (("stamped_at_enqueue", False), ("stamped_after_the_copy", True)):
        dec.gpu_complete_lifetime_events = wait
        dec.lifetime_events.clear()
        one_step(args.warmup + args.steps + (1 if wait else 0))
        spans = [transmission_seconds(ev) for ev in dec.lifetime_events.values()]
        transmission_us[name] = round(sum(spans) / len(spans) * 1e6, 2)
    dec.gpu_complete_lifetime_events = False
    # the tables the BlockManagers produced are the workload's own
    same_tables = all(ci == c.ctx_idx and di == c.dec_idx for (ci, di), c in zip(tables, w.calls))
    dw = dec.workers[0][0]
    src_k = [[x.k_cache for x in row] for row in ctx.workers]
    src_v = [[x.v_cache for x in row] for row in ctx.workers]
    bit_exact = verify(w, src_k, src_v, dw.k_cache, dw.v_cache) if not args.no_verify else None
    ms_per_step = total_s / args.steps * 1e3
    hbm_gbps = 2 * w.payload_bytes / (ms_per_step * 1e-3) / 1e9
    cabi.reset()
    # the engines were frozen into the collector's permanent generation with everything else;
    # thaw and collect, or their pools (cycles hold them) stay allocated for the rest of the run
    driven_by_scheduler = sched is not None
    del src_k, src_v, dw, sched
    ctx.workers, dec.workers = [], []
    gc.unfreeze()
    gc.collect()
    torch.cuda.empty_cache()
    return {
        "metric": f"KV migration hand-off GB/s + us/request, {w.name}", "value": round(hbm_gbps, 2), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"{w.name}: {len(w.calls)} requests, {w.total_blocks} blocks",
                   "pattern": (("bridge queue -> DecodingStageFCFSScheduler.post_process -> " if driven_by_scheduler else "")
                               + "BlockManager.allocate_blocks + Worker.migrate_blocks (torch op) + release of the "
                               "context blocks, " + ("one migrate call per batch" if batched else "one per request")),
                   "value_counts": "HBM bytes read + written per second of host wall clock (allocation to GPU idle)"},
        "us_per_request": round(ms_per_step * 1e3 / len(w.calls), 2),
        "host_us_per_request": round(host_s / args.steps / len(w.calls) * 1e6, 2),
        "host_us_per_request_by_step": host_breakdown,
        "transmission_us_per_request": transmission_us["stamped_after_the_copy"],
        "transmission_us_per_request_stamped_at_enqueue": transmission_us["stamped_at_enqueue"],
        "transmission_note": ("mean of migration_end - migration_begin over the requests of one step, as the reference's "
                              "plots compute it; batched: every request of the call spans the whole call"),
        "frac_of_hbm_peak": round(hbm_gbps / HBM_PEAK_GBPS, 4),
        "block_tables_equal_workload": same_tables, "bit_exact": bit_exact,
    }


def run_handoff_by_size(args):
    """The hand-off pattern over requests of one size, for every size asked for: per request
    the wall clock to GPU idle, the host's share, where the host's share goes, and beside
    them the copy alone (the same block lists through the C ABI, HIP events) -- so that it
    shows from which prompt length on the GPU, not the host, is the longer leg."""
    import torch

    from distserve_amd import cabi, workloads

    by_size = {}
    for n in args.request_blocks:
        w = workloads.fixed_size_requests(n)
        h = run_handoff_bench(args, w)
        # the copy alone: same lists, one call per request, nothing but the launches timed
        s = w.shape
        src_k = workloads.fill_uniform(w.src_pool_shape(), 1, "cuda")
        src_v = workloads.fill_uniform(w.src_pool_shape(), 2, "cuda")
        dst_k, dst_v = torch.empty_like(src_k), torch.empty_like(src_v)
        cabi.reset()
        cabi.register_source(1, 1, 0, 0, s.num_layers, s.num_kv_heads, src_k.data_ptr(), src_v.data_ptr(),
                             src_k.numel() * s.dtype_bytes)
        geom = cabi.geom(s.num_layers, s.num_kv_heads, s.block_size, s.head_dim, s.dtype_bytes)
        calls = [(cabi.index_array(c.ctx_idx), cabi.index_array(c.dec_idx)) for c in w.calls]
        stream = torch.cuda.current_stream()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for timed in (False, True):
            e0.record(stream)
            for _ in range(args.steps):
                for ci, di in calls:
                    cabi.migrate(geom, ci, di, dst_k.data_ptr(), dst_v.data_ptr(), w.dst_blocks, stream.cuda_stream)
            e1.record(stream)
            torch.cuda.synchronize()
        copy_us = e0.elapsed_time(e1) * 1e3 / (args.steps * len(calls))
        cabi.reset()
        del src_k, src_v, dst_k, dst_v
        torch.cuda.empty_cache()
        by_size[str(n)] = {
            "prompt_tokens": n * s.block_size, "requests_per_step": len(w.calls),
            "us_per_request": h["us_per_request"], "host_us_per_request": h["host_us_per_request"],
            "host_us_per_request_by_step": h["host_us_per_request_by_step"],
            "copy_alone_us_per_request": round(copy_us, 2), "GBps": h["value"], "bit_exact": h["bit_exact"],
            "block_tables_equal_workload": h["block_tables_equal_workload"],
            "longer_leg": "host" if h["host_us_per_request"] > copy_us else "gpu"}
    first = by_size[str(args.request_blocks[0])]
    return {"metric": "KV migration hand-off us/request by request size, LLaMA-2-7B shape", "value": first["us_per_request"],
            "unit": "us/request", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(first["us_per_request"] * first["requests_per_step"] * 1e-3, 4),
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "48 requests of N blocks each (8 MiB per block, K+V), scattered block lists, TP1 -> TP1; "
                                   f"value is N = {args.request_blocks[0]}",
                       "pattern": args.pattern},
            "by_request_blocks": by_size}


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
