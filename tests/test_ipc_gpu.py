"""Memory handles across a process boundary (reference distserve/worker.py:133-134, 229-248;
distserve/single_stage_engine.py:211-221, 469-483): the context instance lives in a child
process, its handles and block tables arrive as JSON over a pipe, and this process, as the
decoding instance, binds them and pulls every decoding rank's share.  One GPU, two processes.
"""
from __future__ import annotations

import json
import os
import queue
import subprocess
import sys
import threading

import pytest
import torch

import oracle
from distserve_amd import (CacheConfig, DecodingStageLLMEngine, MigratingRequest, ModelConfig, ParallelConfig,
                           create_request, workloads)
from helpers import canary_pool, same_bits

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
CHILD = os.path.join(HERE, "ipc_context_child.py")


DECODING_CHILD = os.path.join(HERE, "ipc_decoding_child.py")


class ContextProcess:
    """A child and a line-at-a-time conversation with it; every wait has a limit."""

    def __init__(self, spec: dict, log_path: str, script: str = CHILD):
        self.log = open(log_path, "w")
        self.proc = subprocess.Popen([sys.executable, "-u", script], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                                     stderr=self.log, text=True, cwd=os.path.dirname(HERE))
        self.lines: "queue.Queue[str]" = queue.Queue()
        threading.Thread(target=self._pump, daemon=True).start()
        self.log_path = log_path
        self.hello = self.ask(spec, timeout=240)     # the child's first import of torch can take minutes

    def _pump(self):
        for line in self.proc.stdout:
            self.lines.put(line)
        self.lines.put("")

    def ask(self, msg: dict, timeout: float = 60) -> dict:
        self.proc.stdin.write(json.dumps(msg) + "\n")
        self.proc.stdin.flush()
        try:
            line = self.lines.get(timeout=timeout)
        except queue.Empty:
            line = ""
        if not line:
            self.close(kill=True)
            raise AssertionError("the child process did not answer; its stderr:\n" + open(self.log_path).read()[-3000:])
        return json.loads(line)

    def read(self, timeout: float = 60) -> dict:
        """The next line the child prints without having been asked."""
        try:
            line = self.lines.get(timeout=timeout)
        except queue.Empty:
            line = ""
        if not line:
            raise AssertionError("the child process said nothing more; its stderr:\n" + open(self.log_path).read()[-3000:])
        return json.loads(line)

    def close(self, kill: bool = False):
        if self.proc.poll() is None:
            try:
                if kill:
                    self.proc.kill()
                else:
                    self.proc.stdin.write(json.dumps({"cmd": "exit"}) + "\n")
                    self.proc.stdin.flush()
                self.proc.wait(timeout=60)
            except Exception:
                self.proc.kill()
        self.log.close()


SPEC = {"layers": 8, "kv_heads": 8, "head_dim": 64, "tp": 2, "pp": 2, "blocks": 24, "seed": 300,
        "busy_blocks": 3, "prompts": [40, 16, 97, 33]}


def sealed(words) -> int:
    """The check word of a handle, as the library computes it over the 17 words before it."""
    mask = (1 << 64) - 1
    x = 0x5A5A5A5A5A5A5A5A
    for w in words[:17]:
        x = (((x << 7) | (x >> 57)) & mask) ^ (w & mask)
    return x - (1 << 64) if x >> 63 else x


def child_sources(spec):
    """The pools the child holds, remade here on the CPU from the seed: src[pp][tp]."""
    import ipc_context_child as child

    g = oracle.Geom(spec["layers"], spec["kv_heads"], 16, spec["head_dim"], 2, spec["pp"], spec["tp"])
    shape = g.ctx_pool_shape(spec["blocks"])
    src_k = [[workloads.fill_uniform(shape, child.pool_seed(spec["seed"], p * spec["tp"] + t, False))
              for t in range(spec["tp"])] for p in range(spec["pp"])]
    src_v = [[workloads.fill_uniform(shape, child.pool_seed(spec["seed"], p * spec["tp"] + t, True))
              for t in range(spec["tp"])] for p in range(spec["pp"])]
    return src_k, src_v


def test_context_instance_in_another_process_tp2pp2_to_tp4_every_rank_against_oracle(kvm, tmp_path):
    kvm.reset()
    ctx = ContextProcess(SPEC, str(tmp_path / "context_process.log"))
    try:
        hello = ctx.hello
        assert hello["pid"] != os.getpid()
        assert hello["pool_bytes"] < kvm.KVM_IPC_MAX_ALLOC_BYTES
        handles = hello["handles"]
        assert len(handles) == 2 and all(len(row) == 2 for row in handles)
        assert all(len(h) == kvm.KVM_HANDLE_WORDS for row in handles for pair in row for h in pair)
        tables = {int(k): v for k, v in hello["tables"].items()}
        src_k, src_v = child_sources(SPEC)

        model = ModelConfig.from_kv_shape(num_layers=8, num_heads=8, head_dim=64, num_kv_heads=8)
        cache = CacheConfig(16, 64)
        ctx_config = ParallelConfig(2, 0, 2, 0)
        released = []

        def release_in_child(migrating_req, migrate_events=()):
            # the copies must have finished before the other process may reuse the blocks: its
            # streams know nothing of this process's events
            for e in migrate_events:
                e.synchronize()
            released.append(ctx.ask({"cmd": "release", "id": migrating_req.req.request_id})["released"])

        dec = DecodingStageLLMEngine(model, ParallelConfig(4, 0, 1, 0), cache,
                                     clear_migrated_blocks_callback=release_in_child)
        dec._init_kvcache(32, 4)
        dec.block_manager.allocate_blocks(create_request(20, 901))      # decoding tables do not start at 0
        for cycle in range(2):
            # bind the other process's pools; close them again at the end of the cycle
            assert kvm.opened_handles() == 0
            dec.register_kvcache_mem_handles(ctx_config, handles)
            assert 1 <= kvm.opened_handles() <= 8
            for w in dec.workers[0]:
                w.k_cache.view(torch.int16).fill_(0x7C01)
                w.v_cache.view(torch.int16).fill_(0x7C01)
            want_k = [canary_pool(w.k_cache.shape) for w in dec.workers[0]]
            want_v = [canary_pool(w.v_cache.shape) for w in dec.workers[0]]
            for rid in (0, 1) if cycle == 0 else (2, 3):
                req = create_request(SPEC["prompts"][rid], rid)
                req.add_generated_token("x", 1)
                m = MigratingRequest(req, tables[rid], ctx_config)
                dec._migrate_blocks(m)
                di = dec.block_manager.get_block_table(rid)
                assert len(di) == len(tables[rid]) == -(-SPEC["prompts"][rid] // 16)
                for u in range(4):
                    g = oracle.Geom(8, 8, 16, 64, 2, 2, 2, 1, 4, 0, u)
                    oracle.migrate_c(g, src_k, tables[rid], di, want_k[u])
                    oracle.migrate_c(g, src_v, tables[rid], di, want_v[u])
            torch.cuda.synchronize()
            for u, w in enumerate(dec.workers[0]):
                assert same_bits(w.k_cache.cpu(), want_k[u]) and same_bits(w.v_cache.cpu(), want_v[u]), (cycle, u)
            assert ctx.ask({"cmd": "verify"}, timeout=120)["unchanged"] is True
            kvm.reset()
            assert kvm.opened_handles() == 0
            with pytest.raises(RuntimeError, match="not registered"):
                dec.workers[0][0].migrate_blocks(tables[0], ctx_config, dec.block_manager.get_block_table(0))
        assert released == [0, 1, 2, 3]

        # a pool inside an allocation of 2 GiB or more is never shared between processes: its
        # handle says so, and registration refuses it before anything is opened
        big = ctx.ask({"cmd": "big_handle"}, timeout=120)["handle"]
        with pytest.raises(kvm.KvmError) as e:
            kvm.register_mem_handle(big, big, 8, 8, [1, 0, 1, 0], [1, 0, 1, 0])
        assert e.value.code == kvm.KVM_EHANDLE and "not shared between processes" in str(e.value)
        assert kvm.opened_handles() == 0

        # a well-formed handle that claims a larger allocation than the other process holds is
        # refused once the mapping is there to be measured, and the mapping is closed again
        lie = list(handles[0][0][0])
        lie[6] *= 64                                    # the allocation's size, as the exporter tells it
        lie[4] = lie[6] - (lie[3] - lie[5])             # a pool that runs to the claimed end
        lie[17] = sealed(lie)
        with pytest.raises(kvm.KvmError) as e:
            kvm.register_mem_handle(lie, lie, 8, 8, [1, 0, 1, 0], [1, 0, 1, 0])
        assert e.value.code == kvm.KVM_EHANDLE and "the mapping holds" in str(e.value)
        assert kvm.opened_handles() == 0
        # a registration whose V handle fails after its K handle has been mapped leaves nothing mapped
        k00, v00 = handles[0][0]
        broken = list(v00)
        broken[4] = 0                                   # names no memory
        broken[17] = sealed(broken)
        with pytest.raises(kvm.KvmError) as e:
            kvm.register_mem_handle(k00, broken, 8, 8, [2, 0, 2, 0], [1, 0, 1, 0])
        assert e.value.code == kvm.KVM_EHANDLE and "names no memory" in str(e.value)
        assert kvm.opened_handles() == 0
        # handles whose exporter had no allocation id to give (the id bits cleared here): the rank's K
        # and V pools still share the mapping their registration call opens, and a second
        # registration maps the allocation anew instead of trusting the old mapping
        anonymous = []
        for h in (k00, v00):
            h = list(h)
            h[7] &= 0xFF
            h[17] = sealed(h)
            anonymous.append(h)
        for _ in range(2):
            kvm.register_mem_handle(*anonymous, 8, 8, [2, 0, 2, 0], [1, 0, 1, 0], ctx_instance=5)
            assert kvm.opened_handles() == len({(h[1], h[5]) for h in anonymous})
        kvm.reset()
        assert kvm.opened_handles() == 0
        # ... and while the allocation is open under its true size, it unbinds nothing
        dec.register_kvcache_mem_handles(ctx_config, handles)
        # a pool that is bound again elsewhere leaves its old mapping without a user: it is closed
        # (here instance 5's binding went with the reset above; nothing but instance 0's is open)
        # one mapping per allocation of the other process, however many pools lie in it and
        # however often they are registered
        allocations = {(h[1], h[5]) for row in handles for pair in row for h in pair}
        assert kvm.opened_handles() == len(allocations)
        with pytest.raises(kvm.KvmError) as e:
            kvm.register_mem_handle(lie, lie, 8, 8, [1, 0, 1, 0], [1, 0, 1, 0], ctx_instance=9)
        assert e.value.code == kvm.KVM_EHANDLE and "is open with" in str(e.value)
        assert kvm.opened_handles() == len(allocations)
        # binding the same pools a second time, as another context instance, leaves the first
        # binding alone: both resolve through the mapping that is already open
        k00, v00 = handles[0][0]
        kvm.register_mem_handle(k00, v00, 8, 8, [2, 0, 2, 0], [4, 0, 1, 0], ctx_instance=7)
        assert kvm.opened_handles() == len(allocations)
        dw = dec.workers[0][0]
        dw.migrate_blocks(tables[0], ctx_config, list(range(len(tables[0]))))     # instance 0 is still bound
        torch.cuda.synchronize()
    finally:
        ctx.close()
        kvm.reset()
    assert ctx.proc.returncode == 0, open(ctx.log_path).read()[-3000:]


def test_pools_reallocated_by_the_other_process_replace_their_stale_mappings(kvm, tmp_path):
    """The context process frees its pools and allocates them again (the runtime may hand out
    the same addresses): handles exported afterwards name other allocations, and registering
    them must not resolve through the mappings of the freed ones."""
    kvm.reset()
    spec = dict(SPEC, seed=520, prompts=[48, 80], busy_blocks=0)
    ctx = ContextProcess(spec, str(tmp_path / "context_process.log"))
    try:
        model = ModelConfig.from_kv_shape(num_layers=8, num_heads=8, head_dim=64, num_kv_heads=8)
        ctx_config = ParallelConfig(2, 0, 2, 0)
        dec = DecodingStageLLMEngine(model, ParallelConfig(1, 0, 1, 0), CacheConfig(16, 64))
        dec._init_kvcache(32, 0)
        dw = dec.workers[0][0]
        g = oracle.Geom(8, 8, 16, 64, 2, 2, 2, 1, 1)
        handles, tables, seen = ctx.hello["handles"], ctx.hello["tables"], []
        for generation, seed in enumerate((520, 521, 522)):
            if generation:
                answer = ctx.ask({"cmd": "reallocate", "seed": seed}, timeout=120)
                handles, tables = answer["handles"], answer["tables"]
            seen.append({(h[5], h[7] >> 8) for row in handles for pair in row for h in pair})
            dec.register_kvcache_mem_handles(ctx_config, handles)     # no reset in between
            src_k, src_v = child_sources(dict(spec, seed=seed))
            dw.k_cache.view(torch.int16).fill_(0x7C01)
            dw.v_cache.view(torch.int16).fill_(0x7C01)
            want_k, want_v = canary_pool(dw.k_cache.shape), canary_pool(dw.v_cache.shape)
            for rid in ("0", "1"):
                di = list(range(3 + 8 * int(rid), 3 + 8 * int(rid) + len(tables[rid])))
                dw.migrate_blocks(tables[rid], ctx_config, di)
                oracle.migrate_c(g, src_k, tables[rid], di, want_k)
                oracle.migrate_c(g, src_v, tables[rid], di, want_v)
            torch.cuda.synchronize()
            assert same_bits(dw.k_cache.cpu(), want_k) and same_bits(dw.v_cache.cpu(), want_v), generation
            assert kvm.opened_handles() <= sum(len({base for base, _ in s}) for s in seen)
        reused = [len({b for b, _ in seen[i]} & {b for b, _ in seen[i + 1]}) for i in range(2)]
        print("addresses handed out again from one generation to the next:", reused)
        # every generation's allocations carried ids of their own
        assert not (seen[0] & seen[1]) and not (seen[1] & seen[2])
    finally:
        ctx.close()
        kvm.reset()
    assert ctx.proc.returncode == 0, open(ctx.log_path).read()[-3000:]


def test_context_and_decoding_instances_as_sibling_processes(kvm, tmp_path):
    """The deployed topology: neither instance is this process.  One child holds the TP2/PP2
    context pools, a second child binds their handles, pulls every request into its TP4
    pools and reports a digest of each; this process only carries the JSON between them and
    checks the digests against the oracle's pools."""
    import hashlib

    spec = dict(SPEC, seed=410, prompts=[64, 23, 120])
    ctx = ContextProcess(spec, str(tmp_path / "context_process.log"))
    dec = None
    try:
        tables = {int(k): v for k, v in ctx.hello["tables"].items()}
        requests = [[rid, spec["prompts"][rid], tables[rid]] for rid in sorted(tables)]
        dec = ContextProcess({"layers": 8, "kv_heads": 8, "head_dim": 64, "tp": 4, "blocks": 32, "busy_prompt": 20,
                              "ctx_tp": 2, "ctx_pp": 2, "handles": ctx.hello["handles"], "requests": requests},
                             str(tmp_path / "decoding_process.log"), script=DECODING_CHILD)
        answer = dec.hello
        assert len({os.getpid(), ctx.hello["pid"], answer["pid"]}) == 3
        assert 1 <= answer["opened"] <= 8
        src_k, src_v = child_sources(spec)
        shape = oracle.Geom(8, 8, 16, 64, 2, 2, 2, 1, 4).dec_pool_shape(32)
        for u in range(4):
            g = oracle.Geom(8, 8, 16, 64, 2, 2, 2, 1, 4, 0, u)
            for src, got in ((src_k, answer["digests"][u][0]), (src_v, answer["digests"][u][1])):
                want = canary_pool(shape)
                for rid, _, ctx_table in requests:
                    oracle.migrate_c(g, src, ctx_table, answer["tables"][str(rid)], want)
                assert hashlib.sha256(oracle.bits(want).numpy().tobytes()).hexdigest() == got, u
        assert ctx.ask({"cmd": "verify"}, timeout=120)["unchanged"] is True
        dec.proc.stdin.write(json.dumps({"cmd": "exit"}) + "\n")
        dec.proc.stdin.flush()
        assert dec.read()["opened_after_reset"] == 0
        dec.proc.wait(timeout=60)
    finally:
        if dec is not None:
            dec.close()
        ctx.close()
    assert ctx.proc.returncode == 0 and dec.proc.returncode == 0, (
        open(ctx.log_path).read()[-2000:] + open(dec.log_path).read()[-2000:])


def test_a_handle_with_this_pid_but_another_nonce_is_not_taken_for_a_local_pointer(kvm):
    """Two processes in different pid namespaces can share a pid.  A handle resolves to its raw
    pointer only when pid AND the exporter's random word match this process; otherwise it goes
    the way of every foreign handle (here the runtime refuses to map this process's own
    export, or maps it: either way the pointer in the handle is not dereferenced as local)."""
    kvm.reset()
    g = oracle.Geom(2, 2, 16, 8, 2)
    pool = torch.zeros(g.ctx_pool_shape(4), dtype=torch.float16, device="cuda")
    nbytes = pool.numel() * 2
    own = kvm.get_mem_handle(pool.data_ptr(), nbytes)
    assert own[1] == os.getpid() and own[16] != 0
    kvm.register_mem_handle(own, own, 2, 2, [1, 0, 1, 0], [1, 0, 1, 0])
    assert kvm.opened_handles() == 0                           # its own: the pointer itself
    kvm.reset()
    other = list(own)
    other[16] ^= 0x5555                                        # same pid, another process's random word
    other[17] = sealed(other)
    try:
        kvm.register_mem_handle(other, other, 2, 2, [1, 0, 1, 0], [1, 0, 1, 0])
    except kvm.KvmError as e:
        assert e.code == kvm.KVM_EHANDLE and "could not be opened" in str(e)
        assert kvm.opened_handles() == 0
    else:
        assert kvm.opened_handles() == 1                       # bound through a mapping, not through the raw pointer
    kvm.reset()


def test_own_handles_still_resolve_without_ipc_whatever_the_pool_size(kvm):
    """Inside one process a handle is the pointer itself: no IPC open, also for a pool in an
    allocation far beyond what may be shared."""
    kvm.reset()
    big = torch.empty((2 << 30) + (8 << 20), dtype=torch.uint8, device="cuda")
    nbytes = 4 * 2 * 2 * 16 * 8 * 2
    k, v = big[1 << 30:(1 << 30) + nbytes], big[(1 << 30) + nbytes:(1 << 30) + 2 * nbytes]
    hk = torch.ops.block_migration_ops.get_ipc_mem_handle(k)
    hv = torch.ops.block_migration_ops.get_ipc_mem_handle(v)
    assert len(hk) == kvm.KVM_HANDLE_WORDS
    kvm.register_mem_handle(hk, hv, 2, 2, [1, 0, 1, 0], [1, 0, 1, 0], ctx_instance=5)
    assert kvm.opened_handles() == 0
    # bound under instance 5 only
    g = oracle.Geom(2, 2, 16, 8, 2)
    src = torch.arange(nbytes, dtype=torch.int32).to(torch.uint8)
    k.copy_(src.cuda())
    v.copy_((src + 1).cuda())
    dst_k = torch.zeros(g.dec_pool_shape(4), dtype=torch.float16, device="cuda")
    dst_v = torch.zeros_like(dst_k)
    geom5 = kvm.geom(2, 2, 16, 8, 2, ctx_instance=5)
    with pytest.raises(kvm.KvmError) as e:
        kvm.migrate(kvm.geom(2, 2, 16, 8, 2), [1], [2], dst_k.data_ptr(), dst_v.data_ptr(), 4)
    assert e.value.code == kvm.KVM_ENOTREG
    kvm.migrate(geom5, [1, 3], [2, 0], dst_k.data_ptr(), dst_v.data_ptr(), 4, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    blk = nbytes // 4
    got = dst_k.view(torch.uint8).view(4, blk).cpu()
    assert torch.equal(got[2], src[blk:2 * blk]) and torch.equal(got[0], src[3 * blk:])
    assert not got[1].any() and not got[3].any()
    kvm.reset()


def test_two_context_instances_in_one_process_keep_their_pools_apart(kvm):
    """Two prefill instances of the same layout feed one decoding instance: each one's ranks
    are bound under its own instance id, and a request is pulled from the instance that holds it."""
    from distserve_amd import ContextStageLLMEngine
    from helpers import rand_pool

    kvm.reset()
    model = ModelConfig.from_kv_shape(num_layers=4, num_heads=8, head_dim=64, num_kv_heads=8)
    cache = CacheConfig(16, 64)
    ctxs = [ContextStageLLMEngine(model, ParallelConfig(2, 0, 1, 0), cache, instance_id=i) for i in (0, 7)]
    dec = DecodingStageLLMEngine(model, ParallelConfig(1, 0, 1, 0), cache,
                                 clear_migrated_blocks_callback=lambda m, migrate_events=(): None)
    dec._init_kvcache(16, 0)
    srcs = []
    for n, ctx in enumerate(ctxs):
        ctx._init_kvcache(12, 0)
        for t, w in enumerate(ctx.workers[0]):
            w.k_cache.copy_(rand_pool(w.k_cache.shape, 40 + 10 * n + t))
            w.v_cache.copy_(rand_pool(w.v_cache.shape, 80 + 10 * n + t))
        dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles, context_instance=ctx.instance_id)
        srcs.append(([[w.k_cache.cpu() for w in ctx.workers[0]]], [[w.v_cache.cpu() for w in ctx.workers[0]]]))
    dw = dec.workers[0][0]
    dw.k_cache.view(torch.int16).fill_(0x7C01)
    dw.v_cache.view(torch.int16).fill_(0x7C01)
    want_k, want_v = canary_pool(dw.k_cache.shape), canary_pool(dw.v_cache.shape)
    g = oracle.Geom(4, 8, 16, 64, 2, 1, 2)
    # the same context block ids on both instances, so that a mix-up of instances shows
    for rid, n in ((0, 1), (1, 0), (2, 1)):
        req = create_request(35, rid)
        ctxs[n].block_manager.allocate_blocks(req)
        req.add_generated_token("x", 1)
        m = ctxs[n].on_prefill_finished(req)
        dec._migrate_blocks(m)
        di = dec.block_manager.get_block_table(rid)
        oracle.migrate_c(g, srcs[n][0], m.block_indexes, di, want_k)
        oracle.migrate_c(g, srcs[n][1], m.block_indexes, di, want_v)
    torch.cuda.synchronize()
    assert same_bits(dw.k_cache.cpu(), want_k) and same_bits(dw.v_cache.cpu(), want_v)
    assert ctxs[0].block_manager.get_block_table(1) == ctxs[1].block_manager.get_block_table(0) == [0, 1, 2]
    kvm.reset()
