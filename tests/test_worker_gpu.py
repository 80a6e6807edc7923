"""The drop-in surface end to end on the GPU: torch.ops schemas, Worker, BlockManager and
the migration handoff, against the CPU oracle."""
import pytest
import torch

import oracle
from distserve_amd import (BlockManager, CacheConfig, ContextStageLLMEngine, DecodingStageLLMEngine, ModelConfig,
                           ParallelConfig, Worker, create_request)
from distserve_amd.utils import Stage
from helpers import canary_pool, rand_pool, same_bits

pytestmark = pytest.mark.gpu


def fill(worker, seed):
    worker.k_cache.copy_(rand_pool(worker.k_cache.shape, seed))
    worker.v_cache.copy_(rand_pool(worker.v_cache.shape, seed + 1))


def test_ops_registered_and_refuse_cpu_tensors():
    z = torch.zeros(2, 1, 1, 2, 2, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.block_migration_ops.migrate_blocks(1, 1, [0], 1, 1, 0, 0, [0], z, z)
    with pytest.raises(RuntimeError):
        torch.ops.block_migration_ops.get_ipc_mem_handle(z)


def test_handoff_tp2pp2_to_tp4_every_rank_against_oracle(kvm):
    """Context TP2/PP2 -> decoding TP4 (the layout of configuration 4) through Worker,
    BlockManager and the handoff; every decoding rank's pools are checked."""
    kvm.reset()
    model = ModelConfig.from_kv_shape(num_layers=8, num_heads=32, head_dim=64, num_kv_heads=8)
    cache = CacheConfig(16, 64)
    ctx = ContextStageLLMEngine(model, ParallelConfig(2, 0, 2, 0), cache)
    dec = DecodingStageLLMEngine(model, ParallelConfig(4, 0, 1, 0), cache,
                                 clear_migrated_blocks_callback=ctx.clear_migrated_blocks_callback)
    ctx._init_kvcache(24, 0)
    dec._init_kvcache(32, 4)
    dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    for i, w in enumerate(w for row in ctx.workers for w in row):
        fill(w, 100 + 10 * i)
    for w in dec.workers[0]:
        w.k_cache.view(torch.int16).fill_(0x7C01)
        w.v_cache.view(torch.int16).fill_(0x7C01)
    src_k = [[w.k_cache.cpu() for w in row] for row in ctx.workers]
    src_v = [[w.v_cache.cpu() for w in row] for row in ctx.workers]
    want_k = [canary_pool(w.k_cache.shape) for w in dec.workers[0]]
    want_v = [canary_pool(w.v_cache.shape) for w in dec.workers[0]]

    # some context blocks are already in use, so the tables are not 0..n on both sides
    ctx.block_manager.allocate_blocks(create_request(50, 900))
    dec.block_manager.allocate_blocks(create_request(20, 901))
    for rid, prompt_len in enumerate([40, 16, 97]):
        req = create_request(prompt_len, rid)
        ctx.block_manager.allocate_blocks(req)
        req.add_generated_token("x", 1)
        m = ctx.on_prefill_finished(req)
        ci = list(m.block_indexes)
        dec._migrate_blocks(m)
        di = dec.block_manager.get_block_table(rid)
        assert len(ci) == len(di) == -(-prompt_len // 16)
        for u in range(4):
            g = oracle.Geom(8, 8, 16, 64, 2, 2, 2, 1, 4, 0, u)
            oracle.migrate_c(g, src_k, ci, di, want_k[u])
            oracle.migrate_c(g, src_v, ci, di, want_v[u])
        assert rid not in ctx.block_manager.block_table          # source blocks released
    torch.cuda.synchronize()
    for u, w in enumerate(dec.workers[0]):
        assert same_bits(w.k_cache.cpu(), want_k[u]) and same_bits(w.v_cache.cpu(), want_v[u]), u
    kvm.reset()


def test_block_manager_swap_through_worker_round_trip(kvm):
    kvm.reset()
    model = ModelConfig.from_kv_shape(4, 8, 64)
    cache = CacheConfig(16, 64)
    worker = Worker(0, Stage.DECODING, model, cache)
    worker.init_kvcache_and_swap(16, 12)
    fill(worker, 5)
    k0, v0 = worker.k_cache.cpu(), worker.v_cache.cpu()

    def call_all(func_name, *args):
        return [getattr(worker, func_name)(*args)]

    bm = BlockManager(Stage.DECODING, 16, 12, model, ParallelConfig(), cache, call_all)
    a, b = create_request(60, 0), create_request(33, 1)
    bm.allocate_blocks(a)                                        # GPU [0..3]
    bm.allocate_blocks(b)                                        # GPU [4,5,6]
    bm.swap_out_requests([a, b])
    assert bm.get_block_table(0) == [0, 1, 2, 3] and bm.get_location(0).value == "cpu"
    filler = create_request(16 * 9, 2)
    bm.allocate_blocks(filler)                                   # takes GPU [7..15]: free list is empty now
    bm.swap_in_requests([b, a])                                  # must flush the swap-out quarantine
    assert bm.get_block_table(1) == [0, 1, 2] and bm.get_block_table(0) == [3, 4, 5, 6]
    worker.step([0, 1])                                          # compute stream waits for the swap-ins
    torch.cuda.synchronize()
    k1, v1 = worker.k_cache.cpu(), worker.v_cache.cpu()
    assert same_bits(k1[0:3], k0[4:7]) and same_bits(v1[0:3], v0[4:7])       # request b
    assert same_bits(k1[3:7], k0[0:4]) and same_bits(v1[3:7], v0[0:4])       # request a
    assert same_bits(k1[7:], k0[7:])
    assert worker.swap_event_table == {}
    worker.wait_for_all_swap_in()
    worker.wait_for_all_swap_out()
    kvm.reset()


def test_one_request_swaps_out_while_another_swaps_in(kvm):
    """What one pass of the decoding scheduler produces (reference
    decoding_stage_scheduler.py:190-215): a swap-out of request A on one side stream and a
    swap-in of request B on the other, both in flight at once, at the LLaMA-2-7B block
    shape so that each takes milliseconds.  Checked block for block against oracle.swap_c
    driven with the id lists the BlockManager produced."""
    kvm.reset()
    model = ModelConfig.from_kv_shape(num_layers=32, num_heads=32, head_dim=128)      # 4 MiB per pool per block
    cache = CacheConfig(16, 256)
    worker = Worker(0, Stage.DECODING, model, cache)
    n_gpu, n_cpu = 120, 80      # enough free blocks on both sides that no call has to wait for an earlier swap
    worker.init_kvcache_and_swap(n_gpu, n_cpu)
    fill(worker, 41)
    worker.k_swap.view(torch.int16).fill_(0x7C01)
    worker.v_swap.view(torch.int16).fill_(0x7C01)
    want = {"gpu_k": worker.k_cache.cpu(), "gpu_v": worker.v_cache.cpu(),
            "host_k": worker.k_swap.clone(), "host_v": worker.v_swap.clone()}
    issued = []

    def call_all(func_name, *args):
        if func_name == "swap_blocks":
            issued.append((list(args[1]), list(args[2]), args[3]))
        return [getattr(worker, func_name)(*args)]

    def mirror(src, dst, is_swap_in):
        for x in ("k", "v"):
            if is_swap_in:
                oracle.swap_c(src, dst, want["host_" + x], want["gpu_" + x])
            else:
                oracle.swap_c(src, dst, want["gpu_" + x], want["host_" + x])

    bm = BlockManager(Stage.DECODING, n_gpu, n_cpu, model, ParallelConfig(), cache, call_all)
    a, b = create_request(16 * 40, 0), create_request(16 * 36, 1)
    bm.allocate_blocks(a)
    bm.allocate_blocks(b)
    bm.swap_out_requests([b])                                    # B goes to the host first ...
    worker.wait_for_all_swap_out()
    mirror(*issued[-1])
    # ... then, in one pass and without any wait between them: A out, B back in
    e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    e[0].record(worker.swap_out_stream)
    bm.swap_out_requests([a])
    e[1].record(worker.swap_out_stream)
    out_call = issued[-1]
    e[2].record(worker.swap_in_stream)
    bm.swap_in_requests([b])
    e[3].record(worker.swap_in_stream)
    in_call = issued[-1]
    assert out_call[2] is False and in_call[2] is True and len(out_call[0]) == 40 and len(in_call[0]) == 36
    # disjoint on both sides: nothing orders the two copies against each other
    assert not set(out_call[0]) & set(in_call[1]) and not set(out_call[1]) & set(in_call[0])
    worker.step([0, 1])                                          # the compute stream waits for both
    torch.cuda.synchronize()
    mirror(*out_call)
    mirror(*in_call)
    assert same_bits(worker.k_cache.cpu(), want["gpu_k"]) and same_bits(worker.v_cache.cpu(), want["gpu_v"])
    assert same_bits(worker.k_swap, want["host_k"]) and same_bits(worker.v_swap, want["host_v"])
    # the two copies overlapped in time: each started before the other ended
    assert e[0].elapsed_time(e[3]) > 0 and e[2].elapsed_time(e[1]) > 0, \
        "a timing relation, not a correctness failure: the swap-out and the swap-in did not overlap"
    assert bm.get_location(0).value == "cpu" and bm.get_location(1).value == "gpu"
    kvm.reset()


def test_profile_and_block_bytes():
    model = ModelConfig("meta-llama/Llama-2-7b-hf")
    worker = Worker(0, Stage.DECODING, model, CacheConfig(16, 256, cpu_swap_space=2))
    assert worker._get_block_size_in_bytes(16, model, ParallelConfig()) == 8 * 1024 * 1024
    assert worker._get_block_size_in_bytes(16, model, ParallelConfig(2, 0, 2, 0)) == 2 * 1024 * 1024
    n_gpu, n_cpu = worker._profile_num_available_blocks(16, 0.5, 2 << 30)
    assert n_cpu == 256 and n_gpu > 1000


@pytest.mark.parametrize("batched", [False, True])
def test_scheduler_driven_migration_matches_oracle(kvm, batched):
    """Requests flow bridge queue -> scheduler.post_process -> engine -> op.  With
    batch_migrations the accepted requests share ONE migrate call; the copied bytes and the
    block tables are the same either way."""
    from distserve_amd import DecodingStageFCFSScheduler, DecodingStageSchedConfig

    kvm.reset()
    model = ModelConfig.from_kv_shape(num_layers=4, num_heads=8, head_dim=64)
    cache = CacheConfig(16, 64)
    ctx = ContextStageLLMEngine(model, ParallelConfig(2, 0, 1, 0), cache)
    dec = DecodingStageLLMEngine(model, ParallelConfig(1, 0, 1, 0), cache,
                                 clear_migrated_blocks_callback=ctx.clear_migrated_blocks_callback)
    ctx._init_kvcache(40, 0)
    dec._init_kvcache(48, 8)
    dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    for i, w in enumerate(ctx.workers[0]):
        fill(w, 300 + 10 * i)
    dw = dec.workers[0][0]
    dw.k_cache.view(torch.int16).fill_(0x7C01)
    dw.v_cache.view(torch.int16).fill_(0x7C01)
    src_k = [[w.k_cache.cpu() for w in ctx.workers[0]]]
    src_v = [[w.v_cache.cpu() for w in ctx.workers[0]]]
    want_k, want_v = canary_pool(dw.k_cache.shape), canary_pool(dw.v_cache.shape)

    calls = []
    real = dw.migrate_blocks
    dw.migrate_blocks = lambda ci, pc, di: (calls.append(len(ci)), real(ci, pc, di))[1]
    sched = DecodingStageFCFSScheduler(
        DecodingStageSchedConfig("fcfs", 8, 4096, waiting_block_prop_threshold=1.0), dec.parallel_config,
        dec.block_manager, dec._migrate_blocks,
        engine_migrate_blocks_batched_callback=dec._migrate_blocks_batched, batch_migrations=batched)
    g = oracle.Geom(4, 8, 16, 64, 2, 1, 2, 1, 1)
    tables = {}
    for rid, prompt_len in enumerate([70, 16, 33, 120]):
        req = create_request(prompt_len, rid)
        ctx.block_manager.allocate_blocks(req)
        req.add_generated_token("x", 1)
        m = ctx.on_prefill_finished(req)
        tables[rid] = list(m.block_indexes)
        sched.add_request(m)
    sched.post_process()
    assert sched.unaccepted_queue == [] and [r.request_id for r in sched.waiting_queue] == [0, 1, 2, 3]
    assert calls == ([5 + 1 + 3 + 8] if batched else [5, 1, 3, 8])
    for rid, ci in tables.items():
        di = dec.block_manager.get_block_table(rid)
        oracle.migrate_c(g, src_k, ci, di, want_k)
        oracle.migrate_c(g, src_v, ci, di, want_v)
        assert rid not in ctx.block_manager.block_table
    torch.cuda.synchronize()
    assert same_bits(dw.k_cache.cpu(), want_k) and same_bits(dw.v_cache.cpu(), want_v)
    assert [str(e.event_type) for e in dec.lifetime_events[3]] == ["migration_begin", "migration_end"]
    kvm.reset()


def _paged_decode_attention(q, k_pool, v_pool, block_table, layer, n_tokens):
    """What the forward pass does with the pools (reference worker.py:217-223 hands it
    k_cache, v_cache and the block table): gather the request's blocks of one layer through
    the block table, [block, head, slot, dim] -> [head, token, dim], attend."""
    idx = torch.tensor(block_table, device=k_pool.device)
    k = k_pool[idx, layer].permute(1, 0, 2, 3).reshape(k_pool.shape[2], -1, k_pool.shape[4])[:, :n_tokens].float()
    v = v_pool[idx, layer].permute(1, 0, 2, 3).reshape(v_pool.shape[2], -1, v_pool.shape[4])[:, :n_tokens].float()
    scores = torch.einsum("hd,htd->ht", q, k) / k.shape[-1] ** 0.5
    return torch.einsum("ht,htd->hd", torch.softmax(scores, dim=-1), v)


def test_consumer_reads_migrated_blocks_through_the_block_table(kvm):
    """Consumer contract: paged attention over the decoding rank's pools + its block table
    gives, head for head, what it gives over the context ranks' pools + their block table
    (context TP2/PP2 -> decoding TP2: layers re-joined, heads re-split)."""
    kvm.reset()
    L, H, D, B = 4, 8, 64, 16
    model = ModelConfig.from_kv_shape(L, H, D)
    cache = CacheConfig(B, 64)
    ctx = ContextStageLLMEngine(model, ParallelConfig(2, 0, 2, 0), cache)
    dec = DecodingStageLLMEngine(model, ParallelConfig(2, 0, 1, 0), cache,
                                 clear_migrated_blocks_callback=None)      # keep the source blocks
    ctx._init_kvcache(20, 0)
    dec._init_kvcache(24, 2)
    dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    for i, w in enumerate(w for row in ctx.workers for w in row):
        fill(w, 700 + 10 * i)
    ctx.block_manager.allocate_blocks(create_request(40, 50))              # shift the tables apart
    dec.block_manager.allocate_blocks(create_request(100, 51))
    prompt_len = 75
    req = create_request(prompt_len, 0)
    ctx.block_manager.allocate_blocks(req)
    m = ctx.on_prefill_finished(req)
    ctx_table = list(m.block_indexes)
    dec._migrate_blocks(m)
    dec_table = dec.block_manager.get_block_table(0)
    assert ctx_table != dec_table and len(dec_table) == 5
    torch.cuda.synchronize()
    q = (torch.rand((H, D), generator=torch.Generator().manual_seed(9)) * 2 - 1).cuda()
    for layer in range(L):
        p, ll = divmod(layer, L // 2)                                       # context pipeline rank, local layer
        for u, dw in enumerate(dec.workers[0]):                             # decoding TP ranks: 4 heads each
            heads = slice(u * 4, (u + 1) * 4)
            got = _paged_decode_attention(q[heads], dw.k_cache, dw.v_cache, dec_table, layer, prompt_len)
            cw = ctx.workers[p][u]                                          # context TP rank u owns the same heads
            want = _paged_decode_attention(q[heads], cw.k_cache, cw.v_cache, ctx_table, ll, prompt_len)
            assert torch.equal(got, want), (layer, u)
    kvm.reset()


def test_random_serving_loop_against_an_oracle_mirror(kvm):
    """A few hundred random steps of what the path sees in service -- prefill hand-offs
    (TP2 -> TP1), swap-outs, swap-ins, frees -- through Worker, BlockManager and the hand-off,
    mirrored step by step on CPU pools with the oracle; at the end every pool must agree
    bit for bit."""
    import random

    kvm.reset()
    rng = random.Random(1234)
    L, H, D, B = 2, 8, 32, 16
    model = ModelConfig.from_kv_shape(L, H, D)
    cache = CacheConfig(B, 64)
    ctx = ContextStageLLMEngine(model, ParallelConfig(2, 0, 1, 0), cache)
    dec = DecodingStageLLMEngine(model, ParallelConfig(1, 0, 1, 0), cache,
                                 clear_migrated_blocks_callback=ctx.clear_migrated_blocks_callback)
    N_CTX, N_DEC, N_HOST = 48, 40, 32
    ctx._init_kvcache(N_CTX, 0)
    dec._init_kvcache(N_DEC, N_HOST)
    dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    dw = dec.workers[0][0]
    for t in (dw.k_cache, dw.v_cache):
        t.view(torch.int16).fill_(0x7C01)
    for t in (dw.k_swap, dw.v_swap):
        t.view(torch.int16).fill_(0x7C01)
    g = oracle.Geom(L, H, B, D, 2, 1, 2, 1, 1)
    # the mirror
    m_ctx_k = [[torch.zeros(w.k_cache.shape, dtype=torch.float16) for w in ctx.workers[0]]]
    m_ctx_v = [[torch.zeros(w.v_cache.shape, dtype=torch.float16) for w in ctx.workers[0]]]
    m_dec_k, m_dec_v = canary_pool(dw.k_cache.shape), canary_pool(dw.v_cache.shape)
    m_host_k, m_host_v = canary_pool(dw.k_swap.shape), canary_pool(dw.v_swap.shape)
    for t, w in enumerate(ctx.workers[0]):
        w.k_cache.zero_()
        w.v_cache.zero_()

    live, next_id, seed = {}, 0, 1000
    counts = {"migrate": 0, "swap_out": 0, "swap_in": 0, "free": 0}
    for step in range(300):
        on_gpu = [r for r in live.values() if dec.block_manager.get_location(r.request_id).value == "gpu"]
        on_cpu = [r for r in live.values() if dec.block_manager.get_location(r.request_id).value == "cpu"]
        op = rng.choice(["migrate", "migrate", "swap_out", "swap_in", "free"])
        if op == "migrate":
            prompt_len = rng.randint(1, 6 * B)
            need = -(-prompt_len // B)
            if need > ctx.block_manager.get_num_avail_gpu_blocks() or need > dec.block_manager.get_num_avail_gpu_blocks():
                continue
            req = create_request(prompt_len, next_id)
            next_id += 1
            ctx.block_manager.allocate_blocks(req)
            table = ctx.block_manager.get_block_table(req.request_id)
            # "prefill": fresh contents for the request's context blocks, on both sides
            for t, w in enumerate(ctx.workers[0]):
                seed += 1
                fresh_k = rand_pool((len(table),) + tuple(w.k_cache.shape[1:]), seed)
                fresh_v = rand_pool((len(table),) + tuple(w.v_cache.shape[1:]), seed + 50000)
                idx = torch.tensor(table)
                m_ctx_k[0][t][idx] = fresh_k
                m_ctx_v[0][t][idx] = fresh_v
                w.k_cache[idx.cuda()] = fresh_k.cuda()
                w.v_cache[idx.cuda()] = fresh_v.cuda()
            req.add_generated_token("t", 1)
            mreq = ctx.on_prefill_finished(req)
            ci = list(mreq.block_indexes)
            dec._migrate_blocks(mreq)
            di = list(dec.block_manager.get_block_table(req.request_id))
            oracle.migrate_c(g, m_ctx_k, ci, di, m_dec_k)
            oracle.migrate_c(g, m_ctx_v, ci, di, m_dec_v)
            live[req.request_id] = req
        elif op == "swap_out" and on_gpu:
            req = rng.choice(on_gpu)
            old = list(dec.block_manager.get_block_table(req.request_id))
            if len(old) > dec.block_manager.get_num_avail_cpu_blocks():
                continue
            dec.block_manager.swap_out_requests([req])
            new = list(dec.block_manager.get_block_table(req.request_id))
            oracle.swap_c(old, new, m_dec_k, m_host_k)
            oracle.swap_c(old, new, m_dec_v, m_host_v)
        elif op == "swap_in" and on_cpu:
            req = rng.choice(on_cpu)
            old = list(dec.block_manager.get_block_table(req.request_id))
            if len(old) > dec.block_manager.get_num_avail_gpu_blocks():
                continue
            dec.block_manager.swap_in_requests([req])
            new = list(dec.block_manager.get_block_table(req.request_id))
            oracle.swap_c(old, new, m_host_k, m_dec_k)
            oracle.swap_c(old, new, m_host_v, m_dec_v)
            dw.step([req.request_id])               # the compute stream waits for the swap-in
        elif op == "free" and live:
            req = rng.choice(list(live.values()))
            dec._free_request_resources(req.request_id)
            del live[req.request_id]
        else:
            continue
        counts[op] += 1
    torch.cuda.synchronize()
    assert min(counts.values()) >= 10, counts
    assert same_bits(dw.k_cache.cpu(), m_dec_k) and same_bits(dw.v_cache.cpu(), m_dec_v)
    assert same_bits(dw.k_swap, m_host_k) and same_bits(dw.v_swap, m_host_v)
    for t, w in enumerate(ctx.workers[0]):
        assert same_bits(w.k_cache.cpu(), m_ctx_k[0][t]) and same_bits(w.v_cache.cpu(), m_ctx_v[0][t])
    kvm.reset()


def test_migrate_op_replays_inside_a_hip_graph(kvm):
    """The op allocates nothing and only launches kernels on the current stream, so it can
    be captured; every replay must copy what the sources hold at that time."""
    kvm.reset()
    g = oracle.Geom(2, 8, 16, 64, 2, 1, 2, 1, 1)
    nb = 24
    src_k = [[rand_pool(g.ctx_pool_shape(nb), 60 + t).cuda() for t in range(2)]]
    src_v = [[rand_pool(g.ctx_pool_shape(nb), 70 + t).cuda() for t in range(2)]]
    for t in range(2):
        torch.ops.block_migration_ops.register_ipc_mem_handle(
            torch.ops.block_migration_ops.get_ipc_mem_handle(src_k[0][t]),
            torch.ops.block_migration_ops.get_ipc_mem_handle(src_v[0][t]), 2, 8, [2, t, 1, 0], [1, 0, 1, 0])
    dst_k = canary_pool(g.dec_pool_shape(nb)).cuda()
    dst_v = canary_pool(g.dec_pool_shape(nb)).cuda()
    ci, di = [5, 0, 17, 9, 23], [1, 22, 4, 8, 0]
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):                   # warm-up outside the capture
        torch.ops.block_migration_ops.migrate_blocks(1, 2, ci, 1, 1, 0, 0, di, dst_k, dst_v)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        torch.ops.block_migration_ops.migrate_blocks(1, 2, ci, 1, 1, 0, 0, di, dst_k, dst_v)
    for replay in range(3):
        for t in range(2):                          # new source contents, eager work between replays
            src_k[0][t].copy_(rand_pool(g.ctx_pool_shape(nb), 100 * replay + t).cuda())
            src_v[0][t].copy_(rand_pool(g.ctx_pool_shape(nb), 100 * replay + 10 + t).cuda())
        dst_k.view(torch.int16).fill_(0x7C01)
        dst_v.view(torch.int16).fill_(0x7C01)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want_k, want_v = canary_pool(g.dec_pool_shape(nb)), canary_pool(g.dec_pool_shape(nb))
        oracle.migrate_c(g, [[t.cpu() for t in src_k[0]]], ci, di, want_k)
        oracle.migrate_c(g, [[t.cpu() for t in src_v[0]]], ci, di, want_v)
        assert same_bits(dst_k.cpu(), want_k) and same_bits(dst_v.cpu(), want_v), replay
    kvm.reset()


@pytest.mark.parametrize("dtype,block_size,head_dim", [("fp32", 16, 64), ("fp16", 8, 128), ("fp16", 32, 80),
                                                       ("fp32", 4, 24)])
def test_ops_with_other_dtypes_block_sizes_and_head_sizes(kvm, dtype, block_size, head_dim):
    """fp32 pools (reference config.py:20-29 allows fp16 and fp32), block sizes other than 16
    and head sizes that are not powers of two, through the torch ops and the Worker."""
    kvm.reset()
    model = ModelConfig.from_kv_shape(num_layers=4, num_heads=6, head_dim=head_dim, dtype=dtype)
    cache = CacheConfig(block_size, 64)
    ctx = ContextStageLLMEngine(model, ParallelConfig(3, 0, 2, 0), cache)          # TP3 / PP2
    dec = DecodingStageLLMEngine(model, ParallelConfig(2, 0, 1, 0), cache,          # TP2
                                 clear_migrated_blocks_callback=ctx.clear_migrated_blocks_callback)
    ctx._init_kvcache(14, 0)
    dec._init_kvcache(18, 6)
    dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    tdtype = model.get_torch_dtype()
    for i, w in enumerate(w for row in ctx.workers for w in row):
        w.k_cache.copy_(rand_pool(w.k_cache.shape, 900 + i, tdtype))
        w.v_cache.copy_(rand_pool(w.v_cache.shape, 950 + i, tdtype))
    for w in dec.workers[0]:
        oracle.bits(w.k_cache).fill_(0x7C01)
        oracle.bits(w.v_cache).fill_(0x7C01)
    src_k = [[w.k_cache.cpu() for w in row] for row in ctx.workers]
    src_v = [[w.v_cache.cpu() for w in row] for row in ctx.workers]
    want_k = [canary_pool(w.k_cache.shape, tdtype) for w in dec.workers[0]]
    want_v = [canary_pool(w.v_cache.shape, tdtype) for w in dec.workers[0]]
    ctx.block_manager.allocate_blocks(create_request(3 * block_size, 70))
    for rid, prompt_len in enumerate([5 * block_size + 1, 1, 2 * block_size]):
        req = create_request(prompt_len, rid)
        ctx.block_manager.allocate_blocks(req)
        m = ctx.on_prefill_finished(req)
        ci = list(m.block_indexes)
        dec._migrate_blocks(m)
        di = dec.block_manager.get_block_table(rid)
        for u in range(2):
            g = oracle.Geom(4, 6, block_size, head_dim, model.get_dtype_size(), 2, 3, 1, 2, 0, u)
            oracle.migrate_c(g, src_k, ci, di, want_k[u])
            oracle.migrate_c(g, src_v, ci, di, want_v[u])
    # and a swap round trip of request 0 on both decoding ranks
    req0 = create_request(5 * block_size + 1, 0)
    old = list(dec.block_manager.get_block_table(0))
    dec.block_manager.swap_out_requests([req0])
    host = list(dec.block_manager.get_block_table(0))
    dec.block_manager.swap_in_requests([req0])
    new = list(dec.block_manager.get_block_table(0))
    for u, w in enumerate(dec.workers[0]):
        hk, hv = canary_pool(w.k_swap.shape, tdtype), canary_pool(w.v_swap.shape, tdtype)
        oracle.swap_c(old, host, want_k[u], hk)
        oracle.swap_c(old, host, want_v[u], hv)
        oracle.swap_c(host, new, hk, want_k[u])
        oracle.swap_c(host, new, hv, want_v[u])
    torch.cuda.synchronize()
    for u, w in enumerate(dec.workers[0]):
        assert same_bits(w.k_cache.cpu(), want_k[u]) and same_bits(w.v_cache.cpu(), want_v[u]), u
    kvm.reset()


def test_tokens_written_by_the_producer_come_back_token_for_token(kvm):
    """Producer-to-consumer contract at token level.  A prefill stand-in writes each token's
    K and V vectors into the context ranks' pools the way the layout prescribes
    (block = table[t // B], slot = t % B, rank-local layer and head); after the hand-off
    (context TP2/PP2 -> decoding TP4), a swap-out and a swap-in, every decoding rank must
    hold exactly those vectors at the slots its own block table names."""
    kvm.reset()
    L, H, D, B = 4, 8, 32, 16
    model = ModelConfig.from_kv_shape(L, H, D)
    cache = CacheConfig(B, 64)
    ctx = ContextStageLLMEngine(model, ParallelConfig(2, 0, 2, 0), cache)
    dec = DecodingStageLLMEngine(model, ParallelConfig(4, 0, 1, 0), cache,
                                 clear_migrated_blocks_callback=ctx.clear_migrated_blocks_callback)
    ctx._init_kvcache(16, 0)
    dec._init_kvcache(20, 12)
    dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    ctx.block_manager.allocate_blocks(create_request(20, 90))               # shift both tables
    dec.block_manager.allocate_blocks(create_request(50, 91))
    n_tokens = 83
    gen = torch.Generator().manual_seed(77)
    tok_k = (torch.rand((n_tokens, L, H, D), generator=gen) * 2 - 1).half()  # [token, layer, head, dim]
    tok_v = (torch.rand((n_tokens, L, H, D), generator=gen) * 2 - 1).half()
    req = create_request(n_tokens, 0)
    ctx.block_manager.allocate_blocks(req)
    table = ctx.block_manager.get_block_table(0)
    for p, row in enumerate(ctx.workers):                                   # the producer
        for t, w in enumerate(row):
            layers, heads = slice(p * 2, p * 2 + 2), slice(t * 4, t * 4 + 4)
            for tok in range(n_tokens):
                w.k_cache[table[tok // B], :, :, tok % B, :] = tok_k[tok, layers, heads].cuda()
                w.v_cache[table[tok // B], :, :, tok % B, :] = tok_v[tok, layers, heads].cuda()
    req.add_generated_token("x", 1)
    dec._migrate_blocks(ctx.on_prefill_finished(req))
    assert 0 not in ctx.block_manager.block_table

    def check(where):
        table = dec.block_manager.get_block_table(0)
        idx = torch.tensor([table[tok // B] for tok in range(n_tokens)])
        slot = torch.tensor([tok % B for tok in range(n_tokens)])
        for u, w in enumerate(dec.workers[0]):                              # the consumer: 2 heads per rank
            heads = slice(u * 2, u * 2 + 2)
            k_pool, v_pool = (w.k_cache, w.v_cache) if where == "gpu" else (w.k_swap, w.v_swap)
            got_k = k_pool.cpu()[idx, :, :, slot, :]                        # [token, layer, head, dim]
            got_v = v_pool.cpu()[idx, :, :, slot, :]
            assert same_bits(got_k, tok_k[:, :, heads]) and same_bits(got_v, tok_v[:, :, heads]), (where, u)

    torch.cuda.synchronize()
    check("gpu")
    dec.block_manager.swap_out_requests([req])
    dec._remote_call_all_workers_async("wait_for_all_swap_out")
    check("host")
    dec.block_manager.swap_in_requests([req])
    dec._remote_call_all_workers_async("wait_for_all_swap_in")
    check("gpu")
    kvm.reset()


class _TimedWorker(Worker):
    """A worker that brackets its migrate call with timing events on the launch stream."""

    def migrate_blocks(self, *args, **kwargs):
        self.copy_start = torch.cuda.Event(enable_timing=True)
        self.copy_stop = torch.cuda.Event(enable_timing=True)
        self.copy_start.record(torch.cuda.current_stream())
        super().migrate_blocks(*args, **kwargs)
        self.copy_stop.record(torch.cuda.current_stream())


@pytest.mark.parametrize("gpu_complete", [True, False], ids=["stamped-after-the-copy", "stamped-at-enqueue"])
def test_transmission_from_lifetime_events_covers_the_copy_only_when_asked_to(kvm, gpu_complete):
    """MigrationEnd - MigrationBegin is what the reference's plots call "Transmission"
    (evaluation/ae-scripts/e2e/_plot.py:323-341).  With gpu_complete_lifetime_events the
    decoding engine waits for the copy before it stamps MigrationEnd, so the interval is at
    least the copy's own duration (HIP events around the launch) and exceeds it by host work
    only; without, it is stamped when the asynchronous call returns and covers the enqueue."""
    from distserve_amd.lifetime import json_encode_lifetime_events, transmission_seconds

    kvm.reset()
    model = ModelConfig.from_kv_shape(num_layers=32, num_heads=32, head_dim=128)      # 8 MiB per block, K+V
    cache = CacheConfig(16, 256)
    ctx = ContextStageLLMEngine(model, ParallelConfig(), cache)
    dec = DecodingStageLLMEngine(model, ParallelConfig(), cache, worker_factory=_TimedWorker,
                                 clear_migrated_blocks_callback=ctx.clear_migrated_blocks_callback,
                                 gpu_complete_lifetime_events=gpu_complete)
    ctx._init_kvcache(160, 0)
    dec._init_kvcache(160, 0)
    dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    fill(ctx.workers[0][0], 77)
    dw = dec.workers[0][0]
    transmissions, copies = [], []
    for rid in range(6):                                   # the first request warms everything up
        req = create_request(2048, rid)                    # 128 blocks = 1 GiB, about 0.3 ms of copy
        ctx.block_manager.allocate_blocks(req)
        req.add_generated_token("x", 1)
        m = ctx.on_prefill_finished(req)
        ci = list(m.block_indexes)
        torch.cuda.synchronize()
        dec._migrate_blocks(m)
        di = dec.block_manager.get_block_table(rid)
        torch.cuda.synchronize()
        events = dec.get_and_pop_request_lifetime_events(rid)
        assert [d["event_type"] for d in json_encode_lifetime_events(events)] == ["migration_begin", "migration_end"]
        transmissions.append(transmission_seconds(events))
        copies.append(dw.copy_start.elapsed_time(dw.copy_stop) * 1e-3)
        assert torch.equal(dw.k_cache[di].view(torch.int16), ctx.workers[0][0].k_cache[ci].view(torch.int16))
        dec.block_manager.free_blocks(rid)
    # timing relations on a shared box: judged on the medians of the repetitions after the warm-up,
    # with margins a busy host does not eat; the bit-exactness asserts above stay hard
    med = lambda xs: sorted(xs)[len(xs) // 2]    # noqa: E731
    t, c = med(transmissions[1:]), med(copies[1:])
    note = f"a timing relation, not a correctness failure: transmissions {transmissions[1:]}, copies {copies[1:]}"
    assert 100e-6 < c < 10e-3, note                        # 2 GiB of traffic: the copy was really timed
    if gpu_complete:
        # two clocks (host wall clock, GPU events): allow a few microseconds between them
        assert t >= c - 20e-6, note
        assert t <= c + 10e-3, note                        # the rest is host work: call, wait, wake-up
    else:
        assert min(transmissions[1:]) < c, note            # stamped while the copy was still running
    kvm.reset()


def test_freed_source_blocks_are_reused_only_after_a_migration_on_another_stream_has_read_them(kvm):
    """The decoding worker pulls on a side stream; the context worker, on the default stream,
    makes its stream wait on the migration's mark and then overwrites the freed blocks (the
    next prefill would).  The destination must hold what the blocks held before.  A mark made
    off the default stream records its event at once (a late one would make the waiting stream
    wait for whatever the side stream got after the copy, too); on the default stream it
    costs nothing: no event is recorded until somebody asks, and one mark serves every
    migration until then."""
    kvm.reset()
    model = ModelConfig.from_kv_shape(num_layers=32, num_heads=32, head_dim=128)
    cache = CacheConfig(16, 256)
    ctx_w = Worker(0, Stage.CONTEXT, model, cache)
    dec_w = Worker(1, Stage.DECODING, model, cache)
    hk, hv = ctx_w.init_kvcache_and_swap(96, 1)
    dec_w.init_kvcache_and_swap(96, 1)
    dec_w.register_kvcache_mem_handles(ParallelConfig(), [[(hk, hv)]])
    ctx_w.k_cache.view(torch.int16).fill_(0x1234)
    ctx_w.v_cache.view(torch.int16).fill_(0x2345)
    dec_w.k_cache.view(torch.int16).fill_(0x7C01)
    dec_w.v_cache.view(torch.int16).fill_(0x7C01)
    ci, di = list(range(10, 90)), list(range(5, 85))           # 80 blocks = 640 MiB, about 0.2 ms of copy
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    for attempt in range(3):
        with torch.cuda.stream(side):
            dec_w.migrate_blocks(ci, ParallelConfig(), di)
        mark = dec_w.latest_migrate_event
        assert mark._event is not None and not mark.pending     # recorded right behind the copy
        with torch.cuda.stream(side):
            torch.cuda._sleep(2_000_000)                        # later work of the side stream: not waited for
        ctx_w.wait_stream_for_migration(mark)                   # default stream now waits for the side stream's copy
        ctx_w.k_cache[ci] = 0                                    # the "next prefill" overwrites the freed blocks
        ctx_w.v_cache[ci] = 0
        torch.cuda.synchronize()
        assert bool((dec_w.k_cache[di].view(torch.int16) == 0x1234).all()), attempt
        assert bool((dec_w.v_cache[di].view(torch.int16) == 0x2345).all()), attempt
        ctx_w.k_cache.view(torch.int16).fill_(0x1234)
        ctx_w.v_cache.view(torch.int16).fill_(0x2345)
        dec_w.k_cache.view(torch.int16).fill_(0x7C01)
        torch.cuda.synchronize()
    # same stream: ordering is the stream's own, and the mark stays unrecorded
    dec_w.migrate_blocks(ci, ParallelConfig(), di)
    mark = dec_w.latest_migrate_event
    ctx_w.wait_stream_for_migration(mark)
    assert mark._event is None and mark.pending
    dec_w.migrate_blocks(ci, ParallelConfig(), di)
    assert dec_w.latest_migrate_event is mark                   # one pending mark serves the next migration too
    ctx_w.k_cache[ci] = 0
    torch.cuda.synchronize()
    assert bool((dec_w.k_cache[di].view(torch.int16) == 0x1234).all())
    mark.synchronize()                                          # asked for, it is a real event
    assert mark._event is not None and mark.query() is True
    dec_w.migrate_blocks(ci, ParallelConfig(), di)
    assert dec_w.latest_migrate_event is not mark               # a recorded mark does not cover later copies
    kvm.reset()
