"""Parity of the swap path (HBM <-> pinned host) against the CPU oracle through the C ABI,
in both implementations (hipMemcpyAsync per run, copy kernel over pinned memory), and
its overlap with a migration on another stream."""
import pytest
import torch

import oracle
from distserve_amd import workloads
from gpu_helpers import GUARD, kvm_geom, upload_and_register
from helpers import canary_pool, geom_of, make_src_pools, rand_pool, same_bits

pytestmark = pytest.mark.gpu

BLOCK = (3, 4, 16, 32)          # layers, heads, block_size, head_dim -> 12 KiB slabs


@pytest.fixture(params=[0, 1, 2, 3], ids=["memcpy", "kernel", "memcpy-forked", "auto"])
def swap_mode(kvm, request):
    old = kvm.get_option("swap_mode")
    kvm.set_option("swap_mode", request.param)
    yield request.param
    kvm.set_option("swap_mode", old)


def pools(n_gpu, n_host, seed, block=BLOCK):
    k_gpu = rand_pool((n_gpu,) + block, seed).cuda()
    v_gpu = rand_pool((n_gpu,) + block, seed + 1).cuda()
    k_host = canary_pool((n_host,) + block).pin_memory()
    v_host = canary_pool((n_host,) + block).pin_memory()
    return k_gpu, v_gpu, k_host, v_host


def guarded_pools(n_gpu, n_host, seed, block):
    """Like pools(), with canary margins on both sides of every pool; also returns a check
    that the margins still hold the canary (no write strayed past a pool's ends)."""
    def inside(whole, n):
        return whole[GUARD:GUARD + n * whole_block].view((n,) + block)

    whole_block = 1
    for d in block:
        whole_block *= d
    wholes = [canary_pool((n_gpu * whole_block + 2 * GUARD,)).cuda() for _ in range(2)]
    wholes += [canary_pool((n_host * whole_block + 2 * GUARD,)).pin_memory() for _ in range(2)]
    k_gpu, v_gpu = inside(wholes[0], n_gpu), inside(wholes[1], n_gpu)
    k_gpu.copy_(rand_pool((n_gpu,) + block, seed))
    v_gpu.copy_(rand_pool((n_gpu,) + block, seed + 1))
    k_host, v_host = inside(wholes[2], n_host), inside(wholes[3], n_host)
    margin = canary_pool((GUARD,))

    def margins_intact():
        return all(same_bits(w[:GUARD].cpu(), margin) and same_bits(w[-GUARD:].cpu(), margin) for w in wholes)

    return k_gpu, v_gpu, k_host, v_host, margins_intact


def do_swap(kvm, src, dst, swap_in, k_gpu, v_gpu, k_host, v_host, stream=None):
    slab = k_gpu[0].numel() * k_gpu.element_size()
    s = (stream or torch.cuda.current_stream()).cuda_stream
    kvm.swap(src, dst, swap_in, k_gpu.data_ptr(), v_gpu.data_ptr(), k_host.data_ptr(), v_host.data_ptr(),
             slab, k_gpu.shape[0], k_host.shape[0], s)


def test_swap_out_then_in_matches_oracle_and_round_trips(kvm, swap_mode):
    k_gpu, v_gpu, k_host, v_host = pools(12, 9, seed=3)
    k0, v0 = k_gpu.cpu(), v_gpu.cpu()
    out_src, out_dst = [7, 0, 1, 2, 11, 5], [3, 8, 4, 5, 0, 6]        # holds a run 0,1,2 -> 4,5 (partly)
    do_swap(kvm, out_src, out_dst, False, k_gpu, v_gpu, k_host, v_host)
    torch.cuda.synchronize()
    want_k, want_v = canary_pool(k_host.shape), canary_pool(v_host.shape)
    oracle.swap_c(out_src, out_dst, k0, want_k)
    oracle.swap_c(out_src, out_dst, v0, want_v)
    assert same_bits(k_host, want_k) and same_bits(v_host, want_v)
    assert same_bits(k_gpu.cpu(), k0) and same_bits(v_gpu.cpu(), v0)       # swap-out only reads HBM

    in_dst = [4, 9, 10, 3, 6, 8]                                         # other slots than they left
    do_swap(kvm, out_dst, in_dst, True, k_gpu, v_gpu, k_host, v_host)
    torch.cuda.synchronize()
    exp_k, exp_v = k0.clone(), v0.clone()
    oracle.swap_c(out_dst, in_dst, want_k, exp_k)
    oracle.swap_c(out_dst, in_dst, want_v, exp_v)
    assert same_bits(k_gpu.cpu(), exp_k) and same_bits(v_gpu.cpu(), exp_v)
    for a, b in zip(out_src, in_dst):                                     # the round trip itself
        assert same_bits(k_gpu[b].cpu(), k0[a]) and same_bits(v_gpu[b].cpu(), v0[a])


def test_consecutive_ids_coalesce_without_changing_the_result(kvm, swap_mode):
    k_gpu, v_gpu, k_host, v_host = pools(16, 16, seed=5)
    k0 = k_gpu.cpu()
    src = list(range(2, 12)) + [15, 0]
    dst = list(range(4, 14)) + [1, 15]
    do_swap(kvm, src, dst, False, k_gpu, v_gpu, k_host, v_host)
    torch.cuda.synchronize()
    want = canary_pool(k_host.shape)
    oracle.swap_lib(src, dst, k0, want)
    assert same_bits(k_host, want)


def test_empty_and_single_and_whole_pool(kvm, swap_mode):
    k_gpu, v_gpu, k_host, v_host = pools(5, 5, seed=9)
    do_swap(kvm, [], [], False, k_gpu, v_gpu, k_host, v_host)
    torch.cuda.synchronize()
    assert same_bits(k_host, canary_pool(k_host.shape))
    do_swap(kvm, [4], [0], False, k_gpu, v_gpu, k_host, v_host)
    do_swap(kvm, [0, 1, 2, 3], [1, 2, 3, 4], False, k_gpu, v_gpu, k_host, v_host)
    torch.cuda.synchronize()
    assert same_bits(k_host[0], k_gpu[4].cpu())
    assert same_bits(v_host[1:], v_gpu[:4].cpu())


def test_swap_errors(kvm, swap_mode):
    k_gpu, v_gpu, k_host, v_host = pools(4, 3, seed=1)
    for src, dst, swap_in, code in [([4], [0], False, kvm.KVM_ERANGE), ([0], [3], False, kvm.KVM_ERANGE),
                                    ([3], [0], True, kvm.KVM_ERANGE), ([0, 1], [2, 2], False, kvm.KVM_EDUP),
                                    ([-1], [0], True, kvm.KVM_ERANGE)]:
        with pytest.raises(kvm.KvmError) as e:
            do_swap(kvm, src, dst, swap_in, k_gpu, v_gpu, k_host, v_host)
        assert e.value.code == code
    pageable = canary_pool(k_host.shape)                                   # not pinned: refused
    with pytest.raises(kvm.KvmError) as e:
        do_swap(kvm, [0], [0], False, k_gpu, v_gpu, pageable, v_host)
    assert e.value.code == kvm.KVM_EINVAL and "pinned" in str(e.value)
    torch.cuda.synchronize()
    assert same_bits(k_host, canary_pool(k_host.shape))


def test_config5_shape_swap_overlapping_a_migration(kvm, swap_mode):
    """Configuration 5 on a thinner model (2 layers) and smaller pools: swap out, swap back
    into other slots on side streams while a migration runs on the main stream."""
    shape = workloads.KvShape(2, 32, 128)
    w = workloads.config5(gpu_blocks=512, host_blocks=512, swap_blocks=256, migrate_requests=4,
                          migrate_src_blocks=160, shape=shape, min_len=64, max_len=512)
    g = geom_of(w.migrate)
    kvm.reset()
    block = shape.pool_shape(1)[1:]
    k_gpu, v_gpu, k_host, v_host = pools(w.gpu_blocks, w.host_blocks, seed=w.seed, block=block)
    k0, v0 = k_gpu.cpu(), v_gpu.cpu()
    src_k, src_v = make_src_pools(g, w.migrate.src_blocks, 77), make_src_pools(g, w.migrate.src_blocks, 78)
    keep = upload_and_register(g, src_k, src_v)
    out_stream, in_stream = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()

    do_swap(kvm, w.out_gpu_ids, w.out_host_ids, False, k_gpu, v_gpu, k_host, v_host, out_stream)
    out_done = torch.cuda.Event()
    out_done.record(out_stream)
    for call in w.migrate.calls:                     # main stream, concurrent with the swaps
        kvm.migrate(kvm_geom(g), call.ctx_idx, call.dec_idx, k_gpu.data_ptr(), v_gpu.data_ptr(), w.gpu_blocks,
                    torch.cuda.current_stream().cuda_stream)
    in_stream.wait_event(out_done)                   # swap-in reuses slots the swap-out frees
    do_swap(kvm, w.out_host_ids, w.in_gpu_ids, True, k_gpu, v_gpu, k_host, v_host, in_stream)
    torch.cuda.synchronize()

    exp_k, exp_v = k0.clone(), v0.clone()
    host_k, host_v = canary_pool(k_host.shape), canary_pool(v_host.shape)
    oracle.swap_c(w.out_gpu_ids, w.out_host_ids, k0, host_k)
    oracle.swap_c(w.out_gpu_ids, w.out_host_ids, v0, host_v)
    oracle.swap_c(w.out_host_ids, w.in_gpu_ids, host_k, exp_k)
    oracle.swap_c(w.out_host_ids, w.in_gpu_ids, host_v, exp_v)
    for call in w.migrate.calls:
        oracle.migrate_c(g, src_k, call.ctx_idx, call.dec_idx, exp_k)
        oracle.migrate_c(g, src_v, call.ctx_idx, call.dec_idx, exp_v)
    assert same_bits(k_host, host_k) and same_bits(v_host, host_v)
    assert same_bits(k_gpu.cpu(), exp_k) and same_bits(v_gpu.cpu(), exp_v)
    for a, b in zip(w.out_gpu_ids, w.in_gpu_ids):
        assert a != b and same_bits(k_gpu[b].cpu(), k0[a])
    del keep
    kvm.reset()


def test_config5_full_size_round_trip_beside_a_migration(kvm):
    """Configuration 5 at full size with the default swap mode: 2048 blocks of the
    LLaMA-2-7B shape (16 GiB) out to a 4096-block pinned pool and back into other slots, on
    side streams, while 8 requests migrate on the main stream.  Checked by the round trip
    itself (every block that came back equals the block that left), by canaries on host
    blocks no swap named, and by the oracle on a sample."""
    w = workloads.config5()
    shape = w.shape
    kvm.reset()
    k_gpu = workloads.fill_uniform(shape.pool_shape(w.gpu_blocks), w.seed, "cuda")
    v_gpu = workloads.fill_uniform(shape.pool_shape(w.gpu_blocks), w.seed + 500, "cuda")
    k_ref, v_ref = k_gpu.clone(), v_gpu.clone()
    k_host = torch.empty(shape.pool_shape(w.host_blocks), dtype=shape.dtype, pin_memory=True)
    v_host = torch.empty(shape.pool_shape(w.host_blocks), dtype=shape.dtype, pin_memory=True)
    k_host.view(torch.int16).fill_(workloads.CANARY_BITS)
    v_host.view(torch.int16).fill_(workloads.CANARY_BITS)
    mig = w.migrate
    g = geom_of(mig)
    src_k = workloads.fill_uniform(mig.src_pool_shape(), 77, "cuda")
    src_v = workloads.fill_uniform(mig.src_pool_shape(), 78, "cuda")
    kvm.register_source(1, 1, 0, 0, g.num_layers, g.num_kv_heads, src_k.data_ptr(), src_v.data_ptr(),
                        src_k.numel() * 2)
    out_stream, in_stream = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    do_swap(kvm, w.out_gpu_ids, w.out_host_ids, False, k_gpu, v_gpu, k_host, v_host, out_stream)
    out_done = torch.cuda.Event()
    out_done.record(out_stream)
    for call in mig.calls:
        kvm.migrate(kvm_geom(g), call.ctx_idx, call.dec_idx, k_gpu.data_ptr(), v_gpu.data_ptr(), w.gpu_blocks,
                    torch.cuda.current_stream().cuda_stream)
    in_stream.wait_event(out_done)
    do_swap(kvm, w.out_host_ids, w.in_gpu_ids, True, k_gpu, v_gpu, k_host, v_host, in_stream)
    torch.cuda.synchronize()
    for ref, pool in ((k_ref, k_gpu), (v_ref, v_gpu)):
        for i0 in range(0, len(w.out_gpu_ids), 256):
            a = torch.tensor(w.out_gpu_ids[i0:i0 + 256], device="cuda")
            b = torch.tensor(w.in_gpu_ids[i0:i0 + 256], device="cuda")
            assert torch.equal(pool.view(torch.int16)[b], ref.view(torch.int16)[a])
    for call in mig.calls:
        a = torch.tensor(call.ctx_idx, device="cuda")
        b = torch.tensor(call.dec_idx, device="cuda")
        assert torch.equal(k_gpu.view(torch.int16)[b], src_k.view(torch.int16)[a])
        assert torch.equal(v_gpu.view(torch.int16)[b], src_v.view(torch.int16)[a])
    named = torch.zeros(w.host_blocks, dtype=torch.bool)
    named[torch.tensor(w.out_host_ids)] = True
    for b in (~named).nonzero().flatten().tolist()[::64]:
        assert bool((k_host[b].view(torch.int16) == workloads.CANARY_BITS).all())
    # oracle on a sample of the swapped blocks: host copy and returned copy
    pick = list(range(0, len(w.out_gpu_ids), 128))
    src_ids = [w.out_gpu_ids[i] for i in pick]
    small_ref = k_ref[torch.tensor(src_ids, device="cuda")].cpu()
    want_host = canary_pool((len(pick),) + tuple(small_ref.shape[1:]))
    oracle.swap_c(list(range(len(pick))), list(range(len(pick))), small_ref, want_host)
    assert same_bits(k_host[torch.tensor([w.out_host_ids[i] for i in pick])], want_host)
    assert same_bits(k_gpu[torch.tensor([w.in_gpu_ids[i] for i in pick], device="cuda")].cpu(), want_host)
    kvm.reset()


def test_random_slab_sizes_lists_and_pool_sizes(kvm, swap_mode):
    """60 seeded draws per implementation: slabs from 2 bytes (2-byte vectors in the kernel)
    to 160 KiB, lists with runs of consecutive blocks, out and back into other slots."""
    import random

    rng = random.Random(50 + swap_mode)
    for case in range(60):
        block = (rng.choice([1, 2, 5]), rng.choice([1, 3, 4]), rng.choice([1, 2, 16]), rng.choice([1, 3, 8, 40, 128]))
        n_gpu, n_host = rng.randint(2, 14), rng.randint(1, 14)
        k_gpu, v_gpu, k_host, v_host, margins_intact = guarded_pools(n_gpu, n_host, 100 + case, block)
        k0, v0 = k_gpu.cpu(), v_gpu.cpu()
        n = rng.randint(0, min(n_gpu, n_host))
        if rng.random() < 0.5:                       # a run of consecutive blocks on both sides
            a, b = rng.randint(0, n_gpu - n), rng.randint(0, n_host - n)
            out_src, out_dst = list(range(a, a + n)), list(range(b, b + n))
        else:
            out_src, out_dst = rng.sample(range(n_gpu), n), rng.sample(range(n_host), n)
        do_swap(kvm, out_src, out_dst, False, k_gpu, v_gpu, k_host, v_host)
        torch.cuda.synchronize()
        want_k, want_v = canary_pool(k_host.shape), canary_pool(v_host.shape)
        oracle.swap_c(out_src, out_dst, k0, want_k)
        oracle.swap_c(out_src, out_dst, v0, want_v)
        assert same_bits(k_host, want_k) and same_bits(v_host, want_v), (case, block, out_src, out_dst)
        in_dst = rng.sample(range(n_gpu), n)
        do_swap(kvm, out_dst, in_dst, True, k_gpu, v_gpu, k_host, v_host)
        torch.cuda.synchronize()
        exp_k, exp_v = k0.clone(), v0.clone()
        oracle.swap_c(out_dst, in_dst, want_k, exp_k)
        oracle.swap_c(out_dst, in_dst, want_v, exp_v)
        assert same_bits(k_gpu.cpu(), exp_k) and same_bits(v_gpu.cpu(), exp_v), (case, block, out_dst, in_dst)
        assert margins_intact(), (case, block)


def test_swap_pools_that_claim_more_than_their_allocation_are_refused(kvm, swap_mode):
    block = (8, 8, 16, 128)                                  # 256 KiB slabs, 64 MiB pools
    k_gpu, v_gpu, k_host, v_host = pools(256, 256, seed=2, block=block)
    slab = k_gpu[0].numel() * 2
    s = torch.cuda.current_stream().cuda_stream
    ptrs = (k_gpu.data_ptr(), v_gpu.data_ptr(), k_host.data_ptr(), v_host.data_ptr())
    with pytest.raises(kvm.KvmError) as e:
        kvm.swap([1], [2], False, *ptrs, slab, 64 * 256, 256, s)          # GPU pool said to be 64 times its size
    assert e.value.code == kvm.KVM_ERANGE
    torch.cuda.synchronize()
    assert same_bits(k_host, canary_pool(k_host.shape))
    kvm.swap([1], [2], False, *ptrs, slab, 256, 256, s)                   # true sizes still work afterwards
    torch.cuda.synchronize()
    assert same_bits(k_host[2], k_gpu[1].cpu())


def test_swap_kernel_replays_inside_a_hip_graph(kvm):
    """The copy-kernel form of the swap is one launch on the current stream, so it can be
    captured; every replay must move what the GPU pool holds at that time."""
    old = kvm.get_option("swap_mode")
    kvm.set_option("swap_mode", 1)
    try:
        k_gpu, v_gpu, k_host, v_host = pools(10, 8, seed=21)
        src, dst = [9, 2, 3, 4, 0], [1, 5, 6, 7, 3]
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):                   # warm-up outside the capture
            do_swap(kvm, src, dst, False, k_gpu, v_gpu, k_host, v_host, stream=side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            do_swap(kvm, src, dst, False, k_gpu, v_gpu, k_host, v_host)
        for replay in range(3):
            k_gpu.copy_(rand_pool(k_gpu.shape, 300 + replay).cuda())      # eager work between replays
            v_gpu.copy_(rand_pool(v_gpu.shape, 400 + replay).cuda())
            k_host.copy_(canary_pool(k_host.shape))
            v_host.copy_(canary_pool(v_host.shape))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            want_k, want_v = canary_pool(k_host.shape), canary_pool(v_host.shape)
            oracle.swap_c(src, dst, k_gpu.cpu(), want_k)
            oracle.swap_c(src, dst, v_gpu.cpu(), want_v)
            assert same_bits(k_host, want_k) and same_bits(v_host, want_v), replay
    finally:
        kvm.set_option("swap_mode", old)


def test_swaps_and_a_migration_from_several_host_threads(kvm, swap_mode):
    """The library may be entered concurrently: two threads swap their own pools out and
    back on their own streams while a third migrates, each result checked on its own."""
    import threading

    kvm.reset()
    g = oracle.Geom(2, 4, 16, 64, 2)
    nb = 48
    src_k, src_v = make_src_pools(g, nb, 61), make_src_pools(g, nb, 62)
    keep = upload_and_register(g, src_k, src_v)
    errors, results = [], {}

    def swapper(tid):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            rng = torch.Generator().manual_seed(200 + tid)
            k_gpu, v_gpu, k_host, v_host = pools(24, 20, seed=70 + tid)
            want_gk, want_gv = k_gpu.cpu(), v_gpu.cpu()
            want_hk, want_hv = canary_pool(k_host.shape), canary_pool(v_host.shape)
            for _ in range(12):
                n = int(torch.randint(1, 9, (1,), generator=rng))
                a = torch.randperm(24, generator=rng)[:n].tolist()
                b = torch.randperm(20, generator=rng)[:n].tolist()
                c = torch.randperm(24, generator=rng)[:n].tolist()
                do_swap(kvm, a, b, False, k_gpu, v_gpu, k_host, v_host, stream=stream)
                do_swap(kvm, b, c, True, k_gpu, v_gpu, k_host, v_host, stream=stream)
                oracle.swap_c(a, b, want_gk, want_hk)
                oracle.swap_c(a, b, want_gv, want_hv)
                oracle.swap_c(b, c, want_hk, want_gk)
                oracle.swap_c(b, c, want_hv, want_gv)
            stream.synchronize()
            results[tid] = (same_bits(k_gpu.cpu(), want_gk) and same_bits(v_gpu.cpu(), want_gv)
                            and same_bits(k_host, want_hk) and same_bits(v_host, want_hv))
        except Exception as e:      # noqa: BLE001
            errors.append((tid, repr(e)))

    def migrator():
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            rng = torch.Generator().manual_seed(300)
            dk, dv = canary_pool(g.dec_pool_shape(nb)).cuda(), canary_pool(g.dec_pool_shape(nb)).cuda()
            want_k, want_v = canary_pool(g.dec_pool_shape(nb)), canary_pool(g.dec_pool_shape(nb))
            for _ in range(30):
                n = int(torch.randint(1, 9, (1,), generator=rng))
                ci = torch.randint(0, nb, (n,), generator=rng).tolist()
                di = torch.randperm(nb, generator=rng)[:n].tolist()
                kvm.migrate(kvm_geom(g), ci, di, dk.data_ptr(), dv.data_ptr(), nb, stream.cuda_stream)
                oracle.migrate_c(g, src_k, ci, di, want_k)
                oracle.migrate_c(g, src_v, ci, di, want_v)
            stream.synchronize()
            results["migrate"] = same_bits(dk.cpu(), want_k) and same_bits(dv.cpu(), want_v)
        except Exception as e:      # noqa: BLE001
            errors.append(("migrate", repr(e)))

    threads = [threading.Thread(target=swapper, args=(t,)) for t in range(2)] + [threading.Thread(target=migrator)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert results == {0: True, 1: True, "migrate": True}, results
    del keep
    kvm.reset()
