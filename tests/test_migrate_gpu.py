"""Parity of the HIP migration path against the CPU oracle, called through the C ABI.
Bit-exact: pools are compared as raw 16/32-bit patterns."""
import functools
import itertools
import json
import os

import pytest
import torch

import oracle
from distserve_amd import workloads
from gpu_helpers import gpu_migrate, kvm_geom, oracle_migrate, stream_handle, upload_and_register
from helpers import canary_pool, geom_of, make_src_pools, same_bits

pytestmark = pytest.mark.gpu


def check_case(kvm, g, nb_src, nb_dst, ci, di, seed=1, dtype=torch.float16):
    kvm.reset()
    src_k = make_src_pools(g, nb_src, seed, dtype)
    src_v = make_src_pools(g, nb_src, seed + 500, dtype)
    keep = upload_and_register(g, src_k, src_v, kvm)
    got_k, got_v = gpu_migrate(g, ci, di, nb_dst, dtype, kvm)
    want_k, want_v = oracle_migrate(g, src_k, src_v, ci, di, nb_dst, dtype)
    assert same_bits(got_k, want_k), "K pool differs from the oracle"
    assert same_bits(got_v, want_v), "V pool differs from the oracle"
    # sources are only read
    for p in range(g.ctx_pp):
        for t in range(g.ctx_tp):
            assert same_bits(keep[0][p][t].cpu(), src_k[p][t]) and same_bits(keep[1][p][t].cpu(), src_v[p][t])
    kvm.reset()


def test_config1_gpt2_small_bit_exact(kvm):
    w = workloads.config1()
    call = w.calls[0]
    check_case(kvm, geom_of(w), w.src_blocks, w.dst_blocks, call.ctx_idx, call.dec_idx, seed=w.seed)


@pytest.mark.parametrize("cpp,ctp,dpp,dtp", list(itertools.product((1, 2, 4), repeat=4)))
def test_every_layout_and_every_decoding_rank(kvm, cpp, ctp, dpp, dtp):
    ci, di = [3, 0, 4, 3], [1, 5, 2, 0]
    for q in range(dpp):
        for u in range(dtp):
            g = oracle.Geom(4, 4, 16, 8, 2, cpp, ctp, dpp, dtp, q, u)
            check_case(kvm, g, 5, 6, ci, di, seed=7)


def _uneven_layouts(count=48, seed=5):
    import random
    rng = random.Random(seed)
    every = [c for c in itertools.product((1, 2, 3, 4, 6), repeat=4) if 3 in c or 6 in c]
    return sorted(rng.sample(every, count))


@pytest.mark.parametrize("cpp,ctp,dpp,dtp", _uneven_layouts())
def test_layouts_whose_splits_do_not_nest(kvm, cpp, ctp, dpp, dtp):
    """12 layers and 12 heads split by 3 against 2, 4 against 6, ...: a decoding rank overlaps
    some context ranks only partly, so one call has segments of different widths."""
    ci, di = [3, 0, 4, 3], [1, 5, 2, 0]
    for q in range(dpp):
        for u in range(dtp):
            g = oracle.Geom(12, 12, 4, 8, 2, cpp, ctp, dpp, dtp, q, u)
            check_case(kvm, g, 5, 6, ci, di, seed=17)


@pytest.mark.parametrize("cpp,ctp,dpp,dtp", [(2, 2, 1, 4), (1, 2, 1, 1), (4, 1, 2, 2), (2, 4, 4, 1), (3, 2, 2, 3), (1, 6, 3, 4)])
def test_labelled_elements_arrive_under_their_global_layer_and_head(kvm, cpp, ctp, dpp, dtp):
    """The kernel against expectations written down without any copy arithmetic: every source
    element carries its global (block, layer, head, slot), and the destination must hold, at
    decoding block di[i], the labels of context block ci[i] for this rank's layers and heads."""
    from helpers import expected_labels, labelled_src_pools

    ci, di = [4, 0, 2, 3], [1, 6, 3, 0]
    for q in range(dpp):
        for u in range(dtp):
            g = oracle.Geom(12, 12, 16, 8, 4, cpp, ctp, dpp, dtp, q, u)
            kvm.reset()
            src = labelled_src_pools(g, 5)
            keep = upload_and_register(g, src, src)
            dst_k = torch.full(g.dec_pool_shape(7), -7, dtype=torch.int32, device="cuda")
            dst_v = torch.full(g.dec_pool_shape(7), -7, dtype=torch.int32, device="cuda")
            kvm.migrate(kvm_geom(g), ci, di, dst_k.data_ptr(), dst_v.data_ptr(), 7, stream_handle())
            torch.cuda.synchronize()
            want = expected_labels(g, ci, di, 7, fill=-7)
            assert torch.equal(dst_k.cpu(), want) and torch.equal(dst_v.cpu(), want), (q, u)
            del keep
    kvm.reset()


def test_golden_fixtures(kvm):
    import hashlib
    from golden.make_golden import build_case

    path = os.path.join(os.path.dirname(__file__), "golden", "migrate_golden.json")
    for case in json.load(open(path))["cases"]:
        kvm.reset()
        g, src_k, src_v, ci, di, nb_dst = build_case(case)
        keep = upload_and_register(g, src_k, src_v)
        got_k, got_v = gpu_migrate(g, ci, di, nb_dst)
        for kind, got in (("k", got_k), ("v", got_v)):
            digest = hashlib.sha256(oracle.bits(got.contiguous()).numpy().tobytes()).hexdigest()
            assert digest == case["sha256_" + kind], (case["name"], kind)
        del keep
    kvm.reset()


@pytest.mark.parametrize("B,D,s,dtype", [(16, 128, 2, torch.float16), (16, 64, 4, torch.float32),
                                         (1, 4, 2, torch.float16), (3, 5, 2, torch.float16),
                                         (1, 1, 2, torch.float16), (7, 3, 4, torch.float32)])
def test_block_and_head_sizes_down_to_narrow_vectors(kvm, B, D, s, dtype):
    """Head slabs of 4 KiB down to 2 bytes: the vector width falls from 16 bytes to 2."""
    g = oracle.Geom(4, 6, B, D, s, 2, 3, 1, 2, 0, 1)
    check_case(kvm, g, 9, 11, [8, 2, 0, 5, 7], [10, 0, 3, 6, 1], seed=13, dtype=dtype)
    kvm.reset()


def test_misaligned_pool_bases_pick_a_narrower_vector(kvm):
    g = oracle.Geom(2, 2, 4, 8, 2)                      # 64-byte head slabs
    kvm.reset()
    src_k = make_src_pools(g, 6, 3)[0][0]
    src_v = make_src_pools(g, 6, 4)[0][0]
    n = src_k.numel()
    raw_k = torch.zeros(n + 8, dtype=torch.float16, device="cuda")
    raw_v = torch.zeros(n + 8, dtype=torch.float16, device="cuda")
    dk, dv = raw_k[2:2 + n], raw_v[2:2 + n]             # bases 4 bytes past a 16-byte boundary
    dk.copy_(src_k.flatten())
    dv.copy_(src_v.flatten())
    kvm.register_source(1, 1, 0, 0, 2, 2, dk.data_ptr(), dv.data_ptr(), n * 2)
    dst_k = canary_pool(g.dec_pool_shape(5)).cuda()
    dst_v = canary_pool(g.dec_pool_shape(5)).cuda()
    plan = kvm.migrate_plan(kvm_geom(g), 3, dst_k.data_ptr(), dst_v.data_ptr())
    assert plan["vector_bytes"] == 4
    kvm.migrate(kvm_geom(g), [5, 0, 2], [1, 4, 0], dst_k.data_ptr(), dst_v.data_ptr(), 5, stream_handle())
    torch.cuda.synchronize()
    want_k, want_v = oracle_migrate(g, [[src_k]], [[src_v]], [5, 0, 2], [1, 4, 0], 5)
    assert same_bits(dst_k.cpu(), want_k) and same_bits(dst_v.cpu(), want_v)
    kvm.reset()


@pytest.mark.parametrize("n", [0, 1, 431, 432, 433, 863, 864, 865, 1000, 1729, 2000])
def test_list_lengths_around_the_per_launch_limit(kvm, n):
    """One launch carries 864 index pairs (pools of at most 65536 blocks: a pair packs into 32
    bits); longer lists split into several launches."""
    g = oracle.Geom(2, 2, 16, 8, 2)
    gen = torch.Generator().manual_seed(n)
    ci = torch.randint(0, 64, (n,), generator=gen).tolist()          # context blocks may repeat
    di = torch.randperm(2100, generator=gen)[:n].tolist()
    check_case(kvm, g, 64, 2100, ci, di, seed=5)


@pytest.mark.parametrize("n", [1, 432, 433, 900])
@pytest.mark.parametrize("big", ["destination", "source"])
def test_pools_of_more_than_65536_blocks_take_wide_index_pairs(kvm, n, big):
    """Block ids beyond 16 bits travel as two int32 (432 pairs per launch).  The blocks are
    64 bytes here, so that 70000 of them are a small pool; the top ids are used."""
    g = oracle.Geom(1, 1, 4, 4, 2)
    nb_src, nb_dst = (64, 70000) if big == "destination" else (70000, 1200)
    gen = torch.Generator().manual_seed(n)
    ci = (torch.randint(0, nb_src, (n,), generator=gen)).tolist()
    di = torch.randperm(nb_dst, generator=gen)[:n].tolist()
    ci[0], di[0] = nb_src - 1, nb_dst - 1
    kvm.reset()
    keep = upload_and_register(g, make_src_pools(g, nb_src, 1), make_src_pools(g, nb_src, 2), kvm)
    dst = canary_pool(g.dec_pool_shape(nb_dst)).cuda()
    plan = kvm.migrate_plan(kvm_geom(g), n, dst.data_ptr(), dst.data_ptr(), nb_dst)
    assert plan["pairs_per_launch"] == 432 and plan["launches"] == -(-n // 432)
    del keep, dst
    check_case(kvm, g, nb_src, nb_dst, ci, di, seed=9)


@pytest.mark.parametrize("order", ["scattered", "neighbours", "descending"])
def test_many_segments_times_many_pairs_split_into_launches_both_ways(kvm, order):
    """pp4 x tp4 context ranks feed one decoding rank (16 segments: two groups of 8) and the
    list has 1800 pairs (three launches of 864 per group): the launch splitter's two loops
    multiply, and a mostly-neighbouring list keeps its order over all six launches."""
    g = oracle.Geom(8, 8, 4, 8, 2, 4, 4, 1, 1, 0, 0)
    n, nb_src, nb_dst = 1800, 2000, 2200
    gen = torch.Generator().manual_seed(3)
    if order == "scattered":
        ci = torch.randperm(nb_src, generator=gen)[:n].tolist()
    elif order == "neighbours":
        ci = list(range(7, 7 + 700)) + list(range(1200, 1200 + 600)) + list(range(800, 800 + 500))
    else:
        ci = list(range(nb_src - 1, nb_src - 1 - n, -1))
    di = torch.randperm(nb_dst, generator=gen)[:n].tolist()
    kvm.reset()
    keep = upload_and_register(g, make_src_pools(g, nb_src, 1), make_src_pools(g, nb_src, 2), kvm)
    dst = canary_pool(g.dec_pool_shape(nb_dst)).cuda()
    plan = kvm.migrate_plan(kvm_geom(g), n, dst.data_ptr(), dst.data_ptr(), nb_dst)
    assert plan["segments"] == 16 and plan["pairs_per_launch"] == 864 and plan["launches"] == 2 * 3
    del keep, dst
    check_case(kvm, g, nb_src, nb_dst, ci, di, seed=31)


@pytest.mark.parametrize("sort_pairs", [0, 1, 2])
@pytest.mark.parametrize("n,nb_src", [(40, 64), (200, 256), (200, 4000), (1000, 1100)])
def test_the_order_of_the_pairs_is_the_librarys_to_choose(kvm, sort_pairs, n, nb_src):
    """A call that names a quarter of the context pool or more has its pairs put in the order
    of their context blocks before they reach the kernel ("sort_pairs" 1; 2 always, 0
    never); the copy is the same whatever the order, repeated context blocks included."""
    g = oracle.Geom(2, 4, 16, 32, 2, 1, 2, 1, 1)
    gen = torch.Generator().manual_seed(n + nb_src)
    ci = torch.randint(0, nb_src, (n,), generator=gen).tolist()      # with repeats
    di = torch.randperm(n + 50, generator=gen)[:n].tolist()
    old = kvm.get_option("sort_pairs")
    kvm.set_option("sort_pairs", sort_pairs)
    try:
        check_case(kvm, g, nb_src, n + 50, ci, di, seed=13)
    finally:
        kvm.set_option("sort_pairs", old)


def test_more_context_ranks_than_one_launch_holds(kvm):
    """pp4 x tp4 context ranks all feed one decoding rank: 16 segments, 8 per launch."""
    g = oracle.Geom(8, 8, 16, 8, 2, 4, 4, 1, 1, 0, 0)
    check_case(kvm, g, 7, 9, [6, 1, 3], [0, 8, 4], seed=17)
    kvm.reset()
    keep = upload_and_register(g, make_src_pools(g, 7, 1), make_src_pools(g, 7, 2))
    dst = canary_pool(g.dec_pool_shape(9)).cuda()
    plan = kvm.migrate_plan(kvm_geom(g), 3, dst.data_ptr(), dst.data_ptr(), 9)
    assert plan["segments"] == 16 and plan["launches"] == 2
    del keep
    kvm.reset()


@pytest.mark.parametrize("tile_bytes,threads,unroll,flavours", [
    (0, 64, 1, ((1, 1, 0), (0, 0, 0))),          # the default: one-shot single-wave workgroups
    (0, 64, 2, ((1, 1, 0),)), (0, 128, 1, ((1, 1, 0),)), (4096, 256, 1, ((1, 1, 0),)),
    (0, 256, 4, ((1, 1, 0), (0, 0, 0))), (32768, 256, 4, ((1, 1, 0),)), (0, 256, 8, ((1, 1, 0), (1, 1, 1))),
    (8192, 512, 2, ((1, 1, 0),)), (1 << 20, 512, 8, ((1, 1, 0), (0, 0, 0))), (16384, 1024, 4, ((1, 1, 0),)),
    (1024, 64, 4, ((1, 1, 1),)), (2048, 64, 1, ((1, 1, 0),))])
def test_every_tuning_choice_copies_the_same_bytes(kvm_explore, tile_bytes, threads, unroll, flavours):
    """Through the exploration build: the product carries the first flavour only."""
    kvm = kvm_explore
    names = ("tile_bytes", "threads", "unroll", "nt_load", "nt_store", "wave_contig")
    saved = {k: kvm.get_option(k) for k in names}
    try:
        kvm.set_option("tile_bytes", tile_bytes)
        kvm.set_option("threads", threads)
        kvm.set_option("unroll", unroll)
        for ntl, nts, contig in flavours:
            kvm.set_option("nt_load", ntl)
            kvm.set_option("nt_store", nts)
            kvm.set_option("wave_contig", contig)
            # 24 KiB rows (cfg1 shape), 80 KiB rows (TP2->1) and 8 KiB strided rows (GQA slice)
            check_case(kvm, oracle.Geom(3, 12, 16, 64, 2), 6, 7, [5, 1, 2], [0, 6, 3], seed=3)
            check_case(kvm, oracle.Geom(4, 40, 16, 128, 2, 1, 2, 1, 1), 4, 5, [3, 1], [0, 4], seed=4)
            check_case(kvm, oracle.Geom(12, 8, 16, 128, 2, 2, 2, 1, 4, 0, 1), 5, 6, [4, 0, 2], [1, 5, 3], seed=5)
    finally:
        for k, v in saved.items():
            kvm.set_option(k, v)


def test_a_flavour_that_was_not_built_is_refused(kvm_explore):
    kvm = kvm_explore
    g = oracle.Geom(2, 2, 16, 8, 2)
    kvm.reset()
    keep = upload_and_register(g, make_src_pools(g, 3, 1), make_src_pools(g, 3, 2), kvm)
    dst = canary_pool(g.dec_pool_shape(3)).cuda()
    old = kvm.get_option("unroll")
    try:
        kvm.set_option("nt_load", 0)            # plain loads with nontemporal stores: built for a few shapes only
        kvm.set_option("unroll", 16)
        with pytest.raises(kvm.KvmError) as e:
            kvm.migrate(kvm_geom(g), [0], [1], dst.data_ptr(), dst.data_ptr(), 3, stream_handle())
        assert e.value.code == kvm.KVM_EINVAL and "no kernel was built" in str(e.value)
    finally:
        kvm.set_option("unroll", old)
        kvm.set_option("nt_load", 1)
    torch.cuda.synchronize()
    assert same_bits(dst.cpu(), canary_pool(g.dec_pool_shape(3)))
    del keep
    kvm.reset()


def test_errors_leave_the_destination_untouched(kvm):
    g = oracle.Geom(2, 4, 16, 8, 2, 1, 2, 1, 1)
    kvm.reset()
    src_k, src_v = make_src_pools(g, 4, 1), make_src_pools(g, 4, 2)
    keep = upload_and_register(g, src_k, src_v)
    dst_k = canary_pool(g.dec_pool_shape(6)).cuda()
    dst_v = canary_pool(g.dec_pool_shape(6)).cuda()
    args = (dst_k.data_ptr(), dst_v.data_ptr(), 6, stream_handle())
    cases = [
        ([0, 1], [2, 2], kvm.KVM_EDUP),             # decoding block named twice
        ([4], [0], kvm.KVM_ERANGE),                 # context index == pool size
        ([-1], [0], kvm.KVM_ERANGE),
        ([0], [6], kvm.KVM_ERANGE),
        ([0], [-3], kvm.KVM_ERANGE),
        ([0, 1], [0], kvm.KVM_EINVAL),              # lists of different length
    ]
    for ci, di, code in cases:
        with pytest.raises(kvm.KvmError) as e:
            kvm.migrate(kvm_geom(g), ci, di, *args)
        assert e.value.code == code, (ci, di, str(e.value))
    # geometry that disagrees with what was registered
    with pytest.raises(kvm.KvmError) as e:
        kvm.migrate(kvm_geom(oracle.Geom(2, 4, 16, 8, 2, 1, 1, 1, 1)), [0], [0], *args)
    assert e.value.code in (kvm.KVM_EMISMATCH, kvm.KVM_ENOTREG)
    # a geometry whose blocks do not tile the registered pools
    with pytest.raises(kvm.KvmError) as e:
        kvm.migrate(kvm_geom(oracle.Geom(2, 4, 16, 24, 2, 1, 2, 1, 1)), [0], [0], *args)
    assert e.value.code == kvm.KVM_EMISMATCH
    # a host pointer is not a pool
    host = torch.zeros(1024, dtype=torch.float16)
    with pytest.raises(kvm.KvmError) as e:
        kvm.migrate(kvm_geom(g), [0], [0], host.data_ptr(), host.data_ptr(), 1, stream_handle())
    assert e.value.code == kvm.KVM_EINVAL
    torch.cuda.synchronize()
    assert same_bits(dst_k.cpu(), canary_pool(g.dec_pool_shape(6)))
    assert same_bits(dst_v.cpu(), canary_pool(g.dec_pool_shape(6)))
    del keep
    kvm.reset()


@pytest.mark.parametrize("make,layers", [(workloads.config2, 2), (workloads.config3, 2), (workloads.config4, 4)])
def test_configs_2_3_4_block_tables_on_a_thinner_model(kvm, make, layers):
    """The measured configurations' real block tables, rank layouts, head counts and head
    size on a model with fewer layers, so that the oracle finishes in seconds.  Calls that
    recycle block ids are verified one by one."""
    w = workloads.scaled(make(), num_layers=layers)
    g = geom_of(w)
    kvm.reset()
    src_k = make_src_pools(g, w.src_blocks, w.seed)
    src_v = make_src_pools(g, w.src_blocks, w.seed + 500)
    keep = upload_and_register(g, src_k, src_v)
    dst_k = canary_pool(g.dec_pool_shape(w.dst_blocks)).cuda()
    dst_v = canary_pool(g.dec_pool_shape(w.dst_blocks)).cuda()
    want_k = canary_pool(g.dec_pool_shape(w.dst_blocks))
    want_v = canary_pool(g.dec_pool_shape(w.dst_blocks))
    for call in w.calls:
        kvm.migrate(kvm_geom(g), call.ctx_idx, call.dec_idx, dst_k.data_ptr(), dst_v.data_ptr(), w.dst_blocks,
                    stream_handle())
        oracle.migrate_c(g, src_k, call.ctx_idx, call.dec_idx, want_k)
        oracle.migrate_c(g, src_v, call.ctx_idx, call.dec_idx, want_v)
        if w.recycles_blocks:
            torch.cuda.synchronize()
            idx = torch.tensor(call.dec_idx)
            assert same_bits(dst_k.cpu()[idx], want_k[idx]) and same_bits(dst_v.cpu()[idx], want_v[idx]), call.request_id
    torch.cuda.synchronize()
    assert same_bits(dst_k.cpu(), want_k) and same_bits(dst_v.cpu(), want_v)
    del keep
    kvm.reset()


def test_config2_full_size_properties(kvm):
    """LLaMA-2-7B shape at full size (two 32 GiB pool pairs): every migrated block equals its
    source (checked on the GPU with torch's own gather), every other destination block
    still holds the canary, and sampled blocks agree with the oracle on the CPU."""
    w = workloads.config2()
    g = geom_of(w)
    kvm.reset()
    shape_src, shape_dst = w.src_pool_shape(), w.dst_pool_shape()
    src_k = workloads.fill_uniform(shape_src, w.seed, "cuda")
    src_v = workloads.fill_uniform(shape_src, w.seed + 500, "cuda")
    dst_k = workloads.fill_canary(shape_dst, "cuda")
    dst_v = workloads.fill_canary(shape_dst, "cuda")
    kvm.register_source(1, 1, 0, 0, g.num_layers, g.num_kv_heads, src_k.data_ptr(), src_v.data_ptr(),
                        src_k.numel() * 2)
    for call in w.calls:                                   # one call per request, as the engine does
        kvm.migrate(kvm_geom(g), call.ctx_idx, call.dec_idx, dst_k.data_ptr(), dst_v.data_ptr(), w.dst_blocks,
                    stream_handle())
    torch.cuda.synchronize()
    ctx = torch.tensor([b for c in w.calls for b in c.ctx_idx], device="cuda")
    dec = torch.tensor([b for c in w.calls for b in c.dec_idx], device="cuda")
    for src, dst in ((src_k, dst_k), (src_v, dst_v)):
        for i0 in range(0, ctx.numel(), 128):
            a = dst.view(torch.int16)[dec[i0:i0 + 128]]
            b = src.view(torch.int16)[ctx[i0:i0 + 128]]
            assert torch.equal(a, b)
        untouched = torch.ones(w.dst_blocks, dtype=torch.bool, device="cuda")
        untouched[dec] = False
        rest = untouched.nonzero().flatten()
        for i0 in range(0, rest.numel(), 256):
            assert bool((dst.view(torch.int16)[rest[i0:i0 + 256]] == workloads.CANARY_BITS).all())
    # oracle on a sample: compact the touched blocks into small CPU pools
    pick = list(range(0, ctx.numel(), max(1, ctx.numel() // 24)))[:24]
    ci = [int(ctx[i]) for i in pick]
    di = [int(dec[i]) for i in pick]
    small_src_k = src_k[torch.tensor(ci, device="cuda")].cpu()
    small_src_v = src_v[torch.tensor(ci, device="cuda")].cpu()
    want_k = canary_pool(g.dec_pool_shape(len(pick)))
    want_v = canary_pool(g.dec_pool_shape(len(pick)))
    oracle.migrate_c(g, [[small_src_k]], list(range(len(pick))), list(range(len(pick))), want_k)
    oracle.migrate_c(g, [[small_src_v]], list(range(len(pick))), list(range(len(pick))), want_v)
    assert same_bits(dst_k[torch.tensor(di, device="cuda")].cpu(), want_k)
    assert same_bits(dst_v[torch.tensor(di, device="cuda")].cpu(), want_v)
    kvm.reset()


def test_migration_is_ordered_on_the_stream_it_is_given(kvm):
    """Producer kernel -> migrate -> consumer kernel on one side stream, no host sync in
    between: the copy must see the producer's data and the consumer must see the copy."""
    g = oracle.Geom(4, 8, 16, 128, 2)
    kvm.reset()
    nb = 96
    src_k = torch.zeros(g.ctx_pool_shape(nb), dtype=torch.float16, device="cuda")
    src_v = torch.zeros_like(src_k)
    fresh_k = make_src_pools(g, nb, 31)[0][0].cuda()
    fresh_v = make_src_pools(g, nb, 32)[0][0].cuda()
    dst_k = canary_pool(g.dec_pool_shape(nb)).cuda()
    dst_v = canary_pool(g.dec_pool_shape(nb)).cuda()
    kvm.register_source(1, 1, 0, 0, g.num_layers, g.num_kv_heads, src_k.data_ptr(), src_v.data_ptr(),
                        src_k.numel() * 2)
    gen = torch.Generator().manual_seed(3)
    ci = torch.randperm(nb, generator=gen).tolist()
    di = torch.randperm(nb, generator=gen).tolist()
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for _ in range(20):                       # keep the stream busy ahead of the producer
            fresh_k.add_(0)
        src_k.copy_(fresh_k)                      # producer: the "prefill" writes the blocks
        src_v.copy_(fresh_v)
        kvm.migrate(kvm_geom(g), ci, di, dst_k.data_ptr(), dst_v.data_ptr(), nb, side.cuda_stream)
        seen_k, seen_v = dst_k.clone(), dst_v.clone()     # consumer
    side.synchronize()
    want_k, want_v = oracle_migrate(g, [[fresh_k.cpu()]], [[fresh_v.cpu()]], ci, di, nb)
    assert same_bits(seen_k.cpu(), want_k) and same_bits(seen_v.cpu(), want_v)
    kvm.reset()


def test_calls_from_several_host_threads_on_their_own_streams(kvm):
    """The library may be entered concurrently: four threads, each with its own stream and
    its own destination pools, all reading the same registered source."""
    import threading

    g = oracle.Geom(2, 4, 16, 64, 2)
    kvm.reset()
    nb = 64
    src_k, src_v = make_src_pools(g, nb, 41), make_src_pools(g, nb, 42)
    keep = upload_and_register(g, src_k, src_v)
    results, errors = {}, []

    def work(tid):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            gen = torch.Generator().manual_seed(100 + tid)
            dk = canary_pool(g.dec_pool_shape(nb)).cuda()
            dv = canary_pool(g.dec_pool_shape(nb)).cuda()
            calls = []
            for _ in range(25):
                n = int(torch.randint(1, 9, (1,), generator=gen))
                ci = torch.randint(0, nb, (n,), generator=gen).tolist()
                di = torch.randperm(nb, generator=gen)[:n].tolist()
                kvm.migrate(kvm_geom(g), ci, di, dk.data_ptr(), dv.data_ptr(), nb, stream.cuda_stream)
                calls.append((ci, di))
            stream.synchronize()
            results[tid] = (dk.cpu(), dv.cpu(), calls)
        except Exception as e:      # noqa: BLE001
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for tid, (dk, dv, calls) in results.items():
        want_k, want_v = canary_pool(g.dec_pool_shape(nb)), canary_pool(g.dec_pool_shape(nb))
        for ci, di in calls:
            oracle.migrate_c(g, src_k, ci, di, want_k)
            oracle.migrate_c(g, src_v, ci, di, want_v)
        assert same_bits(dk, want_k) and same_bits(dv, want_v), tid
    del keep
    kvm.reset()


def test_registrations_from_one_thread_while_others_migrate(kvm):
    """A decoding worker may bind a second context instance (and re-bind it, and bind ranks it
    never reads) while its migrations from the first one are running on other threads: the
    registry is read under a shared lock and changed under an exclusive one, and a migration
    always sees the pools of a whole registration."""
    import threading

    g = oracle.Geom(2, 4, 16, 64, 2)
    kvm.reset()
    nb = 48
    src_k, src_v = make_src_pools(g, nb, 51), make_src_pools(g, nb, 52)
    keep = upload_and_register(g, src_k, src_v)                     # context instance 0
    other_k, other_v = make_src_pools(g, nb, 61), make_src_pools(g, nb, 62)
    dev_other = (other_k[0][0].cuda(), other_v[0][0].cuda())
    stop, errors, results = threading.Event(), [], {}

    def register():
        try:
            torch.cuda.set_device(0)
            n = 0
            while not stop.is_set():
                for inst in (1, 2, 3):
                    kvm.register_source(1, 1, 0, 0, g.num_layers, g.num_kv_heads, dev_other[0].data_ptr(),
                                        dev_other[1].data_ptr(), dev_other[0].numel() * 2, ctx_instance=inst)
                h = kvm.get_mem_handle(dev_other[0].data_ptr(), dev_other[0].numel() * 2)
                kvm.register_mem_handle(h, h, g.num_layers, g.num_kv_heads, [1, 0, 1, 0], [1, 0, 1, 0], ctx_instance=4)
                n += 1
            results["registrations"] = n
        except Exception as e:      # noqa: BLE001
            errors.append(("register", repr(e)))

    def work(tid):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            gen = torch.Generator().manual_seed(200 + tid)
            dk = canary_pool(g.dec_pool_shape(nb)).cuda()
            dv = canary_pool(g.dec_pool_shape(nb)).cuda()
            calls = []
            for _ in range(200):
                n = int(torch.randint(1, 9, (1,), generator=gen))
                ci = torch.randint(0, nb, (n,), generator=gen).tolist()
                di = torch.randperm(nb, generator=gen)[:n].tolist()
                kvm.migrate(kvm_geom(g), ci, di, dk.data_ptr(), dv.data_ptr(), nb, stream.cuda_stream)
                calls.append((ci, di))
            stream.synchronize()
            results[tid] = (dk.cpu(), dv.cpu(), calls)
        except Exception as e:      # noqa: BLE001
            errors.append((tid, repr(e)))

    registrar = threading.Thread(target=register)
    workers = [threading.Thread(target=work, args=(t,)) for t in range(3)]
    registrar.start()
    for t in workers:
        t.start()
    for t in workers:
        t.join()
    stop.set()
    registrar.join()
    assert not errors, errors
    assert results["registrations"] >= 1
    for tid in range(3):
        dk, dv, calls = results[tid]
        want_k, want_v = canary_pool(g.dec_pool_shape(nb)), canary_pool(g.dec_pool_shape(nb))
        for ci, di in calls:
            oracle.migrate_c(g, src_k, ci, di, want_k)
            oracle.migrate_c(g, src_v, ci, di, want_v)
        assert same_bits(dk, want_k) and same_bits(dv, want_v), tid
    # the instance bound meanwhile is usable afterwards
    g1 = kvm.geom(g.num_layers, g.num_kv_heads, g.block_size, g.head_dim, g.dtype_bytes, ctx_instance=1)
    dk, dv = canary_pool(g.dec_pool_shape(nb)).cuda(), canary_pool(g.dec_pool_shape(nb)).cuda()
    kvm.migrate(g1, [5, 7], [0, 1], dk.data_ptr(), dv.data_ptr(), nb, stream_handle())
    torch.cuda.synchronize()
    want_k, want_v = oracle_migrate(g, other_k, other_v, [5, 7], [0, 1], nb)
    assert same_bits(dk.cpu(), want_k) and same_bits(dv.cpu(), want_v)
    assert kvm.opened_handles() == 0
    del keep
    kvm.reset()


@pytest.mark.parametrize("make", [
    workloads.config3, workloads.config4,
    functools.partial(workloads.config3, fresh_pools=True), functools.partial(workloads.config4, fresh_pools=True),
], ids=["cfg3", "cfg4", "cfg3-neighbouring-blocks", "cfg4-neighbouring-blocks"])
def test_configs_3_and_4_full_size_properties(kvm, make):
    """OPT-13B (TP2 -> TP1) and LLaMA-2-70B GQA (TP2/PP2 -> TP4 rank 1) at full size: after
    every request's call, each of its blocks equals the source rectangles it was sliced from
    (torch slicing + gather on the GPU); sampled blocks agree with the oracle on the CPU.
    Once with the configurations' scattered block lists and once with the lists of block
    managers that have just started, whose launches hand out their work in plain order."""
    w = make()
    g = geom_of(w)
    kvm.reset()
    src_k = [[workloads.fill_uniform(w.src_pool_shape(), w.seed + 10 * p + t, "cuda") for t in range(w.ctx_tp)]
             for p in range(w.ctx_pp)]
    src_v = [[workloads.fill_uniform(w.src_pool_shape(), w.seed + 500 + 10 * p + t, "cuda") for t in range(w.ctx_tp)]
             for p in range(w.ctx_pp)]
    for p in range(w.ctx_pp):
        for t in range(w.ctx_tp):
            kvm.register_source(w.ctx_pp, w.ctx_tp, p, t, g.num_layers, g.num_kv_heads, src_k[p][t].data_ptr(),
                                src_v[p][t].data_ptr(), src_k[p][t].numel() * 2)
    dst_k = workloads.fill_canary(w.dst_pool_shape(), "cuda")
    dst_v = workloads.fill_canary(w.dst_pool_shape(), "cuda")
    l0, h0 = g.dec_pp_rank * g.dec_layers, g.dec_tp_rank * g.dec_heads
    for n_call, call in enumerate(w.calls):
        kvm.migrate(kvm_geom(g), call.ctx_idx, call.dec_idx, dst_k.data_ptr(), dst_v.data_ptr(), w.dst_blocks,
                    stream_handle())
        ctx = torch.tensor(call.ctx_idx, device="cuda")
        dec = torch.tensor(call.dec_idx, device="cuda")
        for src, dst in ((src_k, dst_k), (src_v, dst_v)):
            got = dst.view(torch.int16)[dec]
            for p in range(w.ctx_pp):
                for t in range(w.ctx_tp):
                    la, lb = max(l0, p * g.ctx_layers), min(l0 + g.dec_layers, (p + 1) * g.ctx_layers)
                    ha, hb = max(h0, t * g.ctx_heads), min(h0 + g.dec_heads, (t + 1) * g.ctx_heads)
                    if la >= lb or ha >= hb:
                        continue
                    want = src[p][t].view(torch.int16)[ctx, la - p * g.ctx_layers:lb - p * g.ctx_layers,
                                                       ha - t * g.ctx_heads:hb - t * g.ctx_heads]
                    assert torch.equal(got[:, la - l0:lb - l0, ha - h0:hb - h0], want), (call.request_id, p, t)
        if n_call % 8 == 0:                                   # oracle on a sample of this call's blocks
            pick = list(range(0, len(call.ctx_idx), max(1, len(call.ctx_idx) // 6)))[:6]
            ci = [call.ctx_idx[i] for i in pick]
            di = [call.dec_idx[i] for i in pick]
            sel = torch.tensor(ci, device="cuda")
            small_k = [[src_k[p][t][sel].cpu() for t in range(w.ctx_tp)] for p in range(w.ctx_pp)]
            small_v = [[src_v[p][t][sel].cpu() for t in range(w.ctx_tp)] for p in range(w.ctx_pp)]
            ident = list(range(len(pick)))
            want_k, want_v = oracle_migrate(g, small_k, small_v, ident, ident, len(pick))
            dsel = torch.tensor(di, device="cuda")
            assert same_bits(dst_k[dsel].cpu(), want_k) and same_bits(dst_v[dsel].cpu(), want_v)
    if not w.recycles_blocks:
        touched = torch.zeros(w.dst_blocks, dtype=torch.bool, device="cuda")
        touched[torch.tensor([b for c in w.calls for b in c.dec_idx], device="cuda")] = True
        rest = (~touched).nonzero().flatten()
        for dst in (dst_k, dst_v):
            for i0 in range(0, rest.numel(), 128):
                assert bool((dst.view(torch.int16)[rest[i0:i0 + 128]] == workloads.CANARY_BITS).all())
    kvm.reset()


@pytest.mark.parametrize("xcd_map,simple", [(0, 0), (0, 1), (1, 0), (1, 1), (2, 0), (2, 1), (3, 1), (1, None), (2, None)])
def test_every_id_to_work_mapping_copies_the_same_bytes(kvm, kvm_explore, xcd_map, simple):
    """Workgroup ids are dealt to XCDs in contiguous chunks; with padding ids when the work
    does not divide by 8 (odd tile counts, odd block counts).  simple None: the product (which
    always takes the short-prologue kernel where the shape allows); 0/1: the exploration build."""
    if simple is None:
        simple = 1
    else:
        kvm = kvm_explore
    saved = {k: kvm.get_option(k) for k in ("xcd_map",) + (("simple",) if kvm is kvm_explore else ())}
    try:
        kvm.set_option("xcd_map", xcd_map)
        if "simple" in saved:
            kvm.set_option("simple", simple)
        gen = torch.Generator().manual_seed(17)
        for g, nb_src, nb_dst, n in [
                (oracle.Geom(2, 16, 16, 128, 2), 40, 48, 37),                   # 128 KiB blocks: 128 tiles
                (oracle.Geom(1, 3, 16, 64, 2), 30, 31, 29),                     # 6 KiB blocks: 6 tiles, 29 blocks
                (oracle.Geom(4, 40, 16, 128, 2, 1, 2, 1, 1), 12, 13, 11),       # two segments of 80 KiB rows
                (oracle.Geom(12, 8, 16, 128, 2, 2, 2, 1, 4, 0, 1), 9, 10, 7),   # strided 8 KiB rows
                (oracle.Geom(16, 32, 16, 128, 2), 6, 7, 5)]:                    # 2 MiB blocks: an eighth is 256 KiB
            ci = torch.randint(0, nb_src, (n,), generator=gen).tolist()
            di = torch.randperm(nb_dst, generator=gen)[:n].tolist()
            check_case(kvm, g, nb_src, nb_dst, ci, di, seed=23)
    finally:
        for k, v in saved.items():
            kvm.set_option(k, v)


@pytest.mark.parametrize("build", ["product", "exploration"])
def test_random_geometries_pools_lists_and_tunings(kvm, kvm_explore, build):
    """300 seeded draws of everything at once: layer/head counts and splits (nesting or not),
    block and head sizes down to one element, 1/2/4-byte elements, pool sizes, index lists
    with repeated sources, and -- in the exploration build -- the kernel flavours, tile
    sizes and table forms (the product has one flavour; its draws vary its own options)."""
    import random

    if build == "product":
        rng = random.Random(21)
        saved = {k: kvm.get_option(k) for k in ("xcd_map", "sort_pairs")}
        try:
            for case in range(300):
                L, H = rng.choice([1, 2, 3, 4, 6, 8, 12]), rng.choice([1, 2, 3, 4, 6, 8, 12])
                div = lambda n: [d for d in range(1, n + 1) if n % d == 0]    # noqa: E731
                cpp, dpp, ctp, dtp = rng.choice(div(L)), rng.choice(div(L)), rng.choice(div(H)), rng.choice(div(H))
                B, D = rng.choice([1, 2, 3, 4, 8, 16, 32]), rng.choice([1, 2, 3, 5, 8, 16, 40, 64, 80, 128])
                s = rng.choice([1, 2, 2, 2, 4])
                g = oracle.Geom(L, H, B, D, s, cpp, ctp, dpp, dtp, rng.randrange(dpp), rng.randrange(dtp))
                nb_src, nb_dst = rng.randint(1, 12), rng.randint(1, 12)
                n = rng.randint(0, nb_dst)
                ci, di = [rng.randrange(nb_src) for _ in range(n)], rng.sample(range(nb_dst), n)
                chosen = dict(xcd_map=rng.randrange(4), sort_pairs=rng.randrange(3))
                for k, v in chosen.items():
                    kvm.set_option(k, v)
                try:
                    check_case(kvm, g, nb_src, nb_dst, ci, di, seed=case + 1,
                               dtype={1: torch.uint8, 2: torch.float16, 4: torch.float32}[s])
                except AssertionError as e:
                    raise AssertionError(f"case {case}: {g} {chosen} ctx {ci} dec {di}: {e}") from None
        finally:
            for k, v in saved.items():
                kvm.set_option(k, v)
        return
    kvm = kvm_explore

    rng = random.Random(20)
    names = ("threads", "unroll", "nt_load", "nt_store", "wave_contig", "tile_bytes", "xcd_map", "simple", "packed",
             "sort_pairs")
    saved = {k: kvm.get_option(k) for k in names}
    flavours = [(64, 1, 1, 1, 0), (64, 2, 1, 1, 0), (128, 1, 1, 1, 0), (256, 1, 1, 1, 0), (256, 4, 1, 1, 0),
                (256, 8, 1, 1, 0), (512, 2, 1, 1, 0), (512, 8, 1, 1, 0), (1024, 4, 1, 1, 0), (64, 1, 0, 0, 0),
                (256, 4, 0, 0, 0), (512, 8, 0, 0, 0), (64, 4, 1, 1, 1), (256, 8, 1, 1, 1)]
    dtypes = {1: torch.uint8, 2: torch.float16, 4: torch.float32}

    def divisors(n):
        return [d for d in range(1, n + 1) if n % d == 0]

    try:
        for case in range(300):
            L, H = rng.choice([1, 2, 3, 4, 6, 8, 12]), rng.choice([1, 2, 3, 4, 6, 8, 12])
            cpp, dpp = rng.choice(divisors(L)), rng.choice(divisors(L))
            ctp, dtp = rng.choice(divisors(H)), rng.choice(divisors(H))
            B, D = rng.choice([1, 2, 3, 4, 8, 16, 32]), rng.choice([1, 2, 3, 5, 8, 16, 40, 64, 80, 128])
            s = rng.choice([1, 2, 2, 2, 4])
            g = oracle.Geom(L, H, B, D, s, cpp, ctp, dpp, dtp, rng.randrange(dpp), rng.randrange(dtp))
            nb_src, nb_dst = rng.randint(1, 12), rng.randint(1, 12)
            n = rng.randint(0, nb_dst)
            ci = [rng.randrange(nb_src) for _ in range(n)]
            di = rng.sample(range(nb_dst), n)
            threads, unroll, nt_load, nt_store, wave_contig = rng.choice(flavours)
            chosen = dict(threads=threads, unroll=unroll, nt_load=nt_load, nt_store=nt_store, wave_contig=wave_contig,
                          tile_bytes=rng.choice([0, 0, 0, 1024, 4096, 16384, 65536]), xcd_map=rng.randrange(4),
                          simple=rng.randrange(2), packed=rng.randrange(2), sort_pairs=rng.randrange(3))
            for k, v in chosen.items():
                kvm.set_option(k, v)
            try:
                check_case(kvm, g, nb_src, nb_dst, ci, di, seed=case + 1, dtype=dtypes[s])
            except AssertionError as e:
                raise AssertionError(f"case {case}: {g} {chosen} ctx {ci} dec {di}: {e}") from None
    finally:
        for k, v in saved.items():
            kvm.set_option(k, v)


def test_a_pool_that_claims_more_than_its_allocation_is_refused_on_the_host(kvm):
    """A wrong block count would send the kernel past mapped memory.  The library asks the
    runtime where the allocation ends and refuses before anything is launched."""
    g = oracle.Geom(2, 4, 16, 64, 2)
    kvm.reset()
    block_bytes = 2 * 4 * 16 * 64 * 2                       # 16 KiB per block and pool kind
    nb = 4096                                               # 64 MiB pools: allocations of their own
    src_k = torch.zeros(g.ctx_pool_shape(nb), dtype=torch.float16, device="cuda")
    src_v = torch.zeros_like(src_k)
    dst_k = canary_pool(g.dec_pool_shape(nb)).cuda()
    dst_v = canary_pool(g.dec_pool_shape(nb)).cuda()
    with pytest.raises(kvm.KvmError) as e:                   # source said to be 64 times its size
        kvm.register_source(1, 1, 0, 0, g.num_layers, g.num_kv_heads, src_k.data_ptr(), src_v.data_ptr(),
                            64 * nb * block_bytes)
    assert e.value.code == kvm.KVM_ERANGE and "allocation ends" in str(e.value)
    kvm.register_source(1, 1, 0, 0, g.num_layers, g.num_kv_heads, src_k.data_ptr(), src_v.data_ptr(), nb * block_bytes)
    s = stream_handle()
    kvm.migrate(kvm_geom(g), [1], [2], dst_k.data_ptr(), dst_v.data_ptr(), nb, s)      # the true size is fine
    with pytest.raises(kvm.KvmError) as e:                   # destination said to hold 64 times its blocks
        kvm.migrate(kvm_geom(g), [1], [3], dst_k.data_ptr(), dst_v.data_ptr(), 64 * nb, s)
    assert e.value.code == kvm.KVM_ERANGE
    torch.cuda.synchronize()
    assert same_bits(dst_k[3].cpu(), canary_pool(g.dec_pool_shape(1))[0])               # nothing was launched
    kvm.migrate(kvm_geom(g), [1], [3], dst_k.data_ptr(), dst_v.data_ptr(), nb, s)      # and the pool is still usable
    torch.cuda.synchronize()
    assert same_bits(dst_k[3].cpu(), src_k[1].cpu())
    kvm.reset()


@pytest.mark.parametrize("cpp,ctp,dpp,dtp,q,u", [(1, 1, 1, 1, 0, 0), (2, 2, 1, 4, 0, 1), (1, 2, 1, 1, 0, 0)])
@pytest.mark.parametrize("lists", ["neighbours", "runs", "scattered", "descending"])
def test_lists_of_neighbouring_and_of_scattered_blocks_copy_the_same_way(kvm, cpp, ctp, dpp, dtp, q, u, lists):
    """The order in which a launch's workgroups take the work is chosen from the context block
    list (in order for mostly neighbouring blocks, per-XCD chunks for scattered ones); the bytes
    copied must not know about it.  Launches large enough for the chunks to differ from the
    plain order: 40 blocks of 64-128 tiles each."""
    import random

    g = oracle.Geom(8, 8, 16, 64, 2, cpp, ctp, dpp, dtp, q, u)
    rng = random.Random(hash((cpp, ctp, dtp, lists)) & 0xFFFF)
    nb_src, nb_dst, n = 48, 64, 40
    if lists == "neighbours":
        ci = list(range(5, 5 + n))                               # one run: ids in order
    elif lists == "runs":
        ci = list(range(30, 44)) + list(range(0, 13)) + list(range(17, 30))   # three runs: still mostly neighbours
    elif lists == "descending":
        ci = list(range(n + 3, 3, -1))                           # adjacent the wrong way round: not neighbours
    else:
        ci = rng.sample(range(nb_src), n)
    di = rng.sample(range(nb_dst), n)
    check_case(kvm, g, nb_src, nb_dst, ci, di, seed=23)
