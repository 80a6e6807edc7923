"""Pins the CPU oracle.  The reference holds no vector for this path (its native op is an
un-vendored library), so the oracle's formulations are checked against each other,
against torch library routines in the cases that reduce to them, by brute force on tiny
shapes, through invariants a wrong index or a dropped term would break, and against the
committed fixtures under tests/golden/."""
import hashlib
import itertools
import json
import os

import pytest
import torch

import oracle
from helpers import canary_pool, make_src_pools, rand_pool, same_bits

SIZES = (1, 2, 4)


def _layouts():
    for cpp, ctp, dpp, dtp in itertools.product(SIZES, SIZES, SIZES, SIZES):
        yield cpp, ctp, dpp, dtp


def _run(fn, g, src, ci, di, nb_dst, dtype=torch.float16):
    dst = canary_pool(g.dec_pool_shape(nb_dst), dtype)
    fn(g, src, ci, di, dst)
    return dst


@pytest.mark.parametrize("cpp,ctp,dpp,dtp", list(_layouts()))
def test_three_formulations_agree_on_every_layout(cpp, ctp, dpp, dtp):
    """C (pull form), torch cat/narrow/index_copy_ and Python push loops, every decoding rank."""
    ci, di = [3, 0, 4], [1, 5, 2]
    for q in range(dpp):
        for u in range(dtp):
            g = oracle.Geom(4, 4, 2, 2, 2, cpp, ctp, dpp, dtp, q, u)
            src = make_src_pools(g, 5, seed=11)
            a = _run(oracle.migrate_c, g, src, ci, di, 6)
            b = _run(oracle.migrate_cat, g, src, ci, di, 6)
            c = _run(oracle.migrate_push_loops, g, src, ci, di, 6)
            assert same_bits(a, b) and same_bits(a, c)


def _uneven_layouts(count=40, seed=3):
    """Layouts over 12 layers and 12 heads in which the two instances' splits do not nest
    (3 against 2, 4 against 6, ...): a decoding rank then overlaps context ranks partly."""
    import random
    rng = random.Random(seed)
    every = [c for c in itertools.product((1, 2, 3, 4, 6), repeat=4) if 3 in c or 6 in c]
    return sorted(rng.sample(every, count))


@pytest.mark.parametrize("cpp,ctp,dpp,dtp", _uneven_layouts())
def test_three_formulations_agree_when_the_splits_do_not_nest(cpp, ctp, dpp, dtp):
    ci, di = [2, 0], [1, 3]
    for q in range(dpp):
        for u in range(dtp):
            g = oracle.Geom(12, 12, 2, 2, 2, cpp, ctp, dpp, dtp, q, u)
            src = make_src_pools(g, 3, seed=13)
            a = _run(oracle.migrate_c, g, src, ci, di, 4)
            b = _run(oracle.migrate_cat, g, src, ci, di, 4)
            c = _run(oracle.migrate_push_loops, g, src, ci, di, 4)
            assert same_bits(a, b) and same_bits(a, c)


@pytest.mark.parametrize("cpp,ctp,dpp,dtp", list(_layouts()) + _uneven_layouts(12, seed=9))
def test_labelled_elements_arrive_under_their_global_layer_and_head(cpp, ctp, dpp, dtp):
    """Every element of the context pools carries its global (block, layer, head, slot) as
    its value, so the expected destination is written down from the meaning of the copy
    alone -- "decoding block di[i] holds context block ci[i]'s layers and heads of this
    rank" -- with none of the oracle's offset arithmetic.  A wrong owner, a wrong local
    offset, a transposed layer/head or a dropped rank all show as a wrong label."""
    from helpers import expected_labels, labelled_src_pools

    L = H = 12 if 3 in (cpp, ctp, dpp, dtp) or 6 in (cpp, ctp, dpp, dtp) else 4
    ci, di = [4, 0, 2], [1, 6, 3]
    for q in range(dpp):
        for u in range(dtp):
            g = oracle.Geom(L, H, 2, 3, 4, cpp, ctp, dpp, dtp, q, u)
            src = labelled_src_pools(g, 5)
            want = expected_labels(g, ci, di, 7, fill=-7)
            for fn in (oracle.migrate_c, oracle.migrate_cat):
                dst = torch.full(g.dec_pool_shape(7), -7, dtype=torch.int32)
                fn(g, src, ci, di, dst)
                assert torch.equal(dst, want), (fn.__name__, q, u)


def test_tp1_pp1_reduces_to_index_copy_of_index_select():
    g = oracle.Geom(3, 5, 4, 8, 2)
    src = make_src_pools(g, 9, seed=3)
    ci, di = [8, 2, 2, 5], [0, 6, 3, 1]          # a context block may be read twice
    got = _run(oracle.migrate_c, g, src, ci, di, 7)
    want = canary_pool(g.dec_pool_shape(7))
    want.index_copy_(0, torch.tensor(di), src[0][0].index_select(0, torch.tensor(ci)))
    assert same_bits(got, want)


def test_decoding_ranks_partition_the_whole_model_block():
    """Union over all decoding ranks == cat of all context ranks (no element lost or doubled)."""
    L, H = 8, 4
    ci, di = [1, 3], [2, 0]
    for cpp, ctp, dpp, dtp in [(2, 2, 1, 4), (4, 1, 2, 2), (1, 4, 4, 1), (2, 4, 4, 2)]:
        g0 = oracle.Geom(L, H, 2, 4, 2, cpp, ctp, dpp, dtp)
        src = make_src_pools(g0, 4, seed=5)
        whole = torch.cat([torch.cat(src[p], dim=2) for p in range(cpp)], dim=1)  # [blocks, L, H, B, D]
        rebuilt = torch.zeros((3, L, H, 2, 4), dtype=torch.float16)
        for q in range(dpp):
            for u in range(dtp):
                g = oracle.Geom(L, H, 2, 4, 2, cpp, ctp, dpp, dtp, q, u)
                dst = _run(oracle.migrate_c, g, src, ci, di, 3)
                rebuilt[:, q * g.dec_layers:(q + 1) * g.dec_layers, u * g.dec_heads:(u + 1) * g.dec_heads] = dst
        for c, d in zip(ci, di):
            assert same_bits(rebuilt[d], whole[c])


def test_untouched_blocks_keep_canary_and_sources_are_unchanged():
    g = oracle.Geom(4, 4, 2, 4, 2, 2, 2, 1, 2, 0, 1)
    src = make_src_pools(g, 6, seed=8)
    before = [[t.clone() for t in row] for row in src]
    dst = _run(oracle.migrate_c, g, src, [5, 1], [3, 0], 5)
    canary = canary_pool(g.dec_pool_shape(1))[0]
    for b in (1, 2, 4):
        assert same_bits(dst[b], canary)
    for b in (0, 3):
        assert not same_bits(dst[b], canary)
    for row, row0 in zip(src, before):
        for t, t0 in zip(row, row0):
            assert same_bits(t, t0)


def test_joint_permutation_of_index_pairs_changes_nothing():
    g = oracle.Geom(4, 2, 2, 4, 2, 2, 1, 1, 2, 0, 1)
    src = make_src_pools(g, 8, seed=2)
    ci, di = [7, 0, 3, 5], [1, 4, 0, 6]
    a = _run(oracle.migrate_c, g, src, ci, di, 7)
    perm = [2, 0, 3, 1]
    b = _run(oracle.migrate_c, g, src, [ci[i] for i in perm], [di[i] for i in perm], 7)
    assert same_bits(a, b)


def test_migrate_there_and_back_restores_the_original():
    """Context (pp2, tp2) -> decoding ranks (tp4), then the roles swapped: identity."""
    L, H = 4, 4
    fwd = dict(ctx_pp=2, ctx_tp=2, dec_pp=1, dec_tp=4)
    g0 = oracle.Geom(L, H, 2, 4, 2, **fwd)
    src = make_src_pools(g0, 5, seed=21)
    ci, mid, back = [4, 1, 2], [0, 2, 1], [3, 0, 4]
    mids = []
    for u in range(4):
        g = oracle.Geom(L, H, 2, 4, 2, dec_tp_rank=u, **fwd)
        mids.append(_run(oracle.migrate_c, g, src, ci, mid, 3))
    for p in range(2):
        for t in range(2):
            g = oracle.Geom(L, H, 2, 4, 2, ctx_pp=1, ctx_tp=4, dec_pp=2, dec_tp=2, dec_pp_rank=p, dec_tp_rank=t)
            out = _run(oracle.migrate_c, g, [mids], mid, back, 5)
            for c, b in zip(ci, back):
                assert same_bits(out[b], src[p][t][c])


def test_swap_formulations_agree_and_round_trip():
    gpu = rand_pool((6, 2, 3, 4, 8), 1)
    host = canary_pool((5, 2, 3, 4, 8))
    gpu0 = gpu.clone()
    a, b = host.clone(), host.clone()
    oracle.swap_c([4, 0, 5], [1, 3, 0], gpu, a)
    oracle.swap_lib([4, 0, 5], [1, 3, 0], gpu, b)
    assert same_bits(a, b)
    assert same_bits(a[1], gpu0[4]) and same_bits(a[3], gpu0[0]) and same_bits(a[0], gpu0[5])
    assert same_bits(a[2], host[2]) and same_bits(a[4], host[4])
    back = canary_pool((6, 2, 3, 4, 8))
    oracle.swap_c([1, 3, 0], [2, 5, 1], a, back)      # back into different slots
    assert same_bits(back[2], gpu0[4]) and same_bits(back[5], gpu0[0]) and same_bits(back[1], gpu0[5])


def test_oracle_rejects_bad_indices_and_accepts_empty_lists():
    g = oracle.Geom(2, 2, 2, 2, 2)
    src = make_src_pools(g, 3, seed=1)
    dst = canary_pool(g.dec_pool_shape(3))
    oracle.migrate_c(g, src, [], [], dst)
    oracle.migrate_cat(g, src, [], [], dst)
    assert same_bits(dst, canary_pool(g.dec_pool_shape(3)))
    with pytest.raises(ValueError):
        oracle.migrate_c(g, src, [3], [0], dst)
    with pytest.raises(ValueError):
        oracle.migrate_c(g, src, [0], [-1], dst)
    with pytest.raises(ValueError):
        oracle.swap_c([0], [9], src[0][0], dst)


def test_fp32_and_odd_shapes():
    g = oracle.Geom(3, 3, 3, 5, 4, 3, 1, 1, 3, 0, 2)
    src = make_src_pools(g, 4, seed=9, dtype=torch.float32)
    a = _run(oracle.migrate_c, g, src, [3, 1], [0, 2], 3, torch.float32)
    b = _run(oracle.migrate_cat, g, src, [3, 1], [0, 2], 3, torch.float32)
    c = _run(oracle.migrate_push_loops, g, src, [3, 1], [0, 2], 3, torch.float32)
    assert same_bits(a, b) and same_bits(a, c)


# ---- committed fixtures (made by tests/golden/make_golden.py from this repository's oracle)

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "migrate_golden.json")


def _sha(t: torch.Tensor) -> str:
    return hashlib.sha256(oracle.bits(t.contiguous()).numpy().tobytes()).hexdigest()


def test_golden_fixture_matches_every_formulation():
    from golden.make_golden import build_case

    cases = json.load(open(GOLDEN))["cases"]
    assert len(cases) >= 5
    for case in cases:
        g, src_k, src_v, ci, di, nb_dst = build_case(case)
        for kind, src in (("k", src_k), ("v", src_v)):
            for fn in (oracle.migrate_c, oracle.migrate_cat):
                dst = canary_pool(g.dec_pool_shape(nb_dst))
                fn(g, src, ci, di, dst)
                assert _sha(dst) == case["sha256_" + kind], (case["name"], kind, fn.__name__)
