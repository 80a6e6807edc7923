"""Shared helpers of the test suite: seeded pools and oracle-side expected results."""
from __future__ import annotations

from typing import List

import torch

import oracle
from distserve_amd.workloads import CANARY_BITS, MigrateWorkload


def geom_of(w: MigrateWorkload, dec_pp_rank=None, dec_tp_rank=None) -> oracle.Geom:
    s = w.shape
    return oracle.Geom(s.num_layers, s.num_kv_heads, s.block_size, s.head_dim, s.dtype_bytes,
                       w.ctx_pp, w.ctx_tp, w.dec_pp, w.dec_tp,
                       w.dec_pp_rank if dec_pp_rank is None else dec_pp_rank,
                       w.dec_tp_rank if dec_tp_rank is None else dec_tp_rank)


def rand_pool(shape, seed: int, dtype=torch.float16) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    if dtype in (torch.float16, torch.float32):
        return (torch.rand(shape, generator=g) * 2 - 1).to(dtype)
    info = torch.iinfo(dtype)
    return torch.randint(info.min, info.max, shape, generator=g, dtype=dtype)


def canary_pool(shape, dtype=torch.float16) -> torch.Tensor:
    t = torch.empty(shape, dtype=dtype)
    oracle.bits(t).fill_(CANARY_BITS if t.element_size() >= 2 else 0x5A)
    return t


def make_src_pools(g: oracle.Geom, num_blocks: int, seed: int, dtype=torch.float16) -> List[List[torch.Tensor]]:
    """src[p][t] for every context rank, each with its own seed."""
    return [[rand_pool(g.ctx_pool_shape(num_blocks), seed * 1000 + p * 37 + t, dtype)
             for t in range(g.ctx_tp)] for p in range(g.ctx_pp)]


def same_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    return a.shape == b.shape and torch.equal(oracle.bits(a.contiguous()), oracle.bits(b.contiguous()))


def labelled_src_pools(g: oracle.Geom, num_blocks: int, dtype=torch.int32) -> List[List[torch.Tensor]]:
    """Context pools whose every element carries its own global coordinates:
    ``label = ((block * L + layer) * H + head) * (B*D) + slot`` with the layer and head counted
    over the WHOLE model.  Built from the rank -> slice rule alone (rank p of P holds layers
    [p*L/P, (p+1)*L/P), rank t of T heads [t*H/T, (t+1)*H/T)), with no copy arithmetic."""
    L, H, BD = g.num_layers, g.num_kv_heads, g.block_size * g.head_dim
    whole = torch.arange(num_blocks * L * H * BD, dtype=torch.int64).view(num_blocks, L, H, g.block_size, g.head_dim)
    Lc, Hc = L // g.ctx_pp, H // g.ctx_tp
    return [[whole[:, p * Lc:(p + 1) * Lc, t * Hc:(t + 1) * Hc].contiguous().to(dtype)
             for t in range(g.ctx_tp)] for p in range(g.ctx_pp)]


def expected_labels(g: oracle.Geom, ci, di, nb_dst: int, fill: int, dtype=torch.int32) -> torch.Tensor:
    """What the decoding rank's pool must hold after migrating labelled pools: at decoding
    block di[i], local (layer, head), the label of context block ci[i] and the GLOBAL layer
    and head that this rank's local ones stand for; ``fill`` everywhere else."""
    L, H, BD = g.num_layers, g.num_kv_heads, g.block_size * g.head_dim
    Ld, Hd = L // g.dec_pp, H // g.dec_tp
    out = torch.full((nb_dst, Ld, Hd, g.block_size, g.head_dim), fill, dtype=torch.int64)
    slot = torch.arange(BD).view(g.block_size, g.head_dim)
    for c, d in zip(ci, di):
        for l in range(Ld):
            for h in range(Hd):
                gl, gh = g.dec_pp_rank * Ld + l, g.dec_tp_rank * Hd + h
                out[d, l, h] = ((c * L + gl) * H + gh) * BD + slot
    return out.to(dtype)
