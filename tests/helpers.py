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
