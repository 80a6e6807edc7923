"""GPU-side helpers: run the HIP path through the C ABI on pools uploaded from the CPU."""
from __future__ import annotations

from typing import List

import torch

import oracle
from distserve_amd import cabi
from helpers import canary_pool


def kvm_geom(g: oracle.Geom) -> cabi.KvmGeom:
    return cabi.geom(g.num_layers, g.num_kv_heads, g.block_size, g.head_dim, g.dtype_bytes,
                     g.ctx_pp, g.ctx_tp, g.dec_pp, g.dec_tp, g.dec_pp_rank, g.dec_tp_rank)


def stream_handle() -> int:
    return torch.cuda.current_stream().cuda_stream


def upload_and_register(g: oracle.Geom, src_k: List[List[torch.Tensor]], src_v: List[List[torch.Tensor]], kvm=cabi):
    """Copies every context rank's pools to the GPU and registers them with `kvm` (the
    product's binding unless another build's is given); returns the GPU tensors (the caller
    keeps them alive)."""
    dev_k = [[t.cuda() for t in row] for row in src_k]
    dev_v = [[t.cuda() for t in row] for row in src_v]
    for p in range(g.ctx_pp):
        for t in range(g.ctx_tp):
            k, v = dev_k[p][t], dev_v[p][t]
            kvm.register_source(g.ctx_pp, g.ctx_tp, p, t, g.num_layers, g.num_kv_heads,
                                k.data_ptr(), v.data_ptr(), k.numel() * k.element_size())
    return dev_k, dev_v


GUARD = 4096   # elements of canary kept on either side of a destination pool


def guarded_canary_pool(shape, dtype=torch.float16):
    """A canary-filled GPU pool that sits in the middle of a larger canary-filled buffer;
    returns (pool view, whole buffer).  The margins must still hold the canary afterwards:
    a write that strays past either end of the pool lands there."""
    n = 1
    for d in shape:
        n *= d
    whole = canary_pool((n + 2 * GUARD,), dtype).cuda()
    return whole[GUARD:GUARD + n].view(shape), whole


def guards_intact(whole: torch.Tensor) -> bool:
    margin = canary_pool((GUARD,), whole.dtype)
    got = whole.cpu()
    return (torch.equal(got[:GUARD].view(torch.uint8), margin.view(torch.uint8))
            and torch.equal(got[-GUARD:].view(torch.uint8), margin.view(torch.uint8)))


def gpu_migrate(g: oracle.Geom, ci, di, nb_dst: int, dtype=torch.float16, kvm=cabi):
    """Runs kvm_migrate into canary-filled destination pools; returns them on the CPU.  The
    pools have canary margins on both sides, which must survive."""
    dst_k, whole_k = guarded_canary_pool(g.dec_pool_shape(nb_dst), dtype)
    dst_v, whole_v = guarded_canary_pool(g.dec_pool_shape(nb_dst), dtype)
    kvm.migrate(kvm_geom(g), ci, di, dst_k.data_ptr(), dst_v.data_ptr(), nb_dst, stream_handle())
    torch.cuda.synchronize()
    assert guards_intact(whole_k) and guards_intact(whole_v), "a write strayed outside the destination pool"
    return dst_k.cpu(), dst_v.cpu()


def oracle_migrate(g: oracle.Geom, src_k, src_v, ci, di, nb_dst: int, dtype=torch.float16):
    want_k = canary_pool(g.dec_pool_shape(nb_dst), dtype)
    want_v = canary_pool(g.dec_pool_shape(nb_dst), dtype)
    oracle.migrate_c(g, src_k, ci, di, want_k)
    oracle.migrate_c(g, src_v, ci, di, want_v)
    return want_k, want_v
