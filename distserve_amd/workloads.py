"""Synthetic KV-movement workloads: the five measured configurations and scaled-down kin.

Everything is derived from a seed with ``torch.Generator`` so that the CPU checker, the
GPU tests and the benchmark see the same block tables.  Pool contents are fp16 values
uniform in [-1, 1); destination pools start from a canary bit pattern so that a stray or
a missing write shows.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import torch

CANARY_BITS = 0x7C01  # an fp16 signalling-NaN pattern that uniform [-1, 1) data never holds


@dataclass(frozen=True)
class KvShape:
    num_layers: int
    num_kv_heads: int
    head_dim: int
    block_size: int = 16
    dtype: torch.dtype = torch.float16

    @property
    def dtype_bytes(self) -> int:
        return torch.empty((), dtype=self.dtype).element_size()

    def pool_shape(self, num_blocks: int, pp: int = 1, tp: int = 1) -> Tuple[int, ...]:
        return (num_blocks, self.num_layers // pp, self.num_kv_heads // tp, self.block_size, self.head_dim)

    def block_bytes(self, pp: int = 1, tp: int = 1) -> int:
        """Bytes of one block of ONE pool kind on a rank of a (pp, tp) instance."""
        return (self.num_layers // pp) * (self.num_kv_heads // tp) * self.block_size * self.head_dim * self.dtype_bytes


@dataclass
class MigrateCall:
    """One ``migrate_blocks`` call: a request's context blocks and the decoding blocks they go to."""

    request_id: int
    prompt_len: int
    ctx_idx: List[int]
    dec_idx: List[int]


@dataclass
class MigrateWorkload:
    name: str
    shape: KvShape
    ctx_pp: int
    ctx_tp: int
    dec_pp: int
    dec_tp: int
    dec_pp_rank: int
    dec_tp_rank: int
    src_blocks: int
    dst_blocks: int
    seed: int
    calls: List[MigrateCall] = field(default_factory=list)
    recycles_blocks: bool = False   # True: calls reuse block ids, verify after each call

    @property
    def total_blocks(self) -> int:
        return sum(len(c.ctx_idx) for c in self.calls)

    @property
    def payload_bytes_per_block(self) -> int:
        """Bytes the decoding rank receives per block, K and V together."""
        return 2 * self.shape.block_bytes(self.dec_pp, self.dec_tp)

    @property
    def payload_bytes(self) -> int:
        return self.total_blocks * self.payload_bytes_per_block

    def src_pool_shape(self) -> Tuple[int, ...]:
        return self.shape.pool_shape(self.src_blocks, self.ctx_pp, self.ctx_tp)

    def dst_pool_shape(self) -> Tuple[int, ...]:
        return self.shape.pool_shape(self.dst_blocks, self.dec_pp, self.dec_tp)


def blocks_for(prompt_len: int, block_size: int) -> int:
    return -(-prompt_len // block_size)


def _lengths(g: torch.Generator, n: int, lo: int, hi: int) -> List[int]:
    return torch.randint(lo, hi + 1, (n,), generator=g).tolist()


def _disjoint_calls(g: torch.Generator, lengths: List[int], block_size: int, src_blocks: int,
                    dst_blocks: int, fresh: bool = False) -> List[MigrateCall]:
    """Per-request slices of two independent random permutations: non-contiguous and disjoint.
    ``fresh``: slices of ``0 .. n-1`` instead, what block managers hand out when they start."""
    src_perm = torch.randperm(src_blocks, generator=g).tolist()
    dst_perm = torch.randperm(dst_blocks, generator=g).tolist()
    if fresh:
        src_perm, dst_perm = list(range(src_blocks)), list(range(dst_blocks))
    calls, at = [], 0
    for rid, length in enumerate(lengths):
        n = blocks_for(length, block_size)
        assert at + n <= min(src_blocks, dst_blocks), "workload does not fit its pools"
        calls.append(MigrateCall(rid, length, src_perm[at:at + n], dst_perm[at:at + n]))
        at += n
    return calls


class _ShuffledFifo:
    """Free list with the block manager's discipline (take from the head, give back at the
    tail) but a shuffled initial order, as a pool looks after it has run for a while.
    ``fresh``: the order a block manager starts with, ``0 .. n-1``."""

    def __init__(self, n: int, g: torch.Generator, fresh: bool = False):
        self.free = list(range(n)) if fresh else torch.randperm(n, generator=g).tolist()

    def take(self, n: int) -> List[int]:
        assert len(self.free) >= n
        out, self.free = self.free[:n], self.free[n:]
        return out

    def give(self, ids: List[int]) -> None:
        self.free += ids


def _recycled_calls(g: torch.Generator, lengths: List[int], block_size: int, src_blocks: int,
                    dst_blocks: int, fresh: bool = False) -> List[MigrateCall]:
    """Sequential hand-offs through pools smaller than the batch: the context side frees a
    request's blocks right after its migration (as the engine does), the decoding side
    frees its oldest requests when it runs short."""
    src, dst = _ShuffledFifo(src_blocks, g, fresh), _ShuffledFifo(dst_blocks, g, fresh)
    resident: List[List[int]] = []
    calls = []
    for rid, length in enumerate(lengths):
        n = blocks_for(length, block_size)
        ctx = src.take(n)
        while len(dst.free) < n:
            dst.give(resident.pop(0))
        dec = dst.take(n)
        resident.append(dec)
        calls.append(MigrateCall(rid, length, ctx, dec))
        src.give(ctx)
    return calls


# ---- the measured configurations


def config1(seed: int = 1) -> MigrateWorkload:
    """GPT-2-small KV shape, 32 blocks, context TP1/PP1 -> decoding TP1 (CPU-sized)."""
    g = torch.Generator().manual_seed(seed)
    shape = KvShape(12, 12, 64)
    w = MigrateWorkload("cfg1-gpt2-small", shape, 1, 1, 1, 1, 0, 0, 256, 512, seed)
    ctx = torch.randperm(256, generator=g)[:32].tolist()
    dec = torch.randperm(512, generator=g)[:32].tolist()
    w.calls = [MigrateCall(0, 32 * 16, ctx, dec)]
    return w


def config2(seed: int = 2, num_requests: int = 16, pool_blocks: int = 4096, fresh_pools: bool = False) -> MigrateWorkload:
    """LLaMA-2-7B KV shape, 16 requests of 64..2048 prompt tokens, TP1 -> TP1."""
    g = torch.Generator().manual_seed(seed)
    shape = KvShape(32, 32, 128)
    w = MigrateWorkload("cfg2-llama2-7b", shape, 1, 1, 1, 1, 0, 0, pool_blocks, pool_blocks, seed)
    w.calls = _disjoint_calls(g, _lengths(g, num_requests, 64, 2048), 16, pool_blocks, pool_blocks, fresh_pools)
    if fresh_pools:
        w.name += "-fresh-pools"
    return w


def fixed_size_requests(blocks_per_request: int, num_requests: int = 48, seed: int = 6,
                        pool_blocks: int = 4096) -> MigrateWorkload:
    """LLaMA-2-7B KV shape, TP1 -> TP1, every request the same number of blocks (scattered,
    disjoint): what the hand-off costs per request as a function of the prompt's length."""
    g = torch.Generator().manual_seed(seed)
    shape = KvShape(32, 32, 128)
    w = MigrateWorkload(f"llama2-7b-{blocks_per_request}-block-requests", shape, 1, 1, 1, 1, 0, 0, pool_blocks,
                        pool_blocks, seed)
    w.calls = _disjoint_calls(g, [blocks_per_request * shape.block_size] * num_requests, shape.block_size,
                              pool_blocks, pool_blocks)
    return w


def config3(seed: int = 3, num_requests: int = 32, fresh_pools: bool = False) -> MigrateWorkload:
    """OPT-13B KV shape, context TP2 -> decoding TP1: two 20-head pools merge into one."""
    g = torch.Generator().manual_seed(seed)
    shape = KvShape(40, 40, 128)
    w = MigrateWorkload("cfg3-opt-13b-tp2to1", shape, 1, 2, 1, 1, 0, 0, 2048, 4096, seed)
    w.calls = _disjoint_calls(g, _lengths(g, num_requests, 128, 1024), 16, 2048, 4096, fresh_pools)
    if fresh_pools:
        w.name += "-fresh-pools"
    return w


def config4(seed: int = 4, num_requests: int = 24, ctx_tp: int = 2, fresh_pools: bool = False) -> MigrateWorkload:
    """LLaMA-2-70B GQA KV shape, context TP2/PP2 -> decoding TP4 rank 1 (2 of 8 KV heads,
    all 80 layers).  The batch needs more blocks than either pool holds, so the calls
    recycle block ids.  ``ctx_tp=4`` is a comparison layout, not the configuration: the same
    block tables and the same bytes, from context pools that hold exactly the two heads
    the decoding rank wants, so the sources are read densely.  ``fresh_pools`` is another
    comparison: the same requests through block managers that have just started, whose free
    lists are still ``0 .. n-1``, so that a request's blocks are neighbours in both pools
    (the configuration itself starts from shuffled lists, the state of a pool in service)."""
    g = torch.Generator().manual_seed(seed)
    shape = KvShape(80, 8, 128)
    name = "cfg4-llama2-70b-tp2pp2to-tp4r1" if ctx_tp == 2 else f"cfg4-variant-tp{ctx_tp}pp2to-tp4r1"
    if fresh_pools:
        name += "-fresh-pools"
    w = MigrateWorkload(name, shape, 2, ctx_tp, 1, 4, 0, 1, 1024, 2048, seed,
                        recycles_blocks=True)
    w.calls = _recycled_calls(g, _lengths(g, num_requests, 256, 4096), 16, 1024, 2048, fresh_pools)
    return w


@dataclass
class SwapWorkload:
    """Configuration 5: swap 2048 blocks out and back into other slots while 8 requests migrate."""

    name: str
    shape: KvShape
    gpu_blocks: int
    host_blocks: int
    seed: int
    out_gpu_ids: List[int]        # swap-out sources
    out_host_ids: List[int]       # swap-out targets = swap-in sources
    in_gpu_ids: List[int]         # swap-in targets, disjoint from out_gpu_ids
    migrate: MigrateWorkload      # concurrent migration into blocks disjoint from every swap slot

    @property
    def slab_bytes(self) -> int:
        return self.shape.block_bytes()

    @property
    def bytes_per_direction(self) -> int:
        return 2 * self.slab_bytes * len(self.out_gpu_ids)


def config5(seed: int = 5, gpu_blocks: int = 4096, host_blocks: int = 4096, swap_blocks: int = 2048,
            migrate_requests: int = 8, migrate_src_blocks: int = 1024,
            shape: Optional[KvShape] = None, min_len: int = 64, max_len: int = 2048) -> SwapWorkload:
    """Swap at the LLaMA-2-7B KV shape.  ``out_gpu_ids[i]`` goes to host block
    ``out_host_ids[i]`` and comes back into ``in_gpu_ids[i] != out_gpu_ids[i]``.  The
    concurrent migration writes GPU blocks that no swap touches.  Swap-in targets may be
    slots an *earlier* swap-out freed, so the swap-in is ordered after the whole swap-out
    (what the block manager's quarantine flush enforces)."""
    g = torch.Generator().manual_seed(seed)
    shape = shape or KvShape(32, 32, 128)
    gpu_perm = torch.randperm(gpu_blocks, generator=g).tolist()
    out_gpu, others = gpu_perm[:swap_blocks], gpu_perm[swap_blocks:]
    host_ids = torch.randperm(host_blocks, generator=g)[:swap_blocks].tolist()
    lengths = _lengths(g, migrate_requests, min_len, max_len)
    need = sum(blocks_for(n, shape.block_size) for n in lengths)
    assert need <= len(others), "migration does not fit beside the swap"
    mig_targets, spare = others[:need], others[need:]
    candidates = spare + out_gpu[:max(0, swap_blocks - len(spare))]
    assert len(candidates) >= swap_blocks
    order = torch.randperm(len(candidates), generator=g).tolist()
    in_gpu = [candidates[i] for i in order][:swap_blocks]
    for i in range(swap_blocks):            # "different slots": never back where it came from
        if in_gpu[i] == out_gpu[i]:
            j = (i + 1) % swap_blocks
            in_gpu[i], in_gpu[j] = in_gpu[j], in_gpu[i]
    assert all(a != b for a, b in zip(in_gpu, out_gpu)) or swap_blocks < 3
    assert not set(in_gpu) & set(mig_targets) and not set(out_gpu) & set(mig_targets)
    mig = MigrateWorkload("cfg5-concurrent-migration", shape, 1, 1, 1, 1, 0, 0, migrate_src_blocks,
                          gpu_blocks, seed)
    src_perm = torch.randperm(migrate_src_blocks, generator=g).tolist()
    at = 0
    for rid, length in enumerate(lengths):
        n = blocks_for(length, shape.block_size)
        assert at + n <= migrate_src_blocks, "migration source pool too small"
        mig.calls.append(MigrateCall(rid, length, src_perm[at:at + n], mig_targets[at:at + n]))
        at += n
    name = "cfg5-swap-llama2-7b" if shape == KvShape(32, 32, 128) else (
        f"cfg5-swap-{shape.num_layers}x{shape.num_kv_heads}x{shape.head_dim}")
    return SwapWorkload(name, shape, gpu_blocks, host_blocks, seed, out_gpu, host_ids,
                        in_gpu, mig)


def scaled(w: MigrateWorkload, num_layers: Optional[int] = None, head_dim: Optional[int] = None) -> MigrateWorkload:
    """Same block tables and rank layout on a thinner model, for checks a CPU finishes in seconds."""
    shape = KvShape(num_layers or w.shape.num_layers, w.shape.num_kv_heads, head_dim or w.shape.head_dim,
                    w.shape.block_size, w.shape.dtype)
    return MigrateWorkload(w.name + "-scaled", shape, w.ctx_pp, w.ctx_tp, w.dec_pp, w.dec_tp, w.dec_pp_rank,
                           w.dec_tp_rank, w.src_blocks, w.dst_blocks, w.seed, w.calls, w.recycles_blocks)


# ---- pool contents


def fill_uniform(shape, seed: int, device="cpu", dtype=torch.float16) -> torch.Tensor:
    """fp16 values uniform in [-1, 1) from a seed; generated on ``device``."""
    g = torch.Generator(device=device).manual_seed(seed)
    out = torch.empty(shape, dtype=dtype, device=device)
    # chunked over blocks so that the fp32 intermediate stays small next to a multi-GiB pool
    step = max(1, (256 << 20) // max(1, out[0].numel() * 4)) if out.shape[0] else 1
    for b0 in range(0, out.shape[0], step):
        part = out[b0:b0 + step]
        part.copy_(torch.rand(part.shape, generator=g, device=device, dtype=torch.float32) * 2 - 1)
    return out


def fill_canary(shape, device="cpu", dtype=torch.float16) -> torch.Tensor:
    out = torch.empty(shape, dtype=dtype, device=device)
    assert out.element_size() == 2
    out.view(torch.int16).fill_(CANARY_BITS)
    return out
