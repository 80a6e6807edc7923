"""TEST INFRASTRUCTURE ONLY -- CPU oracle for KV-block migration and swap.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may
import this package, and only as the checker.  The product (``distserve_amd``) never
imports it and has no CPU fallback.

The native op these functions restate (SwiftTransformer ``block_migration_ops`` /
``swapping_ops``, un-vendored and un-pinned, see reference ``distserve/__init__.py:4-16``
and ``README.md:26-28``) is absent from the reference tree and the reference holds no
golden vector for it: with respect to that op itself, PARITY UNPINNED.  What is pinned:
the semantics fixed by the reference's call sites (``distserve/worker.py:250-267,
269-311``), its pool layout (``distserve/worker.py:107-121``) and its rank->slice rule
(``distserve/config.py:225-257, 279-286``).  Three independently written formulations
live here and the tests check them against each other and against library routines:

* ``migrate_c`` / ``swap_c``   -- the C restatement in ``kvmove_oracle.c`` (pull form:
  decoding rank's rectangle, per head slab ``memcpy``).
* ``migrate_cat``              -- torch library routines only: ``index_select`` of the
  context blocks, ``cat`` of context ranks along layers (PP) and heads (TP), ``narrow``
  to the decoding rectangle, ``index_copy_`` into the destination.  This is also the
  CPU baseline that ``bench.py`` times ("torch index_select/copy over the block tables").
* ``migrate_push_loops``       -- pure-Python element loops in *push* form (iterate over
  every element of every context pool, ask which decoding rank owns it); tiny shapes only.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkvmove_oracle.so")
_lib = None


@dataclass(frozen=True)
class Geom:
    """Whole-model KV geometry plus the two instances' parallel layouts."""

    num_layers: int
    num_kv_heads: int
    block_size: int
    head_dim: int
    dtype_bytes: int
    ctx_pp: int = 1
    ctx_tp: int = 1
    dec_pp: int = 1
    dec_tp: int = 1
    dec_pp_rank: int = 0
    dec_tp_rank: int = 0

    # slice rule: distserve/config.py:279-286 (layers / pp), :225-257 (kv heads / tp)
    @property
    def ctx_layers(self) -> int:
        return self.num_layers // self.ctx_pp

    @property
    def ctx_heads(self) -> int:
        return self.num_kv_heads // self.ctx_tp

    @property
    def dec_layers(self) -> int:
        return self.num_layers // self.dec_pp

    @property
    def dec_heads(self) -> int:
        return self.num_kv_heads // self.dec_tp

    def ctx_pool_shape(self, num_blocks: int):
        return (num_blocks, self.ctx_layers, self.ctx_heads, self.block_size, self.head_dim)

    def dec_pool_shape(self, num_blocks: int):
        return (num_blocks, self.dec_layers, self.dec_heads, self.block_size, self.head_dim)


class _CGeom(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in (
        "num_layers", "num_kv_heads", "block_size", "head_dim", "dtype_bytes",
        "ctx_pp", "ctx_tp", "dec_pp", "dec_tp", "dec_pp_rank", "dec_tp_rank")]


def build(force: bool = False) -> str:
    """Compile kvmove_oracle.c with gcc (``make -C oracle``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


def load_c():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        lib = ctypes.CDLL(_LIB_PATH)
        lib.kvo_migrate.restype = ctypes.c_int
        lib.kvo_migrate.argtypes = [
            ctypes.POINTER(_CGeom), ctypes.POINTER(ctypes.c_void_p), ctypes.c_int64,
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64]
        lib.kvo_swap.restype = ctypes.c_int
        lib.kvo_swap.argtypes = [
            ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64,
            ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64]
        _lib = lib
    return _lib


def _i64(a: Sequence[int]) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(list(a), dtype=np.int64))


def _check_pool(t: torch.Tensor, shape) -> None:
    assert t.device.type == "cpu" and t.is_contiguous(), "oracle works on contiguous CPU tensors"
    assert tuple(t.shape) == tuple(shape), f"pool shape {tuple(t.shape)} != {tuple(shape)}"


# --------------------------------------------------------------------------- migrate


def migrate_c(g: Geom, src_pools: List[List[torch.Tensor]], ctx_idx, dec_idx, dst: torch.Tensor) -> None:
    """C restatement (one pool kind).  ``src_pools[p][t]`` is context rank (pp p, tp t)."""
    lib = load_c()
    nb_src = src_pools[0][0].shape[0]
    flat = []
    for p in range(g.ctx_pp):
        for t in range(g.ctx_tp):
            _check_pool(src_pools[p][t], g.ctx_pool_shape(nb_src))
            assert src_pools[p][t].element_size() == g.dtype_bytes
            flat.append(src_pools[p][t].data_ptr())
    _check_pool(dst, g.dec_pool_shape(dst.shape[0]))
    ptrs = (ctypes.c_void_p * len(flat))(*flat)
    ci, di = _i64(ctx_idx), _i64(dec_idx)
    assert len(ci) == len(di)
    cg = _CGeom(g.num_layers, g.num_kv_heads, g.block_size, g.head_dim, g.dtype_bytes,
                g.ctx_pp, g.ctx_tp, g.dec_pp, g.dec_tp, g.dec_pp_rank, g.dec_tp_rank)
    rc = lib.kvo_migrate(ctypes.byref(cg), ptrs, nb_src, ci.ctypes.data, di.ctypes.data, len(ci),
                         dst.data_ptr(), dst.shape[0])
    if rc != 0:
        raise ValueError(f"kvo_migrate rejected its arguments (rc={rc})")


def migrate_cat(g: Geom, src_pools: List[List[torch.Tensor]], ctx_idx, dec_idx, dst: torch.Tensor) -> None:
    """Library-routine formulation: index_select -> cat(PP: layers, TP: heads) -> narrow -> index_copy_."""
    ci = torch.as_tensor(list(ctx_idx), dtype=torch.long)
    di = torch.as_tensor(list(dec_idx), dtype=torch.long)
    assert ci.numel() == di.numel()
    if ci.numel() == 0:
        return
    per_stage = []
    for p in range(g.ctx_pp):
        per_stage.append(torch.cat([src_pools[p][t].index_select(0, ci) for t in range(g.ctx_tp)], dim=2))
    whole = torch.cat(per_stage, dim=1)  # [n, L, H, B, D] of the whole model
    rect = whole.narrow(1, g.dec_pp_rank * g.dec_layers, g.dec_layers) \
                .narrow(2, g.dec_tp_rank * g.dec_heads, g.dec_heads)
    dst.index_copy_(0, di, rect.contiguous())


def migrate_push_loops(g: Geom, src_pools, ctx_idx, dec_idx, dst: torch.Tensor) -> None:
    """Brute force, push form, element by element.  Tiny shapes only."""
    ci, di = list(ctx_idx), list(dec_idx)
    assert len(ci) == len(di)
    for p in range(g.ctx_pp):
        for t in range(g.ctx_tp):
            pool = src_pools[p][t]
            for i in range(len(ci)):
                for ll in range(g.ctx_layers):
                    gl = p * g.ctx_layers + ll          # global layer
                    if gl // g.dec_layers != g.dec_pp_rank:
                        continue
                    for hh in range(g.ctx_heads):
                        gh = t * g.ctx_heads + hh      # global kv head
                        if gh // g.dec_heads != g.dec_tp_rank:
                            continue
                        for b in range(g.block_size):
                            for d in range(g.head_dim):
                                dst[di[i], gl % g.dec_layers, gh % g.dec_heads, b, d] = \
                                    pool[ci[i], ll, hh, b, d]


# ------------------------------------------------------------------------------ swap


def swap_c(src_ids, dst_ids, src_pool: torch.Tensor, dst_pool: torch.Tensor) -> None:
    """C restatement of ``dst_pool[dst_ids[i]] = src_pool[src_ids[i]]`` (worker.py:269-311)."""
    lib = load_c()
    assert src_pool.is_contiguous() and dst_pool.is_contiguous()
    assert src_pool.shape[1:] == dst_pool.shape[1:] and src_pool.dtype == dst_pool.dtype
    slab = src_pool[0].numel() * src_pool.element_size() if src_pool.shape[0] else 0
    si, di = _i64(src_ids), _i64(dst_ids)
    assert len(si) == len(di)
    rc = lib.kvo_swap(si.ctypes.data, di.ctypes.data, len(si), src_pool.data_ptr(), src_pool.shape[0],
                      dst_pool.data_ptr(), dst_pool.shape[0], slab)
    if rc != 0:
        raise ValueError(f"kvo_swap rejected its arguments (rc={rc})")


def swap_lib(src_ids, dst_ids, src_pool: torch.Tensor, dst_pool: torch.Tensor) -> None:
    """Library-routine formulation of swap: index_copy_(index_select)."""
    si = torch.as_tensor(list(src_ids), dtype=torch.long)
    di = torch.as_tensor(list(dst_ids), dtype=torch.long)
    if si.numel():
        dst_pool.index_copy_(0, di, src_pool.index_select(0, si))


# --------------------------------------------------------------------------- helpers


def bits(t: torch.Tensor) -> torch.Tensor:
    """Raw bit pattern view for exact comparison (NaN payloads and -0 are data here)."""
    view = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()]
    return t.view(view)
