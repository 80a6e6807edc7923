"""Block tables of one instance: which pool blocks each request owns, on HBM or on the host.

Host-side mirror of reference ``distserve/block_manager.py``; method names, arguments and
the order in which block ids are handed out are the reference's, because the block-index
lists built here are exactly what ``migrate_blocks`` and ``swap_blocks`` receive.

Hand-out order (reference block_manager.py:44-45, 82-83, 96-97, 157-160): each location
starts with ids ``0..N-1`` in a FIFO list; an allocation takes the head of the list;
freed ids go to the tail.  Blocks that are the *source* of a swap are not free at once:
they wait in a per-location quarantine list until the copy that reads them is known to
have finished, which is forced ("flushed") only when the free list alone cannot serve a
request (reference block_manager.py:66-98, design notes :211-286).

Two departures from the reference, neither changes a block id:
* ``swap_blocks`` is sent the request *ids* (the reference passes ``Request`` objects,
  block_manager.py:313-315, which the worker's id-keyed event table never matches,
  worker.py:204-212, 290-295);
* the workers are reached through a plain callable, there is no Ray hop.
"""
from __future__ import annotations

from enum import Enum
from typing import Callable, Dict, List

from distserve_amd.config import CacheConfig, ModelConfig, ParallelConfig
from distserve_amd.request import BatchedRequests, Request
from distserve_amd.utils import Stage


class BlockLocation(Enum):
    """Where a request's blocks live."""

    GPU = "gpu"
    CPU = "cpu"


class _Shelf:
    """The blocks of one location: a FIFO free list plus the quarantine of swap sources."""

    def __init__(self, capacity: int, name: str, flush_call: str):
        self.capacity = capacity
        self.name = name
        self.flush_call = flush_call   # worker method that waits for the copies reading the quarantine
        self.free: List[int] = list(range(capacity))
        self.quarantine: List[int] = []

    def available(self) -> int:
        return len(self.free) + len(self.quarantine)

    def take(self, count: int, call_workers: Callable) -> List[int]:
        have = self.available()
        assert have >= count, f"not enough free blocks on {self.name}, requested {count}, available {have}"
        if len(self.free) < count:
            # the copies that read the quarantined blocks must be over before they are reused
            call_workers(self.flush_call)
            self.free += self.quarantine
            self.quarantine = []
        # the head of the list, cut off in place: slicing the rest into a new list would copy (and
        # re-count) every free block of the pool on every allocation, microseconds per call
        taken = self.free[:count]
        del self.free[:count]
        return taken

    def used(self) -> int:
        return self.capacity - self.available()


class BlockManager:
    """Maintains the key-value cache at block level (reference block_manager.py:20-330)."""

    def __init__(self, stage: Stage, max_num_gpu_blocks: int, max_num_cpu_blocks: int,
                 model_config: ModelConfig, parallel_config: ParallelConfig, cache_config: CacheConfig,
                 engine_remote_call_all_workers_async: Callable):
        self.stage = stage
        self.max_num_gpu_blocks = max_num_gpu_blocks
        self.max_num_cpu_blocks = max_num_cpu_blocks
        self.model_config = model_config
        self.parallel_config = parallel_config
        self.cache_config = cache_config
        self.engine_remote_call_all_workers_async = engine_remote_call_all_workers_async

        # swap-out reads GPU blocks, so the GPU quarantine is flushed by waiting for swap-outs
        self._shelves: Dict[BlockLocation, _Shelf] = {
            BlockLocation.GPU: _Shelf(max_num_gpu_blocks, "GPU", "wait_for_all_swap_out"),
            BlockLocation.CPU: _Shelf(max_num_cpu_blocks, "CPU", "wait_for_all_swap_in"),
        }
        self.block_table: Dict[int, List[int]] = {}               # request_id -> block ids
        self.request_location: Dict[int, BlockLocation] = {}      # request_id -> where they are

    # ---- views under the reference's attribute names

    @property
    def free_gpu_blocks_list(self) -> List[int]:
        return self._shelves[BlockLocation.GPU].free

    @property
    def free_cpu_blocks_list(self) -> List[int]:
        return self._shelves[BlockLocation.CPU].free

    @property
    def swapping_gpu_blocks_list(self) -> List[int]:
        return self._shelves[BlockLocation.GPU].quarantine

    @property
    def swapping_cpu_blocks_list(self) -> List[int]:
        return self._shelves[BlockLocation.CPU].quarantine

    # ---- counting

    def get_num_avail_gpu_blocks(self) -> int:
        return self._shelves[BlockLocation.GPU].available()

    def get_num_avail_cpu_blocks(self) -> int:
        return self._shelves[BlockLocation.CPU].available()

    def get_allocated_num_blocks(self, request_id: int) -> int:
        return len(self.block_table.get(request_id, []))

    def get_location(self, request_id: int) -> BlockLocation:
        return self.request_location.get(request_id, None)

    def get_num_blocks_needed(self, request: Request) -> int:
        """ceil((prompt + generated) / block_size) (reference block_manager.py:108-115)."""
        tokens = request.get_input_len() + request.get_output_len()
        return -(-tokens // self.cache_config.block_size)

    def get_num_append_blocks_needed(self, request: Request) -> int:
        rid = request.request_id
        assert self.request_location[rid] == BlockLocation.GPU, \
            f"request {rid} is not on GPU when calling get_num_append_blocks_needed"
        return self.get_num_blocks_needed(request) - len(self.block_table[rid])

    # ---- allocation

    def _get_free_blocks(self, num_blocks: int, location: BlockLocation) -> List[int]:
        assert location in (BlockLocation.GPU, BlockLocation.CPU)
        return self._shelves[location].take(num_blocks, self.engine_remote_call_all_workers_async)

    def allocate_blocks(self, request: Request) -> None:
        """Grow the request's table to cover all its tokens (reference block_manager.py:126-147)."""
        rid = request.request_id
        assert rid not in self.block_table or self.request_location.get(rid) == BlockLocation.GPU, \
            f"request {rid} is currently on CPU. Please migrate it to GPU before allocating more blocks"
        needed = self.get_num_blocks_needed(request)
        if rid not in self.block_table:
            self.block_table[rid] = self._get_free_blocks(needed, BlockLocation.GPU)
            self.request_location[rid] = BlockLocation.GPU
            return
        missing = needed - len(self.block_table[rid])
        if missing > 0:
            self.block_table[rid] += self._get_free_blocks(missing, BlockLocation.GPU)

    def allocate_blocks_batched(self, batch_requests: BatchedRequests) -> None:
        for request in batch_requests.requests:
            self.allocate_blocks(request)

    def free_blocks(self, request_id: int) -> None:
        """Give the request's blocks back, at the tail of their location's free list."""
        assert request_id in self.block_table, f"request {request_id} not allocated"
        location = self.request_location.pop(request_id)
        self._shelves[location].free += self.block_table.pop(request_id)

    def free_blocks_batched(self, requests: List[Request]) -> None:
        for request in requests:
            self.free_blocks(request.request_id)

    def get_block_table(self, request_id: int) -> List[int]:
        assert request_id in self.block_table, f"request {request_id} not allocated"
        return self.block_table[request_id]

    def get_partial_block_table(self, request_ids: List[int]) -> List[List[int]]:
        tables = []
        for request_id in request_ids:
            assert request_id in self.block_table, f"request {request_id} not allocated"
            tables.append(self.block_table[request_id])
        return tables

    # ---- swapping ("swap in" = host -> HBM, "swap out" = HBM -> host)

    def swap_requests(self, requests: List[Request], is_swap_in: bool) -> None:
        """Retarget each request's table to fresh blocks on the other side and tell every
        worker to copy (reference block_manager.py:288-315).  ``source_block_ids`` and
        ``target_block_ids`` concatenate the requests' old and new tables in order."""
        here = BlockLocation.CPU if is_swap_in else BlockLocation.GPU
        there = BlockLocation.GPU if is_swap_in else BlockLocation.CPU
        source_block_ids: List[int] = []
        target_block_ids: List[int] = []
        for request in requests:
            rid = request.request_id
            assert rid in self.block_table, f"request {rid} not allocated"
            assert self.request_location[rid] == here, f"request {rid} is on {there} now"
            old_ids = self.block_table[rid]
            new_ids = self._get_free_blocks(len(old_ids), there)
            source_block_ids += old_ids
            target_block_ids += new_ids
            self.block_table[rid] = new_ids
            self.request_location[rid] = there
            self._shelves[here].quarantine += old_ids
        self.engine_remote_call_all_workers_async(
            "swap_blocks", [r.request_id for r in requests], source_block_ids, target_block_ids, is_swap_in)

    def swap_in_requests(self, requests: List[Request]) -> None:
        self.swap_requests(requests, is_swap_in=True)

    def swap_out_requests(self, requests: List[Request]) -> None:
        self.swap_requests(requests, is_swap_in=False)

    def is_all_requests_on_gpu(self, requests: BatchedRequests) -> bool:
        return all(self.request_location[r.request_id] != BlockLocation.CPU for r in requests.requests)

    # ---- reporting

    def __repr__(self) -> str:
        return (f"BlockManager(max_num_gpu_blocks={self.max_num_gpu_blocks}, "
                f"max_num_cpu_blocks={self.max_num_cpu_blocks}, blocksize={self.cache_config.block_size})")

    def block_usage(self) -> Dict[str, int]:
        gpu, cpu = self._shelves[BlockLocation.GPU], self._shelves[BlockLocation.CPU]
        return {"gpu_used": gpu.used(), "gpu_total": gpu.capacity, "gpu_swapping_out": len(gpu.quarantine),
                "cpu_used": cpu.used(), "cpu_total": cpu.capacity, "cpu_swapping_in": len(cpu.quarantine)}

    def print_block_usage(self) -> None:
        u = self.block_usage()
        for side, verb in (("cpu", "in"), ("gpu", "out")):
            total = max(u[f"{side}_total"], 1)
            print(f"({self.stage}) {side.upper()} blocks: {u[f'{side}_used']} / {u[f'{side}_total']} "
                  f"({u[f'{side}_used'] / total * 100:.2f}%) used, "
                  f"({u[f'{side}_swapping_' + verb]} swapping {verb})")
