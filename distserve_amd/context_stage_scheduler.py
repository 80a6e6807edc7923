"""The context (prefill) side's view of the hand-off: which prefilled requests still hold
source blocks because the decoding instance has not pulled them yet.

Host-side mirror of reference ``distserve/context_stage_scheduler.py``
(``ContextStageFCFSScheduler``).  Its tie to the KV movement path is block accounting: a
request that finished prefill keeps its blocks until it has been migrated
(``on_request_migrated``, called from ``clear_migrated_blocks_callback``), and those
blocks count against the next prefill batch (reference :127-172).
"""
from __future__ import annotations

import copy
from typing import List, Optional

from distserve_amd.block_manager import BlockManager
from distserve_amd.config import ParallelConfig
from distserve_amd.request import BatchedRequests, MigratingRequest, Request


class ContextStageSchedConfig:
    """Reference config.py:90-109."""

    def __init__(self, policy: str, max_batch_size: int, max_tokens_per_batch: int,
                 parallel_config: Optional[ParallelConfig] = None):
        assert policy in ["fcfs"], f"policy {policy} not supported"
        self.policy = policy
        self.max_batch_size = max_batch_size
        self.max_tokens_per_batch = max_tokens_per_batch
        self.parallel_config = parallel_config


class ContextStageFCFSScheduler:
    def __init__(self, sched_config: ContextStageSchedConfig, parallel_config: ParallelConfig,
                 block_manager: BlockManager):
        assert sched_config.policy == "fcfs", \
            f"can not initialize a FCFS scheduler with policy {sched_config.policy}"
        self.sched_config = sched_config
        self.parallel_config = copy.deepcopy(parallel_config)
        self.block_manager = block_manager
        self.waiting_queue: List[Request] = []
        self.unaccepted_queue: List[Request] = []    # prefilled, blocks still here, not yet migrated
        self.num_on_fly_request_block = 0            # blocks of the batches being prefilled

    def _get_block_needed(self, length: int) -> int:
        block_size = self.block_manager.cache_config.block_size
        return (length + block_size - 1) // block_size

    def _prompt_blocks(self, requests: List[Request]) -> int:
        return sum(self._get_block_needed(len(r.prompt_token_ids)) for r in requests)

    def add_request(self, request: Request) -> None:
        self.waiting_queue.append(request)

    def abort_request(self, request_id: int) -> None:
        for i, request in enumerate(self.waiting_queue):
            if request.request_id == request_id:
                del self.waiting_queue[i]
                return

    def get_next_batch_and_pop(self) -> BatchedRequests:
        """Head-of-line requests while batch size, token budget and block budget allow; the
        block budget counts this batch, the prefilled requests that are not migrated yet and
        the batches in flight (reference :127-172)."""
        batch = BatchedRequests()
        while self.waiting_queue:
            request = self.waiting_queue[0]
            fits = (len(batch) < self.sched_config.max_batch_size
                    and batch.get_num_input_tokens() + request.get_num_input_tokens()
                    <= self.sched_config.max_tokens_per_batch
                    and self._prompt_blocks(batch.requests + [request]) + self._prompt_blocks(self.unaccepted_queue)
                    + self.num_on_fly_request_block <= self.block_manager.max_num_gpu_blocks)
            if not fits:
                break
            batch.add_request(request)
            self.waiting_queue.pop(0)
        self.num_on_fly_request_block += sum(self._get_block_needed(r.get_input_len()) for r in batch.requests)
        return batch

    def on_finish_requests(self, batch: BatchedRequests) -> None:
        for request in batch.requests:
            if not request.is_finished:
                self.unaccepted_queue.append(request)
        self.num_on_fly_request_block -= sum(self._get_block_needed(r.get_input_len()) for r in batch.requests)

    def on_request_migrated(self, migrated_request: MigratingRequest) -> None:
        for i, request in enumerate(self.unaccepted_queue):
            if request.request_id == migrated_request.req.request_id:
                del self.unaccepted_queue[i]
                return

    def get_num_waiting_requests(self) -> int:
        return len(self.waiting_queue)

    def __repr__(self) -> str:
        return (f"FCFS(max_batch_size={self.sched_config.max_batch_size}, "
                f"max_tokens_per_batch={self.sched_config.max_tokens_per_batch})")


def get_context_stage_scheduler(sched_config: ContextStageSchedConfig, parallel_config: ParallelConfig,
                                block_manager: BlockManager) -> ContextStageFCFSScheduler:
    if sched_config.policy == "fcfs":
        return ContextStageFCFSScheduler(sched_config, parallel_config, block_manager)
    raise NotImplementedError(f"Unknown context scheduler policy {sched_config.policy}")
