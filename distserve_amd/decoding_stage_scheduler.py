"""What triggers the KV movement on the decoding side: the FCFS decoding scheduler's
swap-out / swap-in decisions and its acceptance of migrating requests.

Host-side mirror of reference ``distserve/decoding_stage_scheduler.py``
(``DecodingStageFCFSScheduler``), kept to the parts that *call* the path: ``get_next_batch``
(swap triggers, :183-223), ``post_process`` (migration trigger, :247-260), the admission
test (:131-150) and the queues they move requests between.  Decisions are the
reference's, evaluated in the same order with the same arithmetic, so the block tables
handed to ``swap_blocks`` / ``migrate_blocks`` are the same.

One addition: with ``batch_migrations=True`` the requests that ``post_process`` accepts in
one pass are migrated by a single call (one kernel launch per decoding worker for the
whole group) instead of one call each.  Acceptance is still decided request by request,
each after the previous one's blocks have been allocated, exactly as in the reference.
"""
from __future__ import annotations

import copy
from typing import Callable, List, Optional

from distserve_amd.block_manager import BlockManager
from distserve_amd.config import ParallelConfig
from distserve_amd.request import BatchedRequests, MigratingRequest, Request


class DecodingStageSchedConfig:
    """Reference config.py:111-139."""

    def __init__(self, policy: str, max_batch_size: int, max_tokens_per_batch: int,
                 model_name: Optional[str] = None, waiting_block_prop_threshold: float = 0.05):
        assert policy in ["fcfs", "srpt", "mlfq", "sj-mlfq"], f"policy {policy} not supported"
        self.policy = policy
        self.max_batch_size = max_batch_size
        self.max_tokens_per_batch = max_tokens_per_batch
        self.model_name = model_name
        self.waiting_block_prop_threshold = waiting_block_prop_threshold


class DecodingStageFCFSScheduler:
    """First come, first served; one batch per pipeline stage in flight."""

    def __init__(self, sched_config: DecodingStageSchedConfig, parallel_config: ParallelConfig,
                 block_manager: BlockManager, engine_migrate_block_callback: Callable,
                 engine_migrate_blocks_batched_callback: Optional[Callable] = None,
                 batch_migrations: bool = False):
        assert sched_config.policy == "fcfs", \
            f"can not initialize a FCFS scheduler with policy {sched_config.policy}"
        self.sched_config = sched_config
        self.parallel_config = copy.deepcopy(parallel_config)
        self.block_manager = block_manager
        self.engine_migrate_block_callback = engine_migrate_block_callback
        self.engine_migrate_blocks_batched_callback = engine_migrate_blocks_batched_callback
        self.batch_migrations = batch_migrations and engine_migrate_blocks_batched_callback is not None
        self.unaccepted_queue: List[MigratingRequest] = []   # blocks still on the context instance
        self.waiting_queue: List[Request] = []               # migrated, not yet in a batch
        self.swapped_queue: List[Request] = []               # was in a batch, now on the host
        self.cur_index = -1
        self.batch_queues = [BatchedRequests() for _ in range(parallel_config.pipeline_parallel_size)]

    # ---- block arithmetic

    def _get_block_needed(self, length: int) -> int:
        block_size = self.block_manager.cache_config.block_size
        return (length + block_size - 1) // block_size

    def _blocks_of_batches(self) -> int:
        """Blocks of every request in every in-flight batch, generated tokens included."""
        return sum(self._get_block_needed(r.get_input_len() + r.get_output_len())
                   for batch in self.batch_queues for r in batch.requests)

    def _blocks_of_waiting(self) -> int:
        """Blocks of the waiting requests' prompts."""
        return sum(self._get_block_needed(r.get_input_len()) for r in self.waiting_queue)

    def _check_add_to_cur_batch(self, request: Request) -> bool:
        """Admission test of reference :131-150: batch size, token budget, block budget."""
        batch = self.batch_queues[self.cur_index]
        if len(batch) >= self.sched_config.max_batch_size:
            return False
        if batch.get_num_input_tokens() + request.get_num_input_tokens() > self.sched_config.max_tokens_per_batch:
            return False
        demand = (self._blocks_of_batches() + self._blocks_of_waiting()
                  + self._get_block_needed(request.get_input_len() + request.get_output_len()))
        return demand <= self.block_manager.max_num_gpu_blocks

    # ---- requests

    def add_request(self, migrating_req: MigratingRequest) -> None:
        self.unaccepted_queue.append(migrating_req)

    def abort_request(self, request_id: int) -> None:
        for batch in self.batch_queues:
            for request in batch.requests:
                if request.request_id == request_id:
                    request.is_finished = True      # released when its batch pops finished requests
                    return
        for i, request in enumerate(self.waiting_queue):
            if request.request_id == request_id:
                del self.waiting_queue[i]
                return

    def pop_finished_requests(self) -> List[Request]:
        last_stage = (self.cur_index + 1) % self.parallel_config.pipeline_parallel_size
        return self.batch_queues[last_stage].pop_finished_requests()

    def get_next_batch(self) -> BatchedRequests:
        """Pick the next batch.  Swap-out while the resident and waiting requests need more
        blocks than the GPU has (victim: the last request of the current batch); then admit
        swapped requests first (swap-in), then waiting ones (reference :183-223)."""
        self.cur_index = (self.cur_index + 1) % self.parallel_config.pipeline_parallel_size
        batch = self.batch_queues[self.cur_index]
        while self._blocks_of_batches() + self._blocks_of_waiting() > self.block_manager.max_num_gpu_blocks:
            victim = batch.requests.pop(-1)
            self.swapped_queue.append(victim)
            self.block_manager.swap_out_requests([victim])
        while self.swapped_queue or self.waiting_queue:
            from_swap = bool(self.swapped_queue)
            request = self.swapped_queue[0] if from_swap else self.waiting_queue[0]
            if not self._check_add_to_cur_batch(request):
                break
            if from_swap:
                self.block_manager.swap_in_requests([request])
                self.swapped_queue.pop(0)
            else:
                self.waiting_queue.pop(0)
            batch.add_request(request)
        return batch

    def post_process(self) -> None:
        """Accept head-of-line migrating requests while the waiting prompts hold less than
        ``waiting_block_prop_threshold`` of the pool and the next prompt fits the available
        GPU blocks; each accepted request is migrated and joins the waiting queue
        (reference :247-260)."""
        accepted: List[MigratingRequest] = []
        while self.unaccepted_queue:
            migrating_req = self.unaccepted_queue[0]
            limit = self.block_manager.max_num_gpu_blocks * self.sched_config.waiting_block_prop_threshold
            prompt_blocks = self._get_block_needed(len(migrating_req.req.prompt_token_ids))
            if not (self._blocks_of_waiting() < limit
                    and prompt_blocks <= self.block_manager.get_num_avail_gpu_blocks()):
                break
            self.unaccepted_queue.pop(0)
            if self.batch_migrations:
                # allocate now so that the next decision sees the pool as the reference would
                self.engine_migrate_blocks_batched_callback([migrating_req], allocate_only=True)
                accepted.append(migrating_req)
            else:
                self.engine_migrate_block_callback(migrating_req)
            self.waiting_queue.append(migrating_req.req)
        if accepted:
            self.engine_migrate_blocks_batched_callback(accepted, allocate_only=False)

    # ---- getters

    def get_total_num_requests(self) -> int:
        return self.get_processing_num_requests() + self.get_waiting_num_requests()

    def get_processing_num_requests(self) -> int:
        return sum(len(batch.requests) for batch in self.batch_queues)

    def get_waiting_num_requests(self) -> int:
        return len(self.waiting_queue)

    def __repr__(self) -> str:
        return (f"FCFS(max_batch_size={self.sched_config.max_batch_size}, "
                f"max_tokens_per_batch={self.sched_config.max_tokens_per_batch})")


def get_decoding_stage_scheduler(sched_config, parallel_config, block_manager, engine_migrate_block_callback,
                                 **kwargs) -> DecodingStageFCFSScheduler:
    if sched_config.policy == "fcfs":
        return DecodingStageFCFSScheduler(sched_config, parallel_config, block_manager,
                                          engine_migrate_block_callback, **kwargs)
    raise NotImplementedError(f"scheduler policy {sched_config.policy} is not supported")
