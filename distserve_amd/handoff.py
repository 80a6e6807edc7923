"""Block-table handoff between the context (prefill) instance and the decoding instance.

In-process mirror of the parts of reference ``distserve/single_stage_engine.py`` that sit
on the KV movement path: pool set-up and handle exchange (``_init_kvcache`` :194-223,
``register_kvcache_mem_handles`` :469-483), the tail of the context step that turns a
prefilled request into a ``MigratingRequest`` (:393-401), ``_migrate_blocks`` (:490-536)
and ``clear_migrated_blocks_callback`` (:405-410).  Scheduling, batching, the model
forward and the Ray/asyncio plumbing are not part of this path: workers are plain
objects on one GPU and a "remote call" is a direct method call on every worker.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional, Tuple

from distserve_amd.block_manager import BlockManager
from distserve_amd.config import CacheConfig, ModelConfig, ParallelConfig
from distserve_amd.lifetime import LifetimeEvent, LifetimeEventType
from distserve_amd.request import MigratingRequest, Request
from distserve_amd.utils import MemoryHandle, Stage
from distserve_amd.worker import Worker


class SingleStageLLMEngine:
    """What both instances share: a [pp][tp] grid of workers and one block manager."""

    stage: Stage = None

    def __init__(self, model_config: ModelConfig, parallel_config: ParallelConfig, cache_config: CacheConfig,
                 worker_factory: Callable[..., Worker] = Worker):
        self.model_config = model_config
        self.parallel_config = parallel_config
        self.cache_config = cache_config
        self.workers: List[List[Worker]] = []
        for pp_rank in range(parallel_config.pipeline_parallel_size):
            row = []
            for tp_rank in range(parallel_config.tensor_parallel_size):
                rank_config = ParallelConfig(parallel_config.tensor_parallel_size, tp_rank,
                                             parallel_config.pipeline_parallel_size, pp_rank)
                worker_id = pp_rank * parallel_config.tensor_parallel_size + tp_rank
                row.append(worker_factory(worker_id, self.stage, model_config, cache_config, rank_config))
            self.workers.append(row)
        self.kv_cache_mem_handles: List[List[Tuple[MemoryHandle, MemoryHandle]]] = []
        self.block_manager: Optional[BlockManager] = None

    def _remote_call_all_workers_async(self, func_name: str, *args) -> list:
        """Call ``func_name`` on every worker, pipeline stage by stage (reference :225-233)."""
        return [getattr(worker, func_name)(*args) for row in self.workers for worker in row]

    def _init_kvcache(self, num_gpu_blocks: int, num_cpu_blocks: int) -> Tuple[int, int]:
        """Allocate every worker's pools and collect the handles as ``[pp][tp]``."""
        if self.stage == Stage.CONTEXT:
            num_cpu_blocks = 1   # the context instance never swaps (reference :206-209)
        flat = self._remote_call_all_workers_async("init_kvcache_and_swap", num_gpu_blocks, num_cpu_blocks)
        tp = self.parallel_config.tensor_parallel_size
        self.kv_cache_mem_handles = [flat[i:i + tp] for i in range(0, len(flat), tp)]
        self.block_manager = BlockManager(self.stage, num_gpu_blocks, num_cpu_blocks, self.model_config,
                                          self.parallel_config, self.cache_config,
                                          self._remote_call_all_workers_async)
        return num_gpu_blocks, num_cpu_blocks

    def _free_request_resources(self, request_id: int) -> None:
        self.block_manager.free_blocks(request_id)
        self._remote_call_all_workers_async("clear_request_resource", request_id)


class ContextStageLLMEngine(SingleStageLLMEngine):
    stage = Stage.CONTEXT

    def __init__(self, *args, instance_id: int = 0, **kwargs):
        super().__init__(*args, **kwargs)
        self.instance_id = instance_id   # names this instance's pools on the decoding side
        self.bridge_queue: List[MigratingRequest] = []
        self.scheduler = None     # optional ContextStageFCFSScheduler, told when a request has left

    def on_prefill_finished(self, request: Request) -> MigratingRequest:
        """Tail of the context step: the request's blocks stay where they are and their
        table travels to the decoding instance (reference :393-401)."""
        migrating_req = MigratingRequest(request, self.block_manager.get_block_table(request.request_id),
                                         self.parallel_config, self.instance_id)
        self.bridge_queue.append(migrating_req)
        return migrating_req

    def clear_migrated_blocks_callback(self, migrated_request: MigratingRequest, migrate_events=()) -> None:
        """Release the source blocks (reference :405-410).  Work the context workers enqueue
        afterwards is ordered behind the migrations that read those blocks."""
        for event in migrate_events:
            self._remote_call_all_workers_async("wait_stream_for_migration", event)
        self._free_request_resources(migrated_request.req.request_id)
        if self.scheduler is not None:
            self.scheduler.on_request_migrated(migrated_request)


class DecodingStageLLMEngine(SingleStageLLMEngine):
    stage = Stage.DECODING

    def __init__(self, *args, clear_migrated_blocks_callback: Optional[Callable] = None,
                 engine_on_new_lifetime_event_callback: Optional[Callable] = None,
                 gpu_complete_lifetime_events: bool = False, **kwargs):
        super().__init__(*args, **kwargs)
        self.clear_migrated_blocks_callback = clear_migrated_blocks_callback
        self.engine_on_new_lifetime_event_callback = engine_on_new_lifetime_event_callback
        # True: MigrationEnd is stamped after the copy's event has completed on the GPU
        self.gpu_complete_lifetime_events = gpu_complete_lifetime_events
        self.lifetime_events: Dict[int, List[LifetimeEvent]] = {}
        self._release_takes_events: Optional[bool] = None

    def _lifetime(self, request_id: int, event_type: LifetimeEventType) -> None:
        event = LifetimeEvent(event_type)
        self.lifetime_events.setdefault(request_id, []).append(event)
        if self.engine_on_new_lifetime_event_callback is not None:
            self.engine_on_new_lifetime_event_callback(request_id, event)

    def _wait_for_copies(self) -> None:
        if not self.gpu_complete_lifetime_events:
            return
        for row in self.workers:
            for w in row:
                event = getattr(w, "latest_migrate_event", None)
                if event is not None and hasattr(event, "synchronize"):
                    event.synchronize()

    def get_and_pop_request_lifetime_events(self, request_id: int) -> List[LifetimeEvent]:
        return self.lifetime_events.pop(request_id, [])

    def register_kvcache_mem_handles(self, context_parallel_config: ParallelConfig,
                                     kv_cache_mem_handles: List[List[Tuple[MemoryHandle, MemoryHandle]]],
                                     context_instance: int = 0) -> None:
        """Hand a context instance's handles to every decoding worker (reference :469-483)."""
        self.kv_cache_mem_handles = kv_cache_mem_handles
        if context_instance:
            self._remote_call_all_workers_async("register_kvcache_mem_handles", context_parallel_config,
                                                kv_cache_mem_handles, context_instance)
        else:
            self._remote_call_all_workers_async("register_kvcache_mem_handles", context_parallel_config,
                                                kv_cache_mem_handles)

    def _call_migrate(self, ctx_idx: List[int], config: ParallelConfig, dec_idx: List[int], instance: int) -> None:
        # the reference's three-argument call unless a second context instance is in play
        extra = (instance,) if instance else ()
        self._remote_call_all_workers_async("migrate_blocks", ctx_idx, config, dec_idx, *extra)

    def _allocate_for_migration(self, migrating_req: MigratingRequest) -> List[int]:
        """Blocks on this side for the request's *prompt* (reference :505-517)."""
        req = migrating_req.req
        # the first generated token already exists; it must not count towards the blocks
        # that are allocated (and copied) now
        kept = (req.generated_tokens, req.generated_token_ids)
        req.generated_tokens, req.generated_token_ids = [], []
        try:
            self.block_manager.allocate_blocks(req)
        finally:
            req.generated_tokens, req.generated_token_ids = kept
        target_block_indexes = self.block_manager.get_block_table(req.request_id)
        assert len(target_block_indexes) == len(migrating_req.block_indexes), (
            f"request {req.request_id}: {len(migrating_req.block_indexes)} context blocks but "
            f"{len(target_block_indexes)} decoding blocks")
        return target_block_indexes

    def _callback_takes_events(self) -> bool:
        """Whether the release callback has a ``migrate_events`` parameter; the reference's
        (``clear_migrated_blocks_callback(migrated_request)``, :405-410) has not."""
        if self._release_takes_events is None:
            import inspect

            try:
                params = inspect.signature(self.clear_migrated_blocks_callback).parameters
                self._release_takes_events = "migrate_events" in params or any(
                    p.kind is inspect.Parameter.VAR_KEYWORD for p in params.values())
            except (TypeError, ValueError):
                self._release_takes_events = False
        return self._release_takes_events

    def _release_source_blocks(self, migrating_reqs: List[MigratingRequest]) -> None:
        if self.clear_migrated_blocks_callback is None:
            return
        events = [w.latest_migrate_event for row in self.workers for w in row
                  if getattr(w, "latest_migrate_event", None) is not None]
        if self._callback_takes_events():
            for migrating_req in migrating_reqs:
                self.clear_migrated_blocks_callback(migrating_req, migrate_events=events)
            return
        # A callback of the reference's shape cannot order the context instance's later work
        # behind the copies, so the blocks are released only once the copies have finished.
        for event in events:
            if hasattr(event, "synchronize"):
                event.synchronize()
        for migrating_req in migrating_reqs:
            self.clear_migrated_blocks_callback(migrating_req)

    def _migrate_blocks(self, migrating_req: MigratingRequest) -> None:
        """Move one request from the context instance to this one (reference :490-536):
        allocate blocks for its *prompt* here, have every decoding rank pull its share,
        then release the blocks on the context side."""
        req = migrating_req.req
        target_block_indexes = self._allocate_for_migration(migrating_req)
        self._lifetime(req.request_id, LifetimeEventType.MigrationBegin)
        self._call_migrate(migrating_req.block_indexes, migrating_req.context_parallel_config,
                           target_block_indexes, getattr(migrating_req, "context_instance", 0))
        self._wait_for_copies()
        self._lifetime(req.request_id, LifetimeEventType.MigrationEnd)
        self._release_source_blocks([migrating_req])

    def _migrate_blocks_batched(self, migrating_reqs: List[MigratingRequest], allocate_only: bool = False) -> None:
        """Several requests of one context instance in ONE ``migrate_blocks`` call per worker:
        their block tables are concatenated.  ``allocate_only`` does the allocation step for
        requests whose copy is issued later together with others (the scheduler decides
        acceptance request by request, each after the previous one's allocation)."""
        if allocate_only:
            for m in migrating_reqs:
                self._allocate_for_migration(m)
            return
        if not migrating_reqs:
            return
        config = migrating_reqs[0].context_parallel_config
        instance = getattr(migrating_reqs[0], "context_instance", 0)
        assert all(m.context_parallel_config.to_list()[0::2] == config.to_list()[0::2]
                   and getattr(m, "context_instance", 0) == instance for m in migrating_reqs), \
            "requests migrated together must come from one context instance"
        ctx_idx: List[int] = []
        dec_idx: List[int] = []
        for m in migrating_reqs:
            rid = m.req.request_id
            if rid not in self.block_manager.block_table:
                self._allocate_for_migration(m)
            target = self.block_manager.get_block_table(rid)
            assert len(target) == len(m.block_indexes)
            ctx_idx += m.block_indexes
            dec_idx += target
            self._lifetime(rid, LifetimeEventType.MigrationBegin)
        self._call_migrate(ctx_idx, config, dec_idx, instance)
        self._wait_for_copies()
        for m in migrating_reqs:
            self._lifetime(m.req.request_id, LifetimeEventType.MigrationEnd)
        self._release_source_blocks(migrating_reqs)
