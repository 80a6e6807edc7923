"""Per-GPU worker: owns the KV pools and the pinned swap pools, and issues the copies.

Host-side mirror of reference ``distserve/worker.py`` (``ParaWorker``), reduced to the KV
movement path: pool allocation, handle export and registration, ``migrate_blocks``,
``swap_blocks`` on two side streams with an event table, and the waits around them.  The
method names and argument order are the reference's; the Ray actor wrapper and the model
forward are not part of this path (``step`` keeps only its swap-event waits and calls an
optional ``forward`` hook).

Ordering differs from the reference where the reference is unsafe, never in what is copied:
* the swap event is recorded *after* the copy is enqueued (the reference records it
  before, worker.py:286-287 vs :302-311, so its event does not cover the copy);
* a side stream first waits for the work already enqueued on the compute stream, so a
  swap-out never reads a block the forward pass is still writing;
* ``migrate_blocks`` leaves a mark (``latest_migrate_event``) that the context instance
  makes its stream wait on before it reuses the freed source blocks.
"""
from __future__ import annotations

import copy
import time
from typing import Callable, Dict, List, Optional, Tuple

import torch

from distserve_amd.config import CacheConfig, ModelConfig, ParallelConfig
from distserve_amd.request import Request
from distserve_amd.streams import side_streams
from distserve_amd.utils import MemoryHandle, Stage


# torch's accessor of the current stream's raw handle (an int), where this build of torch has it
_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _require_gpu() -> None:
    if not torch.cuda.is_available():
        raise RuntimeError("distserve_amd.Worker needs a GPU: the KV movement path has no CPU fallback")


class MigrationMark:
    """Stands for "the copies enqueued on ``stream`` so far" with the interface of an event
    (``wait``, ``synchronize``, ``query``).  On the device's default stream the HIP event
    behind it is only recorded when somebody needs one: work that follows on the same stream
    is behind the copies by stream order alone, and that is the common case (one worker
    thread, one current stream), where an eager event per migrated request would be two
    runtime calls that order nothing.  An event recorded late covers the copies all the same,
    and whatever the stream got since -- which is why a mark made on any OTHER stream records
    at once (``eager``): a worker that migrates on a stream of its own has other streams
    beside it, and one of them waiting on a late event would also wait for everything the
    migration's stream was given after the copies (a long decoding step, say)."""

    def __init__(self, stream: torch.cuda.Stream, eager: bool = False):
        self.stream = stream
        self.raw_stream = stream.cuda_stream   # the hipStream_t as an int: what the hot path compares
        self._event: Optional[torch.cuda.Event] = None
        if eager:
            self._recorded()

    @property
    def pending(self) -> bool:
        """No event has been recorded yet: the mark still stands for everything on its stream."""
        return self._event is None

    def _recorded(self) -> torch.cuda.Event:
        if self._event is None:
            self._event = torch.cuda.Event()
            self._event.record(self.stream)
        return self._event

    def wait(self, stream: torch.cuda.Stream) -> None:
        if stream != self.stream:
            self._recorded().wait(stream)

    def synchronize(self) -> None:
        self._recorded().synchronize()

    def query(self) -> bool:
        return self._recorded().query()


class Worker:
    """One worker per GPU (reference worker.py:24-334)."""

    def __init__(self, worker_id: int, stage: Stage, model_config: ModelConfig, cache_config: CacheConfig,
                 parallel_config: ParallelConfig = ParallelConfig(),
                 tensor_parallel_id: List[int] = None, pipeline_parallel_id: List[int] = None,
                 forward: Optional[Callable] = None) -> None:
        model_config.check_kv_heads_are_split(parallel_config)
        _require_gpu()
        self.worker_id = worker_id
        self.stage = stage
        self.model_config = model_config
        self.cache_config = cache_config
        self.parallel_config = parallel_config
        self.tensor_parallel_id = tensor_parallel_id      # communicator ids belong to the model's
        self.pipeline_parallel_id = pipeline_parallel_id  # TP/PP collectives, unused on this path
        self.forward = forward
        self.device = torch.device("cuda:0")
        torch.cuda.set_device(self.device)
        self._device_index = self.device.index
        self._default_stream = torch.cuda.default_stream(self.device)
        self._default_raw_stream = self._default_stream.cuda_stream
        # the overloads, resolved once: a lookup through torch.ops per call costs microseconds
        self._migrate_op = torch.ops.block_migration_ops.migrate_blocks_from.default
        self._swap_op = torch.ops.swapping_ops.swap.default

        self.k_cache: Optional[torch.Tensor] = None   # [blocks, layers_local, kv_heads_local, B, D] on HBM
        self.v_cache: Optional[torch.Tensor] = None
        self.k_swap: Optional[torch.Tensor] = None    # same block shape, pinned host memory
        self.v_swap: Optional[torch.Tensor] = None
        # default-priority side streams, one per direction (reference worker.py:64-66), picked so
        # that the GPU runs them beside each other and beside the default stream: two streams
        # that share a hardware queue would turn a swap-out and a swap-in into one after the other
        self.swap_in_stream, self.swap_out_stream = side_streams(2, device=self.device)
        self.swap_event_table: Dict[int, torch.cuda.Event] = {}   # request_id -> its latest swap
        self.latest_swap_in_event: Optional[torch.cuda.Event] = None
        self.latest_swap_out_event: Optional[torch.cuda.Event] = None
        self.latest_migrate_event: Optional[MigrationMark] = None
        self.execution_time = 0.0
        self.blocked_swapping_time = 0.0

    def ready(self) -> None:
        pass

    def _current_stream(self) -> torch.cuda.Stream:
        # with the device named, torch does not re-count the devices on every call (tens of
        # microseconds each on ROCm), which matters for a call made once per migrated request
        return torch.cuda.current_stream(self.device)

    def _current_raw_stream(self) -> int:
        """The current stream's hipStream_t as an int, without building a Stream object
        (1-2 microseconds each, twice per migrated request otherwise)."""
        if _RAW_STREAM is not None:
            return _RAW_STREAM(self._device_index)
        return self._current_stream().cuda_stream

    # ---- pools

    def kv_cache_shape(self, num_blocks: int) -> Tuple[int, int, int, int, int]:
        return (num_blocks,
                self.model_config.get_num_layers(self.parallel_config),
                self.model_config.get_num_heads(self.parallel_config),
                self.cache_config.block_size,
                self.model_config.get_head_size())

    def _new_pool(self, num_blocks: int, on_host: bool) -> torch.Tensor:
        shape, dtype = self.kv_cache_shape(num_blocks), self.model_config.get_torch_dtype()
        if on_host:
            # pinned, so that the swap copies are asynchronous to the host
            return torch.empty(shape, dtype=dtype, device="cpu", pin_memory=True)
        return torch.empty(shape, dtype=dtype, device=self.device)

    def init_kvcache_and_swap(self, num_gpu_blocks: int, num_cpu_blocks: int) -> Tuple[MemoryHandle, MemoryHandle]:
        """Allocate the K/V pools on HBM and the pinned K/V swap pools on the host; return the
        memory handles of the two HBM pools (reference worker.py:101-134)."""
        self.k_cache, self.v_cache = (self._new_pool(num_gpu_blocks, on_host=False) for _ in range(2))
        self.k_swap, self.v_swap = (self._new_pool(num_cpu_blocks, on_host=True) for _ in range(2))
        torch.cuda.synchronize()
        export = torch.ops.block_migration_ops.get_ipc_mem_handle
        return export(self.k_cache), export(self.v_cache)

    def _get_block_size_in_bytes(self, block_size: int, model_config: ModelConfig,
                                 parallel_config: ParallelConfig) -> int:
        """Bytes of one block, K and V together (reference worker.py:136-150)."""
        per_pool = (model_config.get_num_layers(parallel_config) * model_config.get_num_heads(parallel_config)
                    * block_size * model_config.get_head_size())
        return 2 * per_pool * model_config.get_dtype_size()

    def _profile_num_available_blocks(self, block_size: int, gpu_memory_utilization: float,
                                      cpu_swap_space: int, model_bytes: int = 0) -> Tuple[int, int]:
        """Blocks that fit (reference worker.py:153-192); the weights' size is an argument
        because the model itself is not part of this path."""
        total = torch.cuda.get_device_properties(self.device).total_memory
        reserved = total * 0.01 + model_bytes
        block_bytes = self._get_block_size_in_bytes(block_size, self.model_config, self.parallel_config)
        num_gpu_blocks = max(int((total * gpu_memory_utilization - reserved) // block_bytes), 0)
        num_cpu_blocks = max(int(cpu_swap_space // block_bytes), 0)
        return num_gpu_blocks, num_cpu_blocks

    # ---- step: only the swap waits of reference worker.py:204-212 belong to this path

    def step(self, request_ids: List[int], input_tokens_batched=None, first_token_indexes=None,
             block_table=None):
        start = time.time()
        for request_id in request_ids:
            event = self.swap_event_table.pop(request_id, None)
            if event is not None:
                # stalls the compute stream, not the host, until the request's blocks are in place
                event.wait(self._current_stream())
        self.blocked_swapping_time += time.time() - start
        if self.forward is None:
            return None
        start = time.time()
        out = self.forward(input_tokens_batched, first_token_indexes, self.k_cache, self.v_cache, block_table)
        self.execution_time += time.time() - start
        return out

    # ---- migration

    def register_kvcache_mem_handles(self, context_parallel_config: ParallelConfig,
                                     kvcache_ipc_mem_handles: List[List[Tuple[MemoryHandle, MemoryHandle]]],
                                     context_instance: int = 0) -> None:
        """Bind every context rank's pools, ``handles[pp_rank][tp_rank] = (k, v)``
        (reference worker.py:229-248).  The handles may come from another process: they are
        plain lists of ints.  ``context_instance`` (not in the reference, where a decoding
        worker serves one context instance) keeps several instances' pools apart."""
        for pp_rank, stage_handles in enumerate(kvcache_ipc_mem_handles):
            for tp_rank, (k_handle, v_handle) in enumerate(stage_handles):
                rank_config = copy.deepcopy(context_parallel_config)
                rank_config.pipeline_parallel_rank = pp_rank
                rank_config.tensor_parallel_rank = tp_rank
                torch.ops.block_migration_ops.register_ipc_mem_handle_from(
                    context_instance, k_handle, v_handle,
                    self.model_config.get_num_layers(), self.model_config.get_num_heads(),
                    rank_config.to_list(), self.parallel_config.to_list())
        torch.cuda.synchronize()

    def migrate_blocks(self, context_block_indexes: List[int], context_parallel_config: ParallelConfig,
                       decoding_block_indexes: List[int], context_instance: int = 0) -> None:
        """Pull this rank's share of the listed context blocks into its own pools, on the
        current stream, without waiting for the GPU (reference worker.py:250-267)."""
        self._migrate_op(
            context_instance,
            context_parallel_config.pipeline_parallel_size,
            context_parallel_config.tensor_parallel_size,
            context_block_indexes,
            self.parallel_config.pipeline_parallel_size,
            self.parallel_config.tensor_parallel_size,
            self.parallel_config.pipeline_parallel_rank,
            self.parallel_config.tensor_parallel_rank,
            decoding_block_indexes,
            self.k_cache,
            self.v_cache,
        )
        raw = self._current_raw_stream()
        mark = self.latest_migrate_event
        # a mark on the same stream that nobody has asked for an event yet stands for these copies too
        if mark is None or mark.raw_stream != raw or not mark.pending:
            self.latest_migrate_event = MigrationMark(self._current_stream(), eager=raw != self._default_raw_stream)

    def wait_stream_for_migration(self, event: Optional[MigrationMark]) -> None:
        """Called on a *context* worker: work it enqueues from now on (the next prefill that
        may overwrite freed blocks) runs after the migration that read them."""
        if event is None:
            return
        if getattr(event, "raw_stream", None) == self._current_raw_stream():
            return                      # the same stream: behind the copies by stream order alone
        event.wait(self._current_stream())

    # ---- swap

    def swap_blocks(self, request_ids: List[int], source_block_ids: List[int], target_block_ids: List[int],
                    is_swap_in: bool) -> None:
        """Copy blocks between the host pools and HBM on the direction's side stream: host
        block ``source_block_ids[i]`` to GPU block ``target_block_ids[i]`` when ``is_swap_in``,
        the other way round otherwise (reference worker.py:269-311)."""
        stream = self.swap_in_stream if is_swap_in else self.swap_out_stream
        # blocks being read or overwritten may still be in use by work on the compute stream
        stream.wait_stream(self._current_stream())
        for request_id in request_ids:
            previous = self.swap_event_table.get(request_id)
            if previous is not None:
                previous.wait(stream)   # the request's earlier swap, possibly on the other stream
        with torch.cuda.stream(stream):
            self._swap_op(source_block_ids, target_block_ids, is_swap_in,
                          self.k_cache, self.v_cache, self.k_swap, self.v_swap)
        event = torch.cuda.Event()
        event.record(stream)
        for request_id in request_ids:
            self.swap_event_table[request_id] = event
        if is_swap_in:
            self.latest_swap_in_event = event
        else:
            self.latest_swap_out_event = event

    def clear_request_resource(self, request_id: int) -> None:
        self.swap_event_table.pop(request_id, None)

    def clear_request_resource_batched(self, requests: List[Request]) -> None:
        for request in requests:
            self.clear_request_resource(request.request_id)

    def wait_for_all_swap_in(self) -> None:
        if self.latest_swap_in_event is not None:
            self.latest_swap_in_event.synchronize()
            self.latest_swap_in_event = None

    def wait_for_all_swap_out(self) -> None:
        if self.latest_swap_out_event is not None:
            self.latest_swap_out_event.synchronize()
            self.latest_swap_out_event = None


# the reference's class name
ParaWorker = Worker
