"""The context scheduler's block accounting around the hand-off (host logic, no GPU).
Expected batches are derived by hand from the reference's rule
(distserve/context_stage_scheduler.py:127-188): prompt blocks of the batch + of the
prefilled-but-unmigrated requests + of the batches in flight must fit the GPU pool."""
import pytest

from distserve_amd.block_manager import BlockManager
from distserve_amd.config import CacheConfig, ModelConfig, ParallelConfig
from distserve_amd.context_stage_scheduler import (ContextStageFCFSScheduler, ContextStageSchedConfig,
                                                   get_context_stage_scheduler)
from distserve_amd.handoff import ContextStageLLMEngine, DecodingStageLLMEngine
from distserve_amd.request import MigratingRequest, create_request
from distserve_amd.utils import Stage


def make(n_gpu, max_batch=8, max_tokens=4096):
    bm = BlockManager(Stage.CONTEXT, n_gpu, 1, ModelConfig.from_kv_shape(2, 2, 8), ParallelConfig(),
                      CacheConfig(16, 64), lambda *a: None)
    return get_context_stage_scheduler(ContextStageSchedConfig("fcfs", max_batch, max_tokens), ParallelConfig(), bm), bm


def test_unmigrated_requests_hold_blocks_against_the_next_batch():
    sched, bm = make(n_gpu=10)
    reqs = [create_request(n, i) for i, n in enumerate([64, 48, 32, 64, 16])]    # 4, 3, 2, 4, 1 blocks
    for r in reqs:
        sched.add_request(r)
    b0 = sched.get_next_batch_and_pop()
    # 4 + 3 + 2 = 9 <= 10; adding request 3 (4 blocks) would make 13
    assert [r.request_id for r in b0.requests] == [0, 1, 2] and sched.num_on_fly_request_block == 9
    assert sched.get_next_batch_and_pop().requests == []          # 9 in flight: not even request 3 (4) fits
    for r in b0.requests:
        r.add_generated_token("t", 1)
    sched.on_finish_requests(b0)                                   # prefilled, waiting to be migrated
    assert sched.num_on_fly_request_block == 0 and [r.request_id for r in sched.unaccepted_queue] == [0, 1, 2]
    assert sched.get_next_batch_and_pop().requests == []          # still 9 blocks held by the unmigrated
    sched.on_request_migrated(MigratingRequest(reqs[0], [0, 1, 2, 3], ParallelConfig()))
    b1 = sched.get_next_batch_and_pop()                            # 5 held: 4 fits (9), then 1 more (10)
    assert [r.request_id for r in b1.requests] == [3, 4] and sched.get_num_waiting_requests() == 0
    sched.on_request_migrated(MigratingRequest(create_request(1, 99), [], ParallelConfig()))   # unknown id: no-op
    assert [r.request_id for r in sched.unaccepted_queue] == [1, 2]


def test_batch_size_token_budget_and_finished_requests():
    sched, _ = make(n_gpu=100, max_batch=2)
    for i in range(3):
        sched.add_request(create_request(16, i))
    assert [r.request_id for r in sched.get_next_batch_and_pop().requests] == [0, 1]
    sched2, _ = make(n_gpu=100, max_tokens=40)
    for i, n in enumerate([30, 10, 5]):
        sched2.add_request(create_request(n, i))
    b = sched2.get_next_batch_and_pop()                            # 30 + 10 = 40 tokens, the third would be 45
    assert [r.request_id for r in b.requests] == [0, 1]
    b.requests[0].is_finished = True                               # finished in prefill: nothing to migrate
    sched2.on_finish_requests(b)
    assert [r.request_id for r in sched2.unaccepted_queue] == [1]
    sched2.abort_request(2)
    assert sched2.get_num_waiting_requests() == 0
    with pytest.raises(AssertionError):
        ContextStageSchedConfig("srpt", 1, 1)


def test_the_handoff_tells_the_context_scheduler_when_a_request_has_left():
    from test_handoff_cpu import FakeWorker

    model, cache = ModelConfig.from_kv_shape(4, 4, 16), CacheConfig(16, 64)
    ctx = ContextStageLLMEngine(model, ParallelConfig(), cache, worker_factory=FakeWorker)
    dec = DecodingStageLLMEngine(model, ParallelConfig(), cache, worker_factory=FakeWorker,
                                 clear_migrated_blocks_callback=ctx.clear_migrated_blocks_callback)
    ctx._init_kvcache(8, 0)
    dec._init_kvcache(8, 2)
    ctx.scheduler = ContextStageFCFSScheduler(ContextStageSchedConfig("fcfs", 4, 1024), ctx.parallel_config,
                                              ctx.block_manager)
    req = create_request(40, 0)
    ctx.scheduler.add_request(req)
    batch = ctx.scheduler.get_next_batch_and_pop()
    ctx.block_manager.allocate_blocks_batched(batch)
    req.add_generated_token("t", 1)
    ctx.scheduler.on_finish_requests(batch)
    assert [r.request_id for r in ctx.scheduler.unaccepted_queue] == [0]
    dec._migrate_blocks(ctx.on_prefill_finished(req))
    assert ctx.scheduler.unaccepted_queue == [] and 0 not in ctx.block_manager.block_table
