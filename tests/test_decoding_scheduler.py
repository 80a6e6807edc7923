"""The decoding scheduler's triggers of the KV movement path (host logic, no GPU).  Expected
decisions are derived by hand from the reference's rules
(distserve/decoding_stage_scheduler.py:131-150, 183-223, 247-260): note that the admission
test counts a waiting request twice (once in the waiting sum, once as the candidate) and
that the swap-out victim is the LAST request of the current batch."""
import pytest

from distserve_amd.block_manager import BlockLocation, BlockManager
from distserve_amd.config import CacheConfig, ModelConfig, ParallelConfig
from distserve_amd.decoding_stage_scheduler import DecodingStageSchedConfig, get_decoding_stage_scheduler
from distserve_amd.request import MigratingRequest, create_request
from distserve_amd.utils import Stage


class Harness:
    """A block manager with recording fake workers and the two engine callbacks."""

    def __init__(self, n_gpu, n_cpu=64, pp=1, batch_migrations=False, max_batch_size=8, max_tokens=4096,
                 threshold=0.05):
        self.worker_calls = []
        self.migrations = []          # one entry per migrate "call": list of request ids
        self.bm = BlockManager(Stage.DECODING, n_gpu, n_cpu, ModelConfig.from_kv_shape(2, 2, 8),
                               ParallelConfig(1, 0, pp, 0), CacheConfig(16, 64),
                               lambda name, *a: self.worker_calls.append((name,) + a))
        cfg = DecodingStageSchedConfig("fcfs", max_batch_size, max_tokens, waiting_block_prop_threshold=threshold)
        self.sched = get_decoding_stage_scheduler(cfg, ParallelConfig(1, 0, pp, 0), self.bm, self.migrate_one,
                                                  engine_migrate_blocks_batched_callback=self.migrate_many,
                                                  batch_migrations=batch_migrations)

    def _allocate_prompt(self, m):
        req = m.req
        kept = (req.generated_tokens, req.generated_token_ids)
        req.generated_tokens, req.generated_token_ids = [], []
        self.bm.allocate_blocks(req)
        req.generated_tokens, req.generated_token_ids = kept

    def migrate_one(self, m):
        self._allocate_prompt(m)
        self.migrations.append([m.req.request_id])

    def migrate_many(self, ms, allocate_only=False):
        if allocate_only:
            for m in ms:
                self._allocate_prompt(m)
        else:
            self.migrations.append([m.req.request_id for m in ms])

    def arrive(self, rid, prompt_len):
        req = create_request(prompt_len, rid)
        req.add_generated_token("t", 1)             # prefill produced the first token
        m = MigratingRequest(req, list(range(100 * rid, 100 * rid + -(-prompt_len // 16))), ParallelConfig())
        self.sched.add_request(m)
        return req


def grow(req, tokens):
    for _ in range(tokens):
        req.add_generated_token("t", 1)


@pytest.mark.parametrize("batched", [False, True])
def test_post_process_accepts_head_of_line_until_waiting_prompts_reach_the_threshold(batched):
    h = Harness(n_gpu=40, batch_migrations=batched)           # threshold: 40 * 0.05 = 2 blocks
    r0, r1, r2 = h.arrive(0, 16), h.arrive(1, 32), h.arrive(2, 16)
    h.sched.post_process()
    # r0: waiting 0 < 2 -> accept (1 block); r1: waiting 1 < 2 -> accept (2 blocks); r2: waiting 3 >= 2 -> stop
    assert [r.request_id for r in h.sched.waiting_queue] == [0, 1]
    assert [m.req.request_id for m in h.sched.unaccepted_queue] == [2]
    assert h.bm.get_block_table(0) == [0] and h.bm.get_block_table(1) == [1, 2]
    assert h.migrations == ([[0, 1]] if batched else [[0], [1]])
    h.sched.post_process()                                     # nothing changed: still blocked
    assert len(h.sched.unaccepted_queue) == 1 and len(h.migrations) == (1 if batched else 2)
    assert h.sched.get_waiting_num_requests() == 2 and h.sched.get_total_num_requests() == 2


def test_post_process_stops_when_the_prompt_does_not_fit_the_available_blocks():
    h = Harness(n_gpu=3, threshold=1.0)                       # threshold never binds: 3 blocks
    h.arrive(0, 32)                                            # 2 blocks
    h.arrive(1, 32)                                            # 2 blocks > 1 available after r0
    h.sched.post_process()
    assert [r.request_id for r in h.sched.waiting_queue] == [0]
    assert [m.req.request_id for m in h.sched.unaccepted_queue] == [1]
    assert h.migrations == [[0]]


def test_get_next_batch_admits_swaps_out_the_last_request_and_swaps_it_back_in():
    h = Harness(n_gpu=12, threshold=1.0)
    a, b, c = h.arrive(0, 32), h.arrive(1, 32), h.arrive(2, 16)
    h.sched.post_process()
    assert [r.request_id for r in h.sched.waiting_queue] == [0, 1, 2]       # 2 + 2 + 1 blocks
    batch = h.sched.get_next_batch()
    # a: 0 + waiting 5 + need(33 tokens)=3 = 8 <= 12; b: 3 + 3 + 3 = 9; c: 6 + 1 + need(17)=2 = 9
    assert [r.request_id for r in batch.requests] == [0, 1, 2] and h.sched.waiting_queue == []
    for r in (a, b, c):
        h.bm.allocate_blocks(r)                                # the engine grows the tables before a step
    assert h.bm.get_block_table(0) == [0, 1, 5] and h.bm.get_block_table(2) == [4, 7]

    grow(a, 39)                                                # 32 + 40 tokens -> 5 blocks
    grow(b, 39)                                                # 5 blocks
    grow(c, 19)                                                # 16 + 20 tokens -> 3 blocks: 13 > 12
    h.worker_calls.clear()
    batch = h.sched.get_next_batch()
    assert [r.request_id for r in batch.requests] == [0, 1]                 # victim: the last one
    assert [r.request_id for r in h.sched.swapped_queue] == [2]
    assert h.bm.get_location(2) == BlockLocation.CPU
    assert h.worker_calls == [("swap_blocks", [2], [4, 7], [0, 1], False)]
    # c cannot come back yet: 10 + 0 + 3 = 13 > 12

    a.is_finished = True
    assert [r.request_id for r in h.sched.pop_finished_requests()] == [0]
    h.bm.free_blocks(0)
    h.worker_calls.clear()
    batch = h.sched.get_next_batch()                           # 5 + 0 + 3 = 8 <= 12: swap-in
    assert [r.request_id for r in batch.requests] == [1, 2] and h.sched.swapped_queue == []
    assert h.bm.get_location(2) == BlockLocation.GPU
    assert h.worker_calls[-1][0] == "swap_blocks" and h.worker_calls[-1][1] == [2] and h.worker_calls[-1][4] is True
    assert h.worker_calls[-1][2] == [0, 1]                     # host blocks it was parked in


def test_swapped_requests_are_admitted_before_waiting_ones_and_limits_hold():
    h = Harness(n_gpu=100, threshold=1.0, max_batch_size=2)
    reqs = [h.arrive(i, 16) for i in range(4)]
    h.sched.post_process()
    batch = h.sched.get_next_batch()
    assert [r.request_id for r in batch.requests] == [0, 1]                # max_batch_size
    assert [r.request_id for r in h.sched.waiting_queue] == [2, 3]
    h2 = Harness(n_gpu=100, threshold=1.0, max_tokens=1)
    h2.arrive(0, 16)
    h2.arrive(1, 16)
    h2.sched.post_process()
    assert [r.request_id for r in h2.sched.get_next_batch().requests] == [0]   # 1 decoding token each, budget 1


def test_pipeline_stages_rotate_and_finished_requests_pop_from_the_last_stage():
    h = Harness(n_gpu=100, pp=2, threshold=1.0, max_batch_size=1)
    r0, r1 = h.arrive(0, 16), h.arrive(1, 16)
    h.sched.post_process()
    b0 = h.sched.get_next_batch()                              # cur_index 0
    b1 = h.sched.get_next_batch()                              # cur_index 1
    assert [r.request_id for r in b0.requests] == [0] and [r.request_id for r in b1.requests] == [1]
    assert h.sched.get_processing_num_requests() == 2
    r0.is_finished = True
    # last stage = (cur_index + 1) % 2 = 0
    assert [r.request_id for r in h.sched.pop_finished_requests()] == [0]
    h.sched.abort_request(1)
    assert r1.is_finished
    h.arrive(2, 16)
    h.sched.post_process()
    h.sched.abort_request(2)
    assert h.sched.waiting_queue == []


def test_only_fcfs_is_built():
    with pytest.raises(NotImplementedError):
        get_decoding_stage_scheduler(DecodingStageSchedConfig("srpt", 1, 1), ParallelConfig(), None, None)
    with pytest.raises(AssertionError):
        DecodingStageSchedConfig("random", 1, 1)
