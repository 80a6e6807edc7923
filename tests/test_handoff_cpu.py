"""The migration handoff protocol with fake workers (no GPU): order of the steps, the
fan-out to every decoding rank and the block tables that travel (reference
distserve/single_stage_engine.py:393-410, 469-536)."""
import pytest

from distserve_amd.config import CacheConfig, ModelConfig, ParallelConfig
from distserve_amd.handoff import ContextStageLLMEngine, DecodingStageLLMEngine
from distserve_amd.request import create_request

LOG = []


class FakeWorker:
    def __init__(self, worker_id, stage, model_config, cache_config, parallel_config):
        self.worker_id, self.stage, self.parallel_config = worker_id, stage, parallel_config
        self.latest_migrate_event = None

    def _tag(self):
        return (str(self.stage), self.parallel_config.pipeline_parallel_rank, self.parallel_config.tensor_parallel_rank)

    def init_kvcache_and_swap(self, n_gpu, n_cpu):
        LOG.append(("init",) + self._tag() + (n_gpu, n_cpu))
        return ([1, self.worker_id], [2, self.worker_id])

    def register_kvcache_mem_handles(self, ctx_pc, handles):
        LOG.append(("register",) + self._tag() + (ctx_pc.to_list(), handles))

    def migrate_blocks(self, ctx_idx, ctx_pc, dec_idx):
        LOG.append(("migrate",) + self._tag() + (list(ctx_idx), ctx_pc.to_list(), list(dec_idx)))
        self.latest_migrate_event = ("event", self.worker_id)

    def wait_stream_for_migration(self, event):
        LOG.append(("wait",) + self._tag() + (event,))

    def clear_request_resource(self, request_id):
        LOG.append(("clear",) + self._tag() + (request_id,))


@pytest.fixture()
def engines():
    LOG.clear()
    model = ModelConfig.from_kv_shape(8, 8, 16)
    cache = CacheConfig(16, 128)
    ctx = ContextStageLLMEngine(model, ParallelConfig(2, 0, 2, 0), cache, worker_factory=FakeWorker)
    dec = DecodingStageLLMEngine(model, ParallelConfig(4, 0, 1, 0), cache, worker_factory=FakeWorker,
                                 clear_migrated_blocks_callback=ctx.clear_migrated_blocks_callback)
    ctx._init_kvcache(10, 7)
    dec._init_kvcache(12, 5)
    return ctx, dec


def test_init_collects_handles_as_pp_by_tp_and_context_never_swaps(engines):
    ctx, dec = engines
    inits = [e for e in LOG if e[0] == "init"]
    assert [e[1:4] for e in inits[:4]] == [("context", 0, 0), ("context", 0, 1), ("context", 1, 0), ("context", 1, 1)]
    assert all(e[4:] == (10, 1) for e in inits[:4])          # num_cpu_blocks forced to 1
    assert all(e[4:] == (12, 5) for e in inits[4:])
    assert ctx.kv_cache_mem_handles == [[([1, 0], [2, 0]), ([1, 1], [2, 1])], [([1, 2], [2, 2]), ([1, 3], [2, 3])]]
    dec.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    regs = [e for e in LOG if e[0] == "register"]
    assert [e[2:4] for e in regs] == [(0, 0), (0, 1), (0, 2), (0, 3)]     # every decoding rank
    assert all(e[5] == ctx.kv_cache_mem_handles for e in regs)


def test_migrate_allocates_prompt_blocks_fans_out_then_frees_the_source(engines):
    ctx, dec = engines
    LOG.clear()
    warm = create_request(16, 90)
    ctx.block_manager.allocate_blocks(warm)                       # context block 0 is taken
    req = create_request(40, 7)                                   # 3 blocks
    ctx.block_manager.allocate_blocks(req)                        # context blocks [1,2,3]
    req.add_generated_token("t", 5)                               # prefill produced the first token
    for _ in range(8):
        req.add_generated_token("t", 5)                           # 49 tokens would be 4 blocks
    m = ctx.on_prefill_finished(req)
    assert m.block_indexes == [1, 2, 3] and ctx.bridge_queue == [m]

    dec._migrate_blocks(m)
    # the generated tokens came back and did not size the allocation
    assert req.get_output_len() == 9
    assert dec.block_manager.get_block_table(7) == [0, 1, 2]
    migrates = [e for e in LOG if e[0] == "migrate"]
    assert [(e[2], e[3]) for e in migrates] == [(0, 0), (0, 1), (0, 2), (0, 3)]
    for e in migrates:
        assert e[4] == [1, 2, 3] and e[5] == [2, 0, 2, 0] and e[6] == [0, 1, 2]
    # order: all migrations, then the context workers wait on their events, then the free
    kinds = [e[0] for e in LOG]
    assert kinds.index("wait") > max(i for i, k in enumerate(kinds) if k == "migrate")
    assert kinds.index("clear") > max(i for i, k in enumerate(kinds) if k == "wait")
    assert len([k for k in kinds if k == "wait"]) == 4 * 4          # 4 events x 4 context workers
    assert 7 not in ctx.block_manager.block_table
    assert ctx.block_manager.free_gpu_blocks_list[-3:] == [1, 2, 3]
    assert [str(e.event_type) for e in dec.lifetime_events[7]] == ["migration_begin", "migration_end"]


def test_length_mismatch_is_refused_before_any_copy(engines):
    ctx, dec = engines
    req = create_request(40, 3)
    ctx.block_manager.allocate_blocks(req)
    m = ctx.on_prefill_finished(req)
    m.block_indexes = m.block_indexes[:-1]
    LOG.clear()
    with pytest.raises(AssertionError):
        dec._migrate_blocks(m)
    assert not [e for e in LOG if e[0] == "migrate"]


def test_lifetime_events_keep_the_reference_json_shape(engines):
    from distserve_amd.lifetime import (LifetimeEvent, LifetimeEventType, json_decode_lifetime_events,
                                        json_encode_lifetime_events, transmission_seconds)

    ctx, dec = engines
    seen = []
    dec.engine_on_new_lifetime_event_callback = lambda rid, ev: seen.append((rid, str(ev.event_type)))
    req = create_request(20, 11)
    ctx.block_manager.allocate_blocks(req)
    dec._migrate_blocks(ctx.on_prefill_finished(req))
    assert seen == [(11, "migration_begin"), (11, "migration_end")]
    events = dec.get_and_pop_request_lifetime_events(11)
    assert 11 not in dec.lifetime_events
    encoded = json_encode_lifetime_events(events)
    assert [sorted(d) for d in encoded] == [["event_type", "timestamp"]] * 2
    assert [d["event_type"] for d in encoded] == ["migration_begin", "migration_end"]
    decoded = json_decode_lifetime_events(encoded)
    assert [e.event_type for e in decoded] == [LifetimeEventType.MigrationBegin, LifetimeEventType.MigrationEnd]
    assert transmission_seconds(decoded) == encoded[1]["timestamp"] - encoded[0]["timestamp"] >= 0
    # every stage name of the reference is there
    assert [str(t) for t in LifetimeEventType] == ["issued", "context_begin", "context_end", "migration_begin",
                                                   "migration_end", "decoding_begin", "decoding_end"]
    assert transmission_seconds([LifetimeEvent(LifetimeEventType.MigrationBegin, 1.0),
                                 LifetimeEvent(LifetimeEventType.MigrationEnd, 1.5)]) == 0.5


def test_a_release_callback_of_the_reference_shape_is_called_after_the_copies(engines):
    """The reference's callback takes the migrated request only (single_stage_engine.py:405-410).
    It cannot be told which copies to order its later work behind, so the decoding engine
    waits for them itself before it calls."""
    ctx, dec = engines
    waited, seen = [], []

    class FakeEvent:
        def __init__(self, tag):
            self.tag = tag

        def synchronize(self):
            waited.append(self.tag)

    def reference_shaped(migrated_request):
        seen.append((migrated_request.req.request_id, list(waited)))

    dec2 = DecodingStageLLMEngine(dec.model_config, dec.parallel_config, dec.cache_config, worker_factory=FakeWorker,
                                  clear_migrated_blocks_callback=reference_shaped)
    dec2._init_kvcache(12, 5)
    for row in dec2.workers:
        for w in row:
            w.migrate_blocks = (lambda w: lambda *a: setattr(w, "latest_migrate_event", FakeEvent(w.worker_id)))(w)
    req = create_request(20, 21)
    ctx.block_manager.allocate_blocks(req)
    dec2._migrate_blocks(ctx.on_prefill_finished(req))
    assert seen == [(21, [0, 1, 2, 3])]                     # every rank's copy waited for, then one call


def test_requests_of_a_second_context_instance_carry_its_id_to_every_worker(engines):
    ctx, dec = engines
    model, cache = ctx.model_config, ctx.cache_config
    calls = []

    class InstanceWorker(FakeWorker):
        def register_kvcache_mem_handles(self, ctx_pc, handles, context_instance=0):
            calls.append(("register", context_instance))

        def migrate_blocks(self, ctx_idx, ctx_pc, dec_idx, context_instance=0):
            calls.append(("migrate", context_instance, list(ctx_idx)))

    other = ContextStageLLMEngine(model, ParallelConfig(2, 0, 2, 0), cache, worker_factory=FakeWorker, instance_id=4)
    other._init_kvcache(10, 0)
    dec2 = DecodingStageLLMEngine(model, ParallelConfig(2, 0, 1, 0), cache, worker_factory=InstanceWorker)
    dec2._init_kvcache(12, 0)
    dec2.register_kvcache_mem_handles(ctx.parallel_config, ctx.kv_cache_mem_handles)
    dec2.register_kvcache_mem_handles(other.parallel_config, other.kv_cache_mem_handles, context_instance=4)
    assert calls == [("register", 0)] * 2 + [("register", 4)] * 2
    calls.clear()
    a, b = create_request(20, 31), create_request(20, 32)
    ctx.block_manager.allocate_blocks(create_request(16, 30))
    ctx.block_manager.allocate_blocks(a)
    other.block_manager.allocate_blocks(b)
    ma, mb = ctx.on_prefill_finished(a), other.on_prefill_finished(b)
    assert (ma.context_instance, mb.context_instance) == (0, 4)
    dec2._migrate_blocks(ma)
    dec2._migrate_blocks(mb)
    assert calls == [("migrate", 0, [1, 2])] * 2 + [("migrate", 4, [0, 1])] * 2
    with pytest.raises(AssertionError, match="one context instance"):
        dec2._migrate_blocks_batched([ctx.on_prefill_finished(a), mb])


def test_a_response_of_the_reference_shape_decodes_into_the_plots_five_stages():
    """The committed fixture is a response as the reference's API server returns it; the
    events decode, encode back to the same records, and split into the stages of the
    reference's latency-breakdown plot, "Transmission" being migration_end - migration_begin."""
    import json
    import os

    from distserve_amd.lifetime import (STAGES, LifetimeEventType, json_decode_lifetime_events,
                                        json_encode_lifetime_events, stage_seconds, transmission_seconds)

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "lifetime_events_response.json")
    fixture = json.load(open(path))
    response = fixture["response"]
    assert sorted(response) == ["lifetime_events", "text", "timestamps"]
    events = json_decode_lifetime_events(response["lifetime_events"])
    assert [e.event_type for e in events] == list(LifetimeEventType)
    assert json_encode_lifetime_events(events) == response["lifetime_events"]
    stages = dict(zip(STAGES, stage_seconds(events)))
    assert set(stages) == set(fixture["expected_stage_seconds"])
    for name, want in fixture["expected_stage_seconds"].items():
        assert stages[name] == pytest.approx(want, abs=1e-9), name
    assert transmission_seconds(events) == pytest.approx(0.0005, abs=1e-9)
    # the stages tile the request's life
    assert sum(stages.values()) == pytest.approx(1001.125 - 1000.0, abs=1e-9)
    # the events this build's hand-off stamps take the place of the fixture's two
    ctx_model = ModelConfig.from_kv_shape(8, 8, 16)
    dec = DecodingStageLLMEngine(ctx_model, ParallelConfig(1, 0, 1, 0), CacheConfig(16, 128), worker_factory=FakeWorker)
    ctx = ContextStageLLMEngine(ctx_model, ParallelConfig(1, 0, 1, 0), CacheConfig(16, 128), worker_factory=FakeWorker)
    ctx._init_kvcache(8, 0)
    dec._init_kvcache(8, 0)
    req = create_request(20, 5)
    ctx.block_manager.allocate_blocks(req)
    dec._migrate_blocks(ctx.on_prefill_finished(req))
    mine = json_encode_lifetime_events(dec.get_and_pop_request_lifetime_events(5))
    assert [sorted(d) for d in mine] == [sorted(d) for d in response["lifetime_events"][3:5]]
    assert [d["event_type"] for d in mine] == [d["event_type"] for d in response["lifetime_events"][3:5]]
    merged = response["lifetime_events"][:3] + [
        {"timestamp": 1000.625, "event_type": mine[0]["event_type"]},
        {"timestamp": 1000.625 + (mine[1]["timestamp"] - mine[0]["timestamp"]), "event_type": mine[1]["event_type"]},
    ] + response["lifetime_events"][5:]
    assert len(stage_seconds(json_decode_lifetime_events(merged))) == 5
