"""BlockManager state machine (host logic, no GPU).  Expected id lists are derived by hand
from the reference's rules: FIFO free lists starting at 0..N-1, allocation from the head,
frees to the tail, swap sources quarantined until a flush (reference
distserve/block_manager.py:44-45, 66-98, 154-161, 288-315)."""
import pytest

from distserve_amd.block_manager import BlockLocation, BlockManager
from distserve_amd.config import CacheConfig, ModelConfig, ParallelConfig
from distserve_amd.request import BatchedRequests, create_request
from distserve_amd.utils import Stage


class Calls:
    def __init__(self):
        self.log = []

    def __call__(self, func_name, *args):
        self.log.append((func_name,) + args)
        return []


def make(n_gpu=8, n_cpu=8, block_size=16):
    calls = Calls()
    bm = BlockManager(Stage.DECODING, n_gpu, n_cpu, ModelConfig.from_kv_shape(2, 2, 8), ParallelConfig(),
                      CacheConfig(block_size, 64), calls)
    return bm, calls


def test_blocks_needed_is_ceil_of_all_tokens():
    bm, _ = make()
    r = create_request(33, 0)
    assert bm.get_num_blocks_needed(r) == 3          # ceil(33/16)
    r.add_generated_token("a", 1)
    for _ in range(14):
        r.add_generated_token("a", 1)
    assert bm.get_num_blocks_needed(r) == 3          # 48 tokens
    r.add_generated_token("a", 1)
    assert bm.get_num_blocks_needed(r) == 4          # 49 tokens


def test_fifo_allocation_and_tail_free():
    bm, _ = make()
    a, b = create_request(40, 0), create_request(16, 1)
    bm.allocate_blocks(a)
    bm.allocate_blocks(b)
    assert bm.get_block_table(0) == [0, 1, 2]
    assert bm.get_block_table(1) == [3]
    assert bm.free_gpu_blocks_list == [4, 5, 6, 7]
    bm.free_blocks(0)
    assert bm.free_gpu_blocks_list == [4, 5, 6, 7, 0, 1, 2]
    c = create_request(80, 2)
    bm.allocate_blocks(c)
    assert bm.get_block_table(2) == [4, 5, 6, 7, 0]
    assert bm.get_location(2) == BlockLocation.GPU and bm.get_location(0) is None
    assert bm.get_num_avail_gpu_blocks() == 2


def test_append_blocks_as_request_grows():
    bm, _ = make()
    r = create_request(16, 7)
    bm.allocate_blocks(r)
    assert bm.get_block_table(7) == [0]
    assert bm.get_num_append_blocks_needed(r) == 0
    r.add_generated_token("x", 1)
    assert bm.get_num_append_blocks_needed(r) == 1
    bm.allocate_blocks(r)
    assert bm.get_block_table(7) == [0, 1]
    bm.allocate_blocks(r)                                  # idempotent when enough
    assert bm.get_block_table(7) == [0, 1]
    assert bm.get_allocated_num_blocks(7) == 2 and bm.get_allocated_num_blocks(99) == 0


def test_batched_helpers_and_partial_table():
    bm, _ = make()
    batch = BatchedRequests([create_request(17, 0), create_request(1, 1)])
    bm.allocate_blocks_batched(batch)
    assert bm.get_partial_block_table([1, 0]) == [[2], [0, 1]]
    assert bm.is_all_requests_on_gpu(batch)
    bm.free_blocks_batched(batch.requests)
    assert bm.free_gpu_blocks_list == [3, 4, 5, 6, 7, 0, 1, 2]
    with pytest.raises(AssertionError):
        bm.get_block_table(0)
    with pytest.raises(AssertionError):
        bm.free_blocks(0)


def test_swap_out_then_in_retargets_tables_and_quarantines_sources():
    bm, calls = make(n_gpu=6, n_cpu=5)
    a, b = create_request(32, 0), create_request(16, 1)
    bm.allocate_blocks(a)          # GPU [0,1]
    bm.allocate_blocks(b)          # GPU [2]
    bm.swap_out_requests([a, b])
    # sources are the old tables in request order, targets the head of the CPU free list
    assert calls.log == [("swap_blocks", [0, 1], [0, 1, 2], [0, 1, 2], False)]
    assert bm.get_block_table(0) == [0, 1] and bm.get_location(0) == BlockLocation.CPU
    assert bm.get_block_table(1) == [2] and bm.get_location(1) == BlockLocation.CPU
    assert bm.swapping_gpu_blocks_list == [0, 1, 2]
    assert bm.free_gpu_blocks_list == [3, 4, 5]
    assert bm.get_num_avail_gpu_blocks() == 6               # quarantined blocks count as available
    assert not bm.is_all_requests_on_gpu(BatchedRequests([a]))

    bm.swap_in_requests([b])
    # free list [3,4,5] suffices: no flush, b lands on GPU block 3
    assert calls.log[-1] == ("swap_blocks", [1], [2], [3], True)
    assert bm.get_block_table(1) == [3] and bm.get_location(1) == BlockLocation.GPU
    assert bm.swapping_cpu_blocks_list == [2]
    assert bm.free_cpu_blocks_list == [3, 4]
    assert len(calls.log) == 2


def test_flush_happens_only_when_the_free_list_alone_is_short():
    bm, calls = make(n_gpu=4, n_cpu=4)
    a = create_request(48, 0)                    # 3 blocks
    bm.allocate_blocks(a)                        # GPU [0,1,2], free [3]
    bm.swap_out_requests([a])                    # quarantine [0,1,2]
    b = create_request(32, 1)                    # needs 2 > len(free)=1 -> flush
    bm.allocate_blocks(b)
    assert calls.log[-1] == ("wait_for_all_swap_out",)
    assert bm.swapping_gpu_blocks_list == []
    assert bm.get_block_table(1) == [3, 0]       # free list became [3] + [0,1,2]
    assert bm.free_gpu_blocks_list == [1, 2]
    # CPU side: swap-in sources are quarantined and flushed by wait_for_all_swap_in
    bm.free_blocks(1)                            # GPU free [1,2,3,0]
    bm.swap_in_requests([a])                     # CPU quarantine [0,1,2], CPU free [3]
    assert bm.get_block_table(0) == [1, 2, 3]
    bm.swap_out_requests([a])                    # needs 3 CPU blocks > 1 free -> flush swap-ins
    assert ("wait_for_all_swap_in",) in calls.log
    assert bm.get_block_table(0) == [3, 0, 1]
    assert bm.free_cpu_blocks_list == [2] and bm.swapping_cpu_blocks_list == []


def test_conservation_over_a_scripted_sequence():
    bm, _ = make(n_gpu=16, n_cpu=16)
    reqs = [create_request(16 * (1 + i % 3), i) for i in range(6)]
    for r in reqs:
        bm.allocate_blocks(r)
    bm.swap_out_requests(reqs[:3])
    bm.free_blocks(4)
    bm.swap_in_requests(reqs[1:2])
    bm.swap_out_requests(reqs[5:6])

    def census(loc, free, quarantine, total):
        owned = [b for rid, t in bm.block_table.items() if bm.request_location[rid] == loc for b in t]
        everything = sorted(free + quarantine + owned)
        assert everything == list(range(total)), (loc, everything)

    census(BlockLocation.GPU, bm.free_gpu_blocks_list, bm.swapping_gpu_blocks_list, 16)
    census(BlockLocation.CPU, bm.free_cpu_blocks_list, bm.swapping_cpu_blocks_list, 16)


def test_errors_the_reference_asserts():
    bm, _ = make(n_gpu=2, n_cpu=1)
    big = create_request(16 * 3, 0)
    with pytest.raises(AssertionError, match="not enough free blocks on GPU"):
        bm.allocate_blocks(big)
    a = create_request(32, 1)
    bm.allocate_blocks(a)
    with pytest.raises(AssertionError, match="not enough free blocks on CPU"):
        bm.swap_out_requests([a])
    with pytest.raises(AssertionError):
        bm.swap_in_requests([a])                  # it is on the GPU, not on the host
    with pytest.raises(AssertionError):
        bm.swap_out_requests([create_request(1, 5)])   # never allocated
    bm2, _ = make(n_gpu=4, n_cpu=4)
    r = create_request(16, 0)
    bm2.allocate_blocks(r)
    bm2.swap_out_requests([r])
    with pytest.raises(AssertionError):
        bm2.allocate_blocks(r)                    # on the host: must be swapped in first
    with pytest.raises(AssertionError):
        bm2.get_num_append_blocks_needed(r)
