"""Side streams picked by measurement: whatever the process did with streams before, the two
a Worker swaps on run beside each other and beside the default stream."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_side_streams_run_together_after_the_process_has_made_many_streams():
    from distserve_amd.streams import run_together, side_streams
    default = torch.cuda.default_stream()
    junk = [torch.cuda.Stream() for _ in range(7)]            # shifts what a fresh stream would get
    for s in junk:
        with torch.cuda.stream(s):
            torch.zeros(8, device="cuda")                      # first use binds a stream to its queue
    torch.cuda.synchronize()
    a, b = side_streams(2)
    assert a != b and a != default and b != default
    assert run_together(a, b) and run_together(b, a)
    assert run_together(default, a) and run_together(default, b)
    assert a.priority == 0 and b.priority == 0
    # a stream cannot overlap with itself: the probe says so
    assert not run_together(a, a)


def test_side_streams_hands_out_what_was_asked_for_when_queues_run_out():
    from distserve_amd.streams import side_streams
    got = side_streams(6)                                      # more than the hardware queues of a process
    assert len(got) == 6 and len({s.cuda_stream for s in got}) == 6
