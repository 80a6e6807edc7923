"""Side streams that the GPU really runs beside each other.

A HIP stream is served by one of a few hardware queues (``GPU_MAX_HW_QUEUES``, 4 by default),
picked by the runtime when the stream is first used; streams that share a queue run one after
the other, whatever the program says about them.  Which queue a new stream gets depends on
every stream the process has made before, so two fresh ``torch.cuda.Stream()`` objects are
sometimes a pair that serialises (measured on MI355X with ROCm 7.2: of the first twelve
streams of torch's pool, #2 and #3 share a queue, #6 shares the default stream's).  For the
swap path that is the difference between a swap-out and a swap-in that share the host link
and two that queue behind each other, or behind the forward pass.

``side_streams`` therefore tries candidates and keeps those that overlap, by measurement,
with the default stream and with each other.  The reference creates its two swap streams
unconditionally (reference distserve/worker.py:64-66); on CUDA nothing more is needed.
"""
from __future__ import annotations

import logging
from typing import List, Optional, Sequence

import torch

logger = logging.getLogger(__name__)

_SPIN_CYCLES = 400_000        # first guess for a kernel of a few hundred microseconds
_SPIN_MS = 0.2                # shorter than this and the host's enqueue time blurs the answer
_CANDIDATES = 12              # the mapping repeats with a period of about four streams


def _spin(stream: torch.cuda.Stream, cycles: int) -> None:
    with torch.cuda.stream(stream):
        torch.cuda._sleep(cycles)


def run_together(a: torch.cuda.Stream, b: torch.cuda.Stream) -> bool:
    """True if a kernel on ``b`` starts while a kernel enqueued earlier on ``a`` still runs."""
    cycles = _SPIN_CYCLES
    for _ in range(6):
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        a.synchronize()
        b.synchronize()
        ev[0].record(a)
        _spin(a, cycles)
        ev[1].record(a)
        ev[2].record(b)          # on a queue of its own this is stamped at once, else after the spin
        ev[1].synchronize()
        ev[2].synchronize()
        spin_ms = ev[0].elapsed_time(ev[1])
        if spin_ms >= _SPIN_MS:
            return ev[2].elapsed_time(ev[1]) > 0.5 * spin_ms
        cycles *= 4
    raise RuntimeError("distserve_amd.streams: the spin kernel never ran long enough to time")


def side_streams(count: int, beside: Optional[Sequence[torch.cuda.Stream]] = None,
                 device: Optional[torch.device] = None) -> List[torch.cuda.Stream]:
    """``count`` default-priority streams that run at the same time as each other and as the
    streams in ``beside`` (default: the device's default stream).  With fewer hardware queues
    than that asks for, the remaining streams are plain new ones and a warning says so."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    if beside is None:
        beside = [torch.cuda.default_stream(device)]
    chosen: List[torch.cuda.Stream] = []
    spare: List[torch.cuda.Stream] = []
    for _ in range(_CANDIDATES):
        if len(chosen) == count:
            break
        cand = torch.cuda.Stream(device)
        if all(run_together(other, cand) for other in list(beside) + chosen):
            chosen.append(cand)
        else:
            spare.append(cand)
    if len(chosen) < count:
        logger.warning("only %d of %d side streams got a hardware queue of their own; the others "
                       "will run behind a stream they share one with", len(chosen), count)
        while len(chosen) < count:
            chosen.append(spare.pop(0) if spare else torch.cuda.Stream(device))
    return chosen
