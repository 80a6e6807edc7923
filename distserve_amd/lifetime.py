"""Per-request lifetime events around the migration, in the reference's JSON shape.

Mirror of reference ``distserve/lifetime.py``: the same event names and the same
``{"timestamp": ..., "event_type": ...}`` records that the API server returns
(``distserve_api_server.py:113-119``) and that the evaluation scripts turn into the
"Transmission" share of a request's latency (``evaluation/ae-scripts/e2e/_plot.py:323-341``:
``migration_end - migration_begin``).  As in the reference, ``migration_end`` is taken on the
host when the migrate calls have returned, which for an asynchronous copy is the time to
enqueue it; a decoding engine built with ``gpu_complete_lifetime_events=True`` waits for the
copy's event first, so that the interval covers the copy itself.
"""
from __future__ import annotations

import time
from enum import Enum
from typing import Dict, List, Optional


class LifetimeEventType(Enum):
    Issued = "issued"
    ContextBegin = "context_begin"
    ContextEnd = "context_end"
    MigrationBegin = "migration_begin"
    MigrationEnd = "migration_end"
    DecodingBegin = "decoding_begin"
    DecodingEnd = "decoding_end"

    def __str__(self) -> str:
        return self.value


class LifetimeEvent:
    def __init__(self, event_type: LifetimeEventType, timestamp: Optional[float] = None):
        self.event_type = event_type
        self.timestamp = time.time() if timestamp is None else timestamp

    def __repr__(self) -> str:
        return f"LifetimeEvent({self.event_type}, {self.timestamp:.6f})"


def json_encode_lifetime_events(events: List[LifetimeEvent]) -> List[dict]:
    return [{"timestamp": e.timestamp, "event_type": str(e.event_type)} for e in events]


def json_decode_lifetime_events(json_list: List[dict]) -> List[LifetimeEvent]:
    return [LifetimeEvent(LifetimeEventType(d["event_type"]), d["timestamp"]) for d in json_list]


def transmission_seconds(events: List[LifetimeEvent]) -> float:
    """The "Transmission" stage as the reference's plots compute it."""
    at: Dict[LifetimeEventType, float] = {e.event_type: e.timestamp for e in events}
    return at[LifetimeEventType.MigrationEnd] - at[LifetimeEventType.MigrationBegin]


STAGES = ("Context Queuing", "Context Execution", "Transmission", "Decoding Queuing", "Decoding Execution")


def stage_seconds(events: List[LifetimeEvent]) -> List[float]:
    """A request's latency split into the five stages of the reference's breakdown plot, in the
    order of ``STAGES`` (``evaluation/ae-scripts/e2e/_plot.py:323-341``): the later timestamp
    wins when an event type occurs twice, and decoding queuing is the two waits either side
    of the transmission."""
    at: Dict[LifetimeEventType, float] = {e.event_type: e.timestamp for e in events}
    t = LifetimeEventType

    def delta(a: LifetimeEventType, b: LifetimeEventType) -> float:
        return at[b] - at[a]

    return [delta(t.Issued, t.ContextBegin),
            delta(t.ContextBegin, t.ContextEnd),
            delta(t.MigrationBegin, t.MigrationEnd),
            delta(t.ContextEnd, t.MigrationBegin) + delta(t.MigrationEnd, t.DecodingBegin),
            delta(t.DecodingBegin, t.DecodingEnd)]
