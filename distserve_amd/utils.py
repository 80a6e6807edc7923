"""Small shared definitions (reference ``distserve/utils.py``)."""
from enum import Enum
from typing import List

GB = 1 << 30
MB = 1 << 20

# A memory handle crosses the worker API as a list of ints (reference utils.py:69 gives
# cudaMemoryIpcHandle the same alias).
MemoryHandle = List[int]
cudaMemoryIpcHandle = MemoryHandle


class Stage(Enum):
    """Which instance a worker or engine belongs to."""

    CONTEXT = "context"
    DECODING = "decoding"

    def __str__(self) -> str:
        return self.value
