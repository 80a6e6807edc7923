"""Request objects the block tables are keyed by (reference ``distserve/request.py``).

Only the fields the block manager and the migration handoff read are kept: the prompt
and generated token ids (their lengths size the block table) and the request id.
"""
from __future__ import annotations

from typing import List, Optional

from distserve_amd.config import ParallelConfig


class Request:
    """Reference request.py:161-296, reduced to what sizes a block table."""

    def __init__(self, arrival_time: float, request_id: int, prompt: Optional[str],
                 prompt_token_ids: List[int], sampling_params=None, priority: int = 0):
        self.arrival_time = arrival_time
        self.request_id = request_id
        self.prompt = prompt
        self.prompt_token_ids = prompt_token_ids
        self.sampling_params = sampling_params
        self.generated_tokens: List[str] = []
        self.generated_token_ids: List[int] = []
        self.is_finished = False
        self.is_running = False
        self.priority = priority

    def add_generated_token(self, token: str, token_id: int) -> None:
        self.generated_tokens.append(token)
        self.generated_token_ids.append(token_id)

    def is_context_stage(self) -> bool:
        return len(self.generated_tokens) == 0

    def get_input_len(self) -> int:
        return len(self.prompt_token_ids)

    def get_output_len(self) -> int:
        assert len(self.generated_tokens) == len(self.generated_token_ids)
        return len(self.generated_token_ids)

    def get_kvcache_slots(self) -> int:
        return self.get_input_len() + self.get_output_len()

    def get_num_input_tokens(self) -> int:
        """Tokens the next iteration feeds the model: the whole prompt in the context
        stage, the last generated token afterwards (reference request.py:238-250)."""
        return self.get_input_len() if self.is_context_stage() else 1

    def __repr__(self) -> str:
        return (f"Request(request_id={self.request_id}, input_len={self.get_input_len()}, "
                f"output_len={self.get_output_len()})")


def create_request(prompt_len: int, request_id: int, arrival_time: float = 0.0) -> Request:
    """A synthetic request with ``prompt_len`` prompt tokens (token values do not matter here)."""
    return Request(arrival_time, request_id, None, [0] * prompt_len)


class BatchedRequests:
    """Reference request.py:298-378, the two members the block manager touches."""

    def __init__(self, requests: Optional[List[Request]] = None):
        self.requests = list(requests) if requests else []

    def __len__(self) -> int:
        return len(self.requests)

    def add_request(self, request: Request) -> None:
        self.requests.append(request)

    def get_request_ids(self) -> List[int]:
        return [r.request_id for r in self.requests]

    def get_num_input_tokens(self) -> int:
        return sum(r.get_num_input_tokens() for r in self.requests)

    def pop_finished_requests(self) -> List[Request]:
        """Remove and return the finished requests (reference request.py:324-332)."""
        finished = [r for r in self.requests if r.is_finished]
        self.requests = [r for r in self.requests if not r.is_finished]
        return finished


class MigratingRequest:
    """Element of the bridge queue between the two instances (reference request.py:408-433):
    a request that finished prefill, whose blocks still sit in the context instance's pools."""

    def __init__(self, req: Request, block_indexes: List[int], context_parallel_config: ParallelConfig,
                 context_instance: int = 0):
        self.req = req
        self.block_indexes = block_indexes
        self.context_parallel_config = context_parallel_config
        # which context instance holds the blocks (not in the reference, which has one)
        self.context_instance = context_instance
