"""Configuration objects of the KV movement path (reference ``distserve/config.py``).

Only what the path needs is kept: block size / swap space (``CacheConfig``), the rank
layout (``ParallelConfig``) and the model's KV geometry (``ModelConfig``).  The geometry is
given as numbers (or any object with HuggingFace-style attributes) instead of being
fetched with ``AutoConfig.from_pretrained`` (reference config.py:186-195), which needs a
network.
"""
from __future__ import annotations

from types import SimpleNamespace
from typing import List, Optional

import torch

from distserve_amd.utils import GB

_TORCH_DTYPE = {"fp16": torch.half, "fp32": torch.float32}
_DTYPE_BYTES = {"fp16": 2, "fp32": 4}

# KV geometry of the models the path is measured on:
# (hidden_size, num_attention_heads, num_hidden_layers, num_key_value_heads or None)
KNOWN_KV_SHAPES = {
    "gpt2": (768, 12, 12, None),
    "facebook/opt-125m": (768, 12, 12, None),
    "facebook/opt-13b": (5120, 40, 40, None),
    "meta-llama/Llama-2-7b-hf": (4096, 32, 32, 32),
    "meta-llama/Llama-2-70b-hf": (8192, 64, 80, 8),
}


class CacheConfig:
    """Block size and swap space (reference config.py:9-29; cpu_swap_space is given in GB)."""

    def __init__(self, block_size: int, max_num_blocks_per_req: int,
                 gpu_memory_utilization: float = 0.9, cpu_swap_space: int = 0):
        self.block_size = block_size
        self.max_num_blocks_per_req = max_num_blocks_per_req
        self.gpu_memory_utilization = gpu_memory_utilization
        self.cpu_swap_space = cpu_swap_space * GB


class ParallelConfig:
    """Sizes and this rank's coordinates (reference config.py:32-66)."""

    def __init__(self, tensor_parallel_size: int = 1, tensor_parallel_rank: int = 0,
                 pipeline_parallel_size: int = 1, pipeline_parallel_rank: int = 0) -> None:
        self.tensor_parallel_size = tensor_parallel_size
        self.tensor_parallel_rank = tensor_parallel_rank
        self.pipeline_parallel_size = pipeline_parallel_size
        self.pipeline_parallel_rank = pipeline_parallel_rank
        self.world_size = pipeline_parallel_size * tensor_parallel_size
        self.use_parallel = self.world_size > 1

    def to_list(self) -> List[int]:
        # order fixed by reference config.py:57-63; the native op unpacks it positionally
        return [self.tensor_parallel_size, self.tensor_parallel_rank,
                self.pipeline_parallel_size, self.pipeline_parallel_rank]

    def is_last_stage(self) -> bool:
        return self.pipeline_parallel_rank == self.pipeline_parallel_size - 1

    def __repr__(self) -> str:
        return (f"ParallelConfig(tp={self.tensor_parallel_rank}/{self.tensor_parallel_size}, "
                f"pp={self.pipeline_parallel_rank}/{self.pipeline_parallel_size})")


class DisaggParallelConfig:
    """The two instances' layouts (reference config.py:69-87)."""

    def __init__(self, context: ParallelConfig, decoding: ParallelConfig) -> None:
        self.context = context
        self.decoding = decoding

    def get_num_workers(self) -> int:
        return self.context.world_size + self.decoding.world_size


class ModelConfig:
    """KV geometry of a model (reference config.py:143-286, the getters the path uses).

    ``hf_config`` is any object with ``hidden_size``, ``num_attention_heads``,
    ``num_hidden_layers`` and optionally ``num_key_value_heads`` / ``n_head_kv`` /
    ``multi_query`` / ``model_type``; when omitted, ``model`` must be a key of
    ``KNOWN_KV_SHAPES``.
    """

    def __init__(self, model: str, tokenizer: Optional[str] = None, tokenizer_mode: str = "auto",
                 trust_remote_code: bool = False, dtype: str = "fp16", seed: int = 1,
                 use_dummy_weights: bool = False, hf_config=None):
        self.model = model
        self.tokenizer = tokenizer if tokenizer else model
        self.tokenizer_mode = tokenizer_mode
        self.trust_remote_code = trust_remote_code
        self.dtype = dtype
        self.seed = seed
        self.use_dummy_weights = use_dummy_weights
        if dtype not in _TORCH_DTYPE:
            raise AssertionError("dtype must be either 'fp16' or 'fp32'.")
        if hf_config is None:
            if model not in KNOWN_KV_SHAPES:
                raise ValueError(
                    f"Failed to load the model config, please check the model name or path: {model} "
                    f"(no network here: pass hf_config=... or use one of {sorted(KNOWN_KV_SHAPES)})")
            hidden, heads, layers, kv_heads = KNOWN_KV_SHAPES[model]
            hf_config = SimpleNamespace(hidden_size=hidden, num_attention_heads=heads,
                                        num_hidden_layers=layers, model_type=model)
            if kv_heads is not None:
                hf_config.num_key_value_heads = kv_heads
        self.hf_config = hf_config

    @classmethod
    def from_kv_shape(cls, num_layers: int, num_heads: int, head_dim: int,
                      num_kv_heads: Optional[int] = None, dtype: str = "fp16", name: str = "synthetic"):
        cfg = SimpleNamespace(hidden_size=num_heads * head_dim, num_attention_heads=num_heads,
                              num_hidden_layers=num_layers, model_type=name)
        if num_kv_heads is not None:
            cfg.num_key_value_heads = num_kv_heads
        return cls(name, dtype=dtype, hf_config=cfg)

    def get_dtype_size(self) -> int:
        return _DTYPE_BYTES[self.dtype]

    def get_torch_dtype(self) -> torch.dtype:
        return _TORCH_DTYPE[self.dtype]

    def get_hidden_size(self) -> int:
        return self.hf_config.hidden_size

    def get_head_size(self) -> int:
        return self.hf_config.hidden_size // self.hf_config.num_attention_heads

    def get_num_heads(self, parallel_config: ParallelConfig = ParallelConfig()) -> int:
        """KV heads held by one tensor rank (reference config.py:225-257)."""
        tp = parallel_config.tensor_parallel_size
        cfg = self.hf_config
        new_arch_falcon = getattr(cfg, "model_type", None) == "falcon" and \
            getattr(cfg, "new_decoder_architecture", False)
        if not new_arch_falcon and getattr(cfg, "multi_query", False):
            return 1  # multi-query attention: a single KV head, replicated
        if getattr(cfg, "n_head_kv", None) is not None:
            return cfg.n_head_kv // tp
        if getattr(cfg, "num_key_value_heads", None) is not None:
            return cfg.num_key_value_heads // tp
        total = cfg.num_attention_heads
        assert total % tp == 0, (
            f"Total number of attention heads ({total}) must be divisible by the size of "
            f"tensor parallel group ({tp}).")
        return total // tp

    def kv_heads_replicated(self, parallel_config: ParallelConfig = ParallelConfig()) -> bool:
        """True when every tensor rank holds a copy of the same KV head instead of a slice of
        them: a multi-query model under tensor parallelism (reference config.py:233-237
        returns 1 head per rank whatever the tensor-parallel size)."""
        tp = parallel_config.tensor_parallel_size
        return tp > 1 and self.get_num_heads(parallel_config) * tp != self.get_num_heads()

    def check_kv_heads_are_split(self, parallel_config: ParallelConfig) -> None:
        """The migration re-slices KV heads between tensor ranks that each own a contiguous
        slice ``[t*H/T, (t+1)*H/T)``.  Replicated heads have no such slice: which copy a
        decoding rank should read is a choice the reference's native op makes and its sources
        do not show, so that layout is refused here instead of guessed."""
        if self.kv_heads_replicated(parallel_config):
            raise ValueError(
                f"model {self.model!r} keeps {self.get_num_heads()} KV head(s) replicated on each of "
                f"{parallel_config.tensor_parallel_size} tensor ranks (multi-query attention); KV migration "
                "between instances needs KV heads that are split over the tensor ranks")

    def get_num_layers(self, parallel_config: ParallelConfig = ParallelConfig()) -> int:
        """Layers held by one pipeline rank (reference config.py:279-286)."""
        total = self.hf_config.num_hidden_layers
        pp = parallel_config.pipeline_parallel_size
        assert total % pp == 0, (
            f"Number of layers ({total}) must be divisible by the size of pipeline parallel group ({pp}).")
        return total // pp
