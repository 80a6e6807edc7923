"""distserve_amd -- MI355X-native KV-block migration and swap behind DistServe's worker API.

Importing the package loads the HIP library (``lib/libkvmove.so``) and the torch op shim
(``lib/libkvmove_torch.so``), which registers ``torch.ops.block_migration_ops.*`` and
``torch.ops.swapping_ops.swap`` exactly as DistServe's worker looks them up
(reference ``distserve/__init__.py:4-16`` loads SwiftTransformer's ``libst_pybinding.so``
the same way).  There is no CPU fallback: a missing library is an error here, and every
op refuses tensors that are not on the GPU.
"""
import os

import torch

_LIB_DIR = os.environ.get("KVMOVE_LIB_DIR") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")
KVMOVE_LIB_PATH = os.path.join(_LIB_DIR, "libkvmove.so")
TORCH_LIB_PATH = os.path.join(_LIB_DIR, "libkvmove_torch.so")

for _path in (KVMOVE_LIB_PATH, TORCH_LIB_PATH):
    if not os.path.exists(_path):
        raise RuntimeError(
            f"Could not find {os.path.basename(_path)} at {_path}. "
            "Build it first with `python distserve_amd/csrc/build.py` (hipcc, gfx950)."
        )

torch.ops.load_library(TORCH_LIB_PATH)

from distserve_amd import cabi  # noqa: E402
from distserve_amd.block_manager import BlockLocation, BlockManager  # noqa: E402
from distserve_amd.config import CacheConfig, DisaggParallelConfig, ModelConfig, ParallelConfig  # noqa: E402
from distserve_amd.request import MigratingRequest, Request, create_request  # noqa: E402
from distserve_amd.worker import ParaWorker, Worker  # noqa: E402
from distserve_amd.handoff import ContextStageLLMEngine, DecodingStageLLMEngine  # noqa: E402
from distserve_amd.context_stage_scheduler import (  # noqa: E402
    ContextStageFCFSScheduler, ContextStageSchedConfig, get_context_stage_scheduler)
from distserve_amd.decoding_stage_scheduler import (  # noqa: E402
    DecodingStageFCFSScheduler, DecodingStageSchedConfig, get_decoding_stage_scheduler)

__all__ = [
    "cabi", "BlockLocation", "BlockManager", "CacheConfig", "DisaggParallelConfig", "ModelConfig",
    "ParallelConfig", "MigratingRequest", "Request", "create_request", "ParaWorker", "Worker",
    "ContextStageLLMEngine", "DecodingStageLLMEngine", "DecodingStageFCFSScheduler",
    "DecodingStageSchedConfig", "get_decoding_stage_scheduler", "ContextStageFCFSScheduler",
    "ContextStageSchedConfig", "get_context_stage_scheduler",
]
