"""Slice arithmetic of the model and parallel configurations (reference distserve/config.py:32-66,
197-286): which layers and KV heads a rank holds, and the layouts the migration refuses."""
from types import SimpleNamespace

import pytest

from distserve_amd.config import ModelConfig, ParallelConfig
from distserve_amd.worker import Worker
from distserve_amd.utils import Stage
from distserve_amd.config import CacheConfig


def model(**hf):
    base = dict(hidden_size=4096, num_attention_heads=32, num_hidden_layers=32, model_type="synthetic")
    base.update(hf)
    return ModelConfig("synthetic", hf_config=SimpleNamespace(**base))


def test_heads_and_layers_per_rank_follow_the_reference_getters():
    m = model()
    assert m.get_num_heads() == 32 and m.get_num_heads(ParallelConfig(4, 1, 1, 0)) == 8
    assert m.get_num_layers(ParallelConfig(1, 0, 4, 2)) == 8 and m.get_head_size() == 128
    gqa = model(num_key_value_heads=8, num_attention_heads=64, hidden_size=8192)
    assert gqa.get_num_heads() == 8 and gqa.get_num_heads(ParallelConfig(4, 0, 1, 0)) == 2
    falcon = model(n_head_kv=8)
    assert falcon.get_num_heads(ParallelConfig(2, 0, 1, 0)) == 4
    assert ParallelConfig(2, 1, 4, 3).to_list() == [2, 1, 4, 3]          # [tp_size, tp_rank, pp_size, pp_rank]
    with pytest.raises(AssertionError, match="divisible"):
        model(num_attention_heads=30, hidden_size=3840).get_num_heads(ParallelConfig(4, 0, 1, 0))


def test_multi_query_heads_are_replicated_under_tensor_parallelism_and_refused():
    """A multi-query model keeps its single KV head on every tensor rank (reference
    config.py:233-237 returns 1 whatever the tensor-parallel size): there is no slice to
    re-slice, and a worker for such a layout is refused before it touches the GPU."""
    mqa = model(multi_query=True)
    tp2 = ParallelConfig(2, 1, 1, 0)
    assert mqa.get_num_heads() == 1 and mqa.get_num_heads(tp2) == 1
    assert mqa.kv_heads_replicated(tp2) and not mqa.kv_heads_replicated(ParallelConfig())
    mqa.check_kv_heads_are_split(ParallelConfig())                          # one rank: nothing is replicated
    with pytest.raises(ValueError, match="replicated on each of 2 tensor ranks"):
        mqa.check_kv_heads_are_split(tp2)
    with pytest.raises(ValueError, match="multi-query"):
        Worker(0, Stage.DECODING, mqa, CacheConfig(16, 64), tp2)
    # models whose heads split evenly are never flagged; new-architecture Falcon ignores the flag
    assert not model().kv_heads_replicated(ParallelConfig(8, 3, 1, 0))
    assert not model(num_key_value_heads=8).kv_heads_replicated(ParallelConfig(4, 0, 2, 1))
    new_falcon = model(multi_query=True, model_type="falcon", new_decoder_architecture=True, n_head_kv=8)
    assert new_falcon.get_num_heads(tp2) == 4 and not new_falcon.kv_heads_replicated(tp2)
