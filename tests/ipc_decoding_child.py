"""A decoding instance in a process of its own, for tests/test_ipc_gpu.py.

Started with ``subprocess`` as a fresh interpreter; talks JSON lines over stdin/stdout.
First line in: ``{"layers", "kv_heads", "head_dim", "tp", "blocks", "busy_prompt", "ctx_tp",
"ctx_pp", "handles", "requests": [[request_id, prompt_len, context_block_table], ...]}``.  It
builds a ``DecodingStageLLMEngine`` of ``tp`` ranks on the GPU with canary-filled pools, binds
the memory handles (made by some other process), pulls every request, and answers with its
pid, the decoding block tables, how many foreign allocations it holds open, and the SHA-256
of every rank's K and V pool.  ``{"cmd": "exit"}`` ends it (after ``kvm_reset``).
"""
import hashlib
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main() -> None:
    spec = json.loads(sys.stdin.readline())
    import torch

    from distserve_amd import (CacheConfig, DecodingStageLLMEngine, MigratingRequest, ModelConfig, ParallelConfig,
                               cabi, create_request)

    torch.cuda.set_device(0)
    model = ModelConfig.from_kv_shape(num_layers=spec["layers"], num_heads=spec["kv_heads"],
                                      head_dim=spec["head_dim"], num_kv_heads=spec["kv_heads"])
    cache = CacheConfig(16, 64)
    dec = DecodingStageLLMEngine(model, ParallelConfig(spec["tp"], 0, 1, 0), cache)
    dec._init_kvcache(spec["blocks"], 0)
    if spec.get("busy_prompt"):
        dec.block_manager.allocate_blocks(create_request(spec["busy_prompt"], 9000))
    for w in dec.workers[0]:
        w.k_cache.view(torch.int16).fill_(0x7C01)
        w.v_cache.view(torch.int16).fill_(0x7C01)
    ctx_config = ParallelConfig(spec["ctx_tp"], 0, spec["ctx_pp"], 0)
    dec.register_kvcache_mem_handles(ctx_config, spec["handles"])
    opened = cabi.opened_handles()
    tables = {}
    for rid, prompt_len, ctx_table in spec["requests"]:
        req = create_request(prompt_len, rid)
        req.add_generated_token("x", 1)
        dec._migrate_blocks(MigratingRequest(req, ctx_table, ctx_config))
        tables[rid] = list(dec.block_manager.get_block_table(rid))
    torch.cuda.synchronize()
    digests = [[hashlib.sha256(t.cpu().view(torch.uint8).numpy().tobytes()).hexdigest()
                for t in (w.k_cache, w.v_cache)] for w in dec.workers[0]]
    print(json.dumps({"pid": os.getpid(), "tables": tables, "opened": opened, "digests": digests}), flush=True)
    for line in sys.stdin:
        if json.loads(line)["cmd"] == "exit":
            break
    cabi.reset()
    print(json.dumps({"opened_after_reset": cabi.opened_handles()}), flush=True)


if __name__ == "__main__":
    main()
