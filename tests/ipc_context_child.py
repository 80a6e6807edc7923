"""A context (prefill) instance in a process of its own, for tests/test_ipc_gpu.py.

Started with ``subprocess`` as a fresh interpreter; talks JSON lines over stdin/stdout.
First line in: ``{"layers", "kv_heads", "head_dim", "tp", "pp", "blocks", "seed", "prompts",
"busy_blocks"}``.  It builds a ``ContextStageLLMEngine`` of that layout on the GPU, fills
every worker's pools from the seed (values made on the CPU, so that the other process can
remake them without a copy), allocates blocks for the prompts and answers with its pid, the
memory handles ``[pp][tp] = (k, v)`` and the block tables.  Commands afterwards:

``{"cmd": "verify"}``             are the pools still what the seed says?  -> ``{"unchanged": bool}``
``{"cmd": "release", "id": n}``   free request n's blocks                   -> ``{"released": n}``
``{"cmd": "big_handle"}``         handle of a pool in an allocation of 2 GiB and more -> ``{"handle": [...]}``
``{"cmd": "reallocate", "seed": s}``  free every pool, hand the memory back to the runtime, allocate the pools
                                  again filled from seed s -> ``{"handles": ..., "tables": ...}``
``{"cmd": "exit"}``
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def pool_seed(seed: int, worker_index: int, is_v: bool) -> int:
    return seed + 10 * worker_index + (500 if is_v else 0)


def main() -> None:
    spec = json.loads(sys.stdin.readline())
    import torch

    from distserve_amd import (CacheConfig, ContextStageLLMEngine, ModelConfig, ParallelConfig, create_request,
                               workloads)

    torch.cuda.set_device(0)
    model = ModelConfig.from_kv_shape(num_layers=spec["layers"], num_heads=spec["kv_heads"],
                                      head_dim=spec["head_dim"], num_kv_heads=spec["kv_heads"])
    cache = CacheConfig(16, 64)
    ctx = ContextStageLLMEngine(model, ParallelConfig(spec["tp"], 0, spec["pp"], 0), cache)
    ctx._init_kvcache(spec["blocks"], 0)
    workers = [w for row in ctx.workers for w in row]
    for i, w in enumerate(workers):
        w.k_cache.copy_(workloads.fill_uniform(w.k_cache.shape, pool_seed(spec["seed"], i, False)))
        w.v_cache.copy_(workloads.fill_uniform(w.v_cache.shape, pool_seed(spec["seed"], i, True)))
    torch.cuda.synchronize()
    if spec.get("busy_blocks"):
        ctx.block_manager.allocate_blocks(create_request(16 * spec["busy_blocks"], 9000))
    tables = {}
    for rid, prompt_len in enumerate(spec["prompts"]):
        req = create_request(prompt_len, rid)
        ctx.block_manager.allocate_blocks(req)
        tables[rid] = list(ctx.block_manager.get_block_table(rid))
    print(json.dumps({"pid": os.getpid(), "handles": ctx.kv_cache_mem_handles, "tables": tables,
                      "pool_bytes": workers[0].k_cache.numel() * 2}), flush=True)

    big = None
    for line in sys.stdin:
        msg = json.loads(line)
        if msg["cmd"] == "verify":
            ok = True
            for i, w in enumerate(workers):
                want_k = workloads.fill_uniform(w.k_cache.shape, pool_seed(spec["seed"], i, False))
                want_v = workloads.fill_uniform(w.v_cache.shape, pool_seed(spec["seed"], i, True))
                ok = ok and torch.equal(w.k_cache.cpu().view(torch.int16), want_k.view(torch.int16))
                ok = ok and torch.equal(w.v_cache.cpu().view(torch.int16), want_v.view(torch.int16))
            print(json.dumps({"unchanged": bool(ok)}), flush=True)
        elif msg["cmd"] == "release":
            ctx._free_request_resources(msg["id"])
            print(json.dumps({"released": msg["id"],
                              "free_blocks": len(ctx.block_manager.free_gpu_blocks_list)}), flush=True)
        elif msg["cmd"] == "big_handle":
            # one allocation of a little over 2 GiB; the pool named is a small piece in its middle
            big = torch.empty((2 << 30) + (4 << 20), dtype=torch.uint8, device="cuda")
            piece = big[1 << 30:(1 << 30) + (1 << 20)]
            print(json.dumps({"handle": torch.ops.block_migration_ops.get_ipc_mem_handle(piece)}), flush=True)
        elif msg["cmd"] == "reallocate":
            for w in workers:
                w.k_cache = w.v_cache = w.k_swap = w.v_swap = None
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
            spec["seed"] = msg["seed"]
            ctx._init_kvcache(spec["blocks"], 0)
            for i, w in enumerate(workers):
                w.k_cache.copy_(workloads.fill_uniform(w.k_cache.shape, pool_seed(spec["seed"], i, False)))
                w.v_cache.copy_(workloads.fill_uniform(w.v_cache.shape, pool_seed(spec["seed"], i, True)))
            torch.cuda.synchronize()
            tables = {}
            for rid, prompt_len in enumerate(spec["prompts"]):
                ctx.block_manager.allocate_blocks(create_request(prompt_len, rid))
                tables[rid] = list(ctx.block_manager.get_block_table(rid))
            print(json.dumps({"handles": ctx.kv_cache_mem_handles, "tables": tables}), flush=True)
        elif msg["cmd"] == "exit":
            break
    del big


if __name__ == "__main__":
    main()
