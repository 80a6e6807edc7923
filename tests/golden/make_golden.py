"""Writes tests/golden/migrate_golden.json: seeded cases with the SHA-256 of the expected
destination pools.

The reference has no golden vector for this path and its native op cannot be built or
imported, so these fixtures come from this repository's own oracle (the C restatement),
and test_oracle.py requires the independent torch formulation to reproduce every digest.
They freeze the oracle: a later edit that changes its results fails the suite.

Run from the repository root:  python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.dirname(HERE)):
    if p not in sys.path:
        sys.path.insert(0, p)

import oracle  # noqa: E402
from helpers import canary_pool, make_src_pools  # noqa: E402

# name, L, H, B, D, ctx_pp, ctx_tp, dec_pp, dec_tp, dec_pp_rank, dec_tp_rank, src_blocks, dst_blocks, n, seed
CASES = [
    ("cfg1-gpt2-small-1to1", 12, 12, 16, 64, 1, 1, 1, 1, 0, 0, 256, 512, 32, 1),
    ("tp2-to-tp1-merge-heads", 4, 8, 16, 32, 1, 2, 1, 1, 0, 0, 24, 40, 9, 3),
    ("tp2pp2-to-tp4-rank1-gqa", 8, 8, 16, 16, 2, 2, 1, 4, 0, 1, 16, 32, 7, 4),
    ("pp1-to-pp2-rank1-split-layers", 6, 4, 8, 16, 1, 1, 2, 1, 1, 0, 12, 12, 5, 6),
    ("tp4pp2-to-tp2pp4-rank3-1", 8, 8, 4, 8, 2, 4, 4, 2, 3, 1, 10, 14, 6, 7),
    ("tp1-to-tp4-rank2-split-heads", 2, 8, 16, 8, 1, 1, 1, 4, 0, 2, 8, 8, 8, 8),
]


def build_case(case: dict):
    g = oracle.Geom(case["L"], case["H"], case["B"], case["D"], 2, case["ctx_pp"], case["ctx_tp"],
                    case["dec_pp"], case["dec_tp"], case["dec_pp_rank"], case["dec_tp_rank"])
    src_k = make_src_pools(g, case["src_blocks"], seed=case["seed"])
    src_v = make_src_pools(g, case["src_blocks"], seed=case["seed"] + 500)
    gen = torch.Generator().manual_seed(case["seed"])
    ci = torch.randperm(case["src_blocks"], generator=gen)[:case["n"]].tolist()
    di = torch.randperm(case["dst_blocks"], generator=gen)[:case["n"]].tolist()
    return g, src_k, src_v, ci, di, case["dst_blocks"]


def _sha(t: torch.Tensor) -> str:
    return hashlib.sha256(oracle.bits(t.contiguous()).numpy().tobytes()).hexdigest()


def main() -> None:
    keys = ("name", "L", "H", "B", "D", "ctx_pp", "ctx_tp", "dec_pp", "dec_tp", "dec_pp_rank", "dec_tp_rank",
            "src_blocks", "dst_blocks", "n", "seed")
    out = []
    for row in CASES:
        case = dict(zip(keys, row))
        g, src_k, src_v, ci, di, nb_dst = build_case(case)
        for kind, src in (("k", src_k), ("v", src_v)):
            dst = canary_pool(g.dec_pool_shape(nb_dst))
            oracle.migrate_c(g, src, ci, di, dst)
            case["sha256_" + kind] = _sha(dst)
        case["ctx_idx"], case["dec_idx"] = ci, di
        out.append(case)
    path = os.path.join(HERE, "migrate_golden.json")
    with open(path, "w") as f:
        json.dump({"made_by": "tests/golden/make_golden.py (repository oracle, C restatement)",
                   "pool_fill": "helpers.make_src_pools: (torch.rand(seed)*2-1).half(); K seed s, V seed s+500",
                   "dst_fill": "fp16 bit pattern 0x7C01", "cases": out}, f, indent=1)
    print("wrote", path, len(out), "cases")


if __name__ == "__main__":
    main()
