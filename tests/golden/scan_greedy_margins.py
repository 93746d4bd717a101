"""Find seeds of the 4-layer ``longrun`` synthetic model whose 64-token greedy stream never
passes a thin decision: the CPU float32 step oracle alone (no GPU, nothing of the library but
the seeded model recipe and its bit-exact CPU encoder), one stream per seed, the smallest
top-1 / top-2 logit gap over the 64 picks in units of one bf16 step of the top logit.

    python tests/golden/scan_greedy_margins.py [first_seed] [n_seeds] [workers]

writes ``tests/golden/greedy_margin_seeds.json``: the streams with the widest smallest gap,
their ids and their gaps.  A GPU path whose logits are within a fraction of that gap of the
oracle's at every pick must reproduce such a stream exactly; ``tests/test_decodev2.py`` asserts
that for the seeds listed there.
"""

from __future__ import annotations

import json
import os
import sys
from concurrent.futures import ProcessPoolExecutor

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

PROMPT = [11, 200, 37, 1999, 5, 640, 3, 77]
N_NEW = 64
KEEP = 24


def longrun_spec():
    from deepfold_amd import decodev2 as dv2

    return dv2.ArchSpec("longrun", "llama_swiglu", 4, 512, 8, 2, 64, 1536, 2048, 128, qkv_bias=False)


def cpu_encode(w):
    from oracle import nf4_oracle as oc

    return oc.c_encode(np.ascontiguousarray(w, dtype=np.float32))


def one(seed: int):
    from deepfold_amd.decodev2.synth import build
    from oracle import step_oracle as so

    model = build(longrun_spec(), seed, encode=cpu_encode)
    ids, margins, tops = so.greedy_ids(model, PROMPT, N_NEW, ignore_eos=True, return_margins=True,
                                      return_tops=True)
    steps = [m / 2.0 ** (np.floor(np.log2(max(abs(t), 1e-30))) - 7) for m, t in zip(margins, tops)]
    return {"seed": seed, "min_gap_bf16_steps": float(min(steps)), "min_gap": float(min(margins)),
            "ids": ids}


def main() -> None:
    first = int(sys.argv[1]) if len(sys.argv) > 1 else 0
    count = int(sys.argv[2]) if len(sys.argv) > 2 else 2000
    workers = int(sys.argv[3]) if len(sys.argv) > 3 else 6
    with ProcessPoolExecutor(workers) as pool:
        rows = list(pool.map(one, range(first, first + count), chunksize=8))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "greedy_margin_seeds.json")
    scanned = [[first, first + count]]
    if os.path.exists(path):  # a further range: keep the best of both
        with open(path) as f:
            old = json.load(f)
        seen = {r["seed"] for r in rows}
        rows += [r for r in old["streams"] if r["seed"] not in seen]
        scanned = old["seeds_scanned"] + scanned
    rows.sort(key=lambda r: -r["min_gap_bf16_steps"])
    out = {"spec": "longrun (4 layers, hidden 512, 8 query / 2 kv heads of 64, ffn 1536, vocab 2048)",
           "prompt": PROMPT, "n_new": N_NEW, "seeds_scanned": scanned,
           "streams": rows[:KEEP]}
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("widest smallest gaps (bf16 steps):", [round(r["min_gap_bf16_steps"], 2) for r in rows[:KEEP]])


if __name__ == "__main__":
    main()
