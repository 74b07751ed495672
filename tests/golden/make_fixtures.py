"""Writes the fixtures in this folder.  Run from the repository root: ``python tests/golden/make_fixtures.py``.

``readme_calculate_blocks.json`` is the worked example the reference documents for
``calculate_blocks`` (README.md:49-63 of the reference): inputs and the values the README states.
It is typed in from that text, not computed.

``small_problems.npz`` holds three small seeded problems (inputs as stored bit patterns, so they do
not depend on a random generator's implementation) and the output of the plain-C oracle
(``oracle/scalar.c``: double-precision arithmetic, stored as float32) for them.  The tests check the torch oracle, and on a GPU
the HIP path, against these stored values; they guard against silent changes of either oracle.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

README_EXAMPLE = {
    "source": "reference README.md:49-63",
    "cu_k_seqlens": [0, 32, 61, 100, 134, 157],
    "k_block_size": 16,
    "num_k_block": 12,
    "cu_num_k_block": [0, 2, 4, 7, 10, 12],
    "last_block_sizes": [16, 13, 7, 2, 7],
    "cu_q_seqlens": [0, 32, 64, 96, 128, 160],
    "q_block_size": 32,
    "num_q_block": 5,
}

PROBLEMS = [
    dict(seed=101, q_lens=[32] * 5, k_lens=[32, 29, 39, 34, 23], hq=8, hk=2, d=32, qbs=32, kbs=16, keep=0.7, diag=False,
         causal=True, scale=None),
    dict(seed=102, q_lens=[70, 33], k_lens=[50, 90], hq=4, hk=4, d=64, qbs=48, kbs=80, keep=0.5, diag=True, causal=False,
         scale=0.2),
    dict(seed=103, q_lens=[130], k_lens=[257], hq=2, hk=1, d=128, qbs=64, kbs=128, keep=0.6, diag=True, causal=True,
         scale=None),
]


def main():
    from hbsattn_amd.workloads import make_problem
    from oracle.scalar import hbsa_oracle_scalar

    with open(os.path.join(HERE, "readme_calculate_blocks.json"), "w") as f:
        json.dump(README_EXAMPLE, f, indent=1)
    arrays = {}
    for i, spec in enumerate(PROBLEMS):
        w = make_problem(device="cpu", dtype=torch.bfloat16, **spec)
        out = hbsa_oracle_scalar(w.q, w.k, w.v, w.cu_q, w.cu_k, w.block_mask, w.q_block_size, w.k_block_size, w.causal,
                                 w.softmax_scale)
        arrays[f"p{i}_spec"] = np.frombuffer(json.dumps(spec).encode(), dtype=np.uint8)
        for name in ("q", "k", "v"):
            arrays[f"p{i}_{name}_bf16_bits"] = getattr(w, name).view(torch.int16).numpy()
        arrays[f"p{i}_mask"] = w.block_mask.numpy()
        arrays[f"p{i}_out"] = out.numpy()
    np.savez_compressed(os.path.join(HERE, "small_problems.npz"), **arrays)
    print("wrote", sorted(os.listdir(HERE)))


if __name__ == "__main__":
    main()
