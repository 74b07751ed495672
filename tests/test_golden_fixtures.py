"""The committed fixtures of tests/golden (written by tests/golden/make_fixtures.py).

``readme_calculate_blocks.json`` is the worked example the reference's README prints (a vector the
reference itself holds).  ``small_problems.npz`` is NOT a reference-held vector: its outputs were written
by this repository's own C oracle (``oracle/scalar.c``), so it is a drift guard for the oracle and the
kernels, and pins nothing independently; what pins the oracle is in tests/test_oracle_*.py."""
import json
import os

import numpy as np
import pytest
import torch

from hbsattn_amd.utils import calculate_blocks
from oracle.dense import calculate_blocks_oracle, hbsa_oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _problems():
    z = np.load(os.path.join(GOLDEN, "small_problems.npz"))
    i = 0
    while f"p{i}_spec" in z:
        spec = json.loads(bytes(z[f"p{i}_spec"]).decode())
        q, k, v = (torch.from_numpy(z[f"p{i}_{n}_bf16_bits"].copy()).view(torch.bfloat16) for n in "qkv")
        yield spec, q, k, v, torch.from_numpy(z[f"p{i}_mask"].copy()), torch.from_numpy(z[f"p{i}_out"].copy())
        i += 1


def _cu(lens):
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    return cu


def test_readme_example_of_calculate_blocks():
    ex = json.load(open(os.path.join(GOLDEN, "readme_calculate_blocks.json")))
    for fn in (calculate_blocks_oracle, lambda cu, bs: calculate_blocks(torch.tensor(cu, dtype=torch.int32), bs)):
        nb, cu_block, _, cu_nb = fn(ex["cu_k_seqlens"], ex["k_block_size"])
        cu_block, cu_nb = [int(x) for x in cu_block], [int(x) for x in cu_nb]
        assert nb == ex["num_k_block"] and cu_nb == ex["cu_num_k_block"]
        assert [cu_block[e] - cu_block[e - 1] for e in cu_nb[1:]] == ex["last_block_sizes"]
        assert fn(ex["cu_q_seqlens"], ex["q_block_size"])[0] == ex["num_q_block"]


def test_torch_oracle_reproduces_the_stored_outputs():
    n = 0
    for spec, q, k, v, mask, expect in _problems():
        out = hbsa_oracle(q, k, v, _cu(spec["q_lens"]), _cu(spec["k_lens"]), mask, spec["qbs"], spec["kbs"], spec["causal"],
                          spec["scale"])
        assert torch.allclose(out, expect, atol=2e-6, rtol=1e-5)
        n += 1
    assert n == 3


@pytest.mark.gpu
def test_hip_path_reproduces_the_stored_outputs():
    from hbsattn_amd import HBSAttention
    from tests.helpers import assert_close_to_oracle
    for spec, q, k, v, mask, expect in _problems():
        cu_q = torch.tensor(_cu(spec["q_lens"]), dtype=torch.int32, device="cuda")
        cu_k = torch.tensor(_cu(spec["k_lens"]), dtype=torch.int32, device="cuda")
        out = HBSAttention(q.cuda(), k.cuda(), v.cuda(), cu_q, cu_k, mask.cuda(), spec["qbs"], spec["kbs"], spec["causal"],
                           spec["scale"])
        assert_close_to_oracle(out, expect, f"fixture seed {spec['seed']}")
