"""The two oracle restatements (torch-vectorised, C scalar) agree on the reference's own
test geometry (reference test/test_accuracy.py:17-38: batch 5, equal or mismatched k
lengths, block sizes 16/32/80 x 16/32, GQA 2:2 and 8:2, head dims 16/18) with seeded inputs."""
import itertools

import pytest
import torch

from oracle.dense import calculate_blocks_oracle, hbsa_oracle, visited_block_pairs
from oracle.scalar import hbsa_oracle_scalar

CU_Q = [0, 32, 64, 96, 128, 160]
CU_K_SAME = [0, 32, 64, 96, 128, 160]
CU_K_DIFF = [0, 32, 61, 100, 134, 157]

GRID = list(itertools.product([False, True], [(2, 2), (8, 2)], [None, 0.333], [16, 32, 80], [16, 32], [True, False], [16, 18]))


@pytest.mark.parametrize("causal,heads,scale,qbs,kbs,same,d", GRID)
def test_dense_equals_scalar_on_reference_grid(causal, heads, scale, qbs, kbs, same, d):
    hq, hk = heads
    cu_k = CU_K_SAME if same else CU_K_DIFF
    g = torch.Generator().manual_seed(hash((causal, hq, qbs, kbs, same, d)) % (2 ** 31))
    q = torch.randn(CU_Q[-1], hq, d, generator=g)
    k = torch.randn(cu_k[-1], hk, d, generator=g)
    v = torch.randn(cu_k[-1], hk, d, generator=g)
    nq, nk = calculate_blocks_oracle(CU_Q, qbs)[0], calculate_blocks_oracle(cu_k, kbs)[0]
    mask = torch.rand(hk, nq, nk, generator=g) < 0.7
    a = hbsa_oracle(q, k, v, CU_Q, cu_k, mask, qbs, kbs, causal, scale)
    b = hbsa_oracle_scalar(q, k, v, CU_Q, cu_k, mask, qbs, kbs, causal, scale)
    assert torch.isfinite(a).all() and torch.isfinite(b).all()
    torch.testing.assert_close(a, b, atol=2e-5, rtol=1e-4)
    a64 = hbsa_oracle(q, k, v, CU_Q, cu_k, mask, qbs, kbs, causal, scale, compute_dtype=torch.float64)
    torch.testing.assert_close(a64.float(), b, atol=2e-6, rtol=1e-5)


def test_scalar_row_range():
    g = torch.Generator().manual_seed(3)
    q, k, v = torch.randn(160, 2, 16, generator=g), torch.randn(157, 2, 16, generator=g), torch.randn(157, 2, 16, generator=g)
    mask = torch.rand(2, 5, 12, generator=g) < 0.7
    full = hbsa_oracle_scalar(q, k, v, CU_Q, CU_K_DIFF, mask, 32, 16, True, None)
    part = hbsa_oracle_scalar(q, k, v, CU_Q, CU_K_DIFF, mask, 32, 16, True, None, row_range=(40, 70))
    assert torch.equal(part[40:70], full[40:70]) and torch.isnan(part[:40]).all() and torch.isnan(part[70:]).all()


def test_scalar_rejects_wrong_mask_shape():
    q = torch.randn(32, 1, 8)
    with pytest.raises(ValueError):
        hbsa_oracle_scalar(q, q, q, [0, 32], [0, 32], torch.ones(1, 1, 1, dtype=torch.bool), 16, 16, False, None)


def test_visited_pairs_small_known_answer():
    # one sequence, 3x3 blocks of 16, all kept, causal with equal lengths: 6 visited pairs,
    # 3 diagonal blocks (136 visible elements each) + 3 full blocks (256)
    mask = torch.ones(1, 3, 3, dtype=torch.bool)
    blk, exact = visited_block_pairs([0, 48], [0, 48], mask, 16, 16, True)
    assert blk == 6 * 256 and exact == 3 * 136 + 3 * 256
    blk, exact = visited_block_pairs([0, 48], [0, 48], mask, 16, 16, False)
    assert blk == exact == 9 * 256
