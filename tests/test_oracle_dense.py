"""Pins the attention oracles against library routines and invariants.

Each check is chosen so that a plausible mistake fails it: a transposed mask, a wrong
causal alignment sign, head mapping ``h % ratio`` instead of ``h // ratio``, a missing
scale, global instead of per-sequence block indices, NaN rows instead of zeros.
Both restatements (``oracle.dense`` and the C ``oracle.scalar``) run every check.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle.dense import calculate_blocks_oracle, hbsa_oracle
from oracle.scalar import hbsa_oracle_scalar

ORACLES = [pytest.param(hbsa_oracle, id="dense"), pytest.param(hbsa_oracle_scalar, id="scalar")]
TOL = dict(atol=2e-5, rtol=1e-4)


def _rand(seed, *shape):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def _full_mask(hk, cu_q, cu_k, qbs, kbs):
    nq = calculate_blocks_oracle(cu_q, qbs)[0]
    nk = calculate_blocks_oracle(cu_k, kbs)[0]
    return torch.ones(hk, nq, nk, dtype=torch.bool)


def _sdpa(q, k, v, mask=None, causal=False, scale=None):
    # q [Lq,H,D] -> [1,H,Lq,D]
    o = F.scaled_dot_product_attention(q.permute(1, 0, 2)[None], k.permute(1, 0, 2)[None], v.permute(1, 0, 2)[None],
                                       attn_mask=mask, is_causal=causal, scale=scale)
    return o[0].permute(1, 0, 2)


@pytest.mark.parametrize("oracle", ORACLES)
@pytest.mark.parametrize("scale", [None, 0.333])
def test_all_true_mask_noncausal_is_sdpa(oracle, scale):
    q, k, v = _rand(1, 70, 3, 24), _rand(2, 101, 3, 24), _rand(3, 101, 3, 24)
    cu_q, cu_k = [0, 70], [0, 101]
    out = oracle(q, k, v, cu_q, cu_k, _full_mask(3, cu_q, cu_k, 32, 16), 32, 16, False, scale)
    torch.testing.assert_close(out, _sdpa(q, k, v, scale=scale), **TOL)


@pytest.mark.parametrize("oracle", ORACLES)
def test_all_true_mask_causal_equal_lengths_is_sdpa_causal(oracle):
    q, k, v = _rand(4, 90, 2, 16), _rand(5, 90, 2, 16), _rand(6, 90, 2, 16)
    cu = [0, 90]
    out = oracle(q, k, v, cu, cu, _full_mask(2, cu, cu, 48, 32), 48, 32, True, None)
    torch.testing.assert_close(out, _sdpa(q, k, v, causal=True), **TOL)


@pytest.mark.parametrize("oracle", ORACLES)
@pytest.mark.parametrize("lq,lk", [(40, 75), (75, 40)])
def test_bottom_right_alignment_matches_explicit_tril(oracle, lq, lk):
    q, k, v = _rand(7, lq, 2, 16), _rand(8, lk, 2, 16), _rand(9, lk, 2, 16)
    cu_q, cu_k = [0, lq], [0, lk]
    out = oracle(q, k, v, cu_q, cu_k, _full_mask(2, cu_q, cu_k, 16, 16), 16, 16, True, None)
    vis = torch.tril(torch.ones(lq, lk, dtype=torch.bool), diagonal=lk - lq)
    ref = _sdpa(q, k, v, mask=vis)
    empty = ~vis.any(dim=1)                       # rows with no visible key (lq > lk)
    ref[empty] = 0.0
    assert empty.sum().item() == max(0, lq - lk)
    assert (out[empty] == 0).all(), "rows with no visible key must be exactly 0"
    torch.testing.assert_close(out, ref, **TOL)


@pytest.mark.parametrize("oracle", ORACLES)
def test_gqa_equals_mha_on_repeated_kv(oracle):
    hq, hk, ratio = 6, 2, 3
    q, k, v = _rand(10, 64, hq, 16), _rand(11, 64, hk, 16), _rand(12, 64, hk, 16)
    cu = [0, 30, 64]
    g = torch.Generator().manual_seed(13)
    nq, nk = calculate_blocks_oracle(cu, 16)[0], calculate_blocks_oracle(cu, 32)[0]
    mask = torch.rand(hk, nq, nk, generator=g) < 0.6
    out = oracle(q, k, v, cu, cu, mask, 16, 32, True, None)
    # q head h uses kv head h // ratio: repeat_interleave, not tile
    out_mha = oracle(q, k.repeat_interleave(ratio, 1), v.repeat_interleave(ratio, 1), cu, cu,
                     mask.repeat_interleave(ratio, 0), 16, 32, True, None)
    torch.testing.assert_close(out, out_mha, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("oracle", ORACLES)
def test_block_mask_vs_element_mask_sdpa(oracle):
    """One sequence, random block mask: expand the block mask by hand (rows = q blocks,
    columns = k blocks) and compare with SDPA under that element mask."""
    lq, lk, qbs, kbs = 50, 77, 16, 32
    q, k, v = _rand(14, lq, 1, 8), _rand(15, lk, 1, 8), _rand(16, lk, 1, 8)
    mask = torch.tensor([[[1, 0, 1], [0, 1, 1], [1, 1, 0], [0, 0, 1]]], dtype=torch.bool)   # 4 q blocks x 3 k blocks
    out = oracle(q, k, v, [0, lq], [0, lk], mask, qbs, kbs, False, 0.5)
    elem = torch.zeros(lq, lk, dtype=torch.bool)
    for i in range(lq):
        for j in range(lk):
            elem[i, j] = mask[0, i // qbs, j // kbs]
    torch.testing.assert_close(out, _sdpa(q, k, v, mask=elem, scale=0.5), **TOL)


@pytest.mark.parametrize("oracle", ORACLES)
def test_packed_batch_equals_per_sequence_calls_and_ignores_cross_sequence_bits(oracle):
    cu_q, cu_k = [0, 32, 64, 96, 128, 160], [0, 32, 61, 100, 134, 157]
    hq, hk, d, qbs, kbs = 4, 2, 16, 32, 16
    q, k, v = _rand(17, 160, hq, d), _rand(18, 157, hk, d), _rand(19, 157, hk, d)
    g = torch.Generator().manual_seed(20)
    mask = torch.rand(hk, 5, 12, generator=g) < 0.7
    out = oracle(q, k, v, cu_q, cu_k, mask, qbs, kbs, True, None)
    _, _, _, cu_nqb = calculate_blocks_oracle(cu_q, qbs)
    _, _, _, cu_nkb = calculate_blocks_oracle(cu_k, kbs)
    for b in range(5):
        sub = mask[:, cu_nqb[b]:cu_nqb[b + 1], cu_nkb[b]:cu_nkb[b + 1]]
        o_b = oracle(q[cu_q[b]:cu_q[b + 1]], k[cu_k[b]:cu_k[b + 1]], v[cu_k[b]:cu_k[b + 1]],
                     [0, cu_q[b + 1] - cu_q[b]], [0, cu_k[b + 1] - cu_k[b]], sub, qbs, kbs, True, None)
        torch.testing.assert_close(out[cu_q[b]:cu_q[b + 1]], o_b, atol=1e-6, rtol=1e-6)
    # flipping every mask entry that pairs blocks of different sequences changes nothing
    flipped = mask.clone()
    for bq in range(5):
        for bk in range(5):
            if bq != bk:
                blk = flipped[:, cu_nqb[bq]:cu_nqb[bq + 1], cu_nkb[bk]:cu_nkb[bk + 1]]
                flipped[:, cu_nqb[bq]:cu_nqb[bq + 1], cu_nkb[bk]:cu_nkb[bk + 1]] = ~blk
    assert torch.equal(oracle(q, k, v, cu_q, cu_k, flipped, qbs, kbs, True, None), out)
    # rows with no visible key: sequence 1 (k 29 < q 32) rows 0..2, sequence 4 (k 23) rows 0..8
    assert (out[32:35] == 0).all() and (out[128:137] == 0).all()
    assert torch.isfinite(out).all()


@pytest.mark.parametrize("oracle", ORACLES)
def test_mask_refinement_and_default_scale(oracle):
    """Splitting every 32-row q block into two 16-row blocks with duplicated mask rows is
    the same problem; ``softmax_scale=None`` means headdim**-0.5."""
    cu = [0, 64, 160]
    q, k, v = _rand(21, 160, 2, 32), _rand(22, 160, 2, 32), _rand(23, 160, 2, 32)
    g = torch.Generator().manual_seed(24)
    mask = torch.rand(2, 5, 10, generator=g) < 0.5
    a = oracle(q, k, v, cu, cu, mask, 32, 16, True, None)
    b = oracle(q, k, v, cu, cu, mask.repeat_interleave(2, 1), 16, 16, True, 32 ** -0.5)
    torch.testing.assert_close(a, b, atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("oracle", ORACLES)
def test_output_rows_are_convex_combinations(oracle):
    cu = [0, 48]
    q, k, v = _rand(25, 48, 1, 8), _rand(26, 48, 1, 8), _rand(27, 48, 1, 8)
    mask = torch.tensor([[[1, 0, 0], [1, 1, 0], [0, 1, 1]]], dtype=torch.bool)
    out = oracle(q, k, v, cu, cu, mask, 16, 16, False, None)
    for qb in range(3):
        keys = torch.cat([torch.arange(16 * j, 16 * j + 16) for j in range(3) if mask[0, qb, j]])
        lo, hi = v[keys, 0].min(0).values, v[keys, 0].max(0).values
        rows = out[16 * qb:16 * qb + 16, 0]
        assert (rows >= lo - 1e-5).all() and (rows <= hi + 1e-5).all()


def test_dense_partial_rows_and_heads():
    cu_q, cu_k = [0, 40, 100], [0, 64, 130]
    q, k, v = _rand(28, 100, 4, 16), _rand(29, 130, 2, 16), _rand(30, 130, 2, 16)
    g = torch.Generator().manual_seed(31)
    nq, nk = calculate_blocks_oracle(cu_q, 16)[0], calculate_blocks_oracle(cu_k, 32)[0]
    mask = torch.rand(2, nq, nk, generator=g) < 0.6
    full = hbsa_oracle(q, k, v, cu_q, cu_k, mask, 16, 32, True, None)
    part = hbsa_oracle(q, k, v, cu_q, cu_k, mask, 16, 32, True, None, q_rows=[3, 39, 40, 99], q_heads=[1, 2])
    for r in (3, 39, 40, 99):
        torch.testing.assert_close(part[r, [1, 2]], full[r, [1, 2]], atol=1e-6, rtol=1e-6)
    assert torch.isnan(part[0]).all() and torch.isnan(part[3, 0]).all()


# ---------------------------------------------------------------------------------------
# log-sum-exp output of the oracle
# ---------------------------------------------------------------------------------------
def test_lse_equals_library_logsumexp_on_dense_and_causal_cases():
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(n, 2, 16, generator=g) for n in (48, 80, 80))
    mask = torch.ones(2, 3, 5, dtype=torch.bool)
    out, lse = hbsa_oracle(q, k, v, [0, 48], [0, 80], mask, 16, 16, False, 0.4, return_lse=True)
    s = torch.einsum("qhd,khd->hqk", q, k) * 0.4
    assert torch.allclose(lse, torch.logsumexp(s, -1).T, atol=1e-5)
    assert torch.allclose(out, torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), v), atol=1e-5)
    out_c, lse_c = hbsa_oracle(q, k, v, [0, 48], [0, 80], mask, 16, 16, True, 0.4, return_lse=True)
    vis = torch.ones(48, 80, dtype=torch.bool).tril(diagonal=80 - 48)
    assert torch.allclose(lse_c, torch.logsumexp(s.masked_fill(~vis, float("-inf")), -1).T, atol=1e-5)


def test_lse_merges_attention_over_disjoint_key_sets_and_is_minus_inf_without_keys():
    g = torch.Generator().manual_seed(6)
    q = torch.randn(64, 4, 8, generator=g)
    k, v = (torch.randn(96, 2, 8, generator=g) for _ in range(2))
    cu_q, cu_k = [0, 40, 64], [0, 30, 96]
    mask = torch.rand(2, 5, 7, generator=g) < 0.6
    part_a = mask.clone(); part_a[:, :, 1::2] = False
    part_b = mask.clone(); part_b[:, :, 0::2] = False
    full, lse = hbsa_oracle(q, k, v, cu_q, cu_k, mask, 16, 16, True, None, return_lse=True)
    oa, la = hbsa_oracle(q, k, v, cu_q, cu_k, part_a, 16, 16, True, None, return_lse=True)
    ob, lb = hbsa_oracle(q, k, v, cu_q, cu_k, part_b, 16, 16, True, None, return_lse=True)
    merged_lse = torch.logaddexp(la, lb)
    assert torch.allclose(merged_lse, lse, atol=1e-5, equal_nan=True)
    wa = torch.nan_to_num(torch.exp(la - merged_lse), nan=0.0).unsqueeze(-1)
    wb = torch.nan_to_num(torch.exp(lb - merged_lse), nan=0.0).unsqueeze(-1)
    assert torch.allclose(wa * oa + wb * ob, full, atol=1e-5)
    empty = torch.isinf(lse) & (lse < 0)
    assert empty.any()                                      # causal rows of sequence 0 ahead of every key (q_len > k_len)
    assert torch.equal(empty, (full == 0).all(-1))
