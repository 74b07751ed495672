"""Gradients of the block-sparse attention forward on the CPU (test infrastructure, never a
product path).

The reference has no backward (reference ``hbsattn/hbsa_interface.py:31-32`` raises
``NotImplementedError``), so there is nothing to restate: the oracle is what the mathematics of the
forward it defines (reference ``hbsattn/reference.py:23-107``) fixes.  With ``S = scale * Q K^T``
masked as in the forward, ``P = softmax(S)`` over a row's visible keys (``P = 0`` for a row without
any) and ``O = P V``:

    dV = P^T dO        dP = dO V^T        dS = P * (dP - rowsum(dP * P))
    dQ = scale * dS K  dK = scale * dS^T Q

evaluated per sequence, kv head and q head of its group in ``compute_dtype``.

What pins it (``tests/test_oracle_grads.py``): torch autograd through ``oracle.dense.hbsa_oracle``
(an independent path: reverse-mode differentiation of the masked-dense forward), central finite
differences of that forward in float64, and autograd through
``torch.nn.functional.scaled_dot_product_attention`` for masks that reduce to it.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch

from .dense import calculate_blocks_oracle, visible_mask


def hbsa_oracle_grads(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, dout: torch.Tensor,
                      cu_q_seqlens: Sequence[int], cu_k_seqlens: Sequence[int], block_mask: torch.Tensor,
                      q_block_size: int, k_block_size: int, causal: bool, softmax_scale: Optional[float],
                      compute_dtype: torch.dtype = torch.float32) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``(dq, dk, dv)`` for ``dout = d loss / d out``, shapes of ``q``, ``k``, ``v``, in ``compute_dtype``."""
    cu_q = [int(x) for x in cu_q_seqlens]
    cu_k = [int(x) for x in cu_k_seqlens]
    total_q, hq, d = q.shape
    hk = k.shape[1]
    ratio = hq // hk
    scale = float(softmax_scale) if softmax_scale is not None else d ** -0.5
    _, _, _, cu_nqb = calculate_blocks_oracle(cu_q, q_block_size)
    _, _, _, cu_nkb = calculate_blocks_oracle(cu_k, k_block_size)
    block_mask = block_mask.cpu()
    dq = torch.zeros(q.shape, dtype=compute_dtype)
    dk = torch.zeros(k.shape, dtype=compute_dtype)
    dv = torch.zeros(v.shape, dtype=compute_dtype)
    for b in range(len(cu_q) - 1):
        qs, qe, ks, ke = cu_q[b], cu_q[b + 1], cu_k[b], cu_k[b + 1]
        if qe == qs or ke == ks:
            continue
        for hkv in range(hk):
            vis = visible_mask(block_mask[hkv, cu_nqb[b]:cu_nqb[b + 1], cu_nkb[b]:cu_nkb[b + 1]], qe - qs, ke - ks,
                               q_block_size, k_block_size, causal)
            kb = k[ks:ke, hkv].to(compute_dtype)
            vb = v[ks:ke, hkv].to(compute_dtype)
            for h in range(hkv * ratio, (hkv + 1) * ratio):
                qb = q[qs:qe, h].to(compute_dtype)
                dob = dout[qs:qe, h].to(compute_dtype)
                s = (qb @ kb.T) * scale
                s = s.masked_fill(~vis, float("-inf"))
                p = torch.nan_to_num(torch.softmax(s, dim=1), nan=0.0)
                dp = dob @ vb.T
                ds = p * (dp - (dp * p).sum(dim=1, keepdim=True))
                dv[ks:ke, hkv] += p.T @ dob
                dq[qs:qe, h] = (ds @ kb) * scale
                dk[ks:ke, hkv] += (ds.T @ qb) * scale
    return dq, dk, dv
