"""Vectorised masked-dense CPU oracle (test infrastructure, never a product path).

Restates, without importing it, what the reference's golden implementation
computes:

* block geometry      — reference ``hbsattn/utils.py:7-50``
* attention semantics — reference ``hbsattn/reference.py:23-107`` (v1: fp32 upcast
  ``:52``, in-sequence mask ``:56-60``, bottom-right causal ``:64-77``, block mask
  lookup ``block_mask[q_head // ratio, q_block, k_block]`` ``:80-87``, softmax over
  keys ``:92-95``, ``nan_to_num`` for rows with no visible key ``:97-98``, PV ``:100``)
  and the equivalent whole-matrix formulation ``hbsattn/reference.py:209-258`` (v3).

The formulation here is neither: it works per sequence and per query head, expands
the block mask with ``repeat_interleave`` of the per-block lengths, and never
materialises a ``[rows, total_k, heads]`` tensor, so it scales to the large
configurations when restricted to sampled rows (``q_rows``).

What pins it: ``tests/test_oracle_dense.py`` (SDPA reductions, invariants) and
``tests/test_oracle_cross.py`` (agreement with the independently written C
restatement ``oracle/scalar.c``).
"""
from __future__ import annotations

import math
from typing import Iterable, List, Optional, Sequence, Tuple

import torch


# --------------------------------------------------------------------------- #
# block geometry                                                               #
# --------------------------------------------------------------------------- #
def calculate_blocks_oracle(cu_seqlen: Sequence[int], block_size: int) -> Tuple[int, List[int], List[int], List[int]]:
    """Plain-Python restatement of reference ``hbsattn/utils.py:7-50``.

    Blocks restart at each sequence start; the last block of a sequence may be
    short.  Returns ``(num_block, cu_block[nb+1], block_to_batch[nb], cu_num_block[B+1])``
    as Python lists of ints.
    """
    cu = [int(x) for x in cu_seqlen]
    cu_block = [0]
    block_to_batch: List[int] = []
    cu_num_block = [0]
    for b in range(len(cu) - 1):
        start, end = cu[b], cu[b + 1]
        pos = start
        while pos < end:
            nxt = min(pos + block_size, end)
            cu_block.append(nxt)
            block_to_batch.append(b)
            pos = nxt
        cu_num_block.append(len(block_to_batch))
    return len(block_to_batch), cu_block, block_to_batch, cu_num_block


def _block_lengths(seq_len: int, block_size: int) -> List[int]:
    n = (seq_len + block_size - 1) // block_size
    return [min(block_size, seq_len - i * block_size) for i in range(n)]


# --------------------------------------------------------------------------- #
# attention                                                                    #
# --------------------------------------------------------------------------- #
def visible_mask(block_mask_seq: torch.Tensor, q_len: int, k_len: int, q_block_size: int,
                 k_block_size: int, causal: bool) -> torch.Tensor:
    """Element mask ``[q_len, k_len]`` (True = key visible) of one sequence and one
    kv head from that sequence's slab ``block_mask_seq[nqb_seq, nkb_seq]`` of the
    block mask.  Causal alignment is bottom-right: key ``j`` is visible to query
    ``i`` iff ``i + (k_len - q_len) >= j`` (reference ``hbsattn/reference.py:66-77``).
    """
    ql = torch.tensor(_block_lengths(q_len, q_block_size))
    kl = torch.tensor(_block_lengths(k_len, k_block_size))
    m = block_mask_seq.to(torch.bool)
    m = torch.repeat_interleave(m, ql, dim=0)
    m = torch.repeat_interleave(m, kl, dim=1)
    if causal:
        i = torch.arange(q_len).unsqueeze(1)
        j = torch.arange(k_len).unsqueeze(0)
        m = m & (i + (k_len - q_len) >= j)
    return m


def hbsa_oracle(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                cu_q_seqlens: Sequence[int], cu_k_seqlens: Sequence[int],
                block_mask: torch.Tensor, q_block_size: int, k_block_size: int,
                causal: bool, softmax_scale: Optional[float],
                *, q_rows: Optional[Iterable[int]] = None, q_heads: Optional[Iterable[int]] = None,
                compute_dtype: torch.dtype = torch.float32, row_chunk: int = 2048, return_lse: bool = False):
    """Masked-dense block-sparse attention forward on CPU tensors.

    ``q [total_q, Hq, D]``, ``k, v [total_k, Hk, D]`` (any float dtype, upcast to
    ``compute_dtype``), ``block_mask [Hk, num_q_block, num_k_block]`` over *global*
    block indices.  Returns ``compute_dtype`` output of shape ``[total_q, Hq, D]``;
    with ``q_rows`` / ``q_heads`` only those rows / heads are computed, the rest is
    NaN so an accidental comparison against an uncomputed entry fails.  With ``return_lse`` the
    result is ``(out, lse)``, ``lse [total_q, Hq]`` = natural-log sum of exp(scaled scores) over a
    row's visible keys (-inf for a row without any), NaN where not computed.
    """
    cu_q = [int(x) for x in cu_q_seqlens]
    cu_k = [int(x) for x in cu_k_seqlens]
    assert len(cu_q) == len(cu_k)
    total_q, hq, d = q.shape
    hk = k.shape[1]
    assert hq % hk == 0
    ratio = hq // hk
    scale = float(softmax_scale) if softmax_scale is not None else d ** -0.5
    _, _, _, cu_nqb = calculate_blocks_oracle(cu_q, q_block_size)
    _, _, _, cu_nkb = calculate_blocks_oracle(cu_k, k_block_size)
    assert tuple(block_mask.shape) == (hk, cu_nqb[-1], cu_nkb[-1]), (tuple(block_mask.shape), (hk, cu_nqb[-1], cu_nkb[-1]))
    block_mask = block_mask.cpu()

    partial = q_rows is not None or q_heads is not None
    out = torch.full((total_q, hq, d), float("nan") if partial else 0.0, dtype=compute_dtype)
    lse = torch.full((total_q, hq), float("nan") if partial else float("-inf"), dtype=compute_dtype)
    heads = sorted(set(int(h) for h in q_heads)) if q_heads is not None else list(range(hq))
    row_sel = None
    if q_rows is not None:
        row_sel = torch.zeros(total_q, dtype=torch.bool)
        row_sel[torch.as_tensor(list(q_rows), dtype=torch.long)] = True

    for b in range(len(cu_q) - 1):
        qs, qe, ks, ke = cu_q[b], cu_q[b + 1], cu_k[b], cu_k[b + 1]
        q_len, k_len = qe - qs, ke - ks
        if q_len == 0:
            continue
        if row_sel is not None:
            local_rows = torch.nonzero(row_sel[qs:qe]).flatten()
            if local_rows.numel() == 0:
                continue
        else:
            local_rows = torch.arange(q_len)
        for hkv in range(hk):
            group = [h for h in heads if h // ratio == hkv]
            if not group:
                continue
            kb = k[ks:ke, hkv].to(compute_dtype)
            vb = v[ks:ke, hkv].to(compute_dtype)
            vis_blocks = block_mask[hkv, cu_nqb[b]:cu_nqb[b + 1], cu_nkb[b]:cu_nkb[b + 1]]
            ql = torch.tensor(_block_lengths(q_len, q_block_size))
            kl = torch.tensor(_block_lengths(k_len, k_block_size))
            row_to_qb = torch.repeat_interleave(torch.arange(ql.numel()), ql)
            for c0 in range(0, local_rows.numel(), row_chunk):
                rows = local_rows[c0:c0 + row_chunk]
                vis = torch.repeat_interleave(vis_blocks[row_to_qb[rows]], kl, dim=1)  # [r, k_len]
                if causal:
                    vis = vis & (rows.unsqueeze(1) + (k_len - q_len) >= torch.arange(k_len).unsqueeze(0))
                for h in group:
                    s = (q[qs + rows, h].to(compute_dtype) @ kb.T) * scale
                    s = s.masked_fill(~vis, float("-inf"))
                    p = torch.softmax(s, dim=1)
                    p = torch.nan_to_num(p, nan=0.0)  # rows with no visible key -> exactly 0
                    out[qs + rows, h] = p @ vb
                    lse[qs + rows, h] = torch.logsumexp(s, dim=1)
    return (out, lse) if return_lse else out


# --------------------------------------------------------------------------- #
# work accounting (shared by tests that check the bench's FLOP model)          #
# --------------------------------------------------------------------------- #
def visited_block_pairs(cu_q_seqlens: Sequence[int], cu_k_seqlens: Sequence[int], block_mask: torch.Tensor,
                        q_block_size: int, k_block_size: int, causal: bool) -> Tuple[int, int]:
    """Brute-force count over one kv head group of (a) ``sum rows(qb) * cols(kb)`` over
    visited block pairs and (b) the element-exact number of visible scores, summed
    over kv heads (multiply by the GQA ratio for q heads).  A pair is visited when
    its mask bit is set, both blocks belong to the same sequence and, if causal,
    the first key of the k block is visible to the last row of the q block.
    """
    cu_q = [int(x) for x in cu_q_seqlens]
    cu_k = [int(x) for x in cu_k_seqlens]
    _, _, _, cu_nqb = calculate_blocks_oracle(cu_q, q_block_size)
    _, _, _, cu_nkb = calculate_blocks_oracle(cu_k, k_block_size)
    bm = block_mask.cpu()
    block_elems = 0
    exact_elems = 0
    for b in range(len(cu_q) - 1):
        q_len, k_len = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
        off = k_len - q_len
        ql, kl = _block_lengths(q_len, q_block_size), _block_lengths(k_len, k_block_size)
        for hkv in range(bm.shape[0]):
            slab = bm[hkv, cu_nqb[b]:cu_nqb[b + 1], cu_nkb[b]:cu_nkb[b + 1]]
            for iq, rows in enumerate(ql):
                r0 = iq * q_block_size
                for jk, cols in enumerate(kl):
                    if not bool(slab[iq, jk]):
                        continue
                    c0 = jk * k_block_size
                    if causal:
                        if r0 + rows - 1 + off < c0:
                            continue
                        vis = 0
                        for r in range(r0, r0 + rows):
                            vis += max(0, min(c0 + cols - 1, r + off) - c0 + 1)
                        exact_elems += vis
                    else:
                        exact_elems += rows * cols
                    block_elems += rows * cols
    return block_elems, exact_elems
