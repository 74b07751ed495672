"""Seeded synthetic problems and work accounting for the block-sparse attention forward.

The generators follow the argument order of the reference's own problem builders
(reference ``test/test_accuracy.py:33-62``, ``test/test_speedup.py:88-115``,
``README.md:49-79``): sequence boundaries, then q, k, v ~ N(0,1), block metadata from
``calculate_blocks``, then a Bernoulli block mask.  Named workloads:

``C1``  batch 5, q lengths 32 each, k lengths 32,29,39,34,23, Hq 8 / Hk 2, D 32, blocks 32x16,
        keep 0.7, causal (the reference README's worked example)
``C2``  batch 8 x 8192, H 32, D 128, 128x128, keep 0.1 + diagonal, causal
``C3``  batch 8, lengths U[2048,16384], Hq 32 / Hk 8, D 128, 64x128, keep 0.3 + diagonal, causal
``C4``  batch 8 x 65536, H 32, D 128, 128x128, keep 0.3, non-causal
``C5``  q lengths 3000,5120,777,4096 vs k lengths 6000,5120,4100,8192, Hq 16 / Hk 2, D 64,
        blocks 80x48, keep 0.5, causal, softmax_scale 0.1
``T``   C2 at sequence length 32768 (the 50 %-of-peak target shape)
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from .utils import calculate_blocks


@dataclass
class Workload:
    name: str
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    cu_q: List[int]
    cu_k: List[int]
    cu_q_seqlens: torch.Tensor
    cu_k_seqlens: torch.Tensor
    block_mask: torch.Tensor
    q_block_size: int
    k_block_size: int
    causal: bool
    softmax_scale: Optional[float]
    q_meta: Tuple = field(default_factory=tuple)  # calculate_blocks(cu_q_seqlens, q_block_size)
    k_meta: Tuple = field(default_factory=tuple)

    def args(self, tile_mode: str = "auto", with_meta: bool = True) -> tuple:
        """Positional argument tuple of ``HBSAttention``."""
        base = (self.q, self.k, self.v, self.cu_q_seqlens, self.cu_k_seqlens, self.block_mask, self.q_block_size,
                self.k_block_size, self.causal, self.softmax_scale)
        if not with_meta:
            return base
        return base + (tile_mode,) + tuple(self.q_meta) + tuple(self.k_meta)


SPECS: Dict[str, dict] = {
    "C1": dict(seed=0, q_lens=[32] * 5, k_lens=[32, 29, 39, 34, 23], hq=8, hk=2, d=32, qbs=32, kbs=16, keep=0.7,
               diag=False, causal=True, scale=None),
    "C2": dict(seed=1, q_lens=[8192] * 8, k_lens=[8192] * 8, hq=32, hk=32, d=128, qbs=128, kbs=128, keep=0.1,
               diag=True, causal=True, scale=None),
    "C3": dict(seed=2, q_lens="U[2048,16384]x8", k_lens="same", hq=32, hk=8, d=128, qbs=64, kbs=128, keep=0.3,
               diag=True, causal=True, scale=None),
    "C4": dict(seed=3, q_lens=[65536] * 8, k_lens=[65536] * 8, hq=32, hk=32, d=128, qbs=128, kbs=128, keep=0.3,
               diag=False, causal=False, scale=None),
    "C5": dict(seed=4, q_lens=[3000, 5120, 777, 4096], k_lens=[6000, 5120, 4100, 8192], hq=16, hk=2, d=64, qbs=80,
               kbs=48, keep=0.5, diag=False, causal=True, scale=0.1),
    "T": dict(seed=1, q_lens=[32768] * 8, k_lens=[32768] * 8, hq=32, hk=32, d=128, qbs=128, kbs=128, keep=0.1,
              diag=True, causal=True, scale=None),
}


def _cumulative(lens: List[int]) -> List[int]:
    out = [0]
    for n in lens:
        out.append(out[-1] + int(n))
    return out


def force_diagonal(block_mask: torch.Tensor, cu_q: List[int], cu_k: List[int], q_block_size: int, k_block_size: int) -> None:
    """For every q block switch on the k block that holds the key its first row is aligned
    with (bottom-right alignment, clamped into the sequence), so no q block is left empty."""
    g = 0
    kb0 = 0
    for b in range(len(cu_q) - 1):
        q_len, k_len = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
        nqb = (q_len + q_block_size - 1) // q_block_size
        nkb = (k_len + k_block_size - 1) // k_block_size
        first_rows = torch.arange(nqb) * q_block_size
        key = (first_rows + (k_len - q_len)).clamp_(0, k_len - 1)
        kb = kb0 + torch.div(key, k_block_size, rounding_mode="floor")
        block_mask[:, torch.arange(g, g + nqb, device=block_mask.device), kb.to(block_mask.device)] = True
        g += nqb
        kb0 += nkb


def make_problem(*, seed: int, q_lens, k_lens, hq: int, hk: int, d: int, qbs: int, kbs: int, keep: float, diag: bool,
                 causal: bool, scale: Optional[float], device="cuda", dtype=torch.bfloat16, gen_device: str = "cpu",
                 name: str = "custom") -> Workload:
    """Builds one problem.  ``gen_device='cpu'`` draws every random tensor from a CPU generator
    (bit-reproducible on any machine) and moves it to ``device``; ``gen_device='device'`` draws on
    ``device`` (fast for multi-GiB tensors, reproducible per device type)."""
    device = torch.device(device)
    on_dev = gen_device != "cpu" and device.type != "cpu"
    gdev = device if on_dev else torch.device("cpu")
    g = torch.Generator(device=gdev)
    g.manual_seed(seed)
    if isinstance(q_lens, str):
        lo, hi = 2048, 16384
        cpu_g = torch.Generator().manual_seed(seed)
        q_lens = torch.randint(lo, hi + 1, (8,), generator=cpu_g).tolist()
        k_lens = list(q_lens)
    cu_q, cu_k = _cumulative(q_lens), _cumulative(k_lens)

    def draw(n, h):
        t = torch.randn(n, h, d, generator=g, device=gdev, dtype=torch.float32).to(dtype)
        return t.to(device)

    q, k, v = draw(cu_q[-1], hq), draw(cu_k[-1], hk), draw(cu_k[-1], hk)
    cu_q_t = torch.tensor(cu_q, dtype=torch.int32, device=device)
    cu_k_t = torch.tensor(cu_k, dtype=torch.int32, device=device)
    q_meta = calculate_blocks(cu_q_t, qbs)
    k_meta = calculate_blocks(cu_k_t, kbs)
    mask = (torch.rand(hk, q_meta[0], k_meta[0], generator=g, device=gdev) < keep).to(device)
    if diag:
        force_diagonal(mask, cu_q, cu_k, qbs, kbs)
    return Workload(name, q, k, v, cu_q, cu_k, cu_q_t, cu_k_t, mask, qbs, kbs, causal, scale, q_meta, k_meta)


def make_workload(name: str, device="cuda", dtype=torch.bfloat16, gen_device: str = "cpu", **overrides) -> Workload:
    spec = dict(SPECS[name])
    spec.update(overrides)
    return make_problem(device=device, dtype=dtype, gen_device=gen_device, name=name, **spec)


# --------------------------------------------------------------------------------------
# work accounting
# --------------------------------------------------------------------------------------
def count_work(w: Workload) -> Dict[str, float]:
    """Algorithmic work of one forward call, computed from the realised mask.

    ``flops``        4 * D * sum over q heads and visited block pairs of rows(qb) * cols(kb); a pair
                     is visited when its mask bit is set, both blocks lie in the same sequence and,
                     if causal, the k block's first key is visible to the q block's last row.
                     Blocks straddling the diagonal count in full.
    ``flops_exact``  the same with only visible score elements counted.
    ``bytes``        Q and O once, K and V blocks that at least one visited pair touches once, the
                     in-sequence part of the mask, and the metadata.
    """
    hq, d = w.q.shape[1], w.q.shape[2]
    hk = w.k.shape[1]
    ratio = hq // hk
    esize = w.q.element_size()
    dev = w.block_mask.device
    pairs = 0
    block_elems = 0
    exact_elems = 0
    touched_keys = 0
    mask_bytes = 0
    g0 = 0
    kb0 = 0
    for b in range(len(w.cu_q) - 1):
        q_len, k_len = w.cu_q[b + 1] - w.cu_q[b], w.cu_k[b + 1] - w.cu_k[b]
        shift = k_len - q_len
        nqb = (q_len + w.q_block_size - 1) // w.q_block_size
        nkb = (k_len + w.k_block_size - 1) // w.k_block_size
        r0 = torch.arange(nqb, device=dev) * w.q_block_size
        rows = torch.clamp(q_len - r0, max=w.q_block_size)
        c0 = torch.arange(nkb, device=dev) * w.k_block_size
        cols = torch.clamp(k_len - c0, max=w.k_block_size)
        slab = w.block_mask[:, g0:g0 + nqb, kb0:kb0 + nkb]
        if w.causal:
            reach = (r0 + rows - 1 + shift).unsqueeze(1) >= c0.unsqueeze(0)
            visited = slab & reach.unsqueeze(0)
            # visible elements of pair (i, j): sum over rows r of clamp(r + shift - c0 + 1, 0, cols)
            rr = torch.arange(w.q_block_size, device=dev)
            r_abs = r0.unsqueeze(1) + rr.unsqueeze(0)                      # [nqb, qbs]
            r_ok = rr.unsqueeze(0) < rows.unsqueeze(1)
            per_pair = torch.zeros(nqb, nkb, device=dev, dtype=torch.float64)
            for lo in range(0, nqb, 64):                                   # bound the [chunk, qbs, nkb] temporary
                hi = min(nqb, lo + 64)
                vis = (r_abs[lo:hi].unsqueeze(2) + shift - c0.view(1, 1, -1) + 1).clamp(min=0)
                vis = torch.minimum(vis, cols.view(1, 1, -1)) * r_ok[lo:hi].unsqueeze(2)
                per_pair[lo:hi] = vis.sum(1).double()
        else:
            visited = slab
            per_pair = (rows.unsqueeze(1) * cols.unsqueeze(0)).double()
        full = (rows.unsqueeze(1) * cols.unsqueeze(0)).double()
        vd = visited.double()
        pairs += float(vd.sum())
        block_elems += float((vd * full.unsqueeze(0)).sum())
        exact_elems += float((vd * per_pair.unsqueeze(0)).sum())
        touched_keys += float((visited.any(dim=1).double() * cols.unsqueeze(0).double()).sum())
        mask_bytes += hk * nqb * nkb
        g0 += nqb
        kb0 += nkb
    total_q = w.q.shape[0]
    meta_bytes = 4 * (2 * len(w.cu_q) + 2 * len(w.cu_q) + g0)
    nbytes = 2 * total_q * hq * d * esize + 2 * touched_keys * d * esize + mask_bytes + meta_bytes
    return {
        "visited_pairs": pairs * ratio,
        "flops": 4.0 * d * block_elems * ratio,
        "flops_exact": 4.0 * d * exact_elems * ratio,
        "bytes": float(nbytes),
    }
