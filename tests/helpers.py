"""Shared helpers of the parity tests."""
from __future__ import annotations

import torch

from oracle.dense import hbsa_oracle

# North-star tolerance for 16-bit inputs against the fp32 masked-dense oracle.
MAX_ABS_TOL = 2e-2
MEAN_ABS_TOL = 2e-3


def oracle_for(w, **kw) -> torch.Tensor:
    """fp32 oracle output for a Workload (tensors are copied to the CPU)."""
    return hbsa_oracle(w.q.cpu(), w.k.cpu(), w.v.cpu(), w.cu_q, w.cu_k, w.block_mask.cpu(), w.q_block_size,
                       w.k_block_size, w.causal, w.softmax_scale, **kw)


def assert_close_to_oracle(out: torch.Tensor, ref: torch.Tensor, what: str = "") -> None:
    out = out.detach().float().cpu()
    sel = ~torch.isnan(ref)
    assert sel.any(), "oracle computed nothing"
    assert torch.isfinite(out).all(), f"{what}: non-finite output"
    err = (out[sel] - ref[sel]).abs()
    assert err.max().item() <= MAX_ABS_TOL, f"{what}: max-abs {err.max().item():.3e} > {MAX_ABS_TOL}"
    assert err.mean().item() <= MEAN_ABS_TOL, f"{what}: mean-abs {err.mean().item():.3e} > {MEAN_ABS_TOL}"
