"""Shared helpers of the parity tests."""
from __future__ import annotations

import torch

from oracle.dense import hbsa_oracle

# North-star tolerance for 16-bit inputs against the fp32 masked-dense oracle.
MAX_ABS_TOL = 2e-2
MEAN_ABS_TOL = 2e-3
# fp32 inputs, "fast" mode: 11-bit significands for q, k, v and p (fp32 accumulation and softmax).
F32_MAX_ABS_TOL = 4e-3
F32_MEAN_ABS_TOL = 3e-4
# fp32 inputs, "exact" mode: fp32 operands and matrix instructions, against the fp32 torch oracle
# (both sum in fp32, in different orders; with logits of magnitude ~10 the sums differ in the fifth digit)
F32_EXACT_MAX_ABS_TOL = 1e-4
F32_EXACT_MEAN_ABS_TOL = 1e-5


def oracle_for(w, **kw) -> torch.Tensor:
    """fp32 oracle output for a Workload (tensors are copied to the CPU)."""
    return hbsa_oracle(w.q.cpu(), w.k.cpu(), w.v.cpu(), w.cu_q, w.cu_k, w.block_mask.cpu(), w.q_block_size,
                       w.k_block_size, w.causal, w.softmax_scale, **kw)


def assert_close_to_oracle(out: torch.Tensor, ref: torch.Tensor, what: str = "", max_abs: float = None,
                           mean_abs: float = None) -> None:
    f32 = out.dtype == torch.float32
    if f32:
        from hbsattn_amd import interface
        exact = interface._fp32_mode == "exact"
        dflt = (F32_EXACT_MAX_ABS_TOL, F32_EXACT_MEAN_ABS_TOL) if exact else (F32_MAX_ABS_TOL, F32_MEAN_ABS_TOL)
    else:
        dflt = (MAX_ABS_TOL, MEAN_ABS_TOL)
    max_abs = max_abs if max_abs is not None else dflt[0]
    mean_abs = mean_abs if mean_abs is not None else dflt[1]
    out = out.detach().float().cpu()
    sel = ~torch.isnan(ref)
    assert sel.any(), "oracle computed nothing"
    assert torch.isfinite(out).all(), f"{what}: non-finite output"
    err = (out[sel] - ref[sel]).abs()
    assert err.max().item() <= max_abs, f"{what}: max-abs {err.max().item():.3e} > {max_abs}"
    assert err.mean().item() <= mean_abs, f"{what}: mean-abs {err.mean().item():.3e} > {mean_abs}"
