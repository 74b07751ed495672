"""hbsattn_amd — MI355X (gfx950) block-sparse attention forward.

Drop-in for the ``hbsattn`` operator (reference ``hbsattn/__init__.py:1``):
``HBSAttention(q, k, v, cu_q_seqlens, cu_k_seqlens, block_mask, q_block_size,
k_block_size, causal, softmax_scale, ...)`` and ``utils.calculate_blocks``.
The compute path is hand-written HIP behind a C ABI (``libhbsattn_amd.so``);
there is no Triton, no eager fallback and no CPU path: CUDA/HIP tensors go to the
kernels, anything else raises.
"""
from .interface import (HBSAttention, clear_prepared_cache, set_deterministic, set_fp32_mode, set_onepass,
                        set_prepared_cache_size)
from .utils import calculate_blocks

__all__ = ["HBSAttention", "calculate_blocks", "set_fp32_mode", "set_prepared_cache_size", "clear_prepared_cache",
           "set_deterministic", "set_onepass"]
