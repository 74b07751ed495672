"""Block geometry of a packed variable-length batch.

Same contract as the reference's ``hbsattn.utils.calculate_blocks`` (reference
``hbsattn/utils.py:7-50``): blocks restart at every sequence start, the last block
of a sequence may be short, block indices are global across the packed batch.
"""
from __future__ import annotations

from typing import Tuple

import torch


def calculate_blocks(cu_seqlen: torch.Tensor, block_size: int) -> Tuple[int, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``cu_seqlen`` int tensor ``[B+1]`` (any device), ``block_size`` int.

    Returns ``(num_block, cu_block, block_to_batch, cu_num_block)``:

    * ``num_block``      Python int, total blocks (one device->host read, like the reference's ``.item()``)
    * ``cu_block``       int32 ``[num_block+1]``: block ``j`` spans tokens ``cu_block[j]:cu_block[j+1]``
    * ``block_to_batch`` int32 ``[num_block]``: sequence index of each block
    * ``cu_num_block``   ``cu_seqlen.dtype`` ``[B+1]``: first global block index of each sequence
    """
    dev = cu_seqlen.device
    lengths = cu_seqlen[1:] - cu_seqlen[:-1]
    per_seq = torch.div(lengths + (block_size - 1), block_size, rounding_mode="floor")
    cu_num_block = torch.cat([per_seq.new_zeros(1), per_seq.cumsum(0).to(per_seq.dtype)])
    num_block = int(cu_num_block[-1])

    block_to_batch = torch.repeat_interleave(
        torch.arange(per_seq.numel(), dtype=torch.int32, device=dev), per_seq.to(torch.int64), output_size=num_block)
    b = block_to_batch.long()
    local = torch.arange(num_block, device=dev) - cu_num_block.long()[b]
    ends = torch.minimum(cu_seqlen.long()[b] + (local + 1) * block_size, cu_seqlen.long()[b + 1])
    cu_block = torch.cat([ends.new_zeros(1), ends]).to(torch.int32)
    return num_block, cu_block, block_to_batch, cu_num_block
