"""Block-sparse "attention sink + local window" attention for the CSLA layers: the counterpart of the
reference's ``SparseFlexAttn`` (models/sparvar/basic_sparvar.py:47-194), with the flex-attention call
replaced by the HIP block-sparse kernel.  Same constructor arguments and ``forward`` signature."""
from __future__ import annotations

from typing import Optional, Sequence

import torch

from . import mask_build as mb
from . import sparse_attn_ops as ops

_DEFAULT_SPARSE_BLOCK_SIZE = 128  # torch flex_attention's default block, which the reference relies on


class SparseFlexAttn(torch.nn.Module):
    def __init__(self, scale_schedule: Sequence, kernel_schedule: Sequence[int], q_scale_idx: int, attn_sink_scale: int,
                 block_size: int = _DEFAULT_SPARSE_BLOCK_SIZE, num_heads: int = 16, device=None):
        super().__init__()
        # square blocks, as flex's BLOCK_SIZE=int gives them (basic_sparvar.py:55-72): the sizes the kernel walks
        if block_size not in (64, 128, 256):
            raise ValueError("block_size must be 64, 128 or 256 (the block shapes of the HIP block-sparse kernel)")
        if device is None:
            device = "cuda"     # the reference builds its mask on 'cuda' too (basic_sparvar.py:70); there is no CPU path
        self.block_size = block_size
        self.num_heads = num_heads
        hw = mb._hw(scale_schedule)
        self.q_len = hw[q_scale_idx][0] * hw[q_scale_idx][1]
        self.kv_len = sum(h * w for h, w in hw[:q_scale_idx + 1])
        # bool [nQ, nK] block-level mask: "any element set => whole block set" (basic_sparvar.py:159-173)
        self.block_level_mask = mb.flex_block_mask(q_scale_idx, kernel_schedule, attn_sink_scale, block_size,
                                                   scales=scale_schedule, device=device)
        num, idx = mb.block_mask_to_lists(self.block_level_mask)
        # one list shared by every batch and head (the reference builds its BlockMask with B=1)
        self.register_buffer("kv_num_blocks", num.view(1, 1, -1), persistent=False)
        self.register_buffer("kv_indices", idx.view(1, 1, idx.shape[0], idx.shape[1]), persistent=False)

    @property
    def density(self) -> float:
        return float(self.block_level_mask.float().mean())

    def forward(self, q, k, v, scale: Optional[float] = None):
        if q.shape[-2] != self.q_len or k.shape[-2] != self.kv_len:
            raise ValueError(f"expected Lq={self.q_len}, Lk={self.kv_len}, got {q.shape[-2]}, {k.shape[-2]}")
        if self.kv_num_blocks.device != q.device:
            self.kv_num_blocks = self.kv_num_blocks.to(q.device)
            self.kv_indices = self.kv_indices.to(q.device)
        out, _ = ops.block_sparse_attn(q.to(v.dtype), k.to(v.dtype), v, self.kv_num_blocks, self.kv_indices,
                                       self.block_size, self.block_size, scale)
        return out
