"""Prefix-LM attention (reference: attention_variants/prefix_lm.py)."""
from __future__ import annotations

from typing import Optional

import torch

from .. import _ffi
from ._common import grouped_view, run


def get_prefix_lm_mask(query: torch.Tensor, prefix_lengths: int) -> torch.Tensor:
    """Boolean [N, 1, L, L], True = masked: k > max(prefix_lengths - 1, q) (prefix_lm.py:33-42).
    Not used by the kernel path."""
    pos = torch.arange(query.size(-2), device=query.device)
    last_visible = pos.clamp(min=int(prefix_lengths) - 1)[:, None]
    return (pos[None, :] > last_visible)[None, None].expand(query.size(0), 1, -1, -1)


def attention_pytorch_prefix_lm(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                prefix_lengths: int = 256, scale: Optional[float] = None,
                                enable_gqa=False) -> torch.Tensor:
    """prefix_lm.py:5-30: the first `prefix_lengths` keys are visible to every query, the rest causally
    (attend iff k < prefix_lengths or k <= q); one integer prefix for the whole batch."""
    if query.size(-2) != key.size(-2):
        raise ValueError("prefix-LM attention needs equally long query and key sequences")
    out = run(query, key, value, scale=scale, enable_gqa=enable_gqa, mask_kind=_ffi.MASK_PREFIX_LM,
              prefix=int(prefix_lengths))
    return grouped_view(out, key, enable_gqa)
