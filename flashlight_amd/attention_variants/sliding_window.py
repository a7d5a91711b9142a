"""Causal sliding-window attention (reference: attention_variants/sliding_window.py)."""
from __future__ import annotations

import torch

from .. import _ffi
from ._common import grouped_view, run


def get_sliding_mask(query: torch.Tensor, window_size: int) -> torch.Tensor:
    """Boolean [1, 1, L, L], True = masked: key ahead of the query or more than `window_size` behind it
    (sliding_window.py:4-12).  Not used by the kernel path, which evaluates the predicate per tile."""
    pos = torch.arange(query.size(-2), device=query.device)
    behind = pos[:, None] - pos[None, :]  # q - k
    return ((behind < 0) | (behind > window_size))[None, None]


def attention_pytorch_sliding_window(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                     window_size: int = 1024, scale=None, enable_gqa: bool = False) -> torch.Tensor:
    """sliding_window.py:14-44: query q attends keys with 0 <= q - k <= window_size (window_size + 1 keys).
    Requires L == S like the reference (sliding_window.py:27)."""
    assert query.size(-2) == key.size(-2) == value.size(-2)
    out = run(query, key, value, scale=scale, enable_gqa=enable_gqa, mask_kind=_ffi.MASK_SLIDING,
              window=int(window_size))
    return grouped_view(out, key, enable_gqa)
