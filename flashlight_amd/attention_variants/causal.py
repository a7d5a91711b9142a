"""Causal softmax attention (reference: attention_variants/causal.py)."""
from __future__ import annotations

import torch

from .. import _ffi
from ._common import grouped_view, run


def attention_pytorch_causal(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, attn_mask=None,
                             dropout_p=0.0, is_causal: bool = False, scale=None, enable_gqa=False) -> torch.Tensor:
    """causal.py:4-36: key k is attended by query q iff k <= q (top-left aligned when L != S).  Like the reference,
    the mask is always applied and `attn_mask`, `dropout_p`, `is_causal` are accepted but not used (`dropout_p` is
    applied once `honor_dropout(True)` has been called).
    Result: [N, Hq, L, Ev], or its [N, Hkv, G, L, Ev] view when enable_gqa is set."""
    out = run(query, key, value, scale=scale, enable_gqa=enable_gqa, mask_kind=_ffi.MASK_CAUSAL, dropout_p=dropout_p)
    return grouped_view(out, key, enable_gqa)
