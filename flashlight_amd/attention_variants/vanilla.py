"""Unmasked softmax attention (reference: attention_variants/vanilla.py)."""
from __future__ import annotations

import torch

from .. import _ffi
from ._common import run


def attention_pytorch_nogqa(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, scale=None) -> torch.Tensor:
    """softmax(q k^T * scale) v for equal head counts (vanilla.py:4-17); scale defaults to 1/sqrt(E)."""
    return run(query, key, value, scale=scale, enable_gqa=False, mask_kind=_ffi.MASK_NONE)


def attention_pytorch(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, scale=None,
                      enable_gqa=False) -> torch.Tensor:
    """vanilla.py:20-35.  With enable_gqa the query's Hq heads are grouped over the Hkv key/value heads (query head
    h reads key/value head h // (Hq / Hkv)); the result is [N, Hq, L, Ev] (this variant views it back, vanilla.py:35)."""
    return run(query, key, value, scale=scale, enable_gqa=enable_gqa, mask_kind=_ffi.MASK_NONE)
