"""Shared argument handling for the variant front-ends."""
from __future__ import annotations

from typing import Optional

import torch

from .. import _ffi, ops


def check_heads(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, enable_gqa: bool) -> None:
    if query.dim() != 4 or key.dim() != 4 or value.dim() != 4:
        for name, t in (("query", query), ("key", key), ("value", value)):
            if t.dim() != 4:
                raise ValueError(f"{name} must be [N, H, L, E], got shape {tuple(t.shape)}")
    hq, hkv = query.shape[1], key.shape[1]
    if value.shape[1] != hkv:
        raise ValueError(f"key has {hkv} heads but value has {value.shape[1]}")
    if enable_gqa:
        if hq % hkv:
            raise ValueError(f"enable_gqa: {hq} query heads are not a multiple of {hkv} key/value heads")
    elif hq != hkv and hkv != 1:  # a single key/value head broadcasts in the reference's matmul
        raise ValueError(f"{hq} query heads vs {hkv} key/value heads: pass enable_gqa=True for grouped-query attention")


def grouped_view(out: torch.Tensor, key: torch.Tensor, enable_gqa: bool) -> torch.Tensor:
    """Result layout of the reference's variants under GQA: [N, Hkv, G, L, Ev] (they never view back, e.g.
    attention_variants/causal.py:27-36).  Same memory as the 4-D result."""
    if not enable_gqa:
        return out
    n, hq, l, ev = out.shape
    hkv = key.size(1)
    return out.view(n, hkv, hq // hkv, l, ev)


_honor_dropout = False


class honor_dropout:
    """The reference's variants take `dropout_p` and ignore it (attention_variants/causal.py:4-36, alibi.py:13-33,
    softcap.py:4-53), and so do this package's by default.  `honor_dropout(True)` (also usable as a context manager:
    `with honor_dropout(): ...`) makes them apply it: softmax weights are dropped with probability `dropout_p` and the
    kept ones scaled by 1 / (1 - p), as torch.nn.functional.dropout would.  Seeds come from torch's default CPU
    generator.  The kernels have dropout for every mask kind with the in-kernel ALiBi term, the soft-cap and dense bias
    operands (a `score_mod` tensor) in any combination, at head dims up to 128: the causal, ALiBi, soft-cap and
    document-mask variants take it."""

    def __init__(self, enabled: bool = True):
        global _honor_dropout
        self._previous = _honor_dropout
        _honor_dropout = bool(enabled)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        global _honor_dropout
        _honor_dropout = self._previous
        return False


def run(query, key, value, *, scale: Optional[float], enable_gqa: bool, dropout_p: float = 0.0, **kw) -> torch.Tensor:
    check_heads(query, key, value, enable_gqa)
    if _honor_dropout and dropout_p:
        kw["dropout_p"] = float(dropout_p)
    return ops.dispatch(query, key, value, scale=scale, **kw)
