"""Attention with tanh soft-capping of the logits (reference: attention_variants/softcap.py)."""
from __future__ import annotations

import torch

from .. import _ffi
from ._common import grouped_view, run


class TanhSoftcap:
    """score -> soft_cap * tanh(score / soft_cap), the formula softcap.py:48 states.  Stands in for
    attn_gym.mods.generate_tanh_softcap(soft_cap, approx=False), which the reference's benchmark passes as
    `score_mod` (benchmarks/run_flex_variants.py:133): same call shape (score, b, h, q_idx, kv_idx)."""

    def __init__(self, soft_cap: float):
        if not soft_cap > 0:
            raise ValueError("soft_cap must be positive")
        self.soft_cap = float(soft_cap)

    def __call__(self, score, *_ignored):
        return self.soft_cap * torch.tanh(score / self.soft_cap)

    def __repr__(self) -> str:
        return f"TanhSoftcap({self.soft_cap})"


def generate_tanh_softcap(soft_cap: float, approx: bool = False) -> TanhSoftcap:
    if approx:
        raise NotImplementedError("only the exact tanh form (approx=False) is implemented")
    return TanhSoftcap(soft_cap)


def attention_softcapped(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, score_mod=None, attn_mask=None,
                         dropout_p=0.0, is_causal: bool = False, scale=None, enable_gqa: bool = False,
                         softcap_threshold: float = 30.0) -> torch.Tensor:
    """softcap.py:4-53: softmax(score_mod(q k^T * scale)) v.  `score_mod` must be a `TanhSoftcap`
    (from `generate_tanh_softcap`); None uses `softcap_threshold` as the cap (the reference declares that parameter but
    never reads it).  `is_causal=True` masks k > q (accepted and ignored by the reference)."""
    if score_mod is None:
        score_mod = TanhSoftcap(softcap_threshold)
    if not isinstance(score_mod, TanhSoftcap):
        raise NotImplementedError(
            "score_mod must come from generate_tanh_softcap(): the fused kernel applies cap * tanh(x / cap) in "
            "registers and cannot call an arbitrary Python function on the score matrix")
    out = run(query, key, value, scale=scale, enable_gqa=enable_gqa,
              mask_kind=_ffi.MASK_CAUSAL if is_causal else _ffi.MASK_NONE, softcap=score_mod.soft_cap,
              dropout_p=dropout_p)
    return grouped_view(out, key, enable_gqa)
