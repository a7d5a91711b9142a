"""Differential attention, Ye et al. 2024 (reference: attention_variants/diff_attn.py)."""
from __future__ import annotations

import torch

from .. import _ffi, ops


def diffattn(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale=None, lambda_full=0.2, **kwargs) -> torch.Tensor:
    """diff_attn.py:6-30: q, k are [B, 2H, S, d] and split on the head axis (first H heads -> softmax 0, last H ->
    softmax 1); v is [B, H, S, 2d]; returns softmax(q0 k0^T s) v - lambda_full * softmax(q1 k1^T s) v, [B, H, S, 2d],
    with s = 1/sqrt(d) unless `scale` is given.  Both softmaxes run inside one kernel launch.

    `is_causal=True` (not in the reference, which swallows extra keywords) masks k > q in both softmaxes."""
    causal = bool(kwargs.get("is_causal", False))
    return ops.dispatch(q, k, v, scale=scale, diff=True, lambda_full=float(lambda_full),
                        mask_kind=_ffi.MASK_CAUSAL if causal else _ffi.MASK_NONE)


def make_input(config, attention_name="diffattn"):
    """Inputs of the reference's benchmark (diff_attn.py:33-38): config = (batch, seqlen, nheads, headdim, causal,
    dropout_p); Q, K ~ N(0,1) [batch, nheads, seqlen, headdim], V [batch, nheads // 2, seqlen, 2 * headdim], bf16."""
    batch, seqlen, nheads, headdim = config[:4]
    shapes = [(batch, nheads, seqlen, headdim)] * 2 + [(batch, nheads // 2, seqlen, 2 * headdim)]
    return tuple(torch.randn(s, dtype=torch.bfloat16, device="cuda") for s in shapes)
