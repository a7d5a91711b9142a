"""Attention with ALiBi bias (reference: attention_variants/alibi.py)."""
from __future__ import annotations

from typing import Optional

import torch

from .. import _ffi
from ._common import grouped_view, run


def alibi_bias(h: int, q_len: int, kv_len: int, device="cuda") -> torch.Tensor:
    """Dense fp32 [h, q_len, kv_len] bias: 2^(-8 (i + 1) / h) * (k - q) for head i (alibi.py:5-9).
    The kernel path never builds this tensor; it is here for callers that want the values."""
    slopes = torch.exp2(-8.0 * (torch.arange(1, h + 1, dtype=torch.float32, device=device) / h))
    rel = torch.arange(kv_len, dtype=torch.int32, device=device).unsqueeze(0) - \
        torch.arange(q_len, dtype=torch.int32, device=device).unsqueeze(1)
    return slopes.view(h, 1, 1) * rel


class AlibiBias:
    """What `generate_alibi_bias_pytorch(nheads)` returns: callable like the reference's lambda
    (`score_mod(q_len, kv_len)` -> dense bias, alibi.py:11) and recognised by `attention_pytorch_alibi`, which
    then computes the slopes inside the kernel instead of reading a [H, L, S] tensor."""

    def __init__(self, nheads: int):
        self.nheads = int(nheads)

    def __call__(self, q_len: int, kv_len: int) -> torch.Tensor:
        return alibi_bias(self.nheads, q_len, kv_len)

    def __repr__(self) -> str:
        return f"AlibiBias(nheads={self.nheads})"


def generate_alibi_bias_pytorch(nheads: int) -> AlibiBias:
    return AlibiBias(nheads)


def attention_pytorch_alibi(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, score_mod=None,
                            attn_mask=None, dropout_p=0.0, is_causal: bool = False, scale=None, enable_gqa=False, *,
                            softcap: Optional[float] = None) -> torch.Tensor:
    """alibi.py:13-33: softmax(q k^T * scale + bias) v with bias = score_mod(L, S); `score_mod` must come from
    `generate_alibi_bias_pytorch` (the reference's tests and benchmarks pass nothing else: tests/test_alibi.py:32,
    benchmarks/run_flex_variants.py:129-131) and its head count must equal the number of query heads.

    Two additions over the reference, both off by default: `is_causal=True` masks k > q (the reference accepts the
    flag and ignores it), and `softcap=c` replaces the scaled score x by c * tanh(x / c) before the bias is added."""
    if score_mod is None:
        raise TypeError("attention_pytorch_alibi needs score_mod=generate_alibi_bias_pytorch(num_query_heads)")
    if not isinstance(score_mod, AlibiBias):
        raise NotImplementedError(
            "score_mod must be the object returned by generate_alibi_bias_pytorch(): the fused kernel computes the "
            "ALiBi term from the head index and positions and cannot call an arbitrary Python function per score")
    if score_mod.nheads != query.size(1):
        raise ValueError(f"ALiBi bias was generated for {score_mod.nheads} heads but the query has {query.size(1)}")
    if softcap is not None and not softcap > 0:
        raise ValueError("softcap must be positive")
    out = run(query, key, value, scale=scale, enable_gqa=enable_gqa,
              mask_kind=_ffi.MASK_CAUSAL if is_causal else _ffi.MASK_NONE,
              alibi_heads=score_mod.nheads, softcap=float(softcap or 0.0))
    return grouped_view(out, key, enable_gqa)
