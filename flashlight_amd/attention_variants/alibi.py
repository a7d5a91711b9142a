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
    """alibi.py:13-33: softmax(q k^T * scale + bias) v with bias = score_mod(L, S).

    With `score_mod = generate_alibi_bias_pytorch(num_query_heads)` (what the reference's tests and benchmarks pass:
    tests/test_alibi.py:32, benchmarks/run_flex_variants.py:129-131) the kernel computes the ALiBi term from the head
    index and the positions and no [H, L, S] tensor exists.  Any other callable is called once, as the reference does
    (alibi.py:26), and the dense tensor it returns (bf16 or fp32, broadcastable to [N, Hq, L, S]; viewed
    [Hkv, G, L, S] under GQA like alibi.py:27-28) is added to the scores by the kernel's additive-bias path.

    Two additions over the reference, both off by default: `is_causal=True` masks k > q (the reference accepts the
    flag and ignores it), and `softcap=c` replaces the scaled score x by c * tanh(x / c) before the bias is added."""
    if score_mod is None:
        raise TypeError("attention_pytorch_alibi needs score_mod, e.g. generate_alibi_bias_pytorch(num_query_heads)")
    if softcap is not None and not softcap > 0:
        raise ValueError("softcap must be positive")
    mask_kind = _ffi.MASK_CAUSAL if is_causal else _ffi.MASK_NONE
    if isinstance(score_mod, AlibiBias):
        if score_mod.nheads != query.size(1):
            raise ValueError(f"ALiBi bias was generated for {score_mod.nheads} heads but the query has {query.size(1)}")
        out = run(query, key, value, scale=scale, enable_gqa=enable_gqa, mask_kind=mask_kind,
                  alibi_heads=score_mod.nheads, softcap=float(softcap or 0.0), dropout_p=dropout_p)
        return grouped_view(out, key, enable_gqa)
    if not callable(score_mod):
        raise TypeError("score_mod must be callable as score_mod(q_len, kv_len)")
    bias = dense_bias_operand(score_mod(query.size(-2), key.size(-2)), query, key, enable_gqa)
    out = run(query, key, value, scale=scale, enable_gqa=enable_gqa, mask_kind=mask_kind, biases=[bias],
              softcap=float(softcap or 0.0), dropout_p=dropout_p)
    return grouped_view(out, key, enable_gqa)


def dense_bias_operand(bias, query: torch.Tensor, key: torch.Tensor, enable_gqa: bool = False):
    """Maps a dense additive term, broadcastable to the scores [N, Hq, L, S], onto the kernel's
    ([N|1, Hq|1, L|1, S] tensor, batch divisor) form.  bf16 and fp32 are read as they are (fp32 keeps terms that grow
    with the distance exact); other dtypes are converted to fp32."""
    if not isinstance(bias, torch.Tensor):
        raise TypeError(f"score_mod must return a tensor, got {type(bias).__name__}")
    n, hq, l, s = query.size(0), query.size(1), query.size(-2), key.size(-2)
    if enable_gqa:  # the reference views the tensor as [Hkv, G, L, S] (alibi.py:27-28): same memory as [Hq, L, S]
        bias = bias.reshape(hq, l, s)
    if bias.dim() > 4:
        raise ValueError(f"bias of shape {tuple(bias.shape)} has more axes than the scores")
    bias = bias.reshape((1,) * (4 - bias.dim()) + tuple(bias.shape))
    for got, want in zip(bias.shape, (n, hq, l, s)):
        if got not in (1, want):
            raise ValueError(f"bias of shape {tuple(bias.shape)} does not broadcast to the scores {(n, hq, l, s)}")
    if bias.dtype != torch.float32 and bias.dtype != query.dtype:
        bias = bias.to(torch.float32)
    if bias.device != query.device:
        bias = bias.to(query.device)
    if bias.size(3) != s:
        bias = bias.expand(*bias.shape[:3], s).contiguous()
    return bias, (n if bias.size(0) == 1 else 1)
