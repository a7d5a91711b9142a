"""The benchmark configurations evaluated by the oracle.  TEST INFRASTRUCTURE (see oracle/__init__.py).

`evaluate(name, tensors, params)` maps a benchmark workload's name (the part after "cfgN/") to the oracle function
that restates the reference variant it exercises, with the workload's own arguments; tensors may live on any device
(plain eager PyTorch either way) and are taken as they are (callers convert to fp32 first).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from . import attention as O


def evaluate(name: str, t: Dict[str, torch.Tensor], params: Dict[str, float], q_block: Optional[int] = None) -> torch.Tensor:
    n = name.split("/")[-1]
    q, k, v = t["q"], t["k"], t["v"]
    if n == "vanilla":
        return O.attention_vanilla(q, k, v, q_block=q_block)
    if n == "causal":
        return O.attention_causal(q, k, v, q_block=q_block)
    if n == "sliding_window":
        return O.attention_sliding_window(q, k, v, window_size=int(params["window"]), q_block=q_block)
    if n == "gqa_alibi_softcap_causal":
        return O.attention_alibi(q, k, v, score_mod=q.size(1), is_causal=True, honor_causal=True, enable_gqa=True,
                                 softcap=float(params["softcap"]), q_block=q_block)
    if n == "document_mask_causal":
        return O.attention_document_mask(q, k, v, t["document_id"], is_causal=True, q_block=q_block)
    if n == "prefix_lm":
        return O.attention_prefix_lm(q, k, v, prefix_lengths=int(params["prefix"]), q_block=q_block)
    if n == "diff_attn_causal":
        return O.diff_attention(q, k, v, lambda_full=float(params["lambda_full"]), is_causal=True, q_block=q_block)
    if n == "evoformer_bias_gate":
        return O.attention_evoformer(q, k, v, [t["pair_bias"]], gate=t["gate"], q_block=q_block)
    raise KeyError(name)
