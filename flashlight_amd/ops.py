"""`torch.library` registration of the fused forward, so that the variant functions trace into `torch.compile` graphs
as one opaque operator instead of breaking the graph at the ctypes call.

The reference reaches its fused kernel through `torch.compile(fn)` (benchmarks/run_flex_variants.py:118-124,
tests/test_causal.py:33); callers that keep that wrapper around the functions of this package get a graph that
contains `flashlight_amd::attn_fwd` once, with shapes and strides propagated by the fake implementation below.
Outside of tracing the front-ends call the C ABI directly (no dispatcher overhead).
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _ffi

__all__ = ["attn_fwd", "dispatch"]


def _out_shape(q: torch.Tensor, v: torch.Tensor, diff: bool):
    return q.size(0), q.size(1) // (2 if diff else 1), q.size(2), v.size(3)


def _alloc_out(q: torch.Tensor, v: torch.Tensor, diff: bool, seq_major_out: bool) -> torch.Tensor:
    B, H, L, Dv = _out_shape(q, v, diff)
    if seq_major_out:  # memory order [B, L, H, Dv] (the Evoformer layout), returned as its [B, H, L, Dv] view
        return torch.empty((B, L, H, Dv), dtype=torch.bfloat16, device=q.device).transpose(1, 2)
    return torch.empty((B, H, L, Dv), dtype=torch.bfloat16, device=q.device)


@torch.library.custom_op("flashlight_amd::attn_fwd", mutates_args=())
def attn_fwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, mask_kind: int, window: int, prefix: int,
             doc_ids: Optional[torch.Tensor], alibi_heads: int, softcap: float,
             bias0: Optional[torch.Tensor], bias0_div: int, bias1: Optional[torch.Tensor], bias1_div: int,
             gate: Optional[torch.Tensor], diff: bool, lambda_full: float, seq_major_out: bool) -> torch.Tensor:
    """Same arguments as `_ffi.attn_fwd`, flattened to what an operator schema can carry: scale <= 0 selects the
    default 1/sqrt(Dqk); bias operands with their batch divisors; `seq_major_out` asks for the result in [B, L, H, Dv]
    memory order."""
    out = _alloc_out(q, v, diff, seq_major_out)
    biases = [(b, d) for b, d in ((bias0, bias0_div), (bias1, bias1_div)) if b is not None]
    _ffi.attn_fwd(q, k, v, scale=scale if scale > 0 else None, mask_kind=mask_kind, window=window, prefix=prefix,
                  doc_ids=doc_ids, alibi_heads=alibi_heads, softcap=softcap, biases=biases, gate=gate, diff=diff,
                  lambda_full=lambda_full, out=out)
    return out


@attn_fwd.register_fake
def _attn_fwd_fake(q, k, v, scale, mask_kind, window, prefix, doc_ids, alibi_heads, softcap, bias0, bias0_div, bias1,
                   bias1_div, gate, diff, lambda_full, seq_major_out):
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("query, key and value must be 4-D [batch, heads, seq, dim]")
    return _alloc_out(q, v, diff, seq_major_out)


def dispatch(q, k, v, *, scale=None, mask_kind=_ffi.MASK_NONE, window=0, prefix=0, doc_ids=None, alibi_heads=0,
             softcap=0.0, biases=(), gate=None, diff=False, lambda_full=0.0, seq_major_out=False) -> torch.Tensor:
    """What the front-ends call: the registered operator while `torch.compile` is tracing, the C ABI otherwise."""
    if torch.compiler.is_compiling():
        bl = list(biases) + [(None, 1)] * (2 - len(biases))
        return attn_fwd(q, k, v, float(scale) if scale is not None else -1.0, int(mask_kind), int(window), int(prefix),
                        doc_ids, int(alibi_heads), float(softcap), bl[0][0], int(bl[0][1]), bl[1][0], int(bl[1][1]), gate,
                        bool(diff), float(lambda_full), bool(seq_major_out))
    out = _alloc_out(q, v, diff, seq_major_out) if seq_major_out else None
    return _ffi.attn_fwd(q, k, v, scale=scale, mask_kind=mask_kind, window=window, prefix=prefix, doc_ids=doc_ids,
                         alibi_heads=alibi_heads, softcap=softcap, biases=biases, gate=gate, diff=diff,
                         lambda_full=lambda_full, out=out)
