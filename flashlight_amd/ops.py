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

__all__ = ["attn_fwd", "attn_fwd_lse", "attn_bwd", "dispatch"]


def _out_shape(q: torch.Tensor, v: torch.Tensor, diff: bool):
    return q.size(0), q.size(1) // (2 if diff else 1), q.size(2), v.size(3)


def _alloc_out(q: torch.Tensor, v: torch.Tensor, diff: bool, seq_major_out: bool) -> torch.Tensor:
    B, H, L, Dv = _out_shape(q, v, diff)
    if seq_major_out:  # memory order [B, L, H, Dv] (the Evoformer layout), returned as its [B, H, L, Dv] view
        return torch.empty((B, L, H, Dv), dtype=q.dtype, device=q.device).transpose(1, 2)
    return torch.empty((B, H, L, Dv), dtype=q.dtype, device=q.device)


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


@torch.library.custom_op("flashlight_amd::attn_fwd_lse", mutates_args=())
def attn_fwd_lse(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, mask_kind: int, window: int, prefix: int,
                 doc_ids: Optional[torch.Tensor], alibi_heads: int, softcap: float, dropout_p: float = 0.0,
                 dropout_seed: int = 0) -> tuple[torch.Tensor, torch.Tensor]:
    """The forward for calls that will be differentiated: also returns the row statistics (float32 [B, Hq, Lq], log2 of
    each row's sum of 2^logit) from which `attn_bwd` recomputes the weights.  The reference has no backward; this
    operator carries the autograd rule registered below.  It is also the operator for a forward with dropout: which
    weights are dropped is a function of `dropout_seed`, so the backward needs no mask from the forward."""
    out = _alloc_out(q, v, False, False)
    lse = torch.empty((q.size(0), q.size(1), q.size(2)), dtype=torch.float32, device=q.device)
    _ffi.attn_fwd(q, k, v, scale=scale if scale > 0 else None, mask_kind=mask_kind, window=window, prefix=prefix,
                  doc_ids=doc_ids, alibi_heads=alibi_heads, softcap=softcap, out=out, lse=lse, dropout_p=dropout_p,
                  dropout_seed=dropout_seed)
    return out, lse


@attn_fwd_lse.register_fake
def _attn_fwd_lse_fake(q, k, v, scale, mask_kind, window, prefix, doc_ids, alibi_heads, softcap, dropout_p=0.0,
                       dropout_seed=0):
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("query, key and value must be 4-D [batch, heads, seq, dim]")
    return _alloc_out(q, v, False, False), torch.empty((q.size(0), q.size(1), q.size(2)), dtype=torch.float32, device=q.device)


@torch.library.custom_op("flashlight_amd::attn_bwd", mutates_args=())
def attn_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, lse: torch.Tensor, dout: torch.Tensor,
             scale: float, mask_kind: int, window: int, prefix: int, doc_ids: Optional[torch.Tensor], alibi_heads: int,
             softcap: float, dropout_p: float = 0.0,
             dropout_seed: int = 0) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dq, dk, dv) of `attn_fwd_lse` for the output gradient `dout`."""
    return _ffi.attn_bwd(q, k, v, out, lse, dout, scale=scale if scale > 0 else None, mask_kind=mask_kind, window=window,
                         prefix=prefix, doc_ids=doc_ids, alibi_heads=alibi_heads, softcap=softcap, dropout_p=dropout_p,
                         dropout_seed=dropout_seed)


@attn_bwd.register_fake
def _attn_bwd_fake(q, k, v, out, lse, dout, scale, mask_kind, window, prefix, doc_ids, alibi_heads, softcap,
                   dropout_p=0.0, dropout_seed=0):
    c = torch.contiguous_format
    return torch.empty_like(q, memory_format=c), torch.empty_like(k, memory_format=c), torch.empty_like(v, memory_format=c)


def _setup_context(ctx, inputs, output):
    q, k, v, scale, mask_kind, window, prefix, doc_ids, alibi_heads, softcap, dropout_p, dropout_seed = inputs
    out, lse = output
    ctx.save_for_backward(q, k, v, out, lse)
    ctx.doc_ids = doc_ids
    ctx.args = (scale, mask_kind, window, prefix, alibi_heads, softcap, dropout_p, dropout_seed)


def _backward(ctx, dout, dlse):
    q, k, v, out, lse = ctx.saved_tensors
    scale, mask_kind, window, prefix, alibi_heads, softcap, dropout_p, dropout_seed = ctx.args
    dq, dk, dv = attn_bwd(q, k, v, out, lse, dout.to(q.dtype), scale, mask_kind, window, prefix, ctx.doc_ids,
                          alibi_heads, softcap, dropout_p, dropout_seed)
    return dq, dk, dv, None, None, None, None, None, None, None, None, None


attn_fwd_lse.register_autograd(_backward, setup_context=_setup_context)


def dispatch(q, k, v, *, scale=None, mask_kind=_ffi.MASK_NONE, window=0, prefix=0, doc_ids=None, alibi_heads=0,
             softcap=0.0, biases=(), gate=None, diff=False, lambda_full=0.0, seq_major_out=False, dropout_p=0.0,
             dropout_seed=None) -> torch.Tensor:
    """What the front-ends call: the registered operator while `torch.compile` is tracing, the C ABI otherwise; the
    differentiable operator when a gradient with respect to q, k or v will be asked for.

    `dropout_p` > 0 drops softmax weights (the reference's functions ignore their `dropout_p`; see
    `attention_variants.honor_dropout`).  `dropout_seed=None` draws a fresh 63-bit seed from torch's default CPU
    generator, so `torch.manual_seed` reproduces a run; the same seed gives the same decisions in forward and backward."""
    dropout_p = float(dropout_p)
    _ffi.dropout_threshold(dropout_p)  # range check
    if dropout_p > 0.0:
        if biases or gate is not None or diff or seq_major_out:
            raise NotImplementedError("dropout is built for positional masks, the in-kernel ALiBi term and the soft-cap; not "
                                      "for bias operands, the gate or differential attention")
        if dropout_seed is None:
            if torch.compiler.is_compiling():
                raise NotImplementedError("dropout under torch.compile needs an explicit dropout_seed (a seed drawn "
                                          "while tracing would be frozen into the graph)")
            dropout_seed = int(torch.randint(0, 2 ** 63 - 1, (1,), dtype=torch.int64).item())
    else:
        dropout_seed = 0
    if (torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)) or \
            (dropout_p > 0.0 and torch.compiler.is_compiling()):
        if biases or gate is not None or diff or seq_major_out:
            raise NotImplementedError(
                "no backward is implemented for bias operands, the sigmoid gate or differential attention: call under "
                "torch.no_grad() (or detach the inputs) if only the forward is wanted")
        out, _ = attn_fwd_lse(q, k, v, float(scale) if scale is not None else -1.0, int(mask_kind), int(window),
                              int(prefix), doc_ids, int(alibi_heads), float(softcap), dropout_p, int(dropout_seed))
        return out
    if torch.compiler.is_compiling():
        bl = list(biases) + [(None, 1)] * (2 - len(biases))
        return attn_fwd(q, k, v, float(scale) if scale is not None else -1.0, int(mask_kind), int(window), int(prefix),
                        doc_ids, int(alibi_heads), float(softcap), bl[0][0], int(bl[0][1]), bl[1][0], int(bl[1][1]), gate,
                        bool(diff), float(lambda_full), bool(seq_major_out))
    out = _alloc_out(q, v, diff, seq_major_out) if seq_major_out else None
    return _ffi.attn_fwd(q, k, v, scale=scale, mask_kind=mask_kind, window=window, prefix=prefix, doc_ids=doc_ids,
                         alibi_heads=alibi_heads, softcap=softcap, biases=biases, gate=gate, diff=diff,
                         lambda_full=lambda_full, out=out, dropout_p=dropout_p, dropout_seed=dropout_seed)
