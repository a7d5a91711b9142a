"""`torch.library` registration of the fused forward, so that the variant functions trace into `torch.compile` graphs
as one opaque operator instead of breaking the graph at the ctypes call.

The reference reaches its fused kernel through `torch.compile(fn)` (benchmarks/run_flex_variants.py:118-124,
tests/test_causal.py:33); callers that keep that wrapper around the functions of this package get a graph that
contains `flashlight_amd::attn_fwd` once, with shapes and strides propagated by the fake implementation below.
Outside of tracing the front-ends call the C ABI directly (no dispatcher overhead).
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from . import _ffi

__all__ = ["attn_fwd", "attn_fwd_lse", "attn_bwd", "attn_fwd_bias_lse", "attn_bwd_bias", "dispatch"]


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
             gate: Optional[torch.Tensor], diff: bool, lambda_full: float, seq_major_out: bool, score_fn: int = 0,
             score_p0: float = 0.0, score_p1: float = 0.0, score_p2: float = 0.0, score_p3: float = 0.0) -> torch.Tensor:
    """Same arguments as `_ffi.attn_fwd`, flattened to what an operator schema can carry: scale <= 0 selects the
    default 1/sqrt(Dqk); bias operands with their batch divisors; `seq_major_out` asks for the result in [B, L, H, Dv]
    memory order; a score function as its kind and four constants."""
    out = _alloc_out(q, v, diff, seq_major_out)
    biases = [(b, d) for b, d in ((bias0, bias0_div), (bias1, bias1_div)) if b is not None]
    _ffi.attn_fwd(q, k, v, scale=scale if scale > 0 else None, mask_kind=mask_kind, window=window, prefix=prefix,
                  doc_ids=doc_ids, alibi_heads=alibi_heads, softcap=softcap, biases=biases, gate=gate, diff=diff,
                  lambda_full=lambda_full, out=out,
                  score_fn=(score_fn, (score_p0, score_p1, score_p2, score_p3)) if score_fn else None)
    return out


@attn_fwd.register_fake
def _attn_fwd_fake(q, k, v, scale, mask_kind, window, prefix, doc_ids, alibi_heads, softcap, bias0, bias0_div, bias1,
                   bias1_div, gate, diff, lambda_full, seq_major_out, score_fn=0, score_p0=0.0, score_p1=0.0, score_p2=0.0,
                   score_p3=0.0):
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


@torch.library.custom_op("flashlight_amd::attn_fwd_bias_lse", mutates_args=())
def attn_fwd_bias_lse(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, mask_kind: int, window: int,
                      prefix: int, bias0: Optional[torch.Tensor], bias0_div: int, bias1: Optional[torch.Tensor],
                      bias1_div: int, dropout_p: float = 0.0, dropout_seed: int = 0, doc_ids: Optional[torch.Tensor] = None,
                      alibi_heads: int = 0, softcap: float = 0.0) -> tuple[torch.Tensor, torch.Tensor]:
    """The forward with bias operands for calls that will be differentiated (the reference's Evoformer function and its
    dense `score_mod` tensors, attention_variants/evoformer.py:24-27, alibi.py:26-30; the reference itself has no
    backward): result and row statistics, like `attn_fwd_lse`.  An operator of its own, so that `torch.compile` traces
    the differentiable call and its backward like any other node."""
    out = _alloc_out(q, v, False, False)
    lse = torch.empty((q.size(0), q.size(1), q.size(2)), dtype=torch.float32, device=q.device)
    biases = [(b, d) for b, d in ((bias0, bias0_div), (bias1, bias1_div)) if b is not None]
    _ffi.attn_fwd(q, k, v, scale=scale if scale > 0 else None, mask_kind=mask_kind, window=window, prefix=prefix,
                  biases=biases, out=out, lse=lse, dropout_p=dropout_p, dropout_seed=dropout_seed, doc_ids=doc_ids,
                  alibi_heads=alibi_heads, softcap=softcap)
    return out, lse


@attn_fwd_bias_lse.register_fake
def _attn_fwd_bias_lse_fake(q, k, v, scale, mask_kind, window, prefix, bias0, bias0_div, bias1, bias1_div, dropout_p=0.0,
                            dropout_seed=0, doc_ids=None, alibi_heads=0, softcap=0.0):
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("query, key and value must be 4-D [batch, heads, seq, dim]")
    return _alloc_out(q, v, False, False), torch.empty((q.size(0), q.size(1), q.size(2)), dtype=torch.float32, device=q.device)


@torch.library.custom_op("flashlight_amd::attn_bwd_bias", mutates_args=())
def attn_bwd_bias(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, lse: torch.Tensor,
                  dout: torch.Tensor, scale: float, mask_kind: int, window: int, prefix: int,
                  bias0: Optional[torch.Tensor], bias0_div: int, bias1: Optional[torch.Tensor], bias1_div: int,
                  want_dscores: bool, dropout_p: float = 0.0, dropout_seed: int = 0,
                  doc_ids: Optional[torch.Tensor] = None, alibi_heads: int = 0,
                  softcap: float = 0.0) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dq, dk, dv, dscores) of `attn_fwd_bias_lse`: dscores, float32 [B, Hq, Lq, Lk], is the gradient with respect to
    whatever was added to q k^T scale (empty when `want_dscores` is false: no bias operand asks for a gradient)."""
    biases = [(b, d) for b, d in ((bias0, bias0_div), (bias1, bias1_div)) if b is not None]
    shape = (q.size(0), q.size(1), q.size(2), k.size(2)) if want_dscores else (0,)
    dscores = torch.zeros(shape, dtype=torch.float32, device=q.device)
    dq, dk, dv = _ffi.attn_bwd(q, k, v, out, lse, dout, scale=scale if scale > 0 else None, mask_kind=mask_kind,
                               window=window, prefix=prefix, biases=biases, dscores=dscores if want_dscores else None,
                               dropout_p=dropout_p, dropout_seed=dropout_seed, doc_ids=doc_ids, alibi_heads=alibi_heads,
                               softcap=softcap)
    return dq, dk, dv, dscores


@attn_bwd_bias.register_fake
def _attn_bwd_bias_fake(q, k, v, out, lse, dout, scale, mask_kind, window, prefix, bias0, bias0_div, bias1, bias1_div,
                        want_dscores, dropout_p=0.0, dropout_seed=0, doc_ids=None, alibi_heads=0, softcap=0.0):
    c = torch.contiguous_format
    shape = (q.size(0), q.size(1), q.size(2), k.size(2)) if want_dscores else (0,)
    return (torch.empty_like(q, memory_format=c), torch.empty_like(k, memory_format=c), torch.empty_like(v, memory_format=c),
            torch.empty(shape, dtype=torch.float32, device=q.device))


def _bias_setup_context(ctx, inputs, output):
    q, k, v, scale, mask_kind, window, prefix, bias0, div0, bias1, div1, dropout_p, dropout_seed, doc_ids, alibi_heads, \
        softcap = inputs
    out, lse = output
    ctx.save_for_backward(q, k, v, out, lse, bias0, bias1, doc_ids)
    ctx.args = (scale, mask_kind, window, prefix, div0, div1, dropout_p, dropout_seed, alibi_heads, softcap)


def _bias_backward(ctx, dout, dlse):
    """The gradient of a bias operand is the score gradient summed over the batch entries and axes the operand
    broadcasts over."""
    q, k, v, out, lse, bias0, bias1, doc_ids = ctx.saved_tensors
    scale, mask_kind, window, prefix, div0, div1, dropout_p, dropout_seed, alibi_heads, softcap = ctx.args
    want = [b is not None and ctx.needs_input_grad[7 + 2 * i] for i, b in enumerate((bias0, bias1))]
    dq, dk, dv, dscores = attn_bwd_bias(q, k, v, out, lse, dout.to(q.dtype), scale, mask_kind, window, prefix, bias0, div0,
                                        bias1, div1, any(want), dropout_p, dropout_seed, doc_ids, alibi_heads, softcap)
    dbs = []
    for b, d, w in ((bias0, div0, want[0]), (bias1, div1, want[1])):
        if not w:
            dbs.append(None)
            continue
        g = dscores.view(dscores.size(0) // d, d, *dscores.shape[1:]).sum(1)
        axes = [i for i in range(4) if b.size(i) == 1 and g.size(i) != 1]
        if axes:
            g = g.sum(axes, keepdim=True)
        dbs.append(g.to(b.dtype))
    return dq, dk, dv, None, None, None, None, dbs[0], None, dbs[1], None, None, None, None, None, None


attn_fwd_bias_lse.register_autograd(_bias_backward, setup_context=_bias_setup_context)


def _differentiable(q, k, v, *, scale, mask_kind, window, prefix, doc_ids, alibi_heads, softcap, biases, gate, diff,
                    lambda_full, dropout_p, dropout_seed):
    """The forward as a composition every part of which has a backward: the sigmoid gate and the difference of the two
    softmax branches are applied as tensor operations around the fused calls (one call per branch and per slab of as
    many value columns as the head dim, since the backward kernels take equal head dims)."""
    if diff:
        h, hk, d = q.size(1) // 2, k.size(1) // 2, q.size(3)
        if v.size(3) % d:
            raise NotImplementedError("gradients of differential attention need a value width that is a multiple of the head dim")
        parts = []
        for br in range(2):
            qb, kb = q[:, br * h:(br + 1) * h], k[:, br * hk:(br + 1) * hk]
            parts.append(torch.cat([_differentiable(qb, kb, v[..., c:c + d], scale=scale, mask_kind=mask_kind, window=window,
                                                    prefix=prefix, doc_ids=doc_ids, alibi_heads=alibi_heads, softcap=softcap,
                                                    biases=biases, gate=None, diff=False, lambda_full=0.0,
                                                    dropout_p=dropout_p, dropout_seed=dropout_seed).float()
                                    for c in range(0, v.size(3), d)], dim=-1))
        out = (parts[0] - lambda_full * parts[1]).to(q.dtype)
    elif biases:
        if softcap and any(b.requires_grad for b, _ in biases):
            raise NotImplementedError("gradients of bias operands are not built under a soft-cap (gradients of q, k and v "
                                      "are: pass the operands detached)")
        bl = list(biases) + [(None, 1)] * (2 - len(biases))
        out, _ = attn_fwd_bias_lse(q, k, v, float(scale) if scale is not None else -1.0, int(mask_kind), int(window),
                                   int(prefix), bl[0][0], int(bl[0][1]), bl[1][0], int(bl[1][1]), dropout_p,
                                   int(dropout_seed), doc_ids, int(alibi_heads), float(softcap))
    else:
        out, _ = attn_fwd_lse(q, k, v, float(scale) if scale is not None else -1.0, int(mask_kind), int(window),
                              int(prefix), doc_ids, int(alibi_heads), float(softcap), dropout_p, int(dropout_seed))
    if gate is not None:
        out = (out.float() * torch.sigmoid(gate.float())).to(q.dtype)
    return out


_HEAD_DIMS = (32, 64, 128)


def _pad_head_dims(q, k, v, gate, diff, bias_only=True, min_dim=32):
    """(q, k, v, gate) with zero columns appended up to a compiled head dim, or None when the head dims are compiled as
    they are (32, 64, 128 for q, k and v alike; 256 and 512 for q and k with values in slabs of 128 columns; the 64/128 and
    128/256 pairs of differential attention) or when no padding would help."""
    dqk, dv = q.shape[-1], v.shape[-1]
    if not diff and dqk == dv and dqk in _HEAD_DIMS and not (dqk == 32 and min_dim > 32):
        return None  # the common case, decided first: this runs on every call
    if dqk != k.size(-1) or q.dim() != 4 or v.dim() != 4:
        return None  # left to the binding's own checks
    if diff:
        if dv != 2 * dqk or dqk > 128:
            return None
        pq = next(p for p in (64, 128) if p >= dqk)
        pv = 2 * pq
    elif (dqk, dv) in ((32, 64), (64, 128)) and bias_only:
        # compiled pairs (invariant point attention's channel counts land on them), with dense bias operands as the only
        # score modification; anything else goes to the square head dim, whose instances cover every combination
        return None
    elif dqk > 128 or dv > 128:
        if dqk > 512:
            return None
        pq, pv = (128 if dqk <= 128 else 256 if dqk <= 256 else 512), -(-dv // 128) * 128
    else:
        pq = pv = next(p for p in _HEAD_DIMS if p >= max(dqk, dv, min_dim))
    if (pq, pv) == (dqk, dv):
        return None
    pad = torch.nn.functional.pad
    return (pad(q, (0, pq - dqk)), pad(k, (0, pq - dqk)), pad(v, (0, pv - dv)),
            None if gate is None else pad(gate, (0, pv - dv)))


def _split_over_keys(q, k, v, scale, softcap, biases=()):
    """Few queries against many keys (a decoding step over a long cache): B * Hq workgroups cannot fill 256 CUs, so the
    keys are cut into C chunks that run as C times as many heads of one launch, each leaving a normalised partial result
    and its row statistic, and a second small launch merges the partial results with the weights 2^(lse_c - max).  Returns None when the
    call is not of that shape (enough workgroups already, short or indivisible key length, key / value tensors whose
    heads are not contiguous in memory when there is more than one batch entry), and the caller launches as usual."""
    B, Hq, Lq, D = q.shape
    Hkv, Lk, Dv = k.size(1), k.size(2), v.size(3)
    groups = B * Hq * ((Lq + 127) // 128)
    # (a workgroup walks about 64 keys per microsecond; the copy of q, the row statistics and the merge launch cost
    # about 20: worth it from 4096 keys on)
    if groups >= 256 or Lk < 4096 or Hq % Hkv:
        return None
    whole = k.is_contiguous() and v.is_contiguous()
    # a cache that is a slice of a longer buffer (dense rows, heads further apart): with one batch entry the chunks can
    # be the batch entries of the launch instead of heads
    rows_dense = B == 1 and k.stride(3) == 1 and v.stride(3) == 1 and k.stride(2) == D and v.stride(2) == Dv
    if not (whole or rows_dense):
        return None
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    if rows_dense:
        # one batch entry (also when the cache is one block): the chunks are the batch entries of the launch, which reads
        # the queries with batch stride 0 (no copy).  Chunks of a multiple of 8 keys; what is left over at the end of a key
        # length that does not divide is one more, shorter chunk from a launch of its own
        chunks = next((c for c in (64, 32, 16, 8, 4, 2) if (Lk // c) // 8 * 8 >= 512 and groups * c <= 2048), 0)
        if not chunks:
            return None
        Lc = (Lk // chunks) // 8 * 8
        main = chunks * Lc
        kc = k.as_strided((chunks, Hkv, Lc, D), (Lc * D, k.stride(1), D, 1), k.storage_offset())
        vc = v.as_strided((chunks, Hkv, Lc, Dv), (Lc * Dv, v.stride(1), Dv, 1), v.storage_offset())
        bc = [(b[..., :main].reshape(chunks, 1, 1, Lc), 1) for b, _ in biases]   # ([1, 1, 1, Lk] rows: chunk c is entry c)
        total = chunks + (1 if main < Lk else 0)   # (both launches write into one pair of buffers)
        lse = torch.empty(total, Hq, Lq, dtype=torch.float32, device=q.device)
        part = torch.empty(total, Hq, Lq, Dv, dtype=q.dtype, device=q.device)
        _ffi.attn_fwd(q.expand(chunks, Hq, Lq, D), kc, vc, scale=scale, softcap=softcap, lse=lse[:chunks], biases=bc,
                      out=part[:chunks])
        if main < Lk:
            _ffi.attn_fwd(q, k[:, :, main:], v[:, :, main:], scale=scale, softcap=softcap, lse=lse[chunks:],
                          biases=[(b[..., main:], 1) for b, _ in biases], out=part[chunks:])
        return _ffi.merge_chunks(part.view(1, total, Hq * Lq, Dv), lse.view(1, total, Hq * Lq)).view(1, Hq, Lq, Dv)
    chunks = 0
    for c in (64, 32, 16, 8, 4, 2):
        if Lk % c == 0 and Lk // c >= 512 and (Lk // c) % 8 == 0 and groups * c <= 2048:
            chunks = c
            break
    if not chunks:
        return None
    G, Lc = Hq // Hkv, Lk // chunks
    # chunk c of key / value head h becomes head h * C + c; its G query heads are copies of the G of head h
    qc = q.reshape(B, Hkv, 1, G, Lq, D).expand(B, Hkv, chunks, G, Lq, D).reshape(B, Hkv * chunks * G, Lq, D)
    kc, vc = k.view(B, Hkv * chunks, Lc, D), v.view(B, Hkv * chunks, Lc, Dv)
    # (biases here are rows of keys, [Nb, 1, 1, Lk]: chunk c of a row goes with chunk c of every head)
    bc = [(b.view(b.size(0), 1, chunks, 1, Lc).expand(b.size(0), Hkv, chunks, G, Lc).reshape(b.size(0), Hkv * chunks * G, 1, Lc), d)
          for b, d in biases]
    lse = torch.empty(B, Hkv * chunks * G, Lq, dtype=torch.float32, device=q.device)
    part = _ffi.attn_fwd(qc, kc, vc, scale=scale, softcap=softcap, lse=lse, biases=bc)
    # one small launch: weights 2^(lse_c - max) over the chunks of a row; a chunk, or a row, without keys counts as zeros
    merged = _ffi.merge_chunks(part.view(B * Hkv, chunks, G * Lq, Dv), lse.view(B * Hkv, chunks, G * Lq))
    return merged.view(B, Hq, Lq, Dv)


def _being_traced(*tensors) -> bool:
    """True while Dynamo captures the caller, and while a tracer (AOTAutograd / make_fx under a compiler backend) runs
    it on stand-in tensors: fake, functional or proxy tensors are subclasses and hold no memory to launch on, so such
    calls go through the registered operators, which every tracer records as one node."""
    return torch.compiler.is_compiling() or any(type(t) is not torch.Tensor for t in tensors if t is not None)


def dispatch(q, k, v, *, scale=None, mask_kind=_ffi.MASK_NONE, window=0, prefix=0, doc_ids=None, alibi_heads=0,
             softcap=0.0, biases=(), gate=None, diff=False, lambda_full=0.0, seq_major_out=False, dropout_p=0.0,
             dropout_seed=None, doc_workspace=None, score_fn=None) -> torch.Tensor:
    """What the front-ends call: the registered operator while `torch.compile` is tracing, the C ABI otherwise; the
    differentiable operator when a gradient with respect to q, k or v will be asked for.

    `dropout_p` > 0 drops softmax weights (the reference's functions ignore their `dropout_p`; see
    `attention_variants.honor_dropout`).  `dropout_seed=None` draws a fresh 63-bit seed from torch's default CPU
    generator, so `torch.manual_seed` reproduces a run; the same seed gives the same decisions in forward and backward.
    `doc_workspace` (an `_ffi.DocWorkspace`) is used by the plain forward call only; traced and differentiable calls run
    their pre-pass every time.  `score_fn` = (kind, four constants), see `_ffi.attn_fwd`: forward only."""
    dropout_p = float(dropout_p)
    _ffi.dropout_threshold(dropout_p)  # range check
    if q.dim() == 4 and k.dim() == 4 and v.dim() == 4 and q.is_cuda and (q.numel() == 0 or k.size(2) == 0):
        # no batch entries, heads or queries: an empty result; queries but no keys: zeros (a softmax over nothing times no
        # values), as the eager functions give.  Nothing to launch; the zeros still hang on the operands for autograd.
        out = _alloc_out(q, v, diff, seq_major_out).zero_()
        if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v)):
            out = out + (q.sum() + k.sum() + v.sum()).to(out.dtype) * 0
        return out
    padded = _pad_head_dims(q, k, v, gate, diff,
                            bias_only=not (alibi_heads or softcap or doc_ids is not None or gate is not None or dropout_p > 0.0
                                           or score_fn is not None),
                            # (score functions and dropout are compiled from head dim 64 up)
                            min_dim=64 if (score_fn is not None or dropout_p > 0.0) else 32)
    if padded is not None:
        # head dims between the compiled ones: zero columns change neither q.k nor the columns of the result that are
        # kept (the reference's generated kernel takes any head dim up to 256 in one block, monkeypatch/fusion/_common.py:4,
        # and loops over wider ones, monkeypatch/fusion/reduction_kernel_fusion.py:1102; here up to 512)
        qp, kp, vp, gp = padded
        if scale is None:
            scale = 1.0 / math.sqrt(q.size(-1))
        out = dispatch(qp, kp, vp, scale=scale, mask_kind=mask_kind, window=window, prefix=prefix, doc_ids=doc_ids,
                       alibi_heads=alibi_heads, softcap=softcap, biases=biases, gate=gp, diff=diff, lambda_full=lambda_full,
                       seq_major_out=seq_major_out, dropout_p=dropout_p, dropout_seed=dropout_seed,
                       doc_workspace=doc_workspace, score_fn=score_fn)
        return out[..., :v.size(-1)]
    if dropout_p > 0.0:
        if diff or seq_major_out:
            raise NotImplementedError("dropout is not built for differential attention and sequence-major results")
        if dropout_seed is None:
            if _being_traced(q, k, v):
                raise NotImplementedError("dropout under torch.compile needs an explicit dropout_seed (a seed drawn "
                                          "while tracing would be frozen into the graph)")
            dropout_seed = int(torch.randint(0, 2 ** 63 - 1, (1,), dtype=torch.int64).item())
    else:
        dropout_seed = 0
    wants_grad = torch.is_grad_enabled() and any(
        t is not None and t.requires_grad for t in (q, k, v, gate, *(b for b, _ in biases)))
    if score_fn is not None and (wants_grad or dropout_p > 0.0):
        raise NotImplementedError("score functions other than the tanh soft-cap are forward-only and take no dropout")
    if wants_grad or (dropout_p > 0.0 and _being_traced(q, k, v)):
        # (the result comes back in [B, H, L, Dv] memory order whatever seq_major_out asks for)
        return _differentiable(q, k, v, scale=scale, mask_kind=mask_kind, window=window, prefix=prefix, doc_ids=doc_ids,
                               alibi_heads=alibi_heads, softcap=softcap, biases=biases, gate=gate, diff=diff,
                               lambda_full=lambda_full, dropout_p=dropout_p, dropout_seed=dropout_seed)
    rows_independent = mask_kind == _ffi.MASK_NONE and gate is None and not diff and doc_ids is None and not alibi_heads \
        and score_fn is None and dropout_p == 0.0 and not seq_major_out and \
        all(b.dim() == 4 and b.size(1) == 1 and b.size(2) == 1 for b, _ in biases)
    if rows_independent:
        Hq, Hkv, Lq = q.size(1), k.size(1), q.size(2)
        if Hq > Hkv and Hq % Hkv == 0 and (Hq // Hkv) * Lq <= 128 and q.is_contiguous():
            # few queries per head under grouped heads (a decoding step): without a mask the rows of a score matrix are
            # independent, so the G query heads of one key / value head are G times as many rows of that head (a view
            # of q), and one workgroup reads the keys for all of them instead of G workgroups reading them G times
            # (a bias that is one row of keys per batch entry, a padding mask, is the same for every row and goes along)
            packed = dispatch(q.view(q.size(0), Hkv, (Hq // Hkv) * Lq, q.size(3)), k, v, softcap=softcap, biases=biases,
                              scale=scale if scale is not None else 1.0 / math.sqrt(q.size(-1)))
            return packed.view(q.size(0), Hq, Lq, v.size(3))
    if _being_traced(q, k, v):
        bl = list(biases) + [(None, 1)] * (2 - len(biases))
        fn_kind, fn_c = (int(score_fn[0]), [float(c) for c in score_fn[1]]) if score_fn is not None else (0, [0.0] * 4)
        return attn_fwd(q, k, v, float(scale) if scale is not None else -1.0, int(mask_kind), int(window), int(prefix),
                        doc_ids, int(alibi_heads), float(softcap), bl[0][0], int(bl[0][1]), bl[1][0], int(bl[1][1]), gate,
                        bool(diff), float(lambda_full), bool(seq_major_out), fn_kind, fn_c[0], fn_c[1], fn_c[2], fn_c[3])
    if rows_independent:
        split = _split_over_keys(q, k, v, scale, softcap, biases) if all(b.is_contiguous() for b, _ in biases) else None
        if split is not None:
            return split
    out = _alloc_out(q, v, diff, seq_major_out) if seq_major_out else None
    return _ffi.attn_fwd(q, k, v, scale=scale, mask_kind=mask_kind, window=window, prefix=prefix, doc_ids=doc_ids,
                         alibi_heads=alibi_heads, softcap=softcap, biases=biases, gate=gate, diff=diff,
                         lambda_full=lambda_full, out=out, dropout_p=dropout_p, dropout_seed=dropout_seed,
                         doc_workspace=doc_workspace, score_fn=score_fn)
