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


class _Affine:
    """What a traced score_mod has made of the score x so far: `post * f(pre * x) + bias`, f = tanh or the identity."""

    def __init__(self, pre=1.0, post=1.0, tanh=False, bias=None):
        self.pre, self.post, self.tanh, self.bias = pre, post, tanh, bias

    def scaled(self, c: float) -> "_Affine":
        if self.tanh:
            return _Affine(self.pre, self.post * c, True, None if self.bias is None else self.bias * c)
        return _Affine(self.pre * c, 1.0, False, None if self.bias is None else self.bias * c)

    def shifted(self, b) -> "_Affine":
        return _Affine(self.pre, self.post, self.tanh, b if self.bias is None else self.bias + b)


def analyse_score_mod(score_mod):
    """Finds out what an arbitrary `score_mod(score, b, h, q_idx, kv_idx)` does to the score matrix by tracing it with
    torch.fx on a symbolic score (softcap.py:49 calls it on the whole scaled score matrix).  Understood: products and
    quotients with numbers, one tanh, sums with numbers or tensors — i.e. `post * tanh(pre * x) + bias` or
    `pre * x + bias`, which covers attn_gym's generate_tanh_softcap(cap, approx=False) however it is spelled.
    Returns (scale multiplier, soft cap or 0.0, additive tensor or None); raises NotImplementedError for anything the
    fused kernel cannot apply in registers."""
    import operator

    import torch.fx as fx

    class _Wrap(torch.nn.Module):
        def forward(self, score):
            return score_mod(score, 0, 0, None, None)

    try:
        gm = fx.symbolic_trace(_Wrap())
        graph = gm.graph
    except Exception as e:  # data-dependent control flow, non-torch calls on the score ...
        raise NotImplementedError(f"score_mod could not be traced ({type(e).__name__}: {e})") from e
    val = {}

    def num(a):
        return isinstance(a, (int, float)) and not isinstance(a, bool)

    def get(a):
        return val[a] if isinstance(a, fx.Node) else a

    for n in graph.nodes:
        if n.op == "placeholder":
            val[n] = _Affine()
        elif n.op == "get_attr":
            obj = gm  # tensors the callable closes over are lifted into attributes of the traced module
            for part in n.target.split("."):
                obj = getattr(obj, part)
            val[n] = obj
        elif n.op == "output":
            out = get(n.args[0])
        elif n.op in ("call_function", "call_method"):
            t = n.target if n.op == "call_function" else getattr(torch.Tensor, n.target, n.target)
            a = [get(x) for x in n.args]
            if t in (operator.mul, torch.mul, torch.Tensor.mul) and len(a) == 2:
                x, c = (a[0], a[1]) if isinstance(a[0], _Affine) else (a[1], a[0])
                if isinstance(x, _Affine) and num(c):
                    val[n] = x.scaled(float(c))
                    continue
            if t in (operator.truediv, torch.div, torch.Tensor.div, torch.true_divide) and len(a) == 2:
                if isinstance(a[0], _Affine) and num(a[1]) and a[1] != 0:
                    val[n] = a[0].scaled(1.0 / float(a[1]))
                    continue
            if t in (operator.add, torch.add, torch.Tensor.add) and len(a) == 2 and not n.kwargs:
                x, c = (a[0], a[1]) if isinstance(a[0], _Affine) else (a[1], a[0])
                if isinstance(x, _Affine) and (num(c) or isinstance(c, torch.Tensor)):
                    val[n] = x.shifted(c)
                    continue
            if t in (operator.sub, torch.sub, torch.Tensor.sub) and len(a) == 2 and not n.kwargs:
                if isinstance(a[0], _Affine) and (num(a[1]) or isinstance(a[1], torch.Tensor)):
                    val[n] = a[0].shifted(-a[1])
                    continue
            if t in (torch.tanh, torch.Tensor.tanh) and len(a) == 1 and isinstance(a[0], _Affine):
                if not a[0].tanh and a[0].bias is None:
                    val[n] = _Affine(a[0].pre, 1.0, True, None)
                    continue
            raise NotImplementedError(f"score_mod applies {getattr(t, '__name__', t)} to the scores, which the fused kernel "
                                      "cannot do in registers (understood: * and / by numbers, tanh, + tensors)")
        else:
            raise NotImplementedError(f"score_mod uses {n.op}")
    if not isinstance(out, _Affine):
        raise NotImplementedError("score_mod does not return a function of the score")
    bias = out.bias if isinstance(out.bias, torch.Tensor) else None  # a number added to every score changes nothing
    if out.tanh:
        # post * tanh(pre * x) = cap * tanh((pre * cap) * x / cap) with cap = post
        if not (out.post > 0 and out.pre > 0):
            raise NotImplementedError("soft-cap with a non-positive factor")
        return out.pre * out.post, out.post, bias
    if not out.pre > 0:
        raise NotImplementedError("score_mod multiplies the scores by a non-positive number")
    return out.pre, 0.0, bias


def attention_softcapped(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, score_mod=None, attn_mask=None,
                         dropout_p=0.0, is_causal: bool = False, scale=None, enable_gqa: bool = False,
                         softcap_threshold: float = 30.0) -> torch.Tensor:
    """softcap.py:4-53: softmax(score_mod(q k^T * scale)) v.  `score_mod` is a `TanhSoftcap` (from
    `generate_tanh_softcap`) or any callable `(score, b, h, q_idx, kv_idx) -> score` that `analyse_score_mod` understands
    (e.g. attn_gym's own generate_tanh_softcap closure); None uses `softcap_threshold` as the cap (the reference
    declares that parameter but never reads it).  `is_causal=True` masks k > q (accepted and ignored by the
    reference)."""
    if score_mod is None:
        score_mod = TanhSoftcap(softcap_threshold)
    mask_kind = _ffi.MASK_CAUSAL if is_causal else _ffi.MASK_NONE
    if isinstance(score_mod, TanhSoftcap):
        out = run(query, key, value, scale=scale, enable_gqa=enable_gqa, mask_kind=mask_kind, softcap=score_mod.soft_cap,
                  dropout_p=dropout_p)
        return grouped_view(out, key, enable_gqa)
    if not callable(score_mod):
        raise TypeError("score_mod must be callable as score_mod(score, b, h, q_idx, kv_idx)")
    # any other callable: traced once to see what it does to the scores (raises NotImplementedError when that is
    # something the kernel cannot apply in registers)
    import math

    from .alibi import dense_bias_operand
    mult, cap, bias = analyse_score_mod(score_mod)
    base = 1.0 / math.sqrt(query.size(-1)) if scale is None else float(scale)
    out = run(query, key, value, scale=base * mult, enable_gqa=enable_gqa, mask_kind=mask_kind, softcap=cap,
              biases=[] if bias is None else [dense_bias_operand(bias, query, key, enable_gqa)], dropout_p=dropout_p)
    return grouped_view(out, key, enable_gqa)
