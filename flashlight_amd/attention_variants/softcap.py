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


class _Poly:
    """A traced value that is a polynomial of the score x of degree <= 3, plus an optional tensor addend."""

    def __init__(self, c=(0.0, 1.0, 0.0, 0.0), tensor=None):
        self.c, self.tensor = [float(v) for v in c], tensor

    @property
    def degree(self) -> int:
        return max((i for i, v in enumerate(self.c) if v != 0.0), default=0)


class _Fn:
    """A traced value of the form post * f(a x + b) + shift (+ tensor), f = tanh, sigmoid or clamp to [lo, hi]."""

    def __init__(self, kind, a, b, lo=0.0, hi=0.0, post=1.0, shift=0.0, tensor=None):
        self.kind, self.a, self.b, self.lo, self.hi = kind, float(a), float(b), float(lo), float(hi)
        self.post, self.shift, self.tensor = float(post), float(shift), tensor


def _add_tensor(a, b):
    return b if a is None else (a if b is None else a + b)


def _scaled(v, c: float):
    t = None if v.tensor is None else v.tensor * c
    if isinstance(v, _Poly):
        return _Poly([x * c for x in v.c], t)
    return _Fn(v.kind, v.a, v.b, v.lo, v.hi, v.post * c, v.shift * c, t)


def _shifted(v, b):
    if isinstance(b, torch.Tensor) or v.tensor is not None:  # (a number joins a tensor addend that is already there)
        out = _scaled(v, 1.0)
        out.tensor = _add_tensor(v.tensor, b)
        return out
    if isinstance(v, _Poly):
        return _Poly([v.c[0] + float(b)] + v.c[1:], v.tensor)
    return _Fn(v.kind, v.a, v.b, v.lo, v.hi, v.post, v.shift + float(b), v.tensor)


def _product(p: _Poly, q: _Poly) -> _Poly:
    if p.tensor is not None or q.tensor is not None or p.degree + q.degree > 3:
        raise NotImplementedError("score_mod forms a product the fused kernel has no form for (polynomials up to the cube)")
    c = [0.0] * 4
    for i, x in enumerate(p.c):
        for j, y in enumerate(q.c):
            if x != 0.0 and y != 0.0:
                c[i + j] += x * y
    return _Poly(c)


def analyse_score_mod(score_mod):
    """Finds out what an arbitrary `score_mod(score, b, h, q_idx, kv_idx)` does to the score matrix by tracing it with
    torch.fx on a symbolic score (softcap.py:49 calls it on the whole scaled score matrix).  Understood: sums, products
    and quotients with numbers, sums with tensors, powers and products up to the cube, and one tanh, sigmoid, ReLU or
    clamp of a linear function of the score.
    Returns (scale multiplier, soft cap or 0.0, additive tensor or None, score function or None): either the first
    two describe the call (`mult * x`, or `cap * tanh(mult * x / cap)`: what the soft-cap kernels take, which covers
    attn_gym's generate_tanh_softcap(cap, approx=False) however it is spelled), or the last is
    (`_ffi.SCORE_*` kind, four constants) for `fl_attn_params.score_fn`; raises NotImplementedError for anything the
    fused kernel cannot apply in registers."""
    import math
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
    traced = (_Poly, _Fn)

    def num(a):
        return isinstance(a, (int, float)) and not isinstance(a, bool)

    def get(a):
        return val[a] if isinstance(a, fx.Node) else a

    def linear_arg(x, what):
        if not (isinstance(x, _Poly) and x.tensor is None and x.degree <= 1):
            raise NotImplementedError(f"score_mod applies {what} to something other than a linear function of the score")
        return x.c[1], x.c[0]

    F = torch.nn.functional
    for n in graph.nodes:
        if n.op == "placeholder":
            val[n] = _Poly()
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
            kw = {k: get(v) for k, v in n.kwargs.items()}
            if t in (operator.mul, torch.mul, torch.Tensor.mul) and len(a) == 2:
                if isinstance(a[0], _Poly) and isinstance(a[1], _Poly):
                    val[n] = _product(a[0], a[1])
                    continue
                x, c = (a[0], a[1]) if isinstance(a[0], traced) else (a[1], a[0])
                if isinstance(x, traced) and num(c):
                    val[n] = _scaled(x, float(c))
                    continue
            if t in (operator.truediv, torch.div, torch.Tensor.div, torch.true_divide) and len(a) == 2:
                if isinstance(a[0], traced) and num(a[1]) and a[1] != 0:
                    val[n] = _scaled(a[0], 1.0 / float(a[1]))
                    continue
            if t in (operator.add, torch.add, torch.Tensor.add) and len(a) == 2 and not kw:
                if isinstance(a[0], _Poly) and isinstance(a[1], _Poly):
                    val[n] = _Poly([x + y for x, y in zip(a[0].c, a[1].c)], _add_tensor(a[0].tensor, a[1].tensor))
                    continue
                x, c = (a[0], a[1]) if isinstance(a[0], traced) else (a[1], a[0])
                if isinstance(x, traced) and (num(c) or isinstance(c, torch.Tensor)):
                    val[n] = _shifted(x, c)
                    continue
            if t in (operator.sub, torch.sub, torch.Tensor.sub) and len(a) == 2 and not kw:
                if isinstance(a[0], _Poly) and isinstance(a[1], _Poly):
                    val[n] = _Poly([x - y for x, y in zip(a[0].c, a[1].c)],
                                   _add_tensor(a[0].tensor, None if a[1].tensor is None else -a[1].tensor))
                    continue
                if isinstance(a[0], traced) and (num(a[1]) or isinstance(a[1], torch.Tensor)):
                    val[n] = _shifted(a[0], -a[1])
                    continue
                if isinstance(a[1], traced) and (num(a[0]) or isinstance(a[0], torch.Tensor)):
                    val[n] = _shifted(_scaled(a[1], -1.0), a[0])
                    continue
            if t in (operator.neg, torch.neg, torch.Tensor.neg) and len(a) == 1 and isinstance(a[0], traced):
                val[n] = _scaled(a[0], -1.0)
                continue
            if t in (operator.pow, torch.pow, torch.Tensor.pow) and len(a) == 2 and isinstance(a[0], _Poly) and a[1] in (1, 2, 3):
                r = a[0]
                for _ in range(int(a[1]) - 1):
                    r = _product(r, a[0])
                val[n] = r
                continue
            if t in (torch.square, torch.Tensor.square) and len(a) == 1 and isinstance(a[0], _Poly):
                val[n] = _product(a[0], a[0])
                continue
            if t in (torch.tanh, torch.Tensor.tanh, F.tanh) and len(a) == 1 and isinstance(a[0], traced):
                val[n] = _Fn("tanh", *linear_arg(a[0], "tanh"))
                continue
            if t in (torch.sigmoid, torch.Tensor.sigmoid, F.sigmoid) and len(a) == 1 and isinstance(a[0], traced):
                val[n] = _Fn("sigmoid", *linear_arg(a[0], "sigmoid"))
                continue
            if t in (torch.relu, torch.Tensor.relu, F.relu) and a and isinstance(a[0], traced):
                val[n] = _Fn("clamp", *linear_arg(a[0], "relu"), lo=0.0, hi=math.inf)
                continue
            if t in (torch.clamp, torch.Tensor.clamp, torch.clip, torch.Tensor.clip) and a and isinstance(a[0], traced):
                lo = a[1] if len(a) > 1 else kw.get("min")
                hi = a[2] if len(a) > 2 else kw.get("max")
                if (lo is None or num(lo)) and (hi is None or num(hi)) and not (lo is None and hi is None):
                    val[n] = _Fn("clamp", *linear_arg(a[0], "clamp"), lo=-math.inf if lo is None else lo,
                                 hi=math.inf if hi is None else hi)
                    continue
            if t in (torch.clamp_min, torch.Tensor.clamp_min) and len(a) == 2 and isinstance(a[0], traced) and num(a[1]):
                val[n] = _Fn("clamp", *linear_arg(a[0], "clamp_min"), lo=a[1], hi=math.inf)
                continue
            if t in (torch.clamp_max, torch.Tensor.clamp_max) and len(a) == 2 and isinstance(a[0], traced) and num(a[1]):
                val[n] = _Fn("clamp", *linear_arg(a[0], "clamp_max"), lo=-math.inf, hi=a[1])
                continue
            raise NotImplementedError(f"score_mod applies {getattr(t, '__name__', t)} to the scores in a way the fused kernel "
                                      "has no form for (understood: + - * / with numbers, + tensors, powers up to the cube, "
                                      "one tanh / sigmoid / relu / clamp of a linear function of the score)")
        else:
            raise NotImplementedError(f"score_mod uses {n.op}")
    if not isinstance(out, traced):
        raise NotImplementedError("score_mod does not return a function of the score")
    bias = out.tensor if isinstance(out.tensor, torch.Tensor) else None
    if isinstance(out, _Poly):
        # (a number added to every score changes no softmax: the constant term is dropped where the form has no place for it)
        if out.degree <= 1 and out.c[1] > 0:
            return out.c[1], 0.0, bias, None
        if out.degree == 0:
            raise NotImplementedError("score_mod does not depend on the score")
        return 1.0, 0.0, bias, (_ffi.SCORE_POLY, tuple(out.c))
    if out.kind == "tanh":
        # post * tanh(a x) = cap * tanh((a * cap) * x / cap) with cap = post
        if out.b != 0.0 or not (out.post > 0 and out.a > 0):
            raise NotImplementedError("tanh of a shifted score, or a soft-cap with a non-positive factor")
        return out.a * out.post, out.post, bias, None
    if out.post == 0.0 or out.a == 0.0:
        raise NotImplementedError("score_mod does not depend on the score")
    if out.kind == "sigmoid":
        return 1.0, 0.0, bias, (_ffi.SCORE_SIGMOID, (out.a, out.b, out.post, out.shift))
    # post * clamp(a x + b, lo, hi) + shift is a clamp of its own: the bounds change places under a negative factor
    lo, hi = out.post * out.lo + out.shift, out.post * out.hi + out.shift
    return 1.0, 0.0, bias, (_ffi.SCORE_CLAMP, (out.post * out.a, out.post * out.b + out.shift, min(lo, hi), max(lo, hi)))


def attention_softcapped(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, score_mod=None, attn_mask=None,
                         dropout_p=0.0, is_causal: bool = False, scale=None, enable_gqa: bool = False,
                         softcap_threshold: float = 30.0) -> torch.Tensor:
    """softcap.py:4-53: softmax(score_mod(q k^T * scale)) v.  `score_mod` is a `TanhSoftcap` (from
    `generate_tanh_softcap`) or any callable `(score, b, h, q_idx, kv_idx) -> score` that `analyse_score_mod` understands
    (e.g. attn_gym's own generate_tanh_softcap closure; a sigmoid, ReLU, clamp or polynomial of the score); None uses `softcap_threshold` as the cap (the reference
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
    mult, cap, bias, score_fn = analyse_score_mod(score_mod)
    base = 1.0 / math.sqrt(query.size(-1)) if scale is None else float(scale)
    out = run(query, key, value, scale=base * mult, enable_gqa=enable_gqa, mask_kind=mask_kind, softcap=cap,
              biases=[] if bias is None else [dense_bias_operand(bias, query, key, enable_gqa)], dropout_p=dropout_p,
              **({} if score_fn is None else {"score_fn": score_fn}))
    return grouped_view(out, key, enable_gqa)
