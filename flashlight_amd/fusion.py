"""Graph rewrite: eager attention written out in PyTorch -> one fused launch.

The reference turns `torch.compile(fn)` of an eager attention function (matmul -> score modifications -> softmax ->
matmul, attention_variants/*.py) into one generated kernel by patching TorchInductor
(`from monkeypatch.fusion import ...`, tests/test_causal.py:14-17).  This module is the counterpart for callers who
keep their own eager functions: `torch.compile(fn, backend=flashlight_amd.fusion.backend, dynamic=False)` captures the
function with Dynamo, finds every region of that shape in the FX graph and replaces it by a call into the hand-written
kernel (`flashlight_amd::attn_fwd`); whatever else the function does keeps running as ordinary eager PyTorch.

A call of `torch.nn.functional.scaled_dot_product_attention` in the captured function is a region by itself (mask,
dropout_p, is_causal, scale, enable_gqa as PyTorch defines them).  What a written-out region may contain, from the first
matmul to the second:
  q @ k.transpose(-2, -1)  [* scale | / scale]  [cap * tanh(x / cap)]  {+ bias | masked_fill / where(mask, fill, x)}*
  -> softmax(dim=-1) [-> type_as / to] -> @ v
with q/k/v of any rank >= 3 (leading axes are batch; `query.view(N, Hkv, G, L, E)` with `key.unsqueeze(2)` is
grouped-query attention, and so is a key / value whose heads were repeated to match the query's: `repeat_kv`,
`repeat_interleave`) and masks/biases broadcastable to the scores.

Masks and biases are recognised by what they compute, not by how they were written:
  * a mask that depends on no graph input is evaluated once at compile time and compared with the closed forms of the
    kernel's positional masks (causal, sliding window, prefix-LM); anything else becomes a constant additive -inf bias;
  * a mask that depends on one integer [N, L] input is probed with random ids and compared with the document
    predicates (same document, optionally k <= q); anything else stays in the graph and is converted to an additive
    bias at run time;
  * a constant bias equal to 2^(-8 (h + 1) / H) * (k - q) is ALiBi and is computed inside the kernel; other biases are
    passed to the kernel's bias operands (fp32 or bf16).
A training-mode dropout on the softmax weights becomes the kernel's own dropout (same rate, the kernel's random
stream, a fresh seed per call) where the dropout kernels cover the region: head dims up to 128, no score function
other than the soft-cap.  Regions that do not fit (a softmax whose weights are used elsewhere, dropout
outside that coverage, ...) are left untouched.
"""
from __future__ import annotations

import math
import operator
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch
import torch.fx as fx

from . import _ffi, ops

__all__ = ["backend", "fuse_attention", "fused_attention"]

_NEG_INF = float("-inf")


# ---- node helpers ------------------------------------------------------------------------------------------------------

def _name(n: Any) -> Optional[str]:
    """Canonical operation name of a call node: 'matmul' for torch.matmul / operator.matmul / Tensor.matmul, ..."""
    if not isinstance(n, fx.Node):
        return None
    if n.op == "call_method":
        s = n.target
    elif n.op == "call_function":
        s = getattr(n.target, "__name__", str(n.target))
    else:
        return None
    s = s.strip("_") if s.startswith("__") else s
    return {"imatmul": "matmul", "truediv": "div", "itruediv": "div", "iadd": "add", "imul": "mul", "add_": "add",
            "mul_": "mul", "div_": "div", "masked_fill_": "masked_fill", "bmm": "matmul", "isub": "sub"}.get(s, s)


def _val(n: fx.Node):
    v = n.meta.get("example_value", n.meta.get("val"))
    if v is None:
        raise _NoMatch(f"no example value recorded for {n.name}")
    return v


def _is_number(x) -> bool:
    return isinstance(x, (int, float)) and not isinstance(x, bool)


class _NoMatch(Exception):
    pass


def _arg(n: fx.Node, i: int, kw: str, default=None):
    if len(n.args) > i:
        return n.args[i]
    return n.kwargs.get(kw, default)


def _is_last2_transpose(n: Any) -> Optional[fx.Node]:
    """Returns x when n is x with its last two axes swapped."""
    nm = _name(n)
    if nm == "transpose":
        d0, d1 = _arg(n, 1, "dim0"), _arg(n, 2, "dim1")
        nd = _val(n.args[0]).dim()
        if isinstance(d0, int) and isinstance(d1, int) and {d0 % nd, d1 % nd} == {nd - 1, nd - 2}:
            return n.args[0]
    if nm == "permute":
        dims = n.args[1:] if len(n.args) > 2 else tuple(_arg(n, 1, "dims"))
        nd = len(dims)
        want = list(range(nd - 2)) + [nd - 1, nd - 2]
        if [d % nd for d in dims] == want:
            return n.args[0]
    if n.op == "call_function" and n.target is getattr and n.args[1] == "mT":
        return n.args[0]
    return None


def _placeholders_of(n: fx.Node) -> List[fx.Node]:
    seen, out, stack = set(), [], [n]
    while stack:
        x = stack.pop()
        if x in seen:
            continue
        seen.add(x)
        if x.op == "placeholder":
            out.append(x)
        stack.extend(x.all_input_nodes)
    return out


def _evaluate(n: Any, env: Dict[fx.Node, Any], gm: fx.GraphModule):
    """Runs the subgraph that produces `n` eagerly; `env` maps placeholders (and already computed nodes) to values."""
    if isinstance(n, (tuple, list)):
        return type(n)(_evaluate(x, env, gm) for x in n)
    if isinstance(n, dict):
        return {k: _evaluate(v, env, gm) for k, v in n.items()}
    if isinstance(n, slice):
        return slice(_evaluate(n.start, env, gm), _evaluate(n.stop, env, gm), _evaluate(n.step, env, gm))
    if not isinstance(n, fx.Node):
        return n
    if n in env:
        return env[n]
    if n.op == "placeholder":
        raise _NoMatch(f"subgraph reads graph input {n.name}")
    args, kwargs = _evaluate(n.args, env, gm), _evaluate(n.kwargs, env, gm)
    if n.op == "call_function":
        r = n.target(*args, **kwargs)
    elif n.op == "call_method":
        r = getattr(args[0], n.target)(*args[1:], **kwargs)
    elif n.op == "get_attr":
        r = gm
        for part in n.target.split("."):
            r = getattr(r, part)
    elif n.op == "call_module":
        r = gm.get_submodule(n.target)(*args, **kwargs)
    else:
        raise _NoMatch(f"cannot evaluate {n.op}")
    env[n] = r
    return r


def _try_evaluate(n: fx.Node, gm: fx.GraphModule):
    """Value of a subgraph without graph inputs, or None when it cannot be computed at compile time."""
    try:
        return _evaluate(n, {}, gm)
    except Exception:
        return None


# ---- what the positional masks look like (True = masked) ---------------------------------------------------------------------

def _idx(L: int, S: int, device):
    return torch.arange(L, device=device).view(L, 1), torch.arange(S, device=device).view(1, S)


def _classify_constant_mask(m: torch.Tensor, L: int, S: int):
    """m: bool, broadcastable to [..., L, S], True = masked.  Returns (mask_kind, window, prefix) when it equals one of the
    kernel's positional masks on every leading index, else None."""
    if m.dim() < 2:
        m = m.reshape((1,) * (2 - m.dim()) + tuple(m.shape))
    if m.size(-2) not in (1, L) or m.size(-1) not in (1, S):
        return None
    m = m.reshape(-1, m.size(-2), m.size(-1))
    if m.size(0) > 1 and not bool((m == m[:1]).all()):
        return None
    m = m[0].expand(L, S)
    q, k = _idx(L, S, m.device)
    if not bool(m.any()):
        return _ffi.MASK_NONE, 0, 0
    if bool((m == (k > q)).all()):
        return _ffi.MASK_CAUSAL, 0, 0
    if L == S:
        w = int((~m[L - 1]).sum().item()) - 1
        if w >= 0 and bool((m == ((q < k) | ((q - k) > w))).all()):
            return _ffi.MASK_SLIDING, w, 0
        p = int((~m[0]).sum().item())
        if p >= 1 and bool((m == (k > torch.clamp(q, min=p - 1))).all()):
            return _ffi.MASK_PREFIX_LM, 0, p
    return None


def _classify_document_mask(node: fx.Node, ids_ph: fx.Node, invert: bool, L: int, S: int, gm: fx.GraphModule):
    """Probes the mask subgraph, a function of one integer [N, L] input, with random ids.  Returns MASK_DOCUMENT or
    MASK_DOCUMENT_CAUSAL when its output equals that predicate for every probe, else None."""
    ex = _val(ids_ph)
    if L != S or ex.dim() != 2 or ex.size(1) != L or ex.dtype not in (torch.int64, torch.int32):
        return None
    N, dev = ex.size(0), ex.device
    g = torch.Generator(device="cpu").manual_seed(1234)
    probes = [torch.randint(0, 3, (N, L), generator=g).sort(dim=1).values,
              torch.randint(-5, 7, (N, L), generator=g),
              torch.zeros(N, L, dtype=torch.int64)]
    q, k = _idx(L, S, dev)
    found = None
    for ids in probes:
        ids = ids.to(device=dev, dtype=ex.dtype)
        try:
            m = _evaluate(node, {ids_ph: ids}, gm)
        except Exception:  # the subgraph needs something a probe cannot give it
            return None
        if not isinstance(m, torch.Tensor) or m.dtype != torch.bool:
            return None
        if invert:
            m = ~m
        if m.dim() < 3 or m.size(0) not in (1, N):
            return None
        same = ids.unsqueeze(2) != ids.unsqueeze(1)                                  # [N, L, S], True = masked
        lead = (N,) + (1,) * (m.dim() - 3)
        ok_doc = bool((m == same.view(*lead, L, S)).all())
        ok_causal = bool((m == (same | (k > q)).view(*lead, L, S)).all())
        got = _ffi.MASK_DOCUMENT if ok_doc else _ffi.MASK_DOCUMENT_CAUSAL if ok_causal else None
        if ok_doc and ok_causal:  # a probe that cannot tell the two apart
            continue
        if got is None or (found is not None and found != got):
            return None
        found = got
    return found


def _is_alibi(b: torch.Tensor, H: int, L: int, S: int) -> bool:
    """b broadcastable to [H, L, S] (or [Hkv, G, L, S]) and equal to 2^(-8 (h + 1) / H) (k - q) (alibi.py:5-9)."""
    if b.numel() != H * L * S:
        return False
    b = b.reshape(H, L, S).to(torch.float32)
    slopes = torch.exp2(-8.0 * torch.arange(1, H + 1, device=b.device, dtype=torch.float32) / H)
    q, k = _idx(L, S, b.device)
    want = slopes.view(H, 1, 1) * (k - q).to(torch.float32)
    return bool(((b - want).abs() <= 1e-5 * want.abs() + 1e-6).all())


# ---- the run-time side: what the replacement node calls -----------------------------------------------------------------------

def _kernel_bias(b: torch.Tensor, lead: Tuple[int, ...], heads: Tuple[int, ...], L: int, S: int,
                 qdtype: torch.dtype = torch.bfloat16):
    """Maps a tensor broadcastable to the scores [*lead, *heads, L, S] onto the kernel's ([Nb, H|1, L|1, S], batch divisor)
    form (batch index = flat_batch // divisor), copying only when the broadcast pattern has no such form."""
    nl, nh = len(lead), len(heads)
    nd = nl + nh + 2
    if b.dim() > nd:
        raise ValueError(f"bias of shape {tuple(b.shape)} has more axes than the scores")
    b = b.reshape((1,) * (nd - b.dim()) + tuple(b.shape))
    for got, want in zip(b.shape, (*lead, *heads, L, S)):
        if got not in (1, want):
            raise ValueError(f"bias of shape {tuple(b.shape)} does not broadcast to the scores {(*lead, *heads, L, S)}")
    if b.dtype == torch.bool:
        raise TypeError("boolean biases are masks; use masked_fill / where")
    if b.dtype != torch.float32 and b.dtype != qdtype:
        b = b.to(torch.float32)
    if b.size(-1) != S:
        b = b.expand(*b.shape[:-1], S)
    hs = tuple(b.shape[nl:nl + nh])
    if not (all(h == 1 for h in hs) or hs == tuple(heads)):  # e.g. full over kv heads, broadcast over the group
        b = b.expand(*b.shape[:nl], *heads, *b.shape[nl + nh:])
        hs = tuple(heads)
    H = math.prod(hs)
    bl = tuple(b.shape[:nl])
    split = nl
    while split > 0 and bl[split - 1] == 1:
        split -= 1
    if any(bl[i] != lead[i] for i in range(split)):
        b = b.expand(*lead, *b.shape[nl:])
        bl, split = tuple(lead), nl
    div = math.prod(lead[split:]) if split < nl else 1
    nb = math.prod(bl[:split]) if split else 1
    return b.reshape(nb, H, b.shape[-2], S), int(div)


def fused_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, doc_ids: Optional[torch.Tensor],
                    biases: Sequence[torch.Tensor], masks: Sequence[torch.Tensor], *, scale: float, mask_kind: int,
                    window: int, prefix: int, alibi_heads: int, softcap: float, gqa: bool,
                    mask_invert: Sequence[bool] = (), diff_lambda: Optional[float] = None, score_fn=None,
                    dropout_p: float = 0.0) -> torch.Tensor:
    """Target of the replacement node.  q [*lead, H, L, E] (or [N, Hkv, G, L, E] with `gqa`), k/v likewise with S keys;
    `biases` are added to the scaled scores, `masks` (bool, True = masked unless the matching `mask_invert` entry is
    set) are those the rewrite could not map to a positional or document mask.  Returns what the eager region
    returned: [*q.shape[:-1], Ev].  With `diff_lambda` q and k hold the heads of both softmax branches (first half,
    second half) and the result is branch 0 minus diff_lambda times branch 1.  `dropout_p` > 0 (a training-mode dropout
    on the softmax weights in the eager region) drops weights inside the kernel; each call draws its seed from torch's
    default CPU generator, so `torch.manual_seed` reproduces a run, but the weights dropped are not the ones
    `torch.nn.functional.dropout` would have dropped for that seed."""
    L, S = q.size(-2), k.size(-2)
    result_shape = (*q.shape[:-1], v.size(-1))
    if gqa:
        lead, heads = (q.size(0),), (q.size(1), q.size(2))
        q4 = q.reshape(q.size(0), -1, L, q.size(-1))
        k4, v4 = k.squeeze(2), v.squeeze(2)
    else:
        if q.dim() == 3:  # [N, L, E]: one head; operands with a batch axis of their own get the head axis too
            q = q.unsqueeze(1)
            biases = [b.unsqueeze(-3) if b.dim() == 3 else b for b in biases]
            masks = [m.unsqueeze(-3) if m.dim() == 3 else m for m in masks]
        lead, heads = tuple(q.shape[:-3]), (q.size(-3),)

        def like_q(t):  # key/value with missing or size-1 leading axes broadcast like matmul operands do
            if t.dim() == 3 and len(lead) == 1:
                t = t.unsqueeze(1)
            t = t.reshape((1,) * (q.dim() - t.dim()) + tuple(t.shape))
            return t if tuple(t.shape[:-3]) == lead else t.expand(*lead, *t.shape[-3:])

        q4, k4, v4 = (t.reshape(-1, *t.shape[-3:]) for t in (q, like_q(k), like_q(v)))
    kb = [_kernel_bias(b, lead, heads, L, S, q.dtype) for b in biases]
    for i, m in enumerate(masks):
        if i < len(mask_invert) and mask_invert[i]:
            m = ~m
        add = torch.zeros(m.shape, dtype=q.dtype, device=m.device).masked_fill_(m, _NEG_INF)
        kb.append(_kernel_bias(add, lead, heads, L, S, q.dtype))
    while len(kb) > 2:  # the kernel takes two operands: fold the rest into the last one
        (b1, d1), (b2, d2) = kb[-2], kb[-1]
        if d1 != d2:  # different batch groupings: give both one row per flat batch index
            b1, b2 = (b.repeat_interleave(d, dim=0) if d > 1 else b for b, d in ((b1, d1), (b2, d2)))
            d1 = 1
        kb[-2:] = [(b1.float() + b2.float(), d1)]
    if diff_lambda is None:
        out = ops.dispatch(q4, k4, v4, scale=scale, mask_kind=mask_kind, window=window, prefix=prefix, doc_ids=doc_ids,
                           alibi_heads=alibi_heads, softcap=softcap, biases=kb, score_fn=score_fn, dropout_p=dropout_p)
        return out.reshape(result_shape)
    out = ops.dispatch(q4, k4, v4, scale=scale, mask_kind=mask_kind, window=window, prefix=prefix, doc_ids=doc_ids,
                       alibi_heads=alibi_heads, softcap=softcap, biases=kb, diff=True, lambda_full=float(diff_lambda))
    return out.reshape(*result_shape[:-3], result_shape[-3] // 2, *result_shape[-2:])


def fused_multi_head_attention(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, *, num_heads: int,
                               in_proj_weight, in_proj_bias, q_proj_weight, k_proj_weight, v_proj_weight,
                               out_proj_weight, out_proj_bias, dropout_p: float, key_padding_mask, attn_mask,
                               is_causal: bool):
    """Target of the node that replaces a call of torch.nn.functional.multi_head_attention_forward (what
    torch.nn.MultiheadAttention and the Transformer layers built on it call; Dynamo keeps it as one node, so its
    scaled_dot_product_attention is not visible to the rewrite).  query [L, N, E], key / value [S, N, *] (or without
    the batch axis); the three input projections and the output projection run as torch linears, the attention
    between them on the fused kernel with the heads read in place.  Masks follow that function's conventions: a
    boolean `attn_mask` ([L, S] or [N * H, L, S]) or `key_padding_mask` ([N, S]) is True where a key is NOT attended,
    any other dtype is added to the scores; `is_causal` says that `attn_mask` is the causal mask, and is taken at
    its word only when there is no padding mask, as that function does.  Returns (result [L, N, E], None)."""
    import torch.nn.functional as F
    batched = query.dim() == 3
    if not batched:
        query, key, value = query.unsqueeze(1), key.unsqueeze(1), value.unsqueeze(1)
        if key_padding_mask is not None:
            key_padding_mask = key_padding_mask.unsqueeze(0)
    (L, N, E), S, H = query.shape, key.size(0), num_heads
    if is_causal and attn_mask is None:
        raise RuntimeError("is_causal needs the causal attn_mask it speaks of")
    if q_proj_weight is None:
        wq, wk, wv = in_proj_weight.chunk(3)
    else:
        wq, wk, wv = q_proj_weight, k_proj_weight, v_proj_weight
    bq, bk, bv = in_proj_bias.chunk(3) if in_proj_bias is not None else (None, None, None)
    if q_proj_weight is None and key is query and value is query:
        q, k, v = F.linear(query, in_proj_weight, in_proj_bias).chunk(3, dim=-1)   # self-attention: one product
    else:
        q, k, v = F.linear(query, wq, bq), F.linear(key, wk, bk), F.linear(value, wv, bv)
    hd = E // H
    q, k, v = (t.reshape(t.size(0), N, H, hd).permute(1, 2, 0, 3) for t in (q, k, v))   # [N, H, L | S, hd], in place
    biases, masks = [], []
    kind = _ffi.MASK_NONE
    if is_causal and key_padding_mask is None:
        kind = _ffi.MASK_CAUSAL
    elif attn_mask is not None:
        am = attn_mask if attn_mask.dim() == 2 else attn_mask.reshape(N, H, L, S)
        (masks if am.dtype == torch.bool else biases).append(am)
    if key_padding_mask is not None:
        kp = key_padding_mask.reshape(N, 1, 1, S)
        (masks if kp.dtype == torch.bool else biases).append(kp)
    out = fused_attention(q, k, v, None, biases, masks, scale=1.0 / math.sqrt(hd), mask_kind=kind, window=0, prefix=0,
                          alibi_heads=0, softcap=0.0, gqa=False, dropout_p=dropout_p)
    out = F.linear(out.permute(2, 0, 1, 3).reshape(L * N, E), out_proj_weight, out_proj_bias).reshape(L, N, E)
    return (out if batched else out.squeeze(1)), None


# ---- matching ----------------------------------------------------------------------------------------------------------------

class _Region:
    def __init__(self):
        self.nodes: List[fx.Node] = []      # interior nodes to delete, consumer first
        self.q = self.k = self.v = None
        self.scale = 1.0
        self.softcap = 0.0
        self.score_fn = None                 # (kind, four constants) of fl_attn_params.score_fn
        self.dropout_p = 0.0                 # rate of a training-mode dropout between the softmax and the second matmul
        self.biases: List[fx.Node] = []
        self.masks: List[Tuple[fx.Node, bool]] = []   # (mask node, invert)
        self.out: Optional[fx.Node] = None
        self.causal = False                  # scaled_dot_product_attention(is_causal=True)


_PASS_OPS = ("to", "type", "type_as", "float", "bfloat16", "half", "contiguous", "clone")
_FN_OPS = ("relu", "sigmoid", "tanh", "clamp", "clip", "clamp_min", "clamp_max", "pow", "square", "neg", "sub", "rsub",
           "mul", "div", "add")


def _peel_function(n: fx.Node, r: _Region, qk_memo, mods_below: List[str]):
    """`n` and everything between it and the q k^T matmul is a function of the scores and numbers alone (no tensor
    enters): the chain is handed, as a callable, to the analysis the soft-cap front-end uses for a caller's score_mod
    (scale, tanh soft-cap, or one of the compiled-in score functions: sigmoid, clamp / ReLU, polynomial)."""
    from .attention_variants.softcap import analyse_score_mod
    chain: List[fx.Node] = []
    seen = set()
    root: List[Optional[fx.Node]] = [None]

    def visit(x: fx.Node):
        if x in seen:
            return
        nm = _name(x)
        if nm == "matmul" and len(x.args) >= 2 and _is_last2_transpose(x.args[1]) is not None:
            if root[0] is not None and root[0] is not x:
                raise _NoMatch("a function of two score matrices")
            root[0] = x
            seen.add(x)
            return
        if nm not in _FN_OPS and nm not in _PASS_OPS:
            raise _NoMatch(f"unsupported operation on the scores: {nm}")
        for a in list(x.args) + list(x.kwargs.values()):
            if isinstance(a, fx.Node):
                visit(a)
            elif not (a is None or _is_number(a) or isinstance(a, (torch.dtype, bool))):
                raise _NoMatch(f"{nm} of the scores with an argument that is not a number")
        seen.add(x)
        chain.append(x)

    visit(n)
    if root[0] is None:
        raise _NoMatch("scores do not come from a matmul")

    def fn(score, *_ignored):
        env = {root[0]: score}
        for x in chain:
            if _name(x) in _PASS_OPS:  # casts and copies leave the value as it is
                env[x] = env[x.args[0]]
                continue
            args = [env[a] if isinstance(a, fx.Node) else a for a in x.args]
            kwargs = {k: env[v] if isinstance(v, fx.Node) else v for k, v in x.kwargs.items()}
            env[x] = x.target(*args, **kwargs) if x.op == "call_function" else getattr(args[0], x.target)(*args[1:], **kwargs)
        return env[n]

    try:
        mult, cap, bias, score_fn = analyse_score_mod(fn)
    except NotImplementedError as e:
        raise _NoMatch(str(e)) from e
    if bias is not None or (cap and (r.softcap or "softcap" in mods_below)):
        raise _NoMatch("a second soft-cap, or a tensor inside the score function")
    r.scale *= mult
    if cap:
        r.softcap = cap
    r.score_fn = score_fn
    r.nodes += list(reversed(chain))
    mods_below.append("softcap" if (cap or score_fn is not None) else "scale")
    return _peel_scores(root[0], r, qk_memo, mods_below)


def _as_number(x) -> Optional[float]:
    """x as a float when it is a Python number or a one-element tensor that depends on no graph input (a fill written
    as `torch.tensor(float("-inf"))` or `torch.full((), -1e10)`), else None."""
    if _is_number(x):
        return float(x)
    if isinstance(x, fx.Node) and not _placeholders_of(x):
        ex = _val(x)
        if isinstance(ex, torch.Tensor) and ex.numel() == 1:
            got = _try_evaluate(x, x.graph.owning_module)
            if isinstance(got, torch.Tensor) and got.numel() == 1:
                return float(got.float().item())
    return None


def _peel_scores(n: Any, r: _Region, qk_memo, mods_below: List[str]):
    """Walks from the softmax input up to the q k^T matmul, recording what each step does to the scores."""
    nm = _name(n)
    if nm is None:
        raise _NoMatch("scores do not come from a matmul")
    if nm in _PASS_OPS:
        r.nodes.append(n)
        return _peel_scores(n.args[0], r, qk_memo, mods_below)
    if nm == "matmul":
        a, b = n.args[0], n.args[1]
        kt = _is_last2_transpose(b)
        if kt is None:
            raise _NoMatch("second matmul operand is not a transposed key")
        r.nodes.append(n)
        if len(b.users) == 1:
            r.nodes.append(b)
        r.q, r.k = a, kt
        return
    if nm in ("where",):
        cond, a, b = n.args[0], n.args[1], n.args[2]
        fa, fb = _as_number(a), _as_number(b)
        if isinstance(b, fx.Node) and fb is None and fa is not None and fa <= -1e9:
            r.masks.append((cond, False))
            inner = b
        elif isinstance(a, fx.Node) and fa is None and fb is not None and fb <= -1e9:
            r.masks.append((cond, True))
            inner = a
        else:
            raise _NoMatch("where() is not a mask fill")
        r.nodes.append(n)
        mods_below.append("mask")
        return _peel_scores(inner, r, qk_memo, mods_below)
    if nm == "masked_fill":
        inner, cond, fill = n.args[0], _arg(n, 1, "mask"), _as_number(_arg(n, 2, "value"))
        if fill is None or not fill <= -1e9:
            raise _NoMatch("masked_fill value is not a large negative number")
        r.masks.append((cond, False))
        r.nodes.append(n)
        mods_below.append("mask")
        return _peel_scores(inner, r, qk_memo, mods_below)
    if nm == "add":
        a, b = n.args[0], n.args[1]
        if _is_number(a) or _is_number(b):
            return _peel_function(n, r, qk_memo, mods_below)
        a_has = _contains_qk(a, qk_memo)
        if a_has and _contains_qk(b, qk_memo):
            return _peel_function(n, r, qk_memo, mods_below)  # a sum of two functions of the scores
        inner, bias = (a, b) if a_has else (b, a)
        if not a_has and not _contains_qk(b, qk_memo):
            raise _NoMatch("add without a score operand")
        r.biases.append(bias)
        r.nodes.append(n)
        mods_below.append("bias")
        return _peel_scores(inner, r, qk_memo, mods_below)
    if nm in ("mul", "div"):
        a, b = n.args[0], n.args[1]
        if nm == "mul" and _is_number(a):
            a, b = b, a
        if not _is_number(b) or not isinstance(a, fx.Node):
            if isinstance(n.args[0], fx.Node) and isinstance(n.args[1], fx.Node) and nm == "mul" \
                    and _contains_qk(n.args[0], qk_memo) and _contains_qk(n.args[1], qk_memo):
                return _peel_function(n, r, qk_memo, mods_below)  # a product of two functions of the scores
            raise _NoMatch("scores multiplied by a tensor")
        c = float(b) if nm == "mul" else 1.0 / float(b)
        if _name(a) == "tanh":  # cap * tanh(x / cap)
            t_in = a.args[0]
            nm2 = _name(t_in)
            if nm2 not in ("div", "mul") or not _is_number(t_in.args[1]):
                raise _NoMatch("tanh argument is not scores / cap")
            inv = 1.0 / float(t_in.args[1]) if nm2 == "div" else float(t_in.args[1])
            if not (c > 0 and abs(c * inv - 1.0) < 1e-6):
                raise _NoMatch("tanh soft-cap with mismatched constants")
            if r.softcap or "softcap" in mods_below:
                raise _NoMatch("two soft-caps")
            r.softcap = c
            r.nodes += [n, a, t_in]
            mods_below.append("softcap")
            return _peel_scores(t_in.args[0], r, qk_memo, mods_below)
        if not c > 0 or _name(a) in _FN_OPS and _name(a) not in ("mul", "div", "add"):
            return _peel_function(n, r, qk_memo, mods_below)  # a factor on a function of the scores, or a negative one
        r.scale *= c
        r.nodes.append(n)
        mods_below.append("scale")
        return _peel_scores(a, r, qk_memo, mods_below)
    if nm in _FN_OPS:
        return _peel_function(n, r, qk_memo, mods_below)
    raise _NoMatch(f"unsupported operation on the scores: {nm}")


def _contains_qk(n: Any, memo: Dict[fx.Node, bool]) -> bool:
    """True when `n` is reached from a (x @ transposed y) matmul through score-chain operations only."""
    if not isinstance(n, fx.Node):
        return False
    if n in memo:
        return memo[n]
    nm = _name(n)
    memo[n] = False
    if nm == "matmul" and len(n.args) >= 2 and _is_last2_transpose(n.args[1]) is not None:
        r = True
    elif nm in ("where", "masked_fill") or nm in _FN_OPS or nm in _PASS_OPS:
        r = any(_contains_qk(a, memo) for a in n.args if isinstance(a, fx.Node))
    else:
        r = False
    memo[n] = r
    return r


def _check_order(r: _Region, order_from_softmax: List[str]):
    """Kernel order: scale, soft-cap, then biases and masks (which commute).  Walking up from the softmax the chain must
    therefore read (bias|mask)* softcap? scale*."""
    stage = 0  # 0: biases/masks, 1: softcap seen, 2: scale seen
    for what in order_from_softmax:
        if what in ("bias", "mask"):
            if stage != 0:
                raise _NoMatch("a bias or mask is applied before the scale or the soft-cap")
        elif what == "softcap":
            if stage >= 1:
                raise _NoMatch("soft-cap applied before the scale")
            stage = 1
        elif what == "scale":
            stage = 2


def _match(softmax: fx.Node) -> _Region:
    dim = _arg(softmax, 1, "dim")
    x = softmax.args[0]
    nd = _val(softmax).dim()
    if not isinstance(dim, int) or dim % nd != nd - 1:
        raise _NoMatch("softmax is not over the last axis")
    r = _Region()
    order: List[str] = []
    _peel_scores(x, r, {}, order)
    _check_order(r, order)
    # downstream: [type_as / to]* -> matmul(p, v)
    cur = softmax
    tail = [softmax]
    while True:
        if len(cur.users) != 1:
            raise _NoMatch("the softmax weights have more than one consumer")
        (u,) = cur.users
        nm = _name(u)
        if nm in _PASS_OPS and u.args and u.args[0] is cur:
            tail.append(u)
            cur = u
            continue
        if nm == "dropout":
            p, training = _arg(u, 1, "p", 0.5), _arg(u, 2, "training", True)
            if not _is_number(p) or not isinstance(training, bool) or not 0.0 <= float(p) < 1.0:
                raise _NoMatch("dropout with a rate or mode that is not a constant")
            if training and float(p) > 0.0:
                if r.dropout_p:
                    raise _NoMatch("two dropouts on the softmax weights")
                r.dropout_p = float(p)
            tail.append(u)
            cur = u
            continue
        if nm == "matmul" and u.args[0] is cur and isinstance(u.args[1], fx.Node):
            r.v, r.out = u.args[1], u
            tail.append(u)
            break
        raise _NoMatch(f"softmax weights feed {nm}, not a matmul with the values")
    r.nodes = list(reversed(tail)) + r.nodes
    # interior values must not escape the region
    inside = set(r.nodes)
    for n in r.nodes:
        if n is r.out:
            continue
        for u in n.users:
            if u not in inside:
                raise _NoMatch(f"intermediate {n.name} is used outside the attention region")
    return r


def _match_sdpa(n: fx.Node) -> _Region:
    """torch.nn.functional.scaled_dot_product_attention(query, key, value, attn_mask=None, dropout_p=0.0,
    is_causal=False, scale=None, enable_gqa=False) as a region of its own: a boolean attn_mask is True where a key
    takes part, any other is added to the scaled scores; dropout_p applies whenever it is not 0."""
    q, k, v = (_arg(n, i, name) for i, name in enumerate(("query", "key", "value")))
    mask, p, causal = _arg(n, 3, "attn_mask"), _arg(n, 4, "dropout_p", 0.0), _arg(n, 5, "is_causal", False)
    scale, gqa = _arg(n, 6, "scale"), _arg(n, 7, "enable_gqa", False)
    if not all(isinstance(x, fx.Node) for x in (q, k, v)) or not isinstance(causal, bool) or not isinstance(gqa, bool):
        raise _NoMatch("scaled_dot_product_attention with operands or flags that are not constants of the graph")
    if not (_is_number(p) and 0.0 <= float(p) < 1.0) or not (scale is None or (_is_number(scale) and scale > 0)):
        raise _NoMatch("scaled_dot_product_attention with a dropout rate or scale that is not a constant")
    qs, ks, vs = _val(q), _val(k), _val(v)
    if qs.dim() == 3 and ks.dim() == 3 and vs.dim() == 3:
        if not qs.size(0) == ks.size(0) == vs.size(0):
            raise _NoMatch("scaled_dot_product_attention operands [N, L, E] with different batch sizes")
    elif qs.dim() != 4 or ks.dim() != 4 or vs.dim() != 4 or qs.size(1) % ks.size(1) or ks.size(1) != vs.size(1) or \
            (qs.size(1) != ks.size(1) and not gqa and ks.size(1) != 1):   # (one key / value head broadcasts: multi-query)
        raise _NoMatch("scaled_dot_product_attention operands are not [N, H, L, E] with grouped heads (or [N, L, E])")
    r = _Region()
    r.q, r.k, r.v, r.out, r.nodes = q, k, v, n, [n]
    r.scale = float(scale) if scale is not None else 1.0 / math.sqrt(qs.size(-1))
    r.dropout_p, r.causal = float(p), causal
    if mask is not None:
        if not isinstance(mask, fx.Node) or (causal and mask is not None):
            raise _NoMatch("scaled_dot_product_attention with both a mask and is_causal")
        if _val(mask).dtype == torch.bool:
            r.masks.append((mask, True))
        else:
            r.biases.append(mask)
    return r


_HALF = (torch.bfloat16, torch.float16)


def _undo_upcasts(r: _Region):
    """Model code that multiplies in fp32 (`query.to(torch.float32) @ key.to(torch.float32).transpose(-1, -2)`, GPT-J's
    and GPT-Neo's attention) hands the region fp32 copies of 16-bit tensors.  The kernel multiplies the 16-bit values
    exactly and accumulates in fp32, which is what the upcast product computes, so it takes the tensors as they were:
    applied when that leaves query, key and value in one 16-bit type."""
    def source(n):
        while isinstance(n, fx.Node) and _name(n) in ("to", "float", "type") and _val(n).dtype == torch.float32 and \
                n.args and isinstance(n.args[0], fx.Node) and _val(n.args[0]).dtype in _HALF and \
                _val(n.args[0]).shape == _val(n).shape:
            n = n.args[0]
        return n
    if not all(isinstance(x, fx.Node) for x in (r.q, r.k, r.v)):
        return
    q, k, v = source(r.q), source(r.k), source(r.v)
    if (q, k, v) != (r.q, r.k, r.v) and _val(q).dtype in _HALF and _val(q).dtype == _val(k).dtype == _val(v).dtype:
        r.q, r.k, r.v = q, k, v


def _shapes(r: _Region):
    q, k, v = _val(r.q), _val(r.k), _val(r.v)
    if q.dim() < 3 or k.dim() < 3 or v.dim() < 3:
        raise _NoMatch("operands need at least [batch, seq, dim]")
    gqa = q.dim() == 5 and k.dim() == 5 and v.dim() == 5 and k.size(2) == 1 and v.size(2) == 1 and q.size(2) > 1 and \
        q.size(1) == k.size(1)
    L, S = q.size(-2), k.size(-2)
    if v.size(-2) != S or q.size(-1) != k.size(-1):
        raise _NoMatch("inconsistent operand shapes")
    if q.size(-1) > 512:
        raise _NoMatch("head dims above 512 have no kernel")
    Hq = q.size(1) * q.size(2) if gqa else (q.size(-3) if q.dim() >= 4 else 1)
    return gqa, L, S, Hq


def _unrepeated_kv(n: Any) -> Optional[Tuple[fx.Node, int]]:
    """(x, g) when n is x [N, Hkv, S, E] with every head repeated g times along the head axis, consecutively:
    `x[:, :, None].expand(N, Hkv, g, S, E).reshape(N, Hkv * g, S, E)` (the `repeat_kv` of model code), the same with
    `unsqueeze(2)`, or `x.repeat_interleave(g, dim=1)`.  The kernel groups query heads over key / value heads by itself
    (query head h reads head h // g), so the repeated copy need not be made."""
    if not isinstance(n, fx.Node):
        return None
    nm = _name(n)
    if nm == "repeat_interleave":
        x, g = n.args[0], _arg(n, 1, "repeats")
        dim = _arg(n, 2, "dim")
        if isinstance(x, fx.Node) and isinstance(g, int) and g >= 1 and _val(x).dim() == 4 and dim in (1, -3):
            return x, g
        return None
    if nm not in ("reshape", "view") or not isinstance(n.args[0], fx.Node):
        return None
    ex, out = n.args[0], _val(n)
    if _name(ex) != "expand" or out.dim() != 4 or not isinstance(ex.args[0], fx.Node):
        return None
    un, e5 = ex.args[0], _val(ex)
    if e5.dim() != 5 or _val(un).dim() != 5 or _val(un).size(2) != 1:
        return None
    if _name(un) == "unsqueeze":
        if _arg(un, 1, "dim") not in (2, -3):
            return None
        x = un.args[0]
    elif un.op == "call_function" and un.target is operator.getitem:
        x, idx = un.args
        full = slice(None, None, None)
        if not isinstance(idx, tuple) or [i for i in idx if i is not Ellipsis][:3] != [full, full, None] or \
                any(i is not None and i != full for i in idx):
            return None
    else:
        return None
    if not isinstance(x, fx.Node):
        return None
    xs, g = _val(x), e5.size(2)
    if xs.dim() != 4 or tuple(e5.shape) != (xs.size(0), xs.size(1), g, xs.size(2), xs.size(3)) or \
            tuple(out.shape) != (xs.size(0), xs.size(1) * g, xs.size(2), xs.size(3)):
        return None
    return x, g


def _head_half(n: Any) -> Optional[Tuple[fx.Node, int]]:
    """(x, 0) when n is the first half of x's heads (axis 1), (x, 1) for the second half: x[:, :h], x[:, h:] or
    torch.chunk(x, 2, dim=1)[i]."""
    if not (isinstance(n, fx.Node) and n.op == "call_function" and n.target is operator.getitem):
        return None
    src, idx = n.args
    if _name(src) == "chunk" and isinstance(idx, int):
        if _arg(src, 1, "chunks") == 2 and _arg(src, 2, "dim", 0) in (1, 1 - _val(src.args[0]).dim()):
            return src.args[0], idx
        return None
    if not isinstance(idx, tuple) or len(idx) < 2 or not isinstance(src, fx.Node):
        return None
    full = slice(None, None, None)
    if any(i != full for j, i in enumerate(idx) if j != 1) or not isinstance(idx[1], slice) or idx[1].step is not None:
        return None
    heads = _val(src).size(1)
    if heads % 2:
        return None
    if idx[1].start in (None, 0) and idx[1].stop == heads // 2:
        return src, 0
    if idx[1].start == heads // 2 and idx[1].stop in (None, heads):
        return src, 1
    return None


def _merge_differential(gm: fx.GraphModule) -> int:
    """attn(q[:, :h], k[:, :h], v) - lam * attn(q[:, h:], k[:, h:], v) (diff_attn.py:14-29) -> one launch that keeps both
    softmax states and reads v once."""
    merged = 0
    for sub in [n for n in gm.graph.nodes if _name(n) == "sub"]:
        if len(sub.args) != 2 or sub.kwargs.get("alpha", 1) != 1:
            continue
        a, m = sub.args
        if _name(m) != "mul" or not isinstance(a, fx.Node):
            continue
        lam, b = (m.args[0], m.args[1]) if _is_number(m.args[0]) else (m.args[1], m.args[0])
        if not _is_number(lam) or not isinstance(b, fx.Node):
            continue
        if not all(x.op == "call_function" and x.target is fused_attention for x in (a, b)):
            continue
        if a.kwargs != b.kwargs or a.kwargs.get("gqa") or a.kwargs.get("diff_lambda") is not None or a.kwargs.get("score_fn") \
                or a.kwargs.get("dropout_p"):
            continue
        if a.args[2] is not b.args[2] or a.args[3] is not b.args[3]:
            continue
        if list(a.args[4]) or list(b.args[4]) or list(a.args[5]) or list(b.args[5]):
            continue
        qa, qb, ka, kb = _head_half(a.args[0]), _head_half(b.args[0]), _head_half(a.args[1]), _head_half(b.args[1])
        if None in (qa, qb, ka, kb) or qa[0] is not qb[0] or ka[0] is not kb[0] or (qa[1], qb[1], ka[1], kb[1]) != (0, 1, 0, 1):
            continue
        if _val(qa[0]).dim() != 4 or len(a.users) != 1 or len(b.users) != 1 or len(m.users) != 1:
            continue
        with gm.graph.inserting_before(sub):
            new = gm.graph.call_function(fused_attention, (qa[0], ka[0], a.args[2], a.args[3], [], []),
                                         dict(a.kwargs, diff_lambda=float(lam)))
        new.meta.update(sub.meta)
        sub.replace_all_uses_with(new)
        for n in (sub, m, b, a):
            gm.graph.erase_node(n)
        merged += 1
    return merged


_MHA_PARAMS = ("query", "key", "value", "embed_dim_to_check", "num_heads", "in_proj_weight", "in_proj_bias", "bias_k",
               "bias_v", "add_zero_attn", "dropout_p", "out_proj_weight", "out_proj_bias", "training", "key_padding_mask",
               "need_weights", "attn_mask", "use_separate_proj_weight", "q_proj_weight", "k_proj_weight", "v_proj_weight",
               "static_k", "static_v", "average_attn_weights", "is_causal")
_MHA_DEFAULTS = dict(training=True, key_padding_mask=None, need_weights=True, attn_mask=None, use_separate_proj_weight=False,
                     q_proj_weight=None, k_proj_weight=None, v_proj_weight=None, static_k=None, static_v=None,
                     average_attn_weights=True, is_causal=False)


def _rewrite_multi_head_attention(gm: fx.GraphModule) -> int:
    """Calls of torch.nn.functional.multi_head_attention_forward that return no weights and use neither bias_k / bias_v,
    add_zero_attn nor static keys become `fused_multi_head_attention`; others are left as they are.  Head dims above
    128 are left alone in training mode (no backward kernel there) and with dropout."""
    import torch.nn.functional as F
    replaced = 0
    for n in [x for x in gm.graph.nodes if x.op == "call_function" and x.target is F.multi_head_attention_forward]:
        a = dict(_MHA_DEFAULTS)
        a.update(zip(_MHA_PARAMS, n.args))
        a.update(n.kwargs)
        if any(name not in a for name in _MHA_PARAMS[:13]):
            continue
        if a["need_weights"] is not False or a["bias_k"] is not None or a["bias_v"] is not None or a["add_zero_attn"] is not False \
                or a["static_k"] is not None or a["static_v"] is not None:
            continue
        if not isinstance(a["num_heads"], int) or not _is_number(a["dropout_p"]) or not isinstance(a["training"], bool) \
                or not isinstance(a["is_causal"], bool) or not isinstance(a["use_separate_proj_weight"], bool):
            continue
        if not all(isinstance(a[x], fx.Node) for x in ("query", "key", "value", "out_proj_weight")):
            continue
        qv = _val(a["query"])
        if qv.dim() not in (2, 3) or qv.size(-1) % a["num_heads"] or qv.dtype not in (torch.bfloat16, torch.float16):
            continue
        hd = qv.size(-1) // a["num_heads"]
        p = float(a["dropout_p"]) if a["training"] else 0.0
        if hd > 512 or (hd > 128 and (a["training"] or p > 0.0)) or not 0.0 <= p < 1.0:
            continue
        sep = a["use_separate_proj_weight"]
        if (sep and any(a[x] is None for x in ("q_proj_weight", "k_proj_weight", "v_proj_weight"))) or \
                (not sep and a["in_proj_weight"] is None):
            continue
        kwargs = dict(num_heads=a["num_heads"], in_proj_weight=None if sep else a["in_proj_weight"],
                      in_proj_bias=a["in_proj_bias"], q_proj_weight=a["q_proj_weight"] if sep else None,
                      k_proj_weight=a["k_proj_weight"] if sep else None, v_proj_weight=a["v_proj_weight"] if sep else None,
                      out_proj_weight=a["out_proj_weight"], out_proj_bias=a["out_proj_bias"], dropout_p=p,
                      key_padding_mask=a["key_padding_mask"], attn_mask=a["attn_mask"], is_causal=a["is_causal"])
        with gm.graph.inserting_before(n):
            new = gm.graph.call_function(fused_multi_head_attention, (a["query"], a["key"], a["value"]), kwargs)
        new.meta.update(n.meta)
        n.replace_all_uses_with(new)
        gm.graph.erase_node(n)
        replaced += 1
    return replaced


def _lower_einsums(gm: fx.GraphModule) -> int:
    """Two-operand `torch.einsum` calls that are a batched matrix product — one contracted letter, one letter of the
    result from each operand alone, the rest batch letters present everywhere, e.g. "bhid,bhjd->bhij" and
    "bhij,bhjd->bhid", or with sequence-major operands "bqhd,bkhd->bhqk" — are rewritten as permute / transpose / matmul
    nodes (the same computation), so that attention spelled with einsum meets the matcher as matmuls.  Returns the
    number of calls rewritten."""
    lowered = 0
    for n in list(gm.graph.nodes):
        if _name(n) != "einsum" or not n.args or not isinstance(n.args[0], str) or n.kwargs:
            continue
        operands = tuple(n.args[1]) if len(n.args) == 2 and isinstance(n.args[1], (list, tuple)) else tuple(n.args[1:])
        eq = n.args[0].replace(" ", "")
        if len(operands) != 2 or not all(isinstance(x, fx.Node) for x in operands) or "." in eq or eq.count("->") != 1:
            continue
        lhs, C = eq.split("->")
        if lhs.count(",") != 1:
            continue
        A, B = lhs.split(",")
        sa, sb, sc = set(A), set(B), set(C)
        if len(sa) != len(A) or len(sb) != len(B) or len(sc) != len(C):
            continue
        contracted, only_a, only_b, batch = (sa & sb) - sc, (sa & sc) - sb, (sb & sc) - sa, sa & sb & sc
        if len(contracted) != 1 or len(only_a) != 1 or len(only_b) != 1 or sa != batch | contracted | only_a or \
                sb != batch | contracted | only_b or sc != batch | only_a | only_b:
            continue
        (c,), (i,), (j,) = contracted, only_a, only_b
        lead = [x for x in C if x in batch]
        a, b = operands
        try:
            va, vb = _val(a), _val(b)
            if va.dim() != len(A) or vb.dim() != len(B):
                continue
            perm_a = [A.index(x) for x in lead + [i, c]]
            perm_b = [B.index(x) for x in lead + [j, c]]
            perm_c = [(lead + [i, j]).index(x) for x in C]
            ident = lambda perm: perm == list(range(len(perm)))
            va1 = va if ident(perm_a) else va.permute(*perm_a)
            direct_b = list(B) == lead + [c, j]            # already [.., contracted, j]: the second operand as it is
            vb1 = vb if direct_b or ident(perm_b) else vb.permute(*perm_b)
            vb2 = vb1 if direct_b else vb1.transpose(-2, -1)
            vmm = torch.matmul(va1, vb2)
            vout = vmm if ident(perm_c) else vmm.permute(*perm_c)
        except Exception:  # noqa: BLE001 - an einsum this cannot express stays as it is
            continue

        def node(kind, target, args, value):
            y = gm.graph.call_method(target, args) if kind == "method" else gm.graph.call_function(target, args)
            y.meta["example_value"] = value
            return y

        with gm.graph.inserting_before(n):
            a1 = a if ident(perm_a) else node("method", "permute", (a, *perm_a), va1)
            b1 = b if direct_b or ident(perm_b) else node("method", "permute", (b, *perm_b), vb1)
            b2 = b1 if direct_b else node("method", "transpose", (b1, -2, -1), vb2)
            mm = node("function", torch.matmul, (a1, b2), vmm)
            out = mm if ident(perm_c) else node("method", "permute", (mm, *perm_c), vout)
        n.replace_all_uses_with(out)
        gm.graph.erase_node(n)
        lowered += 1
    return lowered


def fuse_attention(gm: fx.GraphModule) -> int:
    """Rewrites every attention region of `gm` (a Dynamo-captured graph with example values on its nodes) in place.
    Returns the number of regions replaced."""
    lowered = _lower_einsums(gm)
    replaced = _rewrite_multi_head_attention(gm)
    for sm in [n for n in gm.graph.nodes if _name(n) in ("softmax", "scaled_dot_product_attention")]:
        try:
            r = _match(sm) if _name(sm) == "softmax" else _match_sdpa(sm)
            _undo_upcasts(r)
            gqa, L, S, Hq = _shapes(r)
            if not gqa and _val(r.q).dim() == 4:
                # key / value heads that were repeated to match the query heads: hand the kernel the originals
                uk, uv = _unrepeated_kv(r.k), _unrepeated_kv(r.v)
                if uk is not None and uv is not None and uk[1] == uv[1] and _val(uk[0]).size(1) == _val(uv[0]).size(1) \
                        and _val(uk[0]).size(1) * uk[1] == Hq:
                    r.k, r.v = uk[0], uv[0]
            kwargs: Dict[str, Any] = dict(scale=float(r.scale), mask_kind=_ffi.MASK_CAUSAL if r.causal else _ffi.MASK_NONE,
                                          window=0, prefix=0, alibi_heads=0, softcap=float(r.softcap), gqa=gqa)
            # (a score function other than the soft-cap goes with positional masks and dense operands only: document
            # ids and the in-kernel ALiBi term stay dense then)
            plain = r.score_fn is None
            if not plain:
                kwargs["score_fn"] = r.score_fn
            doc_ids = None
            run_masks: List[fx.Node] = []
            run_invert: List[bool] = []
            const_biases: List[torch.Tensor] = []
            run_biases: List[fx.Node] = []
            for node, invert in r.masks:
                phs = _placeholders_of(node)
                got = None
                if not phs:
                    m = _try_evaluate(node, gm)
                    if not isinstance(m, torch.Tensor) or m.dtype != torch.bool:
                        run_masks.append(node)
                        run_invert.append(invert)
                        continue
                    m = ~m if invert else m
                    got = _classify_constant_mask(m, L, S)
                    if got is not None and got[0] != _ffi.MASK_NONE:
                        if kwargs["mask_kind"] != _ffi.MASK_NONE:
                            got = None  # two positional masks: keep the second one dense
                        else:
                            kwargs.update(mask_kind=got[0], window=got[1], prefix=got[2])
                    if got is None:
                        const_biases.append(torch.zeros(m.shape, dtype=_val(r.q).dtype, device=m.device)
                                            .masked_fill_(m, _NEG_INF))
                    continue
                if plain and len(phs) == 1 and kwargs["mask_kind"] == _ffi.MASK_NONE:
                    kind = _classify_document_mask(node, phs[0], invert, L, S, gm)
                    if kind is not None:
                        kwargs["mask_kind"] = kind
                        doc_ids = phs[0]
                        continue
                run_masks.append(node)
                run_invert.append(invert)
            for node in r.biases:
                b = _try_evaluate(node, gm) if not _placeholders_of(node) else None
                if isinstance(b, torch.Tensor):
                    if plain and kwargs["alibi_heads"] == 0 and _is_alibi(b, Hq, L, S):
                        kwargs["alibi_heads"] = Hq
                        continue
                    # a constant additive mask (zeros and fills <= -1e9, the way model code builds its causal mask when
                    # no padding mask is given): the same positional forms as a boolean one
                    as_mask = b <= -1e9
                    if b.is_floating_point() and kwargs["mask_kind"] == _ffi.MASK_NONE and bool(as_mask.any()) and \
                            bool(((b == 0) | as_mask).all()):
                        got = _classify_constant_mask(as_mask, L, S)
                        if got is not None and got[0] != _ffi.MASK_NONE:
                            kwargs.update(mask_kind=got[0], window=got[1], prefix=got[2])
                            continue
                    const_biases.append(b)
                else:
                    run_biases.append(node)
            if r.dropout_p:
                # the dropout kernels cover head dims up to 128 (padded to 64 or 128) and every score modification but the
                # score functions
                E, Ev = _val(r.q).size(-1), _val(r.v).size(-1)
                if not plain or max(E, Ev) > 128:
                    raise _NoMatch("dropout together with this combination of score modifications or head dims")
                kwargs["dropout_p"] = r.dropout_p
        except _NoMatch:
            continue
        bias_nodes: List[fx.Node] = list(run_biases)
        with gm.graph.inserting_before(r.out):
            for i, t in enumerate(const_biases):
                name = f"_flashlight_const_{replaced}_{i}"
                gm.register_buffer(name, t, persistent=False)
                bias_nodes.append(gm.graph.get_attr(name))
            new = gm.graph.call_function(fused_attention, (r.q, r.k, r.v, doc_ids, bias_nodes, run_masks),
                                         dict(kwargs, mask_invert=tuple(run_invert)))
            out_dtype = _val(r.out).dtype
            if out_dtype != _val(r.q).dtype and _val(r.q).dtype in _HALF:
                # (operands that the region upcast to fp32: what follows still gets the region's own result type)
                fused, new = new, gm.graph.call_method("to", (new, out_dtype))
                fused.meta.update(r.out.meta)
        new.meta.update(r.out.meta)
        r.out.replace_all_uses_with(new)
        for n in r.nodes:
            if not n.users:
                gm.graph.erase_node(n)
        replaced += 1
    if replaced:
        _merge_differential(gm)
    if replaced or lowered:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
    return replaced


def backend(gm: fx.GraphModule, example_inputs):
    """`torch.compile(fn, backend=flashlight_amd.fusion.backend, dynamic=False)`, or `backend="flashlight_amd"` once
    this module is imported: attention regions run on the fused kernel, the rest of the captured graph as eager
    PyTorch."""
    fuse_attention(gm)
    return gm.forward


def backend_inductor(gm: fx.GraphModule, example_inputs):
    """`backend="flashlight_amd_inductor"`: the same rewrite, then the rest of the graph goes to Inductor (the reference's
    setting: its fused attention is one kernel inside an Inductor-compiled graph), which traces through the replacement
    nodes down to the registered operators and keeps those as external kernels.  A graph in which a region drops
    weights is not handed on (the seed of each call is drawn when the node runs; a tracer would freeze one into the
    compiled code): it runs like `backend="flashlight_amd"`."""
    fuse_attention(gm)
    for n in gm.graph.nodes:
        if n.op == "call_function" and n.target in (fused_attention, fused_multi_head_attention) and n.kwargs.get("dropout_p", 0.0):
            return gm.forward
    from torch._inductor.compile_fx import compile_fx
    # constants of the rewrite (dense masks it evaluated) become inputs of the graph: the compiler takes tensors through
    # placeholders, not through attributes added to a captured module
    consts: List[torch.Tensor] = []
    last_placeholder = None
    for n in gm.graph.nodes:
        if n.op == "placeholder":
            last_placeholder = n
    for n in list(gm.graph.nodes):
        if n.op == "get_attr" and isinstance(n.target, str) and n.target.startswith("_flashlight_const_"):
            t = getattr(gm, n.target)
            if last_placeholder is None:   # (a graph without inputs: nothing for a compiler to specialise on)
                return gm.forward
            with gm.graph.inserting_after(last_placeholder):
                ph = gm.graph.placeholder(n.target)
            ph.meta.update(n.meta)
            n.replace_all_uses_with(ph)
            gm.graph.erase_node(n)
            last_placeholder = ph
            consts.append(t)
    if not consts:
        return compile_fx(gm, example_inputs)
    gm.graph.lint()
    gm.recompile()
    compiled = compile_fx(gm, list(example_inputs) + consts)
    return lambda *args: compiled(*args, *consts)


torch._dynamo.register_backend(compiler_fn=backend, name="flashlight_amd")
torch._dynamo.register_backend(compiler_fn=backend_inductor, name="flashlight_amd_inductor")
