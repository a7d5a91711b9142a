"""Eager restatement of the reference's attention variants.  TEST INFRASTRUCTURE (see oracle/__init__.py).

Every public function keeps the reference's positional signature and result layout and cites the file it follows.
They all reduce to one routine, `_softmax_attention`, which materialises the score matrix exactly like the
reference's eager code does (optionally in blocks of query rows so that long sequences fit in host memory; the
arithmetic per row is unchanged).  Keyword arguments marked "extension" do not exist in the reference; their
defaults reproduce it.
"""
from __future__ import annotations

import math
from typing import Callable, List, Optional, Sequence

import torch

NEG_INF = float("-inf")
MASK_FILL = -1e10  # the value sliding_window.py:40, prefix_lm.py:26 and document_mask.py:37 write into masked scores

# (q_idx [l,1] int64, k_idx [1,S] int64) -> bool tensor broadcastable to the score block [..., l, S]; True = masked
MaskFn = Callable[[torch.Tensor, torch.Tensor], torch.Tensor]
# same arguments -> additive term (or a sequence of terms, added in order) broadcastable to the score block
BiasFn = Callable[[torch.Tensor, torch.Tensor], torch.Tensor]


def _default_scale(query: torch.Tensor, scale: Optional[float]) -> float:
    return 1.0 / math.sqrt(query.size(-1)) if scale is None else scale


def _group(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, enable_gqa: bool):
    """GQA view used by every reference variant (e.g. causal.py:27-30): q-head h reads kv-head h // G."""
    if not enable_gqa:
        return query, key, value
    n, hkv = query.size(0), key.size(1)
    return query.reshape(n, hkv, -1, query.size(-2), query.size(-1)), key.unsqueeze(2), value.unsqueeze(2)


def _softmax_attention(query, key, value, scale, *, masked: Optional[MaskFn] = None, fill: float = NEG_INF,
                       bias: Optional[BiasFn] = None, softcap: Optional[float] = None,
                       q_block: Optional[int] = None, score_fn=None) -> torch.Tensor:
    """softmax(mask(cap(q k^T * scale) + bias)) v over the last two axes; leading axes broadcast like matmul.
    `score_fn`, a callable on the scaled score block, takes the cap's place (softcap.py:49 applies whatever
    `score_mod` it is given there)."""
    L, S = query.size(-2), key.size(-2)
    step = L if not q_block else q_block
    k_t = key.transpose(-2, -1)
    k_idx = torch.arange(S, device=query.device).view(1, S)
    outs = []
    for a in range(0, L, step):
        b = min(L, a + step)
        q_idx = torch.arange(a, b, device=query.device).view(b - a, 1)
        w = torch.matmul(query[..., a:b, :], k_t) * scale
        if softcap is not None:
            w = softcap * torch.tanh(w / softcap)
        if score_fn is not None:
            w = score_fn(w)
        if bias is not None:
            terms = bias(q_idx, k_idx)
            for term in (terms if isinstance(terms, (tuple, list)) else (terms,)):
                w = w + term
        if masked is not None:
            w = torch.where(masked(q_idx, k_idx), torch.full((), fill, dtype=w.dtype, device=w.device), w)
        outs.append(torch.matmul(torch.softmax(w, dim=-1), value))
    return outs[0] if len(outs) == 1 else torch.cat(outs, dim=-2)


# ---- vanilla ------------------------------------------------------------------------------------------------------------

def attention_vanilla_nogqa(query, key, value, scale=None, *, q_block=None):
    """attention_variants/vanilla.py:4-17 (`attention_pytorch_nogqa`)."""
    return _softmax_attention(query, key, value, _default_scale(query, scale), q_block=q_block)


def attention_vanilla(query, key, value, scale=None, enable_gqa=False, *, q_block=None):
    """attention_variants/vanilla.py:20-35 (`attention_pytorch`): the only variant that views a GQA result back to
    [N, Hq, L, Ev]; tests/test_gqa.py:11-57 (`grouped_query_attention`) is the same computation."""
    q, k, v = _group(query, key, value, enable_gqa)
    out = _softmax_attention(q, k, v, _default_scale(query, scale), q_block=q_block)
    return out.reshape(value.size(0), -1, out.size(-2), value.size(-1))


# ---- causal -------------------------------------------------------------------------------------------------------------

def attention_causal(query, key, value, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None, enable_gqa=False,
                     *, q_block=None):
    """attention_variants/causal.py:4-36 (`attention_pytorch_causal`): always causal; attn_mask, dropout_p and
    is_causal are accepted and ignored; masked scores become -inf (causal.py:32-33)."""
    q, k, v = _group(query, key, value, enable_gqa)
    return _softmax_attention(q, k, v, _default_scale(query, scale), masked=lambda qi, ki: ki > qi, fill=NEG_INF,
                              q_block=q_block)


# ---- sliding window ------------------------------------------------------------------------------------------------------

def attention_sliding_window(query, key, value, window_size=1024, scale=None, enable_gqa=False, *, q_block=None):
    """attention_variants/sliding_window.py:14-44: attends 0 <= q - k <= window_size (window_size + 1 keys)."""
    assert query.size(-2) == key.size(-2) == value.size(-2)  # sliding_window.py:27
    q, k, v = _group(query, key, value, enable_gqa)
    return _softmax_attention(q, k, v, _default_scale(query, scale),
                              masked=lambda qi, ki: (qi < ki) | ((qi - ki) > window_size), fill=MASK_FILL,
                              q_block=q_block)


# ---- prefix-LM -----------------------------------------------------------------------------------------------------------

def attention_prefix_lm(query, key, value, prefix_lengths=256, scale=None, enable_gqa=False, *, q_block=None):
    """attention_variants/prefix_lm.py:5-42: one integer prefix for the whole batch; attends k <= max(P - 1, q)."""
    q, k, v = _group(query, key, value, enable_gqa)
    return _softmax_attention(q, k, v, _default_scale(query, scale),
                              masked=lambda qi, ki: ki > torch.clamp(qi, min=prefix_lengths - 1), fill=MASK_FILL,
                              q_block=q_block)


# ---- document mask --------------------------------------------------------------------------------------------------------

def attention_document_mask(query, key, value, document_id, scale=None, enable_gqa=False, *, is_causal=False,
                            q_block=None):
    """attention_variants/document_mask.py:6-41: `document_id` int64 [N, L]; a pair is attended iff both positions
    carry the same id (bidirectional inside a document).  Extension: is_causal additionally requires k <= q, which is
    what the reference's FlexAttention baseline masks (benchmarks/run_flex_variants.py:66-90)."""
    q, k, v = _group(query, key, value, enable_gqa)
    lead = (document_id.size(0),) + (1,) * (q.dim() - 3)  # broadcast over the head (and group) axes

    def masked(qi, ki):
        dq = document_id[:, qi.view(-1)].reshape(*lead, qi.numel(), 1)
        dk = document_id[:, ki.view(-1)].reshape(*lead, 1, ki.numel())
        m = dq != dk
        return (m | (ki > qi)) if is_causal else m

    return _softmax_attention(q, k, v, _default_scale(query, scale), masked=masked, fill=MASK_FILL, q_block=q_block)


# ---- ALiBi ----------------------------------------------------------------------------------------------------------------

def alibi_slopes(nheads: int, device=None) -> torch.Tensor:
    """2^(-8 (h + 1) / nheads) for h = 0..nheads-1 (attention_variants/alibi.py:5-7)."""
    return torch.exp2(-((torch.arange(nheads, dtype=torch.int32, device=device) + 1) * 8.0 / nheads))


def attention_alibi(query, key, value, score_mod=None, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None,
                    enable_gqa=False, *, softcap=None, honor_causal=False, q_block=None):
    """attention_variants/alibi.py:13-33 with score_mod = generate_alibi_bias_pytorch(Hq) (alibi.py:11): adds
    slope_h * (k - q) to the scaled scores, no mask (is_causal is ignored by the reference).  `score_mod` here is the
    number of heads the slopes are generated for (None = query heads), or a callable (L, S) -> dense tensor.  Extensions: softcap (applied to the scaled
    score before the bias), honor_causal (mask k > q with -inf when is_causal is set)."""
    hq = query.size(1)
    q, k, v = _group(query, key, value, enable_gqa)
    masked = (lambda qi, ki: ki > qi) if (honor_causal and is_causal) else None
    if callable(score_mod):
        # any other callable: its dense result is converted to the scores' dtype and, under GQA, viewed as
        # [Hkv, G, L, S] (alibi.py:26-29)
        dense = score_mod(query.size(-2), key.size(-2)).to(q.dtype)
        if enable_gqa:
            dense = dense.view(q.size(1), q.size(2), query.size(-2), key.size(-2))
        return _softmax_attention(q, k, v, _default_scale(query, scale), softcap=softcap, masked=masked, fill=NEG_INF,
                                  bias=lambda qi, ki: dense if dense.size(-2) == 1 else dense[..., qi.view(-1), :],
                                  q_block=q_block)
    slopes = alibi_slopes(hq if score_mod is None else int(score_mod), device=query.device).to(torch.float32)
    head_shape = (q.size(1), q.size(2), 1, 1) if enable_gqa else (hq, 1, 1)  # alibi.py:27-28

    def bias(qi, ki):
        rel = (ki.to(torch.int32) - qi.to(torch.int32))
        return (slopes.view(-1, 1, 1) * rel).to(q.dtype).reshape(*head_shape[:-2], qi.numel(), ki.numel())

    return _softmax_attention(q, k, v, _default_scale(query, scale), bias=bias, softcap=softcap, masked=masked,
                              fill=NEG_INF, q_block=q_block)


# ---- tanh soft-capping -------------------------------------------------------------------------------------------------------

def tanh_softcap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(x / cap): the formula stated at attention_variants/softcap.py:48 and computed by the FlashInfer
    baseline's logits_soft_cap (attention_variants/flashinfer/softcap.py:3).  The callable the reference passes in
    (attn_gym.mods.generate_tanh_softcap(30, approx=False), benchmarks/run_flex_variants.py:133) lives in a
    dependency that is not vendored; parity of this variant rests on the closed form."""
    return cap * torch.tanh(x / cap)


def attention_softcapped(query, key, value, score_mod=None, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None,
                         enable_gqa=False, softcap_threshold=30.0, *, honor_causal=False, q_block=None):
    """attention_variants/softcap.py:4-53: softmax(score_mod(q k^T * scale)) v.  `score_mod` here is the cap value
    (None = softcap_threshold, which the reference declares but never reads), or a callable of the reference's
    signature `(score, b, h, q_idx, kv_idx)`, which is applied to the scaled scores as softcap.py:49 does."""
    q, k, v = _group(query, key, value, enable_gqa)
    masked = (lambda qi, ki: ki > qi) if (honor_causal and is_causal) else None
    if callable(score_mod):
        return _softmax_attention(q, k, v, _default_scale(query, scale), masked=masked, fill=NEG_INF, q_block=q_block,
                                  score_fn=lambda w: score_mod(w, query.size(0), query.size(1), None, None))
    cap = float(softcap_threshold if score_mod is None else score_mod)
    return _softmax_attention(q, k, v, _default_scale(query, scale), softcap=cap, masked=masked, fill=NEG_INF,
                              q_block=q_block)


# ---- differential attention ---------------------------------------------------------------------------------------------------

def diff_attention(q, k, v, scale=None, lambda_full=0.2, *, is_causal=False, q_block=None, **kwargs):
    """attention_variants/diff_attn.py:6-30 (`diffattn`): q, k [B, 2H, S, d] split on the head axis, v [B, H, S, 2d];
    softmax(q0 k0^T s) v - lambda_full * softmax(q1 k1^T s) v with s = 1/sqrt(d).  Extension: is_causal."""
    s = _default_scale(q, scale)
    hq, hk = q.size(1) // 2, k.size(1) // 2
    masked = (lambda qi, ki: ki > qi) if is_causal else None
    a0 = _softmax_attention(q[:, :hq], k[:, :hk], v, s, masked=masked, q_block=q_block)
    a1 = _softmax_attention(q[:, hq:], k[:, hk:], v, s, masked=masked, q_block=q_block)
    return a0 - lambda_full * a1


# ---- Evoformer row attention ---------------------------------------------------------------------------------------------------

def attention_evoformer(q_input, k_input, v_input, biases: Sequence[torch.Tensor], sm_scale=None, *, gate=None,
                        q_block=None, **kwargs):
    """attention_variants/evoformer.py:8-36 (`attention_reference`): inputs [*, S, H, D]; scores get every tensor of
    `biases` added (each broadcastable to [*, H, S, S]); result is returned as [*, S, H, D].
    Extension: gate (logits shaped like the result) multiplies the result by sigmoid(gate)."""
    q, k, v = (t.transpose(-2, -3) for t in (q_input, k_input, v_input))
    scale = _default_scale(q, sm_scale)
    bl: List[torch.Tensor] = list(biases)

    def bias(qi, ki):  # added one after the other, in the order given (evoformer.py:26-27)
        return [b if b.size(-2) == 1 else b[..., qi.view(-1), :] for b in bl]

    out = _softmax_attention(q, k, v, scale, bias=bias if bl else None, q_block=q_block).transpose(-2, -3)
    if gate is not None:
        out = out * torch.sigmoid(gate.to(out.dtype))
    return out


# ---- invariant point attention ------------------------------------------------------------------------------------------------

def invariant_point_attention(q_scalar, k_scalar, v_scalar, q_points, k_points, v_points, pair_bias, frames=None,
                              mask=None, c_hidden=64, no_qk_points=8):
    """tests/test_ipa.py:57-125.  Scalars [*, H, N, C], points [*, H, N, P, X].  The frame transforms and the mask are
    commented out in the reference (test_ipa.py:84-86, 111-112, 122), so `frames` and `mask` are unused.  Returns the
    two aggregations (output_scalar [*, H, N, C], output_points [*, N, H, Pv, X]) of test_ipa.py:117-122 instead of
    their sum (test_ipa.py:125), which does not broadcast for general sizes."""
    content = torch.matmul(q_scalar / (c_hidden ** 0.5), k_scalar.transpose(-1, -2))     # test_ipa.py:88-100
    diff = q_points.unsqueeze(-3) - k_points.unsqueeze(-4)                               # [*, H, Nq, Nk, P, X]
    dist_sq = (diff ** 2).sum(dim=-1)                                                    # test_ipa.py:102-105
    weight = -0.5 * (9.0 / (2 * no_qk_points)) ** 0.5                                    # test_ipa.py:107
    logits = content + dist_sq.sum(dim=-1) * weight
    if pair_bias is not None:
        logits = logits + pair_bias                                                      # test_ipa.py:110
    attn = torch.softmax(logits, dim=-1)
    out_scalar = torch.matmul(attn, v_scalar)                                            # test_ipa.py:118
    out_points = torch.einsum('...hij,...hjpv->...ihpv', attn, v_points)                 # test_ipa.py:122
    return out_scalar, out_points
