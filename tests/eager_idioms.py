"""Attention written out in eager PyTorch, the way callers of the reference write it (the idioms of
attention_variants/*.py: explicit matmuls, a mask or bias built with tensor operations, softmax, second matmul; GQA by
viewing the query as [N, Hkv, G, L, E]).  Inputs for the graph-rewrite tests: `flashlight_amd.fusion` has to recognise
each of them, and on a GPU the rewritten function has to return what the eager function returns."""
import math

import torch
import torch.nn.functional as F


def _gqa(query, key, value):
    query = query.view(query.size(0), key.size(1), -1, query.size(-2), query.size(-1))
    return query, key.unsqueeze(2), value.unsqueeze(2)


def plain(query, key, value, enable_gqa=False):
    s = 1 / math.sqrt(query.size(-1))
    if enable_gqa:
        query, key, value = _gqa(query, key, value)
    w = torch.softmax(query @ key.transpose(-2, -1) * s, dim=-1)
    return (w @ value).view(value.size(0), -1, value.size(-2), value.size(-1))


def divided_by_sqrt_d(query, key, value):
    return torch.matmul(F.softmax(torch.matmul(query, key.mT) / math.sqrt(query.size(-1)), dim=-1), value)


def causal_triu(query, key, value, enable_gqa=False):
    s = 1 / math.sqrt(query.size(-1))
    if enable_gqa:
        query, key, value = _gqa(query, key, value)
    future = torch.triu(torch.ones(query.size(-2), key.size(-2), device=query.device, dtype=torch.bool), diagonal=1)
    w = torch.where(future, float("-inf"), query @ key.transpose(-2, -1) * s)
    return torch.softmax(w, dim=-1) @ value


def causal_tril_keep(query, key, value):
    keep = torch.ones(query.size(-2), key.size(-2), device=query.device).tril().bool()
    w = torch.where(keep, torch.matmul(query, key.transpose(-1, -2)) * 0.2, -1e30)
    return w.softmax(-1) @ value


def sliding(query, key, value, window, enable_gqa=False):
    s = 1.0 / math.sqrt(query.size(-1))
    if enable_gqa:
        query, key, value = _gqa(query, key, value)
    n = query.size(-2)
    qi = torch.arange(n, device=query.device).view(n, 1)
    ki = torch.arange(n, device=query.device).view(1, n)
    outside = ((qi < ki) | ((qi - ki) > window)).unsqueeze(0).unsqueeze(0)
    w = (torch.matmul(query, key.transpose(-2, -1)) * s).masked_fill(outside, -1e10)
    return torch.softmax(w, dim=-1) @ value


def prefix_lm(query, key, value, prefix, enable_gqa=False):
    s = 1.0 / math.sqrt(query.size(-1))
    n = query.size(-2)
    plen = torch.full((query.size(0),), prefix, dtype=torch.long, device=query.device)
    qi = torch.arange(n, device=query.device).view(1, 1, n, 1)
    ki = torch.arange(n, device=query.device).view(1, 1, 1, n)
    hidden = ki > torch.maximum(plen.view(-1, 1, 1, 1) - 1, qi)
    if enable_gqa:
        query, key, value = _gqa(query, key, value)
        hidden = hidden.unsqueeze(2).expand(hidden.size(0), key.size(1), -1, n, n)
    w = (torch.matmul(query, key.transpose(-2, -1)) * s).masked_fill(hidden, -1e10)
    return torch.softmax(w, dim=-1) @ value


def documents(query, key, value, document_id, causal=False, enable_gqa=False):
    s = 1.0 / math.sqrt(query.size(-1))
    other = (document_id.unsqueeze(2) != document_id.unsqueeze(1)).unsqueeze(1)
    if causal:
        n = query.size(-2)
        other = other | torch.ones(n, n, dtype=torch.bool, device=query.device).triu(1)
    if enable_gqa:
        query, key, value = _gqa(query, key, value)
        other = other.unsqueeze(2).expand(other.size(0), key.size(1), -1, other.size(-2), other.size(-1))
    w = torch.where(other, -1e10, torch.matmul(query, key.transpose(-2, -1)) * s)
    return torch.softmax(w, dim=-1) @ value


def alibi(query, key, value, enable_gqa=False):
    s = 1 / math.sqrt(query.size(-1))
    h = query.size(1)
    if enable_gqa:
        query, key, value = _gqa(query, key, value)
    w = torch.matmul(query, key.transpose(-2, -1)) * s
    slopes = torch.exp2(-((torch.arange(h, dtype=torch.int32, device=query.device) + 1) * 8.0 / h))
    rel = torch.arange(w.size(-1), dtype=torch.int32, device=query.device)[None, :] - \
        torch.arange(w.size(-2), dtype=torch.int32, device=query.device)[:, None]
    bias = (slopes[:, None, None] * rel).to(w.dtype)
    if enable_gqa:
        bias = bias.view(w.size(1), w.size(2), w.size(3), w.size(4))
    return torch.softmax(w + bias, dim=-1) @ value


def softcap(query, key, value, cap, causal=False):
    w = query @ key.transpose(-2, -1) * (1 / math.sqrt(query.size(-1)))
    w = cap * torch.tanh(w / cap)
    if causal:
        w = w.masked_fill(torch.ones(w.size(-2), w.size(-1), dtype=torch.bool, device=w.device).triu(1), float("-inf"))
    return torch.softmax(w, dim=-1) @ value


def learned_bias(query, key, value, bias, key_padding):
    """A run-time additive bias plus a boolean key-padding mask that no closed form covers."""
    w = torch.matmul(query, key.transpose(-2, -1)) / math.sqrt(query.size(-1)) + bias
    w = w.masked_fill(key_padding[:, None, None, :], float("-inf"))
    return torch.matmul(torch.softmax(w, dim=-1), value)


def checkerboard(query, key, value):
    """A constant mask that is none of the positional forms: attend only keys of the query's parity."""
    n = query.size(-2)
    i = torch.arange(n, device=query.device)
    hidden = (i.view(n, 1) + i.view(1, n)) % 2 == 1
    w = (query @ key.transpose(-2, -1) * 0.125).masked_fill(hidden, float("-inf"))
    return torch.softmax(w, dim=-1) @ value


def differential(q, k, v, lam):
    s = 1 / math.sqrt(q.size(-1))
    h, hk = q.size(1) // 2, k.size(1) // 2
    w0 = torch.matmul(q[:, :h], k[:, :hk].transpose(-1, -2)) * s
    w1 = torch.matmul(q[:, h:], k[:, hk:].transpose(-1, -2)) * s
    w0 = torch.softmax(w0, dim=-1).type_as(w0)
    w1 = torch.softmax(w1, dim=-1).type_as(w1)
    return torch.matmul(w0, v) - lam * torch.matmul(w1, v)


def msa_row(q_in, k_in, v_in, biases):
    q, k, v = (t.transpose(-2, -3) for t in (q_in, k_in, v_in))
    a = torch.matmul(q, k.transpose(-1, -2)) * (1 / math.sqrt(q.size(-1)))
    for b in biases:
        a += b
    return torch.matmul(F.softmax(a, dim=-1), v).transpose(-2, -3)


def returns_weights(query, key, value):
    """Not fusable: the caller wants the attention weights as well."""
    w = torch.softmax(query @ key.transpose(-2, -1) * 0.125, dim=-1)
    return w @ value, w


def relu_scores(query, key, value, causal=False):
    """A score function other than the soft-cap (softcap.py:49 takes any callable): ReLU of the scaled scores."""
    w = torch.relu(query @ key.transpose(-2, -1) / math.sqrt(query.size(-1)))
    if causal:
        w = w.masked_fill(torch.ones(w.size(-2), w.size(-1), dtype=torch.bool, device=w.device).triu(1), float("-inf"))
    return torch.softmax(w, dim=-1) @ value


def sigmoid_scores(query, key, value, bias):
    w = torch.matmul(query, key.transpose(-2, -1)) * 0.25
    w = 8.0 * torch.sigmoid(0.5 * w - 1.0) + bias
    return torch.matmul(F.softmax(w, dim=-1), value)


def clamped_scores(query, key, value):
    w = (query @ key.transpose(-2, -1) * (1 / math.sqrt(query.size(-1)))).clamp(min=-2.0, max=3.0) * 2.0
    return torch.softmax(w, dim=-1) @ value


def squared_scores(query, key, value):
    w = query @ key.transpose(-2, -1) * 0.125
    w = -0.5 * w * w + w
    return torch.softmax(w, dim=-1) @ value


def causal_with_dropout(query, key, value, p=0.1, training=True):
    """The usual module code: dropout on the attention weights, active in training mode only."""
    future = torch.triu(torch.ones(query.size(-2), key.size(-2), device=query.device, dtype=torch.bool), diagonal=1)
    w = (query @ key.transpose(-2, -1) / math.sqrt(query.size(-1))).masked_fill(future, float("-inf"))
    w = F.dropout(torch.softmax(w, dim=-1), p=p, training=training)
    return w @ value


def learned_bias_with_dropout(query, key, value, bias, p=0.2):
    w = torch.softmax(query @ key.transpose(-2, -1) * 0.125 + bias, dim=-1)
    return torch.nn.functional.dropout(w, p) @ value


def documents_with_dropout(query, key, value, document_id, p=0.1):
    same = document_id.unsqueeze(2) == document_id.unsqueeze(1)
    w = (query @ key.transpose(-2, -1) / math.sqrt(query.size(-1))).masked_fill(~same.unsqueeze(1), -1e10)
    return torch.dropout(torch.softmax(w, dim=-1), p, True) @ value


def _repeat_kv(hidden_states, n_rep):
    """Key / value heads repeated to match the query heads, as model code does before an eager attention."""
    batch, num_key_value_heads, slen, head_dim = hidden_states.shape
    if n_rep == 1:
        return hidden_states
    hidden_states = hidden_states[:, :, None, :, :].expand(batch, num_key_value_heads, n_rep, slen, head_dim)
    return hidden_states.reshape(batch, num_key_value_heads * n_rep, slen, head_dim)


def decoder_layer_attention(query, key, value, attention_mask, dropout=0.0, training=False):
    """The eager attention of a decoder layer as transformer libraries write it: repeated key / value heads, an additive
    mask [B, 1, L, S] holding the dtype's most negative number, softmax in fp32 cast back, dropout, and the result
    transposed to [B, L, H, E]."""
    n_rep = query.size(1) // key.size(1)
    key_states, value_states = _repeat_kv(key, n_rep), _repeat_kv(value, n_rep)
    attn_weights = torch.matmul(query, key_states.transpose(2, 3)) * query.size(-1) ** -0.5
    causal_mask = attention_mask[:, :, :, : key_states.shape[-2]]
    attn_weights = attn_weights + causal_mask
    attn_weights = F.softmax(attn_weights, dim=-1, dtype=torch.float32).to(query.dtype)
    attn_weights = F.dropout(attn_weights, p=dropout, training=training)
    attn_output = torch.matmul(attn_weights, value_states)
    return attn_output.transpose(1, 2).contiguous()


def decoder_layer_attention_softcapped(query, key, value, attention_mask, softcap=50.0):
    """The same with the logit soft-cap written as three statements and the heads repeated with repeat_interleave."""
    n_rep = query.size(1) // key.size(1)
    key, value = key.repeat_interleave(n_rep, dim=1), torch.repeat_interleave(value, n_rep, dim=1)
    attn_weights = torch.matmul(query, key.transpose(2, 3)) * query.size(-1) ** -0.5
    attn_weights = attn_weights / softcap
    attn_weights = torch.tanh(attn_weights)
    attn_weights = attn_weights * softcap
    attn_weights = attn_weights + attention_mask
    attn_weights = F.softmax(attn_weights, dim=-1, dtype=torch.float32).to(query.dtype)
    return torch.matmul(attn_weights, value)


def einsum_attention(q, k, v, mask=None):
    """Attention spelled with einsum on [B, H, L, E] operands, as research code often writes it."""
    s = torch.einsum("bhid,bhjd->bhij", q, k) * q.size(-1) ** -0.5
    if mask is not None:
        s = s.masked_fill(~mask, float("-inf"))
    return torch.einsum("bhij,bhjd->bhid", s.softmax(dim=-1), v)


def einsum_attention_seq_major(q, k, v):
    """The same on [B, L, H, E] operands (the layout projections produce), causal, result [B, L, H, E]."""
    L, S = q.size(1), k.size(1)
    s = torch.einsum("bqhd,bkhd->bhqk", q, k) / math.sqrt(q.size(-1))
    s = s.masked_fill(torch.ones(L, S, dtype=torch.bool, device=q.device).triu(1), float("-inf"))
    return torch.einsum("bhqk,bkhd->bqhd", torch.softmax(s, dim=-1), v)
