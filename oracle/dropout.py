"""CPU restatement of attention dropout.  TEST INFRASTRUCTURE, NOT PRODUCT CODE (see oracle/__init__.py).

The reference accepts `dropout_p` in several signatures and ignores it (attention_variants/causal.py:4-36,
alibi.py:13-33, softcap.py:4-53); this build's kernels can apply it on request.  Semantics are those of
torch.nn.functional.dropout on the softmax weights: out = ((softmax(S) * keep) / (1 - p)) @ V, the normalisation
taken over all weights, kept or not.

Which weights are kept is a pure function of (seed, batch * Hq + head, query, key), so that forward and backward
kernels and this file agree without exchanging a mask.  One 32-bit hash serves the two keys 2j, 2j + 1 of a query
(low and high half); a weight is kept when its 16 bits are >= round(p * 65536), so the effective rate is a multiple
of 2^-16.  The hash is built from 24-bit multiply-adds, shifts and xors only (full-rate vector instructions on the
GPU); tests/test_dropout.py checks its statistics and pins known values.
"""
from __future__ import annotations

import numpy as np
import torch

_M32 = np.uint64(0xFFFFFFFF)
_U = np.uint64
K_QUERY, K_PAIR = 0x9E3779B1, 0x85EBCA77       # multipliers of the query position and the key-pair index
C_ROUND1, C_ROUND2 = 0xCA6B35, 0xB2AE3D        # 24-bit multipliers of the two mixing rounds


def threshold16(p: float) -> int:
    """16-bit threshold of rate p: a weight is dropped when its 16 hash bits are below it."""
    if not 0.0 <= p < 1.0:
        raise ValueError(f"dropout_p must be in [0, 1), got {p}")
    return min(int(round(p * 65536.0)), 65535)


def effective_rate(p: float) -> float:
    return threshold16(p) / 65536.0


def _fmix32(x):
    x = _U(x) & _M32
    x ^= x >> _U(16)
    x = (x * _U(0x85EBCA6B)) & _M32
    x ^= x >> _U(13)
    x = (x * _U(0xC2B2AE35)) & _M32
    x ^= x >> _U(16)
    return x


def head_seed(seed: int, bh: int) -> int:
    """32-bit start value of (batch * Hq + head) under a 64-bit seed."""
    lo, hi = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
    inner = _fmix32((_U(hi) + _U(0x9E3779B9) * _U(bh + 1)) & _M32)
    return int(_fmix32(_U(lo) ^ inner))


def _mad24(a, c, b):
    return ((a & _U(0xFFFFFF)) * _U(c) + b) & _M32


def pair_hash(s0: int, q, kp):
    """32 bits for query position(s) q and key-pair index(es) kp (numpy uint64 arrays, broadcast together)."""
    x = (_U(s0) + q.astype(np.uint64) * _U(K_QUERY) + kp.astype(np.uint64) * _U(K_PAIR)) & _M32
    x ^= x >> _U(16)
    x = _mad24(x, C_ROUND1, x >> _U(8))
    x ^= x >> _U(13)
    x = _mad24(x >> _U(8), C_ROUND2, x)
    x ^= x >> _U(16)
    return x


def random16(seed: int, bh: int, Lq: int, Lk: int) -> np.ndarray:
    """[Lq, Lk] int64 array of the 16 bits that decide each weight of one (batch, head)."""
    q = np.arange(Lq, dtype=np.uint64)[:, None]
    k = np.arange(Lk, dtype=np.uint64)[None, :]
    x = pair_hash(head_seed(seed, bh), q, k >> _U(1))
    return np.where((k & _U(1)) == 1, x >> _U(16), x & _U(0xFFFF)).astype(np.int64)


def keep_mask(seed: int, B: int, Hq: int, Lq: int, Lk: int, p: float) -> torch.Tensor:
    """bool [B, Hq, Lq, Lk]: True where the weight survives."""
    thr = threshold16(p)
    out = np.empty((B, Hq, Lq, Lk), dtype=bool)
    for b in range(B):
        for h in range(Hq):
            out[b, h] = random16(seed, b * Hq + h, Lq, Lk) >= thr
    return torch.from_numpy(out)


def attention_dropout(query, key, value, keep: torch.Tensor, p: float, scale=None, *, attend=None, bias=None,
                      softcap=None):
    """softmax(S) with dropout, times V.  query [B, Hq, L, E]; key/value [B, H, S, E*]; Hq a multiple of H.
    keep: bool [B, Hq, L, S]; p: the rate whose 1 / (1 - p_effective) rescales the kept weights;
    attend: optional bool [.., L, S] (False = masked out); bias: optional additive [.., L, S] (after the soft-cap);
    softcap: optional cap of cap * tanh(s / cap).  Differentiable (torch autograd) in query, key, value."""
    B, Hq, L, E = query.shape
    H = key.shape[1]
    g = Hq // H
    k = key.repeat_interleave(g, dim=1)
    v = value.repeat_interleave(g, dim=1)
    sc = (1.0 / E ** 0.5) if scale is None else scale
    s = torch.matmul(query, k.transpose(-1, -2)) * sc
    if softcap is not None:
        s = softcap * torch.tanh(s / softcap)
    if bias is not None:
        s = s + bias
    if attend is not None:
        s = s.masked_fill(~attend, float("-inf"))
    w = torch.softmax(s, dim=-1)
    w = torch.nan_to_num(w, nan=0.0)  # rows that attend nothing
    w = w * keep.to(w.dtype) / (1.0 - effective_rate(p))
    return torch.matmul(w, v)
