"""Writes tests/golden/attention_golden.npz: small known-answer vectors for every attention variant.

Expected outputs come from library routines only -- torch.nn.functional.scaled_dot_product_attention in float64 with
masks and biases built by explicit Python loops -- never from oracle/ or flashlight_amd/, and the reference's code is
not imported.  Inputs are N(0,1) draws rounded to bfloat16 and stored as their 16-bit patterns, so a bf16 kernel and
a float64 routine see identical values.  Run from the repo root:  python tests/golden/make_golden.py
"""
from __future__ import annotations

import math
from pathlib import Path

import numpy as np
import torch
import torch.nn.functional as F

OUT = Path(__file__).resolve().parent / "attention_golden.npz"


def bf16_randn(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def loop_mask(L, S, fn):
    m = torch.zeros(L, S, dtype=torch.bool)
    for q in range(L):
        for k in range(S):
            m[q, k] = bool(fn(q, k))
    return m


def sdpa(q, k, v, *, mask=None, scale=None, gqa=False):
    """float64 SDPA; q [N,Hq,L,E], k/v [N,Hkv,S,E]; query head h reads key head h // (Hq/Hkv)."""
    q, k, v = q.double(), k.double(), v.double()
    if gqa:
        g = q.size(1) // k.size(1)
        k, v = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    if mask is not None and mask.dtype != torch.bool:
        mask = mask.double()
    return F.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=scale)


def main():
    g = torch.Generator().manual_seed(20251125)
    rec = {}

    def put(name, inputs: dict, expected: torch.Tensor, **meta):
        for key, t in inputs.items():
            if t.dtype == torch.bfloat16:
                rec[f"{name}/{key}.bf16"] = bits(t)
            else:
                rec[f"{name}/{key}"] = t.numpy()
        rec[f"{name}/expected"] = expected.to(torch.float32).numpy()
        for key, val in meta.items():
            rec[f"{name}/meta.{key}"] = np.asarray(val)

    # vanilla with grouped heads, D=128
    q, k, v = bf16_randn(g, 1, 4, 100, 128), bf16_randn(g, 1, 2, 100, 128), bf16_randn(g, 1, 2, 100, 128)
    put("vanilla_gqa", dict(q=q, k=k, v=v), sdpa(q, k, v, gqa=True))

    # causal, D=64, ragged length
    L = 131
    q, k, v = (bf16_randn(g, 2, 2, L, 64) for _ in range(3))
    put("causal", dict(q=q, k=k, v=v), sdpa(q, k, v, mask=loop_mask(L, L, lambda a, b: b <= a)))

    # sliding window W=17 (attends 0 <= q-k <= 17)
    L, W = 150, 17
    q, k, v = (bf16_randn(g, 1, 2, L, 64) for _ in range(3))
    put("sliding", dict(q=q, k=k, v=v), sdpa(q, k, v, mask=loop_mask(L, L, lambda a, b: 0 <= a - b <= W)), window=W)

    # prefix-LM P=40
    L, P = 140, 40
    q, k, v = (bf16_randn(g, 1, 2, L, 64) for _ in range(3))
    put("prefix_lm", dict(q=q, k=k, v=v), sdpa(q, k, v, mask=loop_mask(L, L, lambda a, b: b < P or b <= a)), prefix=P)

    # document masks: sorted ids with uneven lengths, and unsorted arbitrary ids
    L = 160
    ids_sorted = torch.tensor([0] * 7 + [1] * 50 + [5] * 33 + [9] * 70, dtype=torch.int64)
    ids_mixed = torch.tensor([(i * 7 + i // 13) % 3 - 1 for i in range(L)], dtype=torch.int64)
    for tag, ids in (("sorted", ids_sorted), ("mixed", ids_mixed)):
        q, k, v = (bf16_randn(g, 1, 2, L, 64) for _ in range(3))
        same = loop_mask(L, L, lambda a, b: ids[a] == ids[b])
        put(f"document_{tag}", dict(q=q, k=k, v=v, document_id=ids[None]), sdpa(q, k, v, mask=same))
        put(f"document_causal_{tag}", dict(q=q, k=k, v=v, document_id=ids[None]),
            sdpa(q, k, v, mask=same & loop_mask(L, L, lambda a, b: b <= a)))

    # ALiBi with grouped heads: bias[h, q, k] = 2^(-8 (h+1) / H) * (k - q)
    L, H = 120, 4
    q, k, v = bf16_randn(g, 1, H, L, 64), bf16_randn(g, 1, 2, L, 64), bf16_randn(g, 1, 2, L, 64)
    bias = torch.zeros(H, L, L, dtype=torch.float64)
    for h in range(H):
        for a in range(L):
            for b in range(L):
                bias[h, a, b] = 2.0 ** (-8.0 * (h + 1) / H) * (b - a)
    put("alibi_gqa", dict(q=q, k=k, v=v), sdpa(q, k, v, mask=bias[None], gqa=True))

    # tanh soft-cap (cap 5 so that the cap bites on N(0,1) logits scaled up by 4), explicit float64 math
    L, cap, sc = 100, 5.0, 0.5
    q, k, v = (bf16_randn(g, 1, 2, L, 64) for _ in range(3))
    s = q.double() @ k.double().transpose(-1, -2) * sc
    put("softcap", dict(q=q, k=k, v=v), torch.softmax(cap * torch.tanh(s / cap), -1) @ v.double(), cap=cap, scale=sc)

    # softcap + ALiBi + causal + GQA, D=128 (the combination of benchmark config 2)
    L, H, cap = 130, 4, 50.0
    q, k, v = bf16_randn(g, 1, H, L, 128), bf16_randn(g, 1, 1, L, 128), bf16_randn(g, 1, 1, L, 128)
    s = q.double() @ k.double().repeat_interleave(H, 1).transpose(-1, -2) / math.sqrt(128)
    s = cap * torch.tanh(s / cap)
    for h in range(H):
        for a in range(L):
            for b in range(L):
                s[0, h, a, b] = s[0, h, a, b] + 2.0 ** (-8.0 * (h + 1) / H) * (b - a) if b <= a else float("-inf")
    put("alibi_softcap_causal_gqa", dict(q=q, k=k, v=v), torch.softmax(s, -1) @ v.double().repeat_interleave(H, 1),
        cap=cap)

    # differential attention: heads split in halves, lambda 0.8; plain and causal
    L, H, d, lam = 110, 2, 64, 0.8
    q, k, v = bf16_randn(g, 1, 2 * H, L, d), bf16_randn(g, 1, 2 * H, L, d), bf16_randn(g, 1, H, L, 2 * d)
    for tag, m in (("", None), ("_causal", loop_mask(L, L, lambda a, b: b <= a))):
        e = sdpa(q[:, :H], k[:, :H], v, mask=m) - lam * sdpa(q[:, H:], k[:, H:], v, mask=m)
        put(f"diff_attn{tag}", dict(q=q, k=k, v=v), e, lambda_full=lam)

    # Evoformer row attention: inputs [B, N, S, H, D], mask bias [B, N, 1, 1, S], pair bias [B, 1, H, S, S], gate
    B, N, S, H, D = 2, 3, 70, 2, 32
    q, k, v = (bf16_randn(g, B, N, S, H, D) for _ in range(3))
    b1, b2, gate = bf16_randn(g, B, N, 1, 1, S), bf16_randn(g, B, 1, H, S, S), bf16_randn(g, B, N, S, H, D)
    t = lambda x: x.double().transpose(-2, -3)
    e = F.scaled_dot_product_attention(t(q), t(k), t(v), attn_mask=(b1.double() + b2.double())).transpose(-2, -3)
    put("evoformer", dict(q=q, k=k, v=v, bias1=b1, bias2=b2), e)
    sig = torch.empty_like(e)
    gf = gate.double().flatten()
    sig_flat = torch.tensor([1.0 / (1.0 + math.exp(-x)) for x in gf.tolist()], dtype=torch.float64)
    put("evoformer_gate", dict(q=q, k=k, v=v, bias1=b1, bias2=b2, gate=gate), e * sig_flat.view_as(e))

    np.savez_compressed(OUT, **rec)
    print(f"wrote {OUT} ({OUT.stat().st_size / 1024:.0f} KiB, {len(rec)} arrays)")


if __name__ == "__main__":
    main()
