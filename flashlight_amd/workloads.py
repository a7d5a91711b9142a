"""The five benchmark configurations as seeded synthetic inputs, with exact attended-pair and FLOP counts.

FLOPs are algorithmic: 2 * (sum of Dqk + sum of Dv over the softmax branches) per attended (q, k) pair per query
head; exp, tanh, bias and gate work is not counted.  Pair counts are closed forms of each mask.
"""
from __future__ import annotations

import math
import random
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional

import torch

PEAK_BF16_TFLOPS = 2516.6  # MI355X dense bf16 MFMA: 256 CU x 4096 FLOP/clk x 2.4 GHz
PEAK_HBM_GBPS = 8000.0


def pairs_none(S: int) -> int:
    return S * S


def pairs_causal(S: int) -> int:
    return S * (S + 1) // 2


def pairs_sliding(S: int, W: int) -> int:
    W = min(W, S - 1)
    return (W + 1) * (W + 2) // 2 + (S - W - 1) * (W + 1)


def pairs_prefix(S: int, P: int) -> int:
    P = max(0, min(P, S))
    return P * P + S * (S + 1) // 2 - P * (P + 1) // 2


def pairs_documents(lengths: List[int], causal: bool) -> int:
    return sum(n * (n + 1) // 2 if causal else n * n for n in lengths)


def document_lengths(seq_len: int, seed: int, lo: int = 512, hi: int = 4096) -> List[int]:
    """Lengths uniform in [lo, hi] from random.Random(seed), drawn until they cover seq_len; the last is truncated."""
    rng = random.Random(seed)
    out, total = [], 0
    while total < seq_len:
        n = min(rng.randint(lo, hi), seq_len - total)
        out.append(n)
        total += n
    return out


def document_ids(lengths: List[int], batch: int, device) -> torch.Tensor:
    ids = torch.repeat_interleave(torch.arange(len(lengths), dtype=torch.int64), torch.tensor(lengths, dtype=torch.int64))
    return ids.to(device).unsqueeze(0).expand(batch, -1).contiguous()


@dataclass
class Workload:
    name: str            # e.g. "cfg1/causal"
    config: int          # number of the benchmark configuration (1-4)
    seed: int
    shapes: Dict[str, tuple]
    pairs_per_head: int  # attended (q, k) pairs per query head (per (n, h) for Evoformer)
    heads: int           # batch * query heads the pairs are counted for
    flops_per_pair: int
    min_bytes: int       # q + k + v + out (+ bias + gate + ids), each touched once
    make: Callable[[torch.device], dict] = field(repr=False, default=None)
    call: Callable[[dict], torch.Tensor] = field(repr=False, default=None)
    params: Dict[str, float] = field(default_factory=dict)  # the variant's own arguments (window, prefix, cap, lambda)
    bound: str = "mfma"  # the roofline that bounds the launch: "mfma", or "hbm" where a head's work is a few key tiles

    @property
    def flops(self) -> int:
        return self.flops_per_pair * self.pairs_per_head * self.heads


def _randn(gen: torch.Generator, shape, device) -> torch.Tensor:
    # drawn on the CPU generator so that CPU and GPU runs see the same values, then moved
    return torch.randn(shape, generator=gen, dtype=torch.float32).to(torch.bfloat16).to(device)


def _qkv(seed, B, Hq, Hkv, S, D, Dv=None):
    def make(device):
        g = torch.Generator().manual_seed(seed)
        return {"q": _randn(g, (B, Hq, S, D), device), "k": _randn(g, (B, Hkv, S, D), device),
                "v": _randn(g, (B, Hkv, S, Dv or D), device)}
    return make


def build_workloads(scale_down: int = 1) -> List[Workload]:
    """All variants of benchmark configurations 1-4.  scale_down > 1 shrinks sequence lengths (and windows/prefixes with
    them) for quick parity runs; 1 gives the full sizes."""
    from .attention_variants import (attention_pytorch, attention_pytorch_alibi, attention_pytorch_causal,
                                     attention_pytorch_document_mask, attention_pytorch_prefix_lm,
                                     attention_pytorch_sliding_window, attention_reference, diffattn,
                                     generate_alibi_bias_pytorch)
    sd = scale_down
    W: List[Workload] = []

    # cfg1: B=4 H=16 S=4096 D=128
    B, H, S, D = 4, 16, 4096 // sd, 128
    io = 2 * (3 * B * H * S * D + B * H * S * D)
    win = 256 // sd
    for name, pairs, fn in (
            ("vanilla", pairs_none(S), lambda t: attention_pytorch(t["q"], t["k"], t["v"])),
            ("causal", pairs_causal(S), lambda t: attention_pytorch_causal(t["q"], t["k"], t["v"])),
            ("sliding_window", pairs_sliding(S, win),
             lambda t, win=win: attention_pytorch_sliding_window(t["q"], t["k"], t["v"], window_size=win))):
        W.append(Workload(f"cfg1/{name}", 1, 1001, {"q": (B, H, S, D), "kv": (B, H, S, D)}, pairs, B * H, 4 * D, io,
                          _qkv(1001, B, H, H, S, D), fn, params={"window": win} if name == "sliding_window" else {},
                          bound="hbm" if name == "sliding_window" else "mfma"))

    # cfg2: GQA + ALiBi + softcap 50 + causal, B=2 Hq=32 Hkv=8 S=8192 D=128
    B, Hq, Hkv, S, D = 2, 32, 8, 8192 // sd, 128
    io = 2 * (2 * B * Hq * S * D + 2 * B * Hkv * S * D)
    W.append(Workload("cfg2/gqa_alibi_softcap_causal", 2, 1002, {"q": (B, Hq, S, D), "kv": (B, Hkv, S, D)},
                      pairs_causal(S), B * Hq, 4 * D, io, _qkv(1002, B, Hq, Hkv, S, D),
                      lambda t: attention_pytorch_alibi(t["q"], t["k"], t["v"],
                                                        score_mod=generate_alibi_bias_pytorch(t["q"].size(1)),
                                                        is_causal=True, enable_gqa=True, softcap=50.0),
                      params={"softcap": 50.0}))

    # cfg3a: document mask, causal within each document, B=1 H=16 S=16384 D=64
    B, H, S, D = 1, 16, 16384 // sd, 64
    lengths = document_lengths(S, 1003, 512 // sd, 4096 // sd)
    io = 2 * 4 * B * H * S * D + 8 * B * S

    def make_doc(device, B=B, H=H, S=S, D=D, lengths=lengths):
        t = _qkv(1003, B, H, H, S, D)(device)
        t["document_id"] = document_ids(lengths, B, device)
        return t
    W.append(Workload("cfg3/document_mask_causal", 3, 1003, {"q": (B, H, S, D), "kv": (B, H, S, D), "docs": len(lengths)},
                      pairs_documents(lengths, True), B * H, 4 * D, io, make_doc,
                      lambda t: attention_pytorch_document_mask(t["q"], t["k"], t["v"], t["document_id"], is_causal=True)))

    # cfg3b: prefix-LM, B=4 H=16 S=4096 D=64, prefix 1024
    B, H, S, D = 4, 16, 4096 // sd, 64
    P = 1024 // sd
    io = 2 * 4 * B * H * S * D
    W.append(Workload("cfg3/prefix_lm", 3, 1013, {"q": (B, H, S, D), "kv": (B, H, S, D)}, pairs_prefix(S, P), B * H,
                      4 * D, io, _qkv(1013, B, H, H, S, D),
                      lambda t, P=P: attention_pytorch_prefix_lm(t["q"], t["k"], t["v"], prefix_lengths=P),
                      params={"prefix": P}))

    # cfg4a: differential attention, B=2 H=16 (q, k: 32 heads x 64; v: 16 heads x 128), S=4096, causal, lambda 0.8
    B, H, S, d = 2, 16, 4096 // sd, 64
    io = 2 * (2 * B * 2 * H * S * d + 2 * B * H * S * 2 * d)

    def make_diff(device, B=B, H=H, S=S, d=d):
        g = torch.Generator().manual_seed(1004)
        return {"q": _randn(g, (B, 2 * H, S, d), device), "k": _randn(g, (B, 2 * H, S, d), device),
                "v": _randn(g, (B, H, S, 2 * d), device)}
    W.append(Workload("cfg4/diff_attn_causal", 4, 1004, {"q": (B, 2 * H, S, d), "v": (B, H, S, 2 * d)}, pairs_causal(S),
                      B * H, 2 * (2 * d + 2 * 2 * d), io, make_diff,
                      lambda t: diffattn(t["q"], t["k"], t["v"], lambda_full=0.8, is_causal=True),
                      params={"lambda_full": 0.8}))

    # cfg4b: Evoformer row attention, B=1 N_seq=256 N_res=384 H=8 D=32, pair bias + sigmoid gate
    B, Nseq, S, H, D = 1, 256 // sd, 384, 8, 32
    io = 2 * (4 * B * Nseq * S * H * D + B * H * S * S + B * Nseq * S * H * D)

    def make_evo(device, B=B, Nseq=Nseq, S=S, H=H, D=D):
        g = torch.Generator().manual_seed(1014)
        t = {n: _randn(g, (B, Nseq, S, H, D), device) for n in ("q", "k", "v")}
        t["pair_bias"] = _randn(g, (B, 1, H, S, S), device)
        t["gate"] = _randn(g, (B, Nseq, S, H, D), device)
        return t
    W.append(Workload("cfg4/evoformer_bias_gate", 4, 1014, {"qkv": (B, Nseq, S, H, D), "bias": (B, 1, H, S, S)},
                      pairs_none(S), B * Nseq * H, 4 * D, io, make_evo,
                      lambda t: attention_reference(t["q"], t["k"], t["v"], [t["pair_bias"]], gate=t["gate"]),
                      bound="hbm"))
    return W


def workload_by_name(name: str, scale_down: int = 1) -> Workload:
    for w in build_workloads(scale_down):
        if w.name == name:
            return w
    raise KeyError(name)
