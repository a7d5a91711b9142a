"""Mask predicates of the attention variants as dense boolean matrices, and closed-form attended-pair counts.

TEST INFRASTRUCTURE (see oracle/__init__.py).  "attend" means the pair takes part in the softmax.
Predicates follow the reference line by line:
  causal          masked iff k > q                       attention_variants/causal.py:32-33
  sliding window  masked iff q < k or q - k > W          attention_variants/sliding_window.py:4-12
  prefix-LM       masked iff k > max(P - 1, q)           attention_variants/prefix_lm.py:33-42
  document        masked iff doc[q] != doc[k]            attention_variants/document_mask.py:25-27
  document+causal additionally k <= q                    benchmarks/run_flex_variants.py:66-90 (Flex baseline)
"""
from __future__ import annotations

import random
from typing import Optional, Sequence

import numpy as np

KINDS = ("none", "causal", "sliding", "prefix", "document", "document_causal")


def attend_matrix(kind: str, Lq: int, Lk: int, *, window: int = 0, prefix: int = 0,
                  doc_ids: Optional[Sequence[int]] = None) -> np.ndarray:
    """Boolean [Lq, Lk]; True where query row q attends key column k (positions top-left aligned)."""
    q = np.arange(Lq, dtype=np.int64)[:, None]
    k = np.arange(Lk, dtype=np.int64)[None, :]
    if kind == "none":
        return np.ones((Lq, Lk), dtype=bool)
    if kind == "causal":
        return ~(k > q)
    if kind == "sliding":
        return ~((q < k) | ((q - k) > window))
    if kind == "prefix":
        return ~(k > np.maximum(prefix - 1, q))
    if kind in ("document", "document_causal"):
        d = np.asarray(doc_ids, dtype=np.int64)
        if d.shape != (Lq,) or Lq != Lk:
            raise ValueError("document ids must be one id per position and Lq == Lk")
        same = d[:, None] == d[None, :]
        return same & (k <= q) if kind == "document_causal" else same
    raise ValueError(f"unknown mask kind {kind!r}")


def attended_pairs(kind: str, S: int, *, window: int = 0, prefix: int = 0,
                   doc_lengths: Optional[Sequence[int]] = None) -> int:
    """Closed-form number of attended (q, k) pairs per head for Lq == Lk == S."""
    if kind == "none":
        return S * S
    if kind == "causal":
        return S * (S + 1) // 2
    if kind == "sliding":
        W = min(window, S - 1)
        return (W + 1) * (W + 2) // 2 + (S - W - 1) * (W + 1)
    if kind == "prefix":
        P = max(0, min(prefix, S))
        return P * P + S * (S + 1) // 2 - P * (P + 1) // 2
    if kind == "document":
        assert sum(doc_lengths) == S
        return sum(n * n for n in doc_lengths)
    if kind == "document_causal":
        assert sum(doc_lengths) == S
        return sum(n * (n + 1) // 2 for n in doc_lengths)
    raise ValueError(f"unknown mask kind {kind!r}")


def document_lengths_cfg3(seq_len: int, seed: int, lo: int = 512, hi: int = 4096) -> list[int]:
    """Document lengths drawn uniformly in [lo, hi] from random.Random(seed) until they cover seq_len;
    the last one is truncated so the lengths sum to seq_len."""
    rng = random.Random(seed)
    out: list[int] = []
    total = 0
    while total < seq_len:
        n = rng.randint(lo, hi)
        n = min(n, seq_len - total)
        out.append(n)
        total += n
    return out


def document_ids_from_lengths(lengths: Sequence[int]) -> np.ndarray:
    """int64 [sum(lengths)]: position -> index of its document (non-decreasing)."""
    return np.repeat(np.arange(len(lengths), dtype=np.int64), np.asarray(lengths, dtype=np.int64))
