"""Packed-document attention (reference: attention_variants/document_mask.py)."""
from __future__ import annotations

import random

import torch

from .. import _ffi
from ._common import grouped_view, run


def attention_pytorch_document_mask(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                                    document_id: torch.Tensor, scale=None, enable_gqa=False, *,
                                    is_causal: bool = False, workspace: "_ffi.DocWorkspace | None" = None,
                                    dropout_p: float = 0.0) -> torch.Tensor:
    """document_mask.py:6-41: `document_id` is an integer tensor [N, L]; q attends k iff document_id[n, q] ==
    document_id[n, k] (both directions inside a document).  The ids may be any integers in any order; sorted ids let
    the kernel skip whole key tiles.

    is_causal (not in the reference, default off) additionally requires k <= q: the mask the reference's
    FlexAttention baseline uses for this variant (benchmarks/run_flex_variants.py:66-90).

    workspace (not in the reference): a `DocumentMaskWorkspace()` handle.  Calls that pass the same handle with the
    same `document_id` tensor and shapes derive the key tiles each query tile visits once instead of on every call, as
    that baseline builds its block mask once for all layers (run_flex_variants.py:66-90).

    dropout_p (not in the reference): dropout on the softmax weights, applied once `honor_dropout(True)` has been
    called, like the `dropout_p` of the causal, ALiBi and soft-cap variants."""
    if document_id.dim() != 2:
        raise ValueError(f"document_id must be [N, L], got {tuple(document_id.shape)}")
    kind = _ffi.MASK_DOCUMENT_CAUSAL if is_causal else _ffi.MASK_DOCUMENT
    out = run(query, key, value, scale=scale, enable_gqa=enable_gqa, mask_kind=kind, doc_ids=document_id,
              doc_workspace=workspace, dropout_p=dropout_p)
    return grouped_view(out, key, enable_gqa)


DocumentMaskWorkspace = _ffi.DocWorkspace


def create_document_id(batch_size: int, seq_len: int, num_docs: int = 12,
                       device: torch.device = torch.device("cuda")) -> torch.Tensor:
    """int64 [batch_size, seq_len] of non-decreasing document indices (document_mask.py:44-67): every document gets
    one position, the remaining seq_len - num_docs positions are dealt out with random.randint, one at a time, so a
    seeded `random` module reproduces the reference's lengths.  All batch rows share the ids."""
    if seq_len < num_docs:
        raise ValueError("Sequence length must be at least equal to the number of documents.")
    counts = [1] * num_docs
    for _ in range(seq_len - num_docs):
        counts[random.randint(0, num_docs - 1)] += 1
    ids = torch.repeat_interleave(torch.arange(num_docs, dtype=torch.int64), torch.tensor(counts, dtype=torch.int64))
    return ids.to(device).unsqueeze(0).expand(batch_size, -1)
