"""Row-wise self-attention of the Evoformer with additive biases (reference: attention_variants/evoformer.py)."""
from __future__ import annotations

import math
from typing import List, Optional, Sequence

import torch

from .. import _ffi, ops

N = 256  # number of MSA rows in the reference's benchmark inputs (evoformer.py:39)


def _as_kernel_bias(b: torch.Tensor, lead: Sequence[int], H: int, S: int):
    """Maps a bias broadcastable to [*lead, H, S, S] onto the kernel's ([Bb, H|1, S|1, S], batch_div) form, where the
    kernel reads batch index flat_batch // batch_div.  Works without copying when the bias's leading axes are
    (full ..., 1 ...) against `lead`; otherwise the bias is expanded over the leading axes first."""
    nl = len(lead)
    if b.dim() > nl + 3:
        raise ValueError(f"bias of shape {tuple(b.shape)} has more axes than the scores")
    b = b.reshape((1,) * (nl + 3 - b.dim()) + tuple(b.shape))
    bl, tail = tuple(b.shape[:nl]), tuple(b.shape[nl:])
    for got, want in zip(tail, (H, S, S)):
        if got not in (1, want):
            raise ValueError(f"bias tail {tail} does not broadcast to {(H, S, S)}")
    if tail[2] != S:
        b = b.expand(*bl, tail[0], tail[1], S)
    split = nl
    while split > 0 and bl[split - 1] == 1:
        split -= 1
    if any(bl[i] != lead[i] for i in range(split)):
        b = b.expand(*lead, *b.shape[nl:])
        bl, split = tuple(lead), nl
    div = math.prod(lead[split:]) if split < nl else 1
    nb = math.prod(bl[:split]) if split else 1
    return b.reshape(nb, *b.shape[nl:]), int(div)


def attention_reference(q_input: torch.Tensor, k_input: torch.Tensor, v_input: torch.Tensor,
                        biases: List[torch.Tensor], sm_scale: Optional[float] = None, **kwargs) -> torch.Tensor:
    """evoformer.py:8-36: inputs [*, S, H, D] (e.g. [B, N_seq, N_res, H, D]); every tensor in `biases`
    (broadcastable to [*, H, S, S], e.g. a mask bias [B, N, 1, 1, S] and a pair bias [B, 1, H, S, S]) is added to
    q k^T * sm_scale before the softmax; returns [*, S, H, D].  The [*, S, H, D] layout is read and written in place
    through strides: nothing is transposed in memory.

    `gate=` (not in the reference): bf16 logits shaped like the result; the result is multiplied by sigmoid(gate)
    in the kernel's epilogue."""
    gate = kwargs.get("gate")
    if q_input.dim() < 4:
        raise ValueError("expected inputs of shape [*, S, H, D]")
    lead = tuple(q_input.shape[:-3])
    S, H, D = q_input.shape[-3:]
    Sk = k_input.shape[-3]
    Dv = v_input.shape[-1]

    def heads_first(t):  # [*, S, H, D] -> 4-D view [prod(*), H, S, D]
        return t.reshape(-1, *t.shape[-3:]).transpose(1, 2)

    bl = list(biases)
    if len(bl) > 2:  # the kernel takes two bias operands; fold the rest into the second one, in fp32 (a sum rounded to
        extra = bl[1].float()  # 16 bits would move the logits by the rounding of their largest term)
        for b in bl[2:]:
            extra = extra + b.float()
        bl = [bl[0], extra]
    if S != Sk and bl:
        raise ValueError("biases need equally long query and key sequences")
    kb = [_as_kernel_bias(b, lead, H, S) for b in bl]

    # the result comes back as the [prod(*), H, S, Dv] view of a buffer in [prod(*), S, H, Dv] memory order
    out = ops.dispatch(heads_first(q_input), heads_first(k_input), heads_first(v_input), scale=sm_scale, biases=kb,
                       gate=None if gate is None else heads_first(gate), seq_major_out=True)
    return out.transpose(1, 2).reshape(*lead, S, H, Dv)


def make_input(config, attention_name="ipa"):
    """Inputs of the reference's benchmark (evoformer.py:41-49): config = (batch, seqlen, nheads, headdim, ...);
    Q, K, V ~ N(0,1) [batch, N, seqlen, nheads, headdim], mask bias [batch, N, 1, 1, seqlen] and pair bias
    [batch, 1, nheads, seqlen, seqlen], all bf16."""
    batch, seqlen, nheads, headdim = config[:4]
    qkv = [torch.randn(batch, N, seqlen, nheads, headdim, dtype=torch.bfloat16, device="cuda") for _ in range(3)]
    bias1 = torch.randn(batch, N, 1, 1, seqlen, dtype=torch.bfloat16, device="cuda")
    bias2 = torch.randn(batch, 1, nheads, seqlen, seqlen, dtype=torch.bfloat16, device="cuda")
    return (*qkv, [bias1, bias2])
