"""Invariant point attention as one fused launch (reference: tests/test_ipa.py:57-125, a test-only function).

logits[i, j] = (q_i / sqrt(c_hidden)) . k_j  +  w * sum_p |qp_ip - kp_jp|^2  +  pair_bias[i, j],
w = -0.5 * sqrt(9 / (2 * no_qk_points)), and the softmax weights aggregate both the scalar values and the value points.

The squared distances never exist as an [N, N] tensor here.  Expanding |qp - kp|^2 = |qp|^2 + |kp|^2 - 2 qp . kp:
  * the |qp|^2 term is constant along a softmax row and drops out,
  * the cross term is a dot product, so the point coordinates are appended to the scalar channels of q and k and ride
    the same matrix product (the kernel's scale is -2 w, applied in fp32, and the scalar query channels are
    pre-multiplied so that their share comes out as 1 / sqrt(c_hidden)),
  * the |kp|^2 term is a per-key fp32 row added through the kernel's second bias operand.
Scalar values and value points are concatenated along the value axis, so both aggregations are one P V product.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from .. import _ffi, ops

# (Dqk, Dv) pairs with a kernel instance that takes bias operands, cheapest first
_BIAS_SHAPES = ((32, 32), (32, 64), (64, 64), (64, 128), (128, 128))


def _padded_dims(dqk: int, dv: int) -> Tuple[int, int]:
    for pq, pv in _BIAS_SHAPES:
        if pq >= dqk and pv >= dv:
            return pq, pv
    raise NotImplementedError(f"{dqk} query/key channels and {dv} value channels (scalar + point coordinates) exceed "
                              f"the widest kernel instance {_BIAS_SHAPES[-1]}")


def point_weight(no_qk_points: int) -> float:
    """Weight of the summed squared distances in the logits (tests/test_ipa.py:107)."""
    return -0.5 * (9.0 / (2 * no_qk_points)) ** 0.5


def invariant_point_attention(q_scalar: torch.Tensor, k_scalar: torch.Tensor, v_scalar: torch.Tensor,
                              q_points: torch.Tensor, k_points: torch.Tensor, v_points: torch.Tensor,
                              pair_bias: Optional[torch.Tensor], frames=None, mask=None, c_hidden: int = 64,
                              no_qk_points: int = 8) -> Tuple[torch.Tensor, torch.Tensor]:
    """tests/test_ipa.py:57-125.  q/k/v_scalar [*, H, N, C]; q/k_points [*, H, N, Pqk, X] and v_points
    [*, H, N, Pv, X] (X coordinates per point: 3, or 4 as in the reference's test inputs); pair_bias broadcastable to
    [*, H, N, N] or None.

    Returns (output_scalar [*, H, N, C], output_points [*, N, H, Pv, X]), the two aggregations of
    test_ipa.py:117-122.  The reference's last line adds the two, which only broadcasts for degenerate sizes; its
    commented-out variants return the pair, which is what callers need.

    `frames` and `mask` are accepted and unused, as in the reference (the frame transforms and the mask are commented
    out there: test_ipa.py:84-86, 111-112, 122).  `no_qk_points` enters only through the distance weight."""
    lead = tuple(q_scalar.shape[:-3])
    H, N, C = q_scalar.shape[-3:]
    S = k_scalar.shape[-2]
    if q_points.shape[:-2] != q_scalar.shape[:-1] or k_points.shape[:-2] != k_scalar.shape[:-1] or \
            v_points.shape[:-2] != v_scalar.shape[:-1]:
        raise ValueError("points must be [*, H, N, P, X] with the leading axes of the scalar tensors")
    if q_points.shape[-2:] != k_points.shape[-2:]:
        raise ValueError("query and key points differ in count or coordinates")
    Pv, X = v_points.shape[-2:]
    nq = q_points.shape[-2] * q_points.shape[-1]
    nv = Pv * X
    dqk, dv = _padded_dims(C + nq, v_scalar.shape[-1] + nv)

    w = point_weight(no_qk_points)
    scale = -2.0 * w  # > 0; multiplies the whole q k^T in the kernel
    B = math.prod(lead) if lead else 1

    def flat(t, tail):  # [*, H, n, ...tail] -> [B, H, n, prod(tail)]
        return t.reshape(B, H, t.shape[len(lead) + 1], tail)

    cv = v_scalar.shape[-1]
    q_scale = 1.0 / (math.sqrt(c_hidden) * scale)
    if torch.compiler.is_compiling() or S != N or q_scalar.dtype != torch.bfloat16:
        # traced, fp16, or cross-attention (which the packing kernel's single row count does not cover): tensor code
        qs = (flat(q_scalar, C).float() * q_scale).to(q_scalar.dtype)
        q_cat = F.pad(torch.cat([qs, flat(q_points, nq)], dim=-1), (0, dqk - C - nq))
        k_cat = F.pad(torch.cat([flat(k_scalar, C), flat(k_points, nq)], dim=-1), (0, dqk - C - nq))
        v_cat = F.pad(torch.cat([flat(v_scalar, cv), flat(v_points, nv)], dim=-1), (0, dv - cv - nv))
        key_term = (w * flat(k_points, nq).float().square().sum(-1)).unsqueeze(-2)  # [B, H, 1, S] fp32
    else:
        # one launch builds all four operands
        rows = B * H * N
        q_cat, k_cat, v_cat, key_term = _ffi.ipa_pack(
            q_scalar.reshape(rows, C), k_scalar.reshape(rows, C), v_scalar.reshape(rows, cv), q_points.reshape(rows, nq),
            k_points.reshape(rows, nq), v_points.reshape(rows, nv), dqk, dv, q_scale, w)
        q_cat, k_cat, v_cat = q_cat.view(B, H, N, dqk), k_cat.view(B, H, N, dqk), v_cat.view(B, H, N, dv)
        key_term = key_term.view(B, H, 1, N)
    biases = []
    if pair_bias is not None:
        pb = pair_bias
        if pb.dim() > len(lead) + 3:
            raise ValueError(f"pair_bias of shape {tuple(pb.shape)} has more axes than the logits")
        pb = pb.reshape((1,) * (len(lead) + 3 - pb.dim()) + tuple(pb.shape))
        if any(a != 1 for a in pb.shape[:len(lead)]):
            pb = pb.expand(*lead, *pb.shape[len(lead):])
            pb = pb.reshape(B, *pb.shape[len(lead):])
            div = 1
        else:
            pb = pb.reshape(1, *pb.shape[len(lead):])
            div = B
        if pb.size(-1) != S:
            pb = pb.expand(*pb.shape[:-1], S).contiguous()
        if pb.dtype != torch.float32 and pb.dtype != q_scalar.dtype:
            pb = pb.float()
        biases.append((pb, div))
    biases.append((key_term, 1))

    out = ops.dispatch(q_cat, k_cat, v_cat, scale=scale, biases=biases)  # [B, H, N, dv]
    out_scalar = out[..., :cv].reshape(*lead, H, N, cv)
    out_points = out[..., cv:cv + nv].reshape(*lead, H, N, Pv, X).transpose(-3, -4)
    return out_scalar, out_points
