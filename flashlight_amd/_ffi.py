"""ctypes binding of libflashlight_amd.so (declared in include/flashlight_amd.h).

PyTorch is used only for device memory and the current HIP stream; every compute call goes through the C ABI.
There is no fallback: a missing library or a non-GPU tensor raises.
"""
from __future__ import annotations

import ctypes as C
import math
import os
from pathlib import Path
from typing import Optional, Sequence

import torch

LIB_NAME = "libflashlight_amd.so"
LIB_PATH = Path(os.environ.get("FL_LIB") or Path(__file__).resolve().parent / LIB_NAME)

MASK_NONE, MASK_CAUSAL, MASK_SLIDING, MASK_PREFIX_LM, MASK_DOCUMENT, MASK_DOCUMENT_CAUSAL = range(6)
FL_BF16 = 0
FL_F32 = 1
FL_F16 = 2
ABI_VERSION = 1


class FlAttnParams(C.Structure):
    """Mirror of `fl_attn_params` (include/flashlight_amd.h); field order and types must match."""

    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
        ("q_strides", C.c_int64 * 4), ("k_strides", C.c_int64 * 4),
        ("v_strides", C.c_int64 * 4), ("o_strides", C.c_int64 * 4),
        ("B", C.c_int32), ("Hq", C.c_int32), ("Hkv", C.c_int32), ("Lq", C.c_int32), ("Lk", C.c_int32),
        ("Dqk", C.c_int32), ("Dv", C.c_int32),
        ("scale", C.c_float),
        ("mask_kind", C.c_int32), ("window", C.c_int32), ("prefix", C.c_int32),
        ("doc_ids", C.c_void_p), ("doc_stride", C.c_int64),
        ("alibi_heads", C.c_int32), ("softcap", C.c_float),
        ("bias", C.c_void_p * 2), ("bias_strides", (C.c_int64 * 4) * 2), ("bias_batch_div", C.c_int32 * 2),
        ("gate", C.c_void_p), ("gate_strides", C.c_int64 * 4),
        ("diff", C.c_int32), ("lambda_", C.c_float),
        ("dtype", C.c_int32),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64),
        ("attended_dump", C.c_void_p),
        ("bias_dtype", C.c_int32 * 2),
        ("lse", C.c_void_p),
        ("dropout_threshold", C.c_uint32), ("dropout_seed", C.c_uint32 * 2),
        ("flags", C.c_uint32),
        ("score_fn", C.c_int32), ("score_fn_params", C.c_float * 4),
    ]


class FlAttnBwdParams(C.Structure):
    """Mirror of `fl_attn_bwd_params` (include/flashlight_amd.h)."""

    _fields_ = [
        ("fwd", FlAttnParams),
        ("dout", C.c_void_p), ("dout_strides", C.c_int64 * 4),
        ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
        ("dq_strides", C.c_int64 * 4), ("dk_strides", C.c_int64 * 4), ("dv_strides", C.c_int64 * 4),
        ("delta", C.c_void_p),
        ("dscores", C.c_void_p),
        ("reserved", C.c_int32 * 6),
    ]


class FlIpaPackParams(C.Structure):
    """Mirror of `fl_ipa_pack_params` (include/flashlight_amd.h)."""

    _fields_ = [
        ("q_scalar", C.c_void_p), ("k_scalar", C.c_void_p), ("v_scalar", C.c_void_p),
        ("q_points", C.c_void_p), ("k_points", C.c_void_p), ("v_points", C.c_void_p),
        ("q_cat", C.c_void_p), ("k_cat", C.c_void_p), ("v_cat", C.c_void_p),
        ("key_term", C.c_void_p),
        ("rows", C.c_int64),
        ("c_qk", C.c_int32), ("c_v", C.c_int32), ("n_qk_coords", C.c_int32), ("n_v_coords", C.c_int32),
        ("dqk", C.c_int32), ("dv", C.c_int32),
        ("q_scale", C.c_float), ("point_weight", C.c_float),
    ]


class FlashlightError(RuntimeError):
    """fl_attn_fwd / fl_attn_validate returned non-zero; `.code` holds the return value."""

    def __init__(self, code: int, message: str):
        super().__init__(f"flashlight_amd error {code}: {message}")
        self.code = code


_lib: Optional[C.CDLL] = None
_MAX_DV_DIFF = 128  # widest value slab of a differential-attention kernel instance


def load_library(path: os.PathLike | str | None = None) -> C.CDLL:
    """Loads the in-tree shared library once (or the library at `path`, which then serves every later call).  Raises if
    it has not been built (no silent fallback)."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = Path(path) if path else LIB_PATH
    if not p.exists():
        raise FileNotFoundError(
            f"{p} is missing: build it with `python -m flashlight_amd.build` (needs hipcc); "
            "flashlight_amd has no non-HIP execution path")
    lib = C.CDLL(str(p))
    lib.fl_version.restype = C.c_int
    lib.fl_last_error.restype = C.c_char_p
    lib.fl_params_sizeof.restype = C.c_uint64
    lib.fl_workspace_bytes.restype = C.c_uint64
    lib.fl_workspace_bytes.argtypes = [C.POINTER(FlAttnParams)]
    lib.fl_bwd_workspace_bytes.restype = C.c_uint64
    lib.fl_bwd_workspace_bytes.argtypes = [C.POINTER(FlAttnParams)]
    lib.fl_attn_validate.restype = C.c_int
    lib.fl_attn_validate.argtypes = [C.POINTER(FlAttnParams)]
    lib.fl_attn_plan.restype = C.c_int
    lib.fl_attn_plan.argtypes = [C.POINTER(FlAttnParams), C.POINTER(C.c_int64)]
    lib.fl_attn_fwd.restype = C.c_int
    lib.fl_attn_fwd.argtypes = [C.POINTER(FlAttnParams), C.c_void_p]
    lib.fl_static_scratch_bytes.restype = C.c_uint64
    lib.fl_bwd_params_sizeof.restype = C.c_uint64
    lib.fl_attn_bwd_validate.restype = C.c_int
    lib.fl_attn_bwd_validate.argtypes = [C.POINTER(FlAttnBwdParams)]
    lib.fl_attn_bwd.restype = C.c_int
    lib.fl_attn_bwd.argtypes = [C.POINTER(FlAttnBwdParams), C.c_void_p]
    lib.fl_attn_bwd_static.restype = C.c_int
    lib.fl_attn_bwd_static.argtypes = [C.POINTER(FlAttnBwdParams), C.c_void_p]
    lib.fl_attn_merge_chunks.restype = C.c_int
    lib.fl_attn_merge_chunks.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int64, C.c_int32,
                                         C.c_int32, C.c_void_p]
    lib.fl_ipa_pack.restype = C.c_int
    lib.fl_ipa_pack.argtypes = [C.POINTER(FlIpaPackParams), C.c_void_p]
    if lib.fl_version() != ABI_VERSION:
        raise RuntimeError(f"{p}: ABI version {lib.fl_version()} != expected {ABI_VERSION}")
    if lib.fl_params_sizeof() != C.sizeof(FlAttnParams):
        raise RuntimeError(f"{p}: fl_attn_params is {lib.fl_params_sizeof()} bytes, binding expects {C.sizeof(FlAttnParams)}")
    if lib.fl_bwd_params_sizeof() != C.sizeof(FlAttnBwdParams):
        raise RuntimeError(f"{p}: fl_attn_bwd_params is {lib.fl_bwd_params_sizeof()} bytes, binding expects "
                           f"{C.sizeof(FlAttnBwdParams)}")
    _lib = lib
    return lib


def last_error() -> str:
    return load_library().fl_last_error().decode()


def _check(rc: int) -> None:
    if rc != 0:
        raise FlashlightError(rc, last_error())


def _strides4(t: torch.Tensor) -> Sequence[int]:
    return t.stride()


_HALF_TYPES = {torch.bfloat16: FL_BF16, torch.float16: FL_F16}


def _require_gpu_half(name: str, t: torch.Tensor, like: Optional[torch.Tensor] = None) -> None:
    """`t` must be a bf16 or fp16 GPU tensor (of `like`'s element type when that is given)."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise NotImplementedError(
            f"{name} is on {t.device}: flashlight_amd only runs its HIP kernels on a GPU tensor (no CPU path)")
    if t.dtype not in _HALF_TYPES:
        raise NotImplementedError(f"{name} has dtype {t.dtype}: the HIP kernels take bfloat16 or float16")
    if like is not None and t.dtype != like.dtype:
        raise NotImplementedError(f"{name} has dtype {t.dtype} but the query has {like.dtype}: mixed element types")


def _require_gpu_bf16(name: str, t: torch.Tensor) -> None:
    _require_gpu_half(name, t)
    if t.dtype != torch.bfloat16:
        raise NotImplementedError(f"{name} has dtype {t.dtype}: this entry point takes bfloat16")


def _dim_contiguous(t: torch.Tensor) -> torch.Tensor:
    """The kernels address [batch, head, seq, dim] through strides but need dim contiguous and 16-byte rows."""
    if t.is_contiguous():  # (copying would change nothing; decided first because it is the common case)
        return t
    if t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:-1]) or t.data_ptr() % 16:
        return t.contiguous()
    return t


def _launch_on(device: torch.device, entry, params) -> None:
    """Calls `entry(&params, stream)` with `device` current and torch's current stream of that device."""
    index = device.index
    if index is None or index == torch.cuda.current_device():
        # (the raw-stream getter skips the Stream object; it is what torch's own generated code calls)
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        stream = raw(torch.cuda.current_device()) if raw is not None else torch.cuda.current_stream().cuda_stream
        _check(entry(C.byref(params), C.c_void_p(stream)))
        return
    with torch.cuda.device(device):
        _check(entry(C.byref(params), C.c_void_p(torch.cuda.current_stream().cuda_stream)))


def dropout_threshold(p: float) -> int:
    """16-bit threshold of dropout rate p (0 = off): the kernels drop a weight when its 16 hash bits are below it, so
    the rate in effect is threshold / 65536."""
    if not 0.0 <= p < 1.0:
        raise ValueError(f"dropout_p must be in [0, 1), got {p}")
    return min(int(round(p * 65536.0)), 65535)


class DocWorkspace:
    """Scratch of document-mask forward calls, kept across calls.  The first call made with a handle allocates the
    buffer and runs the pre-pass that lists, from the ids, the key tiles every query tile visits; later calls with the
    same handle, the same ids tensor (same memory, not modified in place since) and the same shapes and options skip the
    pre-pass (FL_FLAG_DOC_PREPARED).  Anything else refills the handle.  The handle keeps the ids tensor alive.  The
    calls must be ordered on the device like any producer and consumer of one buffer (same stream, or events)."""

    def __init__(self):
        self.buffer = None
        self.key = None
        self.ids = None


FLAG_DOC_PREPARED = 1
SCORE_NONE, SCORE_SIGMOID, SCORE_CLAMP, SCORE_POLY = 0, 1, 2, 3  # fl_attn_params.score_fn


def _fill_params(lib, q, k, v, out, Hq, Hkv, scale, mask_kind, window, prefix, doc_ids, alibi_heads, softcap, biases,
                 gate, diff, lambda_full, attended_dump, dropout_p=0.0, dropout_seed=0, alloc_workspace=True,
                 doc_workspace=None):
    """Fills an `fl_attn_params` for validated 4-D tensors; returns it with the tensors that must outlive the launch."""
    B, _, Lq, Dqk = q.shape
    Lk, Dv = k.shape[2], v.shape[3]
    p = FlAttnParams()
    p.q, p.k, p.v, p.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    p.q_strides[:] = _strides4(q)
    p.k_strides[:] = _strides4(k)
    p.v_strides[:] = _strides4(v)
    p.o_strides[:] = _strides4(out)
    p.B, p.Hq, p.Hkv, p.Lq, p.Lk, p.Dqk, p.Dv = B, Hq, Hkv, Lq, Lk, Dqk, Dv
    p.scale = float(1.0 / math.sqrt(Dqk) if scale is None else scale)
    p.mask_kind, p.window, p.prefix = int(mask_kind), int(window), int(prefix)
    p.dropout_threshold = dropout_threshold(float(dropout_p))
    p.dropout_seed[0], p.dropout_seed[1] = int(dropout_seed) & 0xFFFFFFFF, (int(dropout_seed) >> 32) & 0xFFFFFFFF
    keep = [q, k, v, out]
    if doc_ids is not None:
        if doc_ids.dim() != 2 or doc_ids.shape[1] != Lk or doc_ids.shape[0] not in (1, B):
            raise ValueError(f"document ids must be [B, L] = [{B}, {Lk}], got {tuple(doc_ids.shape)}")
        d = doc_ids.to(device=q.device, dtype=torch.int64)
        if d.stride(1) != 1:
            d = d.contiguous()
        p.doc_ids = d.data_ptr()
        p.doc_stride = int(d.stride(0)) if d.shape[0] == B and B > 1 else 0
        keep.append(d)
    p.alibi_heads = int(alibi_heads)
    p.softcap = float(softcap)
    if len(biases) > 2:
        raise ValueError("at most two additive biases are supported")
    for i, (b, div) in enumerate(biases):
        if b.dtype == torch.float32 and b.is_cuda:
            p.bias_dtype[i] = FL_F32
        else:
            _require_gpu_half(f"bias[{i}]", b, q)
            p.bias_dtype[i] = _HALF_TYPES[q.dtype]
        if b.dim() != 4:
            raise ValueError(f"bias[{i}] must be 4-D, got {tuple(b.shape)}")
        want = (B // div, Hq, Lq, Lk)
        if B % div:
            raise ValueError(f"bias[{i}]: batch divisor {div} does not divide {B}")
        strides = []
        for ax, (n, w) in enumerate(zip(b.shape, want)):
            if n == w and n != 1:
                strides.append(int(b.stride(ax)))
            elif n == 1:
                strides.append(0)
            else:
                raise ValueError(f"bias[{i}] shape {tuple(b.shape)} does not broadcast to {want}")
        if strides[3] not in (0, 1):
            b = b.contiguous()
            strides = [int(s) if n != 1 else 0 for s, n in zip(b.stride(), b.shape)]
        p.bias[i] = b.data_ptr()
        p.bias_strides[i][:] = strides
        p.bias_batch_div[i] = int(div)
        keep.append(b)
    if gate is not None:
        _require_gpu_half("gate", gate, q)
        if tuple(gate.shape) != (B, Hq, Lq, Dv):
            raise ValueError(f"gate must have the output's shape {(B, Hq, Lq, Dv)}, got {tuple(gate.shape)}")
        if gate.stride(-1) != 1 or any(s % 4 for s in gate.stride()[:-1]) or gate.data_ptr() % 8:
            gate = gate.contiguous()
        p.gate = gate.data_ptr()
        p.gate_strides[:] = _strides4(gate)
        keep.append(gate)
    p.diff = 1 if diff else 0
    p.lambda_ = float(lambda_full)
    p.dtype = _HALF_TYPES[q.dtype]
    if attended_dump is not None:
        if attended_dump.dtype != torch.uint8 or tuple(attended_dump.shape) != (B, Hq, Lq, Lk) or \
                not attended_dump.is_contiguous() or attended_dump.device != q.device:
            raise ValueError("attended_dump must be a contiguous uint8 [B, Hq, Lq, Lk] tensor on the inputs' device")
        p.attended_dump = attended_dump.data_ptr()
    need = lib.fl_workspace_bytes(C.byref(p)) if alloc_workspace else 0
    if need:
        if doc_workspace is not None:
            d = keep[4]  # the ids as the kernel reads them
            key = (d.data_ptr(), d._version, tuple(d.shape), tuple(d.stride()), B, Hq, Hkv, Lk, Dqk, Dv, q.dtype, int(mask_kind),
                   p.alibi_heads > 0, p.softcap > 0.0, len(biases), gate is not None, bool(diff), attended_dump is not None,
                   int(need), str(q.device))
            if doc_workspace.key == key and doc_workspace.buffer is not None:
                p.flags |= FLAG_DOC_PREPARED
            else:
                doc_workspace.buffer = torch.empty(need, dtype=torch.uint8, device=q.device)
                doc_workspace.key, doc_workspace.ids = key, d
            ws = doc_workspace.buffer
        else:
            ws = torch.empty(need, dtype=torch.uint8, device=q.device)
        p.workspace, p.workspace_bytes = ws.data_ptr(), need
        keep.append(ws)
    return p, keep


def attn_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    *,
    scale: Optional[float] = None,
    mask_kind: int = MASK_NONE,
    window: int = 0,
    prefix: int = 0,
    doc_ids: Optional[torch.Tensor] = None,
    alibi_heads: int = 0,
    softcap: float = 0.0,
    biases: Sequence[tuple[torch.Tensor, int]] = (),
    gate: Optional[torch.Tensor] = None,
    diff: bool = False,
    lambda_full: float = 0.0,
    out: Optional[torch.Tensor] = None,
    attended_dump: Optional[torch.Tensor] = None,
    validate_only: bool = False,
    lse: Optional[torch.Tensor] = None,
    dropout_p: float = 0.0,
    dropout_seed: int = 0,
    doc_workspace: Optional[DocWorkspace] = None,
    score_fn: Optional[tuple] = None,
) -> torch.Tensor:
    """Fused attention forward on 4-D views: q [B, Hq(x2 if diff), Lq, Dqk], k [B, Hkv(x2), Lk, Dqk], v [B, Hkv, Lk, Dv].

    `biases` holds up to two (tensor, batch_div) pairs; each tensor is 4-D, bf16 or fp32, broadcastable to
    [B/batch_div, Hq, Lq, Lk] (size-1 axes broadcast).  q, k, v (and gate, 16-bit biases) are all bf16 or all fp16.  Returns `out` [B, Hq, Lq, Dv]
    in that type, written on the current stream.
    `lse` (float32 [B, Hq, Lq]) receives the row statistics that `attn_bwd` needs.
    `dropout_p` > 0 drops softmax weights (torch.nn.functional.dropout semantics) by a hash of (`dropout_seed`, batch,
    head, query, key); positional masks and GQA only.
    `doc_workspace` (document masks): a `DocWorkspace` handle that keeps the pre-pass's result across calls.
    `score_fn` = (kind, (p0, p1, p2, p3)): a function of the scaled score z from the compiled-in set, in the soft-cap's
    place: SCORE_SIGMOID p2 * sigmoid(p0 z + p1) + p3, SCORE_CLAMP min(max(p0 z + p1, p2), p3), SCORE_POLY
    p0 + p1 z + p2 z^2 + p3 z^3.  Forward only; positional masks and bias operands.
    """
    lib = load_library()
    for name, t in (("query", q), ("key", k), ("value", v)):
        _require_gpu_half(name, t, q if isinstance(q, torch.Tensor) and q.dtype in _HALF_TYPES else None)
        if t.dim() != 4:
            raise ValueError(f"{name} must be 4-D [batch, heads, seq, dim], got shape {tuple(t.shape)}")
    q, k, v = _dim_contiguous(q), _dim_contiguous(k), _dim_contiguous(v)
    B, Hq_all, Lq, Dqk = q.shape
    Bk, Hk_all, Lk, Dk = k.shape
    Bv, Hv, Lv, Dv = v.shape
    if not (B == Bk == Bv) or Dqk != Dk or Lk != Lv:
        raise ValueError(f"inconsistent shapes: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    if diff:
        if Hq_all % 2 or Hk_all % 2:
            raise ValueError("differential attention needs an even number of query and key heads")
        Hq, Hkv = Hq_all // 2, Hk_all // 2
    else:
        Hq, Hkv = Hq_all, Hk_all
    if Hv != Hkv:
        raise ValueError(f"value has {Hv} heads, expected {Hkv}")
    if out is None:
        out = torch.empty((B, Hq, Lq, Dv), dtype=q.dtype, device=q.device)
    elif tuple(out.shape) != (B, Hq, Lq, Dv) or out.dtype != q.dtype or out.device != q.device:
        raise ValueError("out has the wrong shape, dtype or device")
    if Dv > _MAX_DV_DIFF and Dv % _MAX_DV_DIFF == 0 and attended_dump is None and (diff or Dqk >= 128):
        # Value columns are independent of one another, so wide values go in slabs of _MAX_DV_DIFF columns, one launch
        # each, through strided views of v and out: a differential launch keeps two sets of output accumulators (the
        # reference's benchmark shape: q, k [B, 16, S, 128], v [B, 8, S, 256], diff_attn.py:33-38), and at head dim 256
        # the query fragments leave room for 128 output columns per launch.
        if diff and (lse is not None or dropout_p > 0.0):
            # what the single launch refuses for differential attention is refused here too, instead of dropped
            raise NotImplementedError("differential attention produces no lse and takes no dropout")
        for c in range(0, Dv, _MAX_DV_DIFF):
            attn_fwd(q, k, v[..., c:c + _MAX_DV_DIFF], scale=scale, mask_kind=mask_kind, window=window, prefix=prefix,
                     doc_ids=doc_ids, alibi_heads=alibi_heads, softcap=softcap, biases=biases,
                     gate=None if gate is None else gate[..., c:c + _MAX_DV_DIFF], diff=diff, lambda_full=lambda_full,
                     out=out[..., c:c + _MAX_DV_DIFF], validate_only=validate_only,
                     lse=lse if c == 0 else None,  # the row statistics depend on q and k only
                     dropout_p=dropout_p, dropout_seed=dropout_seed,  # so do the dropout decisions
                     doc_workspace=doc_workspace,  # (and the key-tile lists: the slabs share one instance)
                     score_fn=score_fn)
        return out

    p, keep = _fill_params(lib, q, k, v, out, Hq, Hkv, scale, mask_kind, window, prefix, doc_ids, alibi_heads, softcap,
                           biases, gate, diff, lambda_full, attended_dump, dropout_p, dropout_seed,
                           doc_workspace=doc_workspace)
    if score_fn is not None:
        kind, consts = score_fn
        if len(consts) != 4:
            raise ValueError("score_fn takes four constants")
        p.score_fn = int(kind)
        p.score_fn_params[:] = [float(c) for c in consts]
    if lse is not None:
        if lse.dtype != torch.float32 or tuple(lse.shape) != (B, Hq, Lq) or not lse.is_contiguous() or lse.device != q.device:
            raise ValueError("lse must be a contiguous float32 [B, Hq, Lq] tensor on the inputs' device")
        p.lse = lse.data_ptr()
    if validate_only:
        _check(lib.fl_attn_validate(C.byref(p)))
        return out
    _launch_on(q.device, lib.fl_attn_fwd, p)
    # tensors in `keep` were last used on the current stream; the caching allocator orders their reuse after it
    del keep
    return out


def attn_bwd(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor, lse: torch.Tensor, dout: torch.Tensor,
             *, scale: Optional[float] = None, mask_kind: int = MASK_NONE, window: int = 0, prefix: int = 0,
             doc_ids: Optional[torch.Tensor] = None, alibi_heads: int = 0, softcap: float = 0.0,
             validate_only: bool = False, dropout_p: float = 0.0, dropout_seed: int = 0, static_scratch: bool = False,
             grads: Optional[Sequence[torch.Tensor]] = None, biases: Sequence[tuple[torch.Tensor, int]] = (),
             dscores: Optional[torch.Tensor] = None):
    """Gradients (dq, dk, dv) of `attn_fwd` called with the same arguments (dropout rate and seed included); `out` and `lse` are what that call
    returned and filled, `dout` [B, Hq, Lq, Dv] the gradient of its result.  Three launches on the current stream.
    `grads` = (dq, dk, dv) receives the results when given.  `static_scratch` goes through `fl_attn_bwd_static`: nothing
    is allocated here beyond the results, the library's own static device array serves as scratch (calls that may
    overlap on one GPU must not both use it).
    `biases` are the forward's bias operands; `dscores`, a zero-filled contiguous float32 [B, Hq, Lq, Lk] tensor, then
    receives the gradient with respect to the scores, from which the caller sums the gradient of each operand over the
    axes it broadcasts over (not under a soft-cap)."""
    lib = load_library()
    for name, t in (("query", q), ("key", k), ("value", v), ("out", out), ("dout", dout)):
        _require_gpu_half(name, t, q if isinstance(q, torch.Tensor) and q.dtype in _HALF_TYPES else None)
        if t.dim() != 4:
            raise ValueError(f"{name} must be 4-D [batch, heads, seq, dim], got shape {tuple(t.shape)}")
    q, k, v, out, dout = (_dim_contiguous(t) for t in (q, k, v, out, dout))
    B, Hq, Lq, Dqk = q.shape
    Hkv, Lk, Dv = k.shape[1], k.shape[2], v.shape[3]
    if tuple(out.shape) != (B, Hq, Lq, Dv) or tuple(dout.shape) != (B, Hq, Lq, Dv):
        raise ValueError("out and dout must be [B, Hq, Lq, Dv]")
    if lse.dtype != torch.float32 or tuple(lse.shape) != (B, Hq, Lq) or not lse.is_contiguous() or lse.device != q.device:
        raise ValueError("lse must be the contiguous float32 [B, Hq, Lq] tensor the forward filled")
    fwd, keep = _fill_params(lib, q, k, v, out, Hq, Hkv, scale, mask_kind, window, prefix, doc_ids, alibi_heads, softcap,
                             biases, None, False, 0.0, None, dropout_p, dropout_seed,
                             alloc_workspace=validate_only or not static_scratch)
    fwd.lse = lse.data_ptr()
    if dscores is not None:
        if dscores.dtype != torch.float32 or tuple(dscores.shape) != (B, Hq, Lq, Lk) or not dscores.is_contiguous() or \
                dscores.device != q.device:
            raise ValueError("dscores must be a contiguous float32 [B, Hq, Lq, Lk] tensor on the inputs' device")
    if grads is not None:
        dq, dk, dv = grads
        for g, like in ((dq, q), (dk, k), (dv, v)):
            if tuple(g.shape) != tuple(like.shape) or g.dtype != like.dtype or g.device != like.device or g.stride(-1) != 1:
                raise ValueError("grads must match q, k, v in shape, dtype and device")
    else:
        dq, dk, dv = torch.empty_like(q, memory_format=torch.contiguous_format), \
            torch.empty_like(k, memory_format=torch.contiguous_format), torch.empty_like(v, memory_format=torch.contiguous_format)
    use_static = static_scratch and not validate_only
    delta = None if use_static else torch.empty((B, Hq, Lq), dtype=torch.float32, device=q.device)
    b = FlAttnBwdParams()
    b.fwd = fwd
    b.dout, b.dq, b.dk, b.dv = dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    b.delta = None if delta is None else delta.data_ptr()
    b.dscores = None if dscores is None else dscores.data_ptr()
    b.dout_strides[:] = _strides4(dout)
    b.dq_strides[:] = _strides4(dq)
    b.dk_strides[:] = _strides4(dk)
    b.dv_strides[:] = _strides4(dv)
    if validate_only:
        _check(lib.fl_attn_bwd_validate(C.byref(b)))
        return dq, dk, dv
    _launch_on(q.device, lib.fl_attn_bwd_static if use_static else lib.fl_attn_bwd, b)
    del keep, delta
    return dq, dk, dv


def ipa_pack(q_scalar, k_scalar, v_scalar, q_points, k_points, v_points, dqk: int, dv: int, q_scale: float,
             point_weight: float):
    """[rows, *] bf16 tensors -> (q_cat [rows, dqk], k_cat [rows, dqk], v_cat [rows, dv], key_term [rows] fp32), one
    launch on the current stream (see `fl_ipa_pack` in include/flashlight_amd.h)."""
    lib = load_library()
    ts = [q_scalar, k_scalar, v_scalar, q_points, k_points, v_points]
    for i, t in enumerate(ts):
        _require_gpu_bf16("invariant point attention operand", t)
        if t.dim() != 2 or t.size(0) != q_scalar.size(0):
            raise ValueError("operands must be 2-D with one row per (batch, head, residue)")
        ts[i] = t.contiguous()
    rows, dev = q_scalar.size(0), q_scalar.device
    if k_scalar.size(1) != q_scalar.size(1) or k_points.size(1) != q_points.size(1):
        raise ValueError("query and key operands differ in width")
    q_cat = torch.empty((rows, dqk), dtype=torch.bfloat16, device=dev)
    k_cat = torch.empty((rows, dqk), dtype=torch.bfloat16, device=dev)
    v_cat = torch.empty((rows, dv), dtype=torch.bfloat16, device=dev)
    key_term = torch.empty((rows,), dtype=torch.float32, device=dev)
    p = FlIpaPackParams()
    (p.q_scalar, p.k_scalar, p.v_scalar, p.q_points, p.k_points, p.v_points) = (t.data_ptr() for t in ts)
    p.q_cat, p.k_cat, p.v_cat, p.key_term = q_cat.data_ptr(), k_cat.data_ptr(), v_cat.data_ptr(), key_term.data_ptr()
    p.rows = rows
    p.c_qk, p.c_v, p.n_qk_coords, p.n_v_coords = ts[0].size(1), ts[2].size(1), ts[3].size(1), ts[5].size(1)
    p.dqk, p.dv, p.q_scale, p.point_weight = int(dqk), int(dv), float(q_scale), float(point_weight)
    with torch.cuda.device(dev):
        rc = lib.fl_ipa_pack(C.byref(p), C.c_void_p(torch.cuda.current_stream().cuda_stream))
    if rc != 0:
        raise FlashlightError(rc, "fl_ipa_pack rejected its arguments or could not launch")
    del ts
    return q_cat, k_cat, v_cat, key_term


def plan(p: FlAttnParams) -> dict:
    """Tile shape / launch shape the library would use for `p` (host only)."""
    lib = load_library()
    out = (C.c_int64 * 8)()
    _check(lib.fl_attn_plan(C.byref(p), out))
    return {"rows_per_workgroup": out[0], "keys_per_tile": out[1], "threads": out[2], "workgroups": out[3],
            "lds_bytes": out[4], "features": out[5], "streaming": out[6]}


_probe_lib = None


def load_probe_library() -> C.CDLL:
    """Loads the bench-only library of measurement probes (include/flashlight_amd_probe.h), built next to the product
    library; the product library exports none of them."""
    global _probe_lib
    if _probe_lib is None:
        p = LIB_PATH.with_name("libflashlight_amd_probe.so")
        if not p.exists():
            raise FileNotFoundError(f"{p} is missing: build it with `python -m flashlight_amd.build` (needs hipcc)")
        lib = C.CDLL(str(p))
        lib.fl_probe_mfma_rate.restype = C.c_int
        lib.fl_probe_mfma_rate.argtypes = [C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        lib.fl_probe_step.restype = C.c_int
        lib.fl_probe_step.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        lib.fl_probe_coissue.restype = C.c_int
        lib.fl_probe_coissue.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        _probe_lib = lib
    return _probe_lib


def probe_mfma_rate(operands: torch.Tensor, iters: int, n_workgroups: int, sink: torch.Tensor) -> float:
    """Launches the MFMA-only rate probe on the current stream (measurement aid, include/flashlight_amd_probe.h) and returns
    the FLOPs of the launch.  `operands`: bf16 device tensor (multiple of 8 elements, 16-byte aligned) the per-lane
    fragments are read from; `sink`: float32 device tensor of n_workgroups * 512 elements."""
    if operands.dtype != torch.bfloat16 or not operands.is_cuda or not operands.is_contiguous() or operands.numel() % 8:
        raise ValueError("operands must be a contiguous bf16 device tensor with a multiple of 8 elements")
    if sink.dtype != torch.float32 or sink.numel() < n_workgroups * 512 or sink.device != operands.device:
        raise ValueError("sink must be a float32 tensor of n_workgroups * 512 elements on the operands' device")
    stream = torch.cuda.current_stream(operands.device).cuda_stream
    rc = load_probe_library().fl_probe_mfma_rate(operands.data_ptr(), operands.numel() // 8, int(iters), int(n_workgroups),
                                           sink.data_ptr(), C.c_void_p(stream))
    if rc != 0:
        raise FlashlightError(rc, "fl_probe_mfma_rate rejected its arguments" if rc < 0 else "probe launch failed")
    return float(n_workgroups) * 8 * iters * 32 * 32768.0


def probe_step(head_dim: int, level: int, iters: int, n_workgroups: int, sink: torch.Tensor) -> int:
    """Launches the step-structure probe on the current stream (measurement aid, include/flashlight_amd_probe.h) and returns
    the number of 32 x 32 score blocks every wave works through; `sink`: float32 device tensor of n_workgroups * 256
    elements."""
    if sink.dtype != torch.float32 or not sink.is_cuda or sink.numel() < n_workgroups * 256:
        raise ValueError("sink must be a float32 device tensor of n_workgroups * 256 elements")
    stream = torch.cuda.current_stream(sink.device).cuda_stream
    rc = load_probe_library().fl_probe_step(int(head_dim), int(level), int(iters), int(n_workgroups), sink.data_ptr(),
                                      C.c_void_p(stream))
    if rc != 0:
        raise FlashlightError(rc, "fl_probe_step rejected its arguments" if rc < 0 else "probe launch failed")
    return 2 * int(iters)


COISSUE_KINDS = {"fma": 0, "exp": 1, "cvt_pk_bf16": 2, "dot2c": 3, "add": 4}


def probe_coissue(mfma_rows: int, valu_kind: str, valu_per_mfma: int, waves_per_simd: int, iters: int = 2000,
                  device="cuda") -> dict:
    """Runs the co-issue probe (include/flashlight_amd_probe.h) on every compute unit and returns shader cycles per unit
    of matrix work (one 32x32x16 MFMA, or two 16x16x32) per SIMD: from the slowest wave and from the mean wave."""
    n_cu = torch.cuda.get_device_properties(device).multi_processor_count
    n_waves = n_cu * 4 * waves_per_simd
    sink = torch.empty(n_cu * 256 * waves_per_simd, dtype=torch.float32, device=device)
    cyc = torch.zeros(n_waves, dtype=torch.int64, device=device)
    stream = torch.cuda.current_stream(sink.device).cuda_stream
    rc = load_probe_library().fl_probe_coissue(int(mfma_rows), COISSUE_KINDS[valu_kind], int(valu_per_mfma), int(waves_per_simd),
                                               int(iters), n_cu, sink.data_ptr(), cyc.data_ptr(), C.c_void_p(stream))
    if rc != 0:
        raise FlashlightError(rc, "fl_probe_coissue rejected its arguments" if rc < 0 else "probe launch failed")
    torch.cuda.synchronize(sink.device)
    c = cyc.double()
    per = 8.0 * iters * waves_per_simd
    return {"slowest_wave": float(c.max()) / per, "mean_wave": float(c.mean()) / per}


def merge_chunks(part: torch.Tensor, lse: torch.Tensor) -> torch.Tensor:
    """`fl_attn_merge_chunks`: part [outer, chunks, inner, dv] (bf16 / fp16) and lse [outer, chunks, inner] (fp32) of one
    launch over key chunks -> [outer, inner, dv], the attention over all the keys.  One launch on the current stream."""
    _require_gpu_half("part", part, None)
    outer, chunks, inner, dv = part.shape
    if lse.dtype != torch.float32 or tuple(lse.shape) != (outer, chunks, inner) or not (part.is_contiguous() and lse.is_contiguous()):
        raise ValueError("merge_chunks: lse must be float32 [outer, chunks, inner], both operands contiguous")
    out = torch.empty((outer, inner, dv), dtype=part.dtype, device=part.device)
    rc = load_library().fl_attn_merge_chunks(C.c_void_p(part.data_ptr()), C.c_void_p(lse.data_ptr()), C.c_void_p(out.data_ptr()),
                                             outer, chunks, inner, dv, _HALF_TYPES[part.dtype],
                                             C.c_void_p(torch.cuda.current_stream().cuda_stream))
    if rc != 0:
        raise FlashlightError(rc, "fl_attn_merge_chunks rejected its arguments or could not launch")
    return out
