"""The C-ABI library: loads without a GPU, exports what include/flashlight_amd.h declares, and validates arguments
on the host (no launch).  Device pointers are faked with aligned integers; nothing here dereferences them."""
import ctypes as C
import re
from pathlib import Path

import pytest

from flashlight_amd import _ffi

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "flashlight_amd.h"


@pytest.fixture(scope="module")
def lib():
    if not _ffi.LIB_PATH.exists():
        from flashlight_amd import build
        build.build(force=False)
    return _ffi.load_library()


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return re.findall(r"^\s*(?:const\s+)?[\w\s\*]+?\b(fl_\w+)\s*\(", text, flags=re.M)


def test_exports_every_declared_symbol(lib):
    names = declared_functions()
    assert {"fl_version", "fl_last_error", "fl_attn_validate", "fl_workspace_bytes", "fl_attn_fwd", "fl_attn_plan",
            "fl_params_sizeof"} <= set(names)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"


def test_version_and_struct_size(lib):
    assert lib.fl_version() == _ffi.ABI_VERSION
    assert lib.fl_params_sizeof() == C.sizeof(_ffi.FlAttnParams)


def good_params(B=2, Hq=4, Hkv=2, L=300, D=64, Dv=None):
    Dv = Dv or D
    p = _ffi.FlAttnParams()
    p.q, p.k, p.v, p.o = 0x10000, 0x20000, 0x30000, 0x40000
    p.q_strides[:] = (Hq * L * D, L * D, D, 1)
    p.k_strides[:] = (Hkv * L * D, L * D, D, 1)
    p.v_strides[:] = (Hkv * L * Dv, L * Dv, Dv, 1)
    p.o_strides[:] = (Hq * L * Dv, L * Dv, Dv, 1)
    p.B, p.Hq, p.Hkv, p.Lq, p.Lk, p.Dqk, p.Dv = B, Hq, Hkv, L, L, D, Dv
    p.scale = 0.125
    return p


def rc(lib, p):
    return lib.fl_attn_validate(C.byref(p))


def test_every_combination_of_score_modifications_has_a_kernel(lib):
    """Mask kind x ALiBi x soft-cap x bias operands x gate (x dropout at head dims 64 and 128), at every compiled head
    dim and in both element types: the
    reference's functions compose these freely (attention_variants/*.py are plain PyTorch), so no combination of them
    may end in "no kernel instance"."""
    import itertools
    for (D, Dv), dtype in itertools.product(((32, 32), (64, 64), (128, 128), (256, 128), (512, 128)), (_ffi.FL_BF16, _ffi.FL_F16)):
        for kind, alibi, cap, bias, gate, drop in itertools.product(
                (_ffi.MASK_NONE, _ffi.MASK_CAUSAL, _ffi.MASK_SLIDING, _ffi.MASK_PREFIX_LM, _ffi.MASK_DOCUMENT,
                 _ffi.MASK_DOCUMENT_CAUSAL), (0, 4), (0.0, 30.0), (0, 1, 2), (False, True), (0, 6554) if D in (64, 128) else (0,)):
            p = good_params(D=D, Dv=Dv)
            p.dtype = dtype
            p.dropout_threshold = drop  # (dropout kernels exist at head dims 64 and 128)
            p.mask_kind, p.window, p.prefix = kind, 17, 40
            p.alibi_heads, p.softcap = alibi, cap
            for i in range(bias):
                p.bias[i], p.bias_batch_div[i], p.bias_dtype[i] = 0x60000 + 0x100000 * i, 1, dtype
                p.bias_strides[i][:] = (0, 0, 304, 1) if i == 0 else (0, 0, 0, 1)
            if gate:
                p.gate = 0x70000
                p.gate_strides[:] = list(p.o_strides)
            if kind in (_ffi.MASK_DOCUMENT, _ffi.MASK_DOCUMENT_CAUSAL):
                p.doc_ids, p.doc_stride = 0x50000, 300
                p.workspace, p.workspace_bytes = 0x80000, lib.fl_workspace_bytes(C.byref(p))
            assert rc(lib, p) == 0, (D, Dv, dtype, kind, alibi, cap, bias, gate, drop, _ffi.last_error())


def test_valid_params_pass(lib):
    for D in (32, 64, 128):
        assert rc(lib, good_params(D=D)) == 0, _ffi.last_error()
        p = good_params(D=D)
        p.dtype = _ffi.FL_F16
        assert rc(lib, p) == 0, _ffi.last_error()
    p = good_params()  # a 16-bit bias must have the element type of q
    p.dtype = _ffi.FL_F16
    p.bias[0], p.bias_batch_div[0] = 0x60000, 1
    p.bias_strides[0][:] = (0, 0, 304, 1)
    assert rc(lib, p) == -4 and "bias_dtype" in _ffi.last_error()
    p.bias_dtype[0] = _ffi.FL_F16
    assert rc(lib, p) == 0, _ffi.last_error()
    p = good_params()
    p.mask_kind, p.window = _ffi.MASK_SLIDING, 17
    assert rc(lib, p) == 0
    assert _ffi.last_error() == ""


def test_plan_reports_launch_shape(lib):
    p = good_params(B=2, Hq=4, L=300, D=128)
    plan = _ffi.plan(p)
    assert plan["threads"] % 64 == 0 and plan["lds_bytes"] <= 160 * 1024
    bm = plan["rows_per_workgroup"]
    assert plan["workgroups"] == 2 * 4 * ((300 + bm - 1) // bm)


def test_score_function_arguments(lib):
    # fl_attn_params.score_fn: a function of the scaled score from the compiled-in set, in the soft-cap's place
    def with_fn(kind, consts, **kw):
        p = good_params(D=kw.pop("D", 64))
        p.score_fn = kind
        p.score_fn_params[:] = consts
        for name, value in kw.items():
            setattr(p, name, value)
        return p
    inf = float("inf")
    assert rc(lib, with_fn(_ffi.SCORE_SIGMOID, (0.5, -1.0, 3.0, 2.0))) == 0, _ffi.last_error()
    assert rc(lib, with_fn(_ffi.SCORE_CLAMP, (1.0, 0.0, 0.0, inf), D=128, mask_kind=_ffi.MASK_CAUSAL)) == 0, _ffi.last_error()
    assert rc(lib, with_fn(_ffi.SCORE_POLY, (0.0, -1.0, 0.1, 0.01))) == 0, _ffi.last_error()
    assert _ffi.plan(with_fn(_ffi.SCORE_POLY, (0.0, 1.0, 0.0, 0.0)))["features"] & 256
    assert rc(lib, with_fn(4, (0.0,) * 4)) == -5 and "score_fn" in _ffi.last_error()
    assert rc(lib, with_fn(_ffi.SCORE_CLAMP, (1.0, 0.0, 2.0, 1.0))) == -5 and "bound" in _ffi.last_error()
    assert rc(lib, with_fn(_ffi.SCORE_SIGMOID, (1.0, 0.0, inf, 0.0))) == -5 and "finite" in _ffi.last_error()
    assert rc(lib, with_fn(_ffi.SCORE_POLY, (float("nan"), 1.0, 0.0, 0.0))) == -5
    for bad in (dict(softcap=30.0), dict(alibi_heads=4), dict(dropout_threshold=1000), dict(diff=1)):
        assert rc(lib, with_fn(_ffi.SCORE_POLY, (0.0, 1.0, 0.1, 0.0), **bad)) == -4, bad
    assert rc(lib, with_fn(_ffi.SCORE_POLY, (0.0, 1.0, 0.1, 0.0), D=32)) == -4 and "no kernel instance" in _ffi.last_error()


def test_large_unmasked_calls_at_head_dim_128_take_256_row_workgroups(lib):
    # one 8-wave workgroup per compute unit brings each K/V tile in once for 256 query rows; chosen only without a mask
    # or score modification, at head dim 128, and when such workgroups still fill the part twice over
    big = good_params(B=4, Hq=16, Hkv=16, L=4096, D=128)
    assert _ffi.plan(big)["rows_per_workgroup"] == 256 and _ffi.plan(big)["threads"] == 512
    assert _ffi.plan(big)["workgroups"] == 4 * 16 * 16
    for change in (dict(L=1024), dict(D=64), dict(B=1, Hq=8, Hkv=8)):
        assert _ffi.plan(good_params(**{**dict(B=4, Hq=16, Hkv=16, L=4096, D=128), **change}))["rows_per_workgroup"] == 128
    masked = good_params(B=4, Hq=16, Hkv=16, L=4096, D=128)
    masked.mask_kind = _ffi.MASK_CAUSAL
    assert _ffi.plan(masked)["rows_per_workgroup"] == 128
    capped = good_params(B=4, Hq=16, Hkv=16, L=4096, D=128)
    capped.softcap = 30.0
    assert _ffi.plan(capped)["rows_per_workgroup"] == 128


@pytest.mark.parametrize("mutate, code, word", [
    (lambda p: setattr(p, "q", 0), -1, "q pointer is null"),
    (lambda p: setattr(p, "o", None), -1, "o pointer"),
    (lambda p: setattr(p, "k", 0x20008), -7, "16-byte"),
    (lambda p: setattr(p, "Lq", 0), -2, "positive"),
    (lambda p: setattr(p, "Hq", 3), -2, "multiple"),
    (lambda p: p.q_strides.__setitem__(3, 2), -3, "stride must be 1"),
    (lambda p: p.k_strides.__setitem__(2, 63), -7, "multiple of 8"),
    (lambda p: setattr(p, "scale", 0.0), -5, "scale"),
    (lambda p: setattr(p, "scale", float("nan")), -5, "scale"),
    (lambda p: setattr(p, "mask_kind", 9), -5, "mask_kind"),
    (lambda p: (setattr(p, "mask_kind", _ffi.MASK_SLIDING), setattr(p, "window", -1)), -5, "window"),
    (lambda p: (setattr(p, "mask_kind", _ffi.MASK_PREFIX_LM), setattr(p, "Lk", 299)), -2, "Lq == Lk"),
    (lambda p: setattr(p, "mask_kind", _ffi.MASK_DOCUMENT), -1, "doc_ids"),
    (lambda p: (setattr(p, "mask_kind", _ffi.MASK_DOCUMENT), setattr(p, "doc_ids", 0x50000)), -6, "workspace"),
    (lambda p: setattr(p, "softcap", -1.0), -5, "softcap"),
    (lambda p: setattr(p, "alibi_heads", -2), -5, "alibi"),
    (lambda p: setattr(p, "dtype", 3), -4, "dtype"),
    (lambda p: (setattr(p, "Dqk", 48), setattr(p, "Dv", 48)), -4, "no kernel instance"),
    (lambda p: (setattr(p, "diff", 1), setattr(p, "lambda_", float("inf"))), -5, "lambda"),
    (lambda p: setattr(p, "flags", 2), -5, "flags"),
    (lambda p: setattr(p, "flags", 1), -5, "FL_FLAG_DOC_PREPARED"),
    (lambda p: (p.bias.__setitem__(0, 0x60000), p.bias_batch_div.__setitem__(0, 0)), -5, "bias_batch_div"),
    (lambda p: (p.bias.__setitem__(0, 0x60000), p.bias_batch_div.__setitem__(0, 1),
                p.bias_strides[0].__setitem__(3, 2)), -3, "key stride"),
    (lambda p: (p.bias.__setitem__(1, 0x60000), p.bias_batch_div.__setitem__(1, 1),
                p.bias_dtype.__setitem__(1, 2)), -4, "bias_dtype"),
    (lambda p: (p.bias.__setitem__(0, 0x60002), p.bias_batch_div.__setitem__(0, 1),
                p.bias_dtype.__setitem__(0, _ffi.FL_F32)), -7, "4-byte aligned"),
    (lambda p: setattr(p, "gate", 0x70004), -7, "gate"),
])
def test_invalid_arguments_are_rejected_without_a_launch(lib, mutate, code, word):
    p = good_params()
    mutate(p)
    assert rc(lib, p) == code, _ffi.last_error()
    assert word in _ffi.last_error()
    # fl_attn_fwd runs the same check first and must not reach the GPU
    assert lib.fl_attn_fwd(C.byref(p), None) == code


def test_null_params(lib):
    assert lib.fl_attn_validate(None) == -1
    assert lib.fl_workspace_bytes(None) == 0


def test_backward_workspace_and_document_length_limit(lib):
    # the backward needs the table of id ranges only (16 bytes per 32 positions of every batch row), not the forward's lists
    p = good_params(B=3, L=1000)
    assert lib.fl_bwd_workspace_bytes(C.byref(p)) == 0 and lib.fl_bwd_workspace_bytes(None) == 0
    p.mask_kind = _ffi.MASK_DOCUMENT
    assert lib.fl_bwd_workspace_bytes(C.byref(p)) == 3 * ((1000 + 31) // 32) * 16
    assert lib.fl_bwd_workspace_bytes(C.byref(p)) < lib.fl_workspace_bytes(C.byref(p))
    # the forward's pre-pass keeps 20 bytes of LDS per key tile: beyond (160 KiB - 128) / 20 tiles a document-mask call
    # is refused by the host check, with the true maximum in the message, instead of failing at launch
    shape = _ffi.plan(good_params(B=1, L=1000))
    bn = shape["keys_per_tile"]
    max_tiles = (160 * 1024 - 128) // 20
    for L, ok in ((max_tiles * bn, True), ((max_tiles + 1) * bn, False)):
        q = good_params(B=1, Hq=1, Hkv=1, L=L)
        q.mask_kind, q.doc_ids = _ffi.MASK_DOCUMENT_CAUSAL, 0x50000
        q.workspace, q.workspace_bytes = 0x80000, lib.fl_workspace_bytes(C.byref(q))
        if ok:
            assert rc(lib, q) == 0, _ffi.last_error()
        else:
            assert rc(lib, q) == -2 and str(max_tiles * bn) in _ffi.last_error(), _ffi.last_error()


def test_workspace_size_for_document_masks(lib):
    p = good_params(B=3, L=1000)
    assert lib.fl_workspace_bytes(C.byref(p)) == 0
    p.mask_kind = _ffi.MASK_DOCUMENT_CAUSAL
    # the backward's (min, max) table per 32 positions, then per (batch, query tile) the forward's list of key tiles
    # (count + entries, rounded up to 4 words), for the tile shape the library reports for this call
    shape = _ffi.plan(good_params(B=3, L=1000))
    bm, bn = shape["rows_per_workgroup"], shape["keys_per_tile"]
    nq, nk = -(-1000 // bm), -(-1000 // bn)
    need = 3 * ((1000 + 31) // 32) * 16 + 3 * nq * ((nk + 1 + 3) // 4 * 4) * 4 + (3 * nq * 4 + 15) // 16 * 16
    assert lib.fl_workspace_bytes(C.byref(p)) == need
    p.doc_ids, p.workspace, p.workspace_bytes = 0x50000, 0x80000, need
    assert rc(lib, p) == 0, _ffi.last_error()
    p.workspace_bytes -= 1
    assert rc(lib, p) == -6
    p.workspace, p.workspace_bytes = 0x80008, need
    assert rc(lib, p) == -7  # 16-byte alignment


def test_too_many_keys_is_an_error_not_a_fault(lib):
    # key tiles are numbered in 16 bits
    p = good_params(B=1, Hq=1, Hkv=1, L=1 << 26, D=64)
    assert rc(lib, p) == -2 and "maximum" in _ffi.last_error()
    p = good_params(B=1, Hq=1, Hkv=1, L=1 << 20, D=64)
    assert rc(lib, p) == 0, _ffi.last_error()
    assert _ffi.plan(p)["lds_bytes"] <= 160 * 1024


def test_front_end_refuses_cpu_and_fp32_tensors(lib):
    import torch
    from flashlight_amd.attention_variants import attention_pytorch_causal, attention_pytorch_alibi
    q = torch.randn(1, 2, 16, 64)
    with pytest.raises(NotImplementedError, match="no CPU path"):
        attention_pytorch_causal(q.bfloat16(), q.bfloat16(), q.bfloat16())
    with pytest.raises(NotImplementedError, match="no CPU path"):
        attention_pytorch_alibi(q.bfloat16(), q.bfloat16(), q.bfloat16(), score_mod=lambda a, b: torch.zeros(a, b))
    with pytest.raises(TypeError, match="return a tensor"):
        attention_pytorch_alibi(q, q, q, score_mod=lambda a, b: None)
    with pytest.raises(TypeError):
        attention_pytorch_alibi(q, q, q)


def test_ipa_pack_rejects_bad_arguments_without_a_gpu(lib):
    assert "fl_ipa_pack" in declared_functions() and "fl_attn_bwd" in declared_functions()
    assert lib.fl_ipa_pack(None, None) == -1
    p = _ffi.FlIpaPackParams()
    assert lib.fl_ipa_pack(C.byref(p), None) == -1                       # null tensors
    for name in ("q_scalar", "k_scalar", "v_scalar", "q_points", "k_points", "v_points", "q_cat", "k_cat", "v_cat", "key_term"):
        setattr(p, name, 0x10000)
    p.rows, p.c_qk, p.c_v, p.n_qk_coords, p.n_v_coords, p.dqk, p.dv = 10, 16, 16, 12, 24, 24, 64
    assert lib.fl_ipa_pack(C.byref(p), None) == -2                       # 16 + 12 channels do not fit 24 columns
    p.dqk, p.rows = 32, 0
    assert lib.fl_ipa_pack(C.byref(p), None) == -2                       # no rows


def test_merge_chunks_rejects_bad_arguments_without_a_gpu(lib):
    assert "fl_attn_merge_chunks" in declared_functions()
    ptr = C.c_void_p(0x10000)
    merge = lambda part, lse, out, outer, chunks, inner, dv, dtype: lib.fl_attn_merge_chunks(part, lse, out, outer, chunks, inner, dv, dtype, None)
    assert merge(None, ptr, ptr, 1, 2, 3, 64, 0) == -1      # null operands
    assert merge(ptr, None, ptr, 1, 2, 3, 64, 0) == -1
    assert merge(ptr, ptr, None, 1, 2, 3, 64, 0) == -1
    assert merge(ptr, ptr, ptr, 0, 2, 3, 64, 0) == -2       # no rows
    assert merge(ptr, ptr, ptr, 1, 0, 3, 64, 0) == -2       # no chunks
    assert merge(ptr, ptr, ptr, 1, 2, 3, 63, 0) == -2       # odd value width
    assert merge(ptr, ptr, ptr, 1 << 20, 2, 1 << 20, 64, 0) == -2   # more rows than a launch has workgroups
    assert merge(ptr, ptr, ptr, 1, 2, 3, 64, 1) == -4       # fp32 partial results are not produced by any kernel here


def test_probe_library_is_separate_and_rejects_bad_arguments_without_a_gpu(lib):
    # the measurement aids live in a bench-only library: the product library exports none of them, the probe library
    # exports every function its header declares, and each checks its arguments on the host before launching anything
    assert not hasattr(lib, "fl_probe_mfma_rate") and not hasattr(lib, "fl_probe_step")
    lib = _ffi.load_probe_library()
    text = re.sub(r"/\*.*?\*/", "", (HEADER.parent / "flashlight_amd_probe.h").read_text(), flags=re.S)
    declared = re.findall(r"^\s*(?:const\s+)?[\w\s\*]+?\b(fl_\w+)\s*\(", text, flags=re.M)
    assert set(declared) == {"fl_probe_mfma_rate", "fl_probe_step", "fl_probe_coissue"}
    for n in declared:
        assert hasattr(lib, n), f"{n} is declared in flashlight_amd_probe.h but not exported"
    assert lib.fl_probe_mfma_rate(None, 1, 1, 1, None, None) == -5
    buf = (C.c_char * 64)()
    addr = C.addressof(buf)
    aligned = (addr + 15) // 16 * 16
    assert lib.fl_probe_mfma_rate(C.c_void_p(aligned), 0, 1, 1, C.c_void_p(aligned), None) == -5
    assert lib.fl_probe_mfma_rate(C.c_void_p(aligned + 2), 1, 1, 1, C.c_void_p(aligned), None) == -7
    assert lib.fl_probe_step(64, 2, 1, 1, None, None) == -5
    assert lib.fl_probe_step(64, 5, 1, 1, C.c_void_p(aligned), None) == -5
    assert lib.fl_probe_step(96, 2, 1, 1, C.c_void_p(aligned), None) == -4
    assert lib.fl_probe_coissue(32, 0, 2, 1, 1, 1, None, None, None) == -5
    assert lib.fl_probe_coissue(32, 0, 2, 3, 1, 1, C.c_void_p(aligned), C.c_void_p(aligned), None) == -5   # waves per SIMD
    assert lib.fl_probe_coissue(24, 0, 2, 1, 1, 1, C.c_void_p(aligned), C.c_void_p(aligned), None) == -4   # MFMA shape
    assert lib.fl_probe_coissue(32, 7, 2, 1, 1, 1, C.c_void_p(aligned), C.c_void_p(aligned), None) == -4   # vector kind
