"""Backward pass (dq, dk, dv).  The reference is forward-only, so there is nothing of its own to compare with: the
checker is autograd through the CPU oracle's eager functions, which `test_oracle_gradients_against_finite_differences`
pins against central differences in float64 (a wrong formula in the oracle, or in autograd's use of it, fails there).
GPU tests compare the HIP kernels' gradients, through the C ABI, with those."""
import ctypes as C
import math

import pytest
import torch

import flashlight_amd.attention_variants as A
import oracle as O
from flashlight_amd import _ffi
from tests.conftest import assert_parity
from tests.test_abi import good_params

DEV = "cuda"


# ---- the checker itself ----------------------------------------------------------------------------------------------------

def _tiny(dtype=torch.float64, N=1, Hq=2, Hkv=1, L=5, E=4, seed=0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g, dtype=dtype).requires_grad_(True)  # noqa: E731
    return mk(N, Hq, L, E), mk(N, Hkv, L, E), mk(N, Hkv, L, E)


@pytest.mark.parametrize("name,fn", [
    ("vanilla", lambda q, k, v: O.attention_vanilla(q, k, v, enable_gqa=True)),
    ("causal", lambda q, k, v: O.attention_causal(q, k, v, enable_gqa=True)),
    ("sliding", lambda q, k, v: O.attention_sliding_window(q, k, v, window_size=2, enable_gqa=True)),
    ("prefix", lambda q, k, v: O.attention_prefix_lm(q, k, v, prefix_lengths=3, enable_gqa=True)),
    ("document", lambda q, k, v: O.attention_document_mask(q, k, v, torch.tensor([[0, 0, 1, 1, 1]]), enable_gqa=True,
                                                           is_causal=True)),
    ("alibi+softcap", lambda q, k, v: O.attention_alibi(q, k, v, score_mod=2, enable_gqa=True, softcap=1.5,
                                                        is_causal=True, honor_causal=True)),
    ("softcap", lambda q, k, v: O.attention_softcapped(q, k, v, score_mod=0.7, enable_gqa=True)),
])
def test_oracle_gradients_against_finite_differences(name, fn):
    q, k, v = _tiny()
    assert torch.autograd.gradcheck(lambda a, b, c: fn(a, b, c), (q, k, v), eps=1e-6, atol=1e-5, rtol=1e-4), name


def test_oracle_gradients_of_bias_gate_and_branches_against_finite_differences():
    g = torch.Generator().manual_seed(3)
    mk = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).requires_grad_(True)  # noqa: E731
    # Evoformer layout [B, N, S, H, D] with a mask bias, a pair bias and the gate
    q, k, v, gate = (mk(1, 2, 4, 2, 3) for _ in range(4))
    b1, b2 = mk(1, 2, 1, 1, 4), mk(1, 1, 2, 4, 4)
    assert torch.autograd.gradcheck(lambda q, k, v, b1, b2, gate: O.attention_evoformer(q, k, v, [b1, b2], gate=gate),
                                    (q, k, v, b1, b2, gate), eps=1e-6, atol=1e-5, rtol=1e-4)
    # dense score_mod tensor (the ALiBi signature), causal
    q, k, v = _tiny()
    dense = mk(2, 5, 5)
    assert torch.autograd.gradcheck(
        lambda q, k, v, d: O.attention_alibi(q, k, v, score_mod=lambda L, S: d, enable_gqa=True, is_causal=True, honor_causal=True),
        (q, k, v, dense), eps=1e-6, atol=1e-5, rtol=1e-4)
    # differential attention: q, k [B, 2H, S, d], v [B, H, S, 2d]
    q, k, v = mk(1, 4, 5, 3), mk(1, 4, 5, 3), mk(1, 2, 5, 6)
    assert torch.autograd.gradcheck(lambda q, k, v: O.diff_attention(q, k, v, lambda_full=0.6, is_causal=True), (q, k, v),
                                    eps=1e-6, atol=1e-5, rtol=1e-4)


def test_backward_abi_validation():
    lib = _ffi.load_library()
    assert lib.fl_bwd_params_sizeof() == C.sizeof(_ffi.FlAttnBwdParams)

    def params(**kw):
        b = _ffi.FlAttnBwdParams()
        b.fwd = good_params(**kw)
        L, D, Hq, Hkv = b.fwd.Lq, b.fwd.Dqk, b.fwd.Hq, b.fwd.Hkv
        b.fwd.lse = 0x90000
        b.dout, b.dq, b.dk, b.dv, b.delta = 0xA0000, 0xB0000, 0xC0000, 0xD0000, 0xE0000
        b.dout_strides[:] = (Hq * L * D, L * D, D, 1)
        b.dq_strides[:] = (Hq * L * D, L * D, D, 1)
        b.dk_strides[:] = (Hkv * L * D, L * D, D, 1)
        b.dv_strides[:] = (Hkv * L * D, L * D, D, 1)
        return b

    rc = lambda b: lib.fl_attn_bwd_validate(C.byref(b))  # noqa: E731
    for D in (64, 128):
        assert rc(params(D=D)) == 0, _ffi.last_error()
    assert lib.fl_attn_bwd_validate(None) == -1
    cases = [
        (lambda b: setattr(b.fwd, "lse", 0), -1, "lse"),
        (lambda b: setattr(b.fwd, "lse", 0x90004), -7, "lse"),
        (lambda b: setattr(b, "delta", 0), -1, "delta"),
        (lambda b: setattr(b, "dout", 0xA0008), -7, "dout"),
        (lambda b: b.dk_strides.__setitem__(2, 62), -7, "dk"),
        (lambda b: (b.fwd.bias.__setitem__(0, 0x60000), b.fwd.bias_batch_div.__setitem__(0, 1),
                    setattr(b.fwd, "softcap", 30.0), setattr(b, "dscores", 0xF0000)), -4, "soft-cap"),
        (lambda b: setattr(b, "dscores", 0xF0000), -5, "dscores"),
        (lambda b: (setattr(b.fwd, "gate", 0x70000), b.fwd.gate_strides.__setitem__(slice(0, 4), list(b.fwd.o_strides))),
         -4, "not supported"),
        (lambda b: b.reserved.__setitem__(3, 1), -5, "reserved"),
        (lambda b: setattr(b.fwd, "scale", -1.0), -5, "scale"),
    ]
    for mutate, code, word in cases:
        b = params()
        mutate(b)
        assert rc(b) == code and word in _ffi.last_error(), (_ffi.last_error(), word)
        assert lib.fl_attn_bwd(C.byref(b), None) == code  # the same check runs before any launch
    assert rc(params(D=32)) == 0, _ffi.last_error()
    b = params(D=32)
    b.fwd.dropout_threshold = 1000  # no dropout kernels at head dim 32
    assert rc(b) == -4 and "kernel" in _ffi.last_error()
    # bias operands are taken with positional masks, and then dscores may be given
    b = params()
    b.fwd.bias[0], b.fwd.bias_batch_div[0] = 0x60000, 1
    b.fwd.bias_strides[0][:] = (0, 0, b.fwd.Lk, 1)
    b.dscores = 0xF0000
    assert rc(b) == 0, _ffi.last_error()
    b.dscores = 0xF0004
    assert rc(b) == -7 and "dscores" in _ffi.last_error()
    b = params(D=64, Dv=128)
    b.fwd.diff = 0
    assert rc(b) == -4


def test_every_combination_of_score_modifications_has_a_backward_kernel():
    """Mask kind x ALiBi x soft-cap x bias operands (x dropout from head dim 64 up) at head dims 32, 64 and 128, both
    element types (the gate and differential attention are compositions around these calls)."""
    import itertools
    lib = _ffi.load_library()
    for D, dtype in itertools.product((32, 64, 128), (_ffi.FL_BF16, _ffi.FL_F16)):
        for kind, alibi, cap, bias, drop in itertools.product(
                (_ffi.MASK_NONE, _ffi.MASK_CAUSAL, _ffi.MASK_SLIDING, _ffi.MASK_PREFIX_LM, _ffi.MASK_DOCUMENT,
                 _ffi.MASK_DOCUMENT_CAUSAL), (0, 4), (0.0, 30.0), (0, 1, 2), (0, 6554) if D > 32 else (0,)):
            b = _ffi.FlAttnBwdParams()
            b.fwd = good_params(D=D)
            f = b.fwd
            f.dtype, f.mask_kind, f.window, f.prefix, f.alibi_heads, f.softcap = dtype, kind, 17, 40, alibi, cap
            f.dropout_threshold = drop
            for i in range(bias):
                f.bias[i], f.bias_batch_div[i], f.bias_dtype[i] = 0x60000 + 0x100000 * i, 1, dtype
                f.bias_strides[i][:] = (0, 0, 304, 1) if i == 0 else (0, 0, 0, 1)
            if kind in (_ffi.MASK_DOCUMENT, _ffi.MASK_DOCUMENT_CAUSAL):
                f.doc_ids, f.doc_stride = 0x50000, 300
                f.workspace, f.workspace_bytes = 0x80000, lib.fl_workspace_bytes(C.byref(f))
            L, Hq, Hkv = f.Lq, f.Hq, f.Hkv
            f.lse = 0x90000
            b.dout, b.dq, b.dk, b.dv, b.delta = 0xA0000, 0xB0000, 0xC0000, 0xD0000, 0xE0000
            b.dout_strides[:] = (Hq * L * D, L * D, D, 1)
            b.dq_strides[:] = (Hq * L * D, L * D, D, 1)
            b.dk_strides[:] = (Hkv * L * D, L * D, D, 1)
            b.dv_strides[:] = (Hkv * L * D, L * D, D, 1)
            if bias and not cap:
                b.dscores = 0xF0000
            assert lib.fl_attn_bwd_validate(C.byref(b)) == 0, (D, dtype, kind, alibi, cap, bias, drop, _ffi.last_error())


# ---- the kernels ---------------------------------------------------------------------------------------------------------------

def _inputs(B, Hq, Hkv, L, D, seed, S=None):
    g = torch.Generator().manual_seed(seed)
    S = S or L
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(DEV)  # noqa: E731
    return mk(B, Hq, L, D), mk(B, Hkv, S, D), mk(B, Hkv, S, D), mk(B, Hq, L, D)


def _grads(fn, q, k, v, dout, dtype):
    q, k, v = (t.detach().to(dtype).requires_grad_(True) for t in (q, k, v))
    out = fn(q, k, v)
    out.backward(dout.to(out.dtype).reshape(out.shape))
    return out.detach(), q.grad, k.grad, v.grad


def _check(name, hip_fn, oracle_fn, q, k, v, dout):
    out, dq, dk, dv = _grads(hip_fn, q, k, v, dout, torch.bfloat16)
    ref, rq, rk, rv = _grads(oracle_fn, q, k, v, dout, torch.float32)
    torch.cuda.synchronize()
    assert_parity(out.reshape(ref.shape), ref, f"{name}: forward")
    for what, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        assert got.dtype == torch.bfloat16 and got.shape == want.shape
        scale = max(1.0, want.abs().max().item())
        assert_parity(got.float() / scale, want / scale, f"{name}: {what}")


VARIANTS = {
    "vanilla": (lambda q, k, v: A.attention_pytorch(q, k, v, enable_gqa=True),
                lambda q, k, v: O.attention_vanilla(q, k, v, enable_gqa=True)),
    "causal": (lambda q, k, v: A.attention_pytorch_causal(q, k, v, enable_gqa=True),
               lambda q, k, v: O.attention_causal(q, k, v, enable_gqa=True)),
    "sliding": (lambda q, k, v: A.attention_pytorch_sliding_window(q, k, v, window_size=37, enable_gqa=True),
                lambda q, k, v: O.attention_sliding_window(q, k, v, window_size=37, enable_gqa=True)),
    "prefix": (lambda q, k, v: A.attention_pytorch_prefix_lm(q, k, v, prefix_lengths=70, enable_gqa=True),
               lambda q, k, v: O.attention_prefix_lm(q, k, v, prefix_lengths=70, enable_gqa=True)),
    "alibi": (lambda q, k, v: A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(q.size(1)),
                                                        enable_gqa=True),
              lambda q, k, v: O.attention_alibi(q, k, v, score_mod=q.size(1), enable_gqa=True)),
    "softcap": (lambda q, k, v: A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(2.0), enable_gqa=True,
                                                       is_causal=True),
                lambda q, k, v: O.attention_softcapped(q, k, v, score_mod=2.0, enable_gqa=True, is_causal=True,
                                                       honor_causal=True)),
    "alibi+softcap+causal": (
        lambda q, k, v: A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(q.size(1)),
                                                  enable_gqa=True, is_causal=True, softcap=5.0),
        lambda q, k, v: O.attention_alibi(q, k, v, score_mod=q.size(1), enable_gqa=True, is_causal=True,
                                          honor_causal=True, softcap=5.0)),
}


@pytest.mark.gpu
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_gradients_match_the_oracle(name, D):
    hip_fn, oracle_fn = VARIANTS[name]
    # 300 rows: two full owner tiles and a ragged one; 4 query heads on 2 key/value heads
    q, k, v, dout = _inputs(2, 4, 2, 300, D, seed=sum(map(ord, name)) + D)
    _check(f"{name} D={D}", hip_fn, oracle_fn, q, k, v, dout)


@pytest.mark.gpu
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("name", ["vanilla", "causal", "alibi+softcap+causal"])
def test_gradients_fp16(name, D):
    """fp16 elements: same kernels compiled for the other MFMA / conversion instructions; fp16 keeps three more
    mantissa bits than bf16, so the bf16 tolerance holds with room."""
    hip_fn, oracle_fn = VARIANTS[name]
    q, k, v, dout = (t.to(torch.float16) for t in _inputs(2, 4, 2, 200, D, seed=sum(map(ord, name)) + D + 1))
    out, dq, dk, dv = _grads(hip_fn, q, k, v, dout, torch.float16)
    ref, rq, rk, rv = _grads(oracle_fn, q, k, v, dout, torch.float32)
    torch.cuda.synchronize()
    assert out.dtype == torch.float16
    assert_parity(out.reshape(ref.shape), ref, f"{name} fp16: forward")
    for what, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        assert got.dtype == torch.float16 and got.shape == want.shape
        scale = max(1.0, want.abs().max().item())
        assert_parity(got.float() / scale, want / scale, f"{name} fp16: {what}")


@pytest.mark.gpu
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
def test_gradients_document_mask(D, causal):
    q, k, v, dout = _inputs(2, 4, 2, 333, D, seed=77 + D)
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 5, (2, 333), generator=g).sort(dim=1).values.to(DEV)
    _check(f"document causal={causal} D={D}",
           lambda q, k, v: A.attention_pytorch_document_mask(q, k, v, ids, enable_gqa=True, is_causal=causal),
           lambda q, k, v: O.attention_document_mask(q, k, v, ids, enable_gqa=True, is_causal=causal), q, k, v, dout)
    # ids in no order: every tile pair has to be looked at
    ids = torch.randint(0, 3, (2, 333), generator=g).to(DEV)
    _check(f"document unsorted D={D}",
           lambda q, k, v: A.attention_pytorch_document_mask(q, k, v, ids, enable_gqa=True, is_causal=causal),
           lambda q, k, v: O.attention_document_mask(q, k, v, ids, enable_gqa=True, is_causal=causal), q, k, v, dout)


@pytest.mark.gpu
@pytest.mark.parametrize("cap", [None, 12.0])
@pytest.mark.parametrize("D", [64, 128])
def test_gradients_document_mask_with_alibi_and_softcap(D, cap):
    """Document ids in the element predicate together with the in-kernel ALiBi term and / or the soft-cap: the oracle is
    autograd through the eager fp32 composition cap * tanh(q k^T s / cap) + slope_h (k - q), masked where ids differ."""
    import math
    from flashlight_amd import _ffi, ops
    from oracle.attention import _softmax_attention, alibi_slopes
    B, H, S = 2, 4, 600
    q, k, v, dout = _inputs(B, H, H, S, D, seed=123 + D)
    g = torch.Generator().manual_seed(17)
    ids = torch.sort(torch.randint(0, 6, (B, S), generator=g), dim=1).values.to(DEV)
    slopes = alibi_slopes(H).float().view(1, H, 1, 1).to(DEV)
    for causal in (False, True):
        def masked(qi, ki):
            m = ids[:, qi.view(-1)].view(B, 1, -1, 1) != ids[:, ki.view(-1)].view(B, 1, 1, -1)
            return (m | (ki > qi)) if causal else m
        _check(f"document + alibi + cap={cap} causal={causal} D={D}",
               lambda q, k, v: ops.dispatch(q, k, v, mask_kind=_ffi.MASK_DOCUMENT_CAUSAL if causal else _ffi.MASK_DOCUMENT,
                                            doc_ids=ids, alibi_heads=H, softcap=cap or 0.0),
               lambda q, k, v: _softmax_attention(q, k, v, 1.0 / math.sqrt(D), masked=masked, softcap=cap,
                                                  bias=lambda qi, ki: slopes * (ki - qi).float()), q, k, v, dout)


@pytest.mark.gpu
@pytest.mark.parametrize("D", [64, 128])
def test_gradients_document_mask_many_dead_tiles(D):
    """Several documents over many tiles: most (owner block, streamed tile) pairs are dead, and the backward hops from
    one live step to the next; one document has a single position, one ends on a tile edge."""
    L = 1500
    lengths = [128, 1, 300, 255, 416, 400]
    assert sum(lengths) == L
    ids = torch.repeat_interleave(torch.arange(len(lengths)), torch.tensor(lengths))[None].expand(2, L).contiguous().to(DEV)
    q, k, v, dout = _inputs(2, 4, 2, L, D, seed=99 + D)
    for causal in (False, True):
        _check(f"document long causal={causal} D={D}",
               lambda q, k, v: A.attention_pytorch_document_mask(q, k, v, ids, enable_gqa=True, is_causal=causal),
               lambda q, k, v: O.attention_document_mask(q, k, v, ids, enable_gqa=True, is_causal=causal), q, k, v, dout)


@pytest.mark.gpu
@pytest.mark.parametrize("L,S", [(1, 1), (31, 31), (64, 200), (200, 64), (129, 257), (1000, 1000)])
def test_gradients_ragged_and_cross_lengths(L, S):
    for D in (64, 128):
        q, k, v, dout = _inputs(1, 2, 2, L, D, seed=L + S + D, S=S)
        _check(f"vanilla {L}x{S} D={D}", lambda q, k, v: A.attention_pytorch(q, k, v),
               lambda q, k, v: O.attention_vanilla(q, k, v), q, k, v, dout)
        _check(f"causal {L}x{S} D={D}", lambda q, k, v: A.attention_pytorch_causal(q, k, v),
               lambda q, k, v: O.attention_causal(q, k, v), q, k, v, dout)


@pytest.mark.gpu
def test_gradient_properties_at_benchmark_size():
    # B=1 H=4 S=4096 D=128 causal: too large for the CPU oracle in a test, so check what the mathematics fixes:
    # (1) dv is linear in dout; (2) sum_k dk . k == sum_q dq . q (both equal sum_{q,k} dS[q,k] S[q,k] / scale, since the
    # logits are bilinear in q and k); (3) a row's dq is orthogonal to nothing in particular, but dout = 0 gives zeros
    g = torch.Generator().manual_seed(9)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(DEV)  # noqa: E731
    q, k, v, d1, d2 = mk(1, 4, 4096, 128), mk(1, 4, 4096, 128), mk(1, 4, 4096, 128), mk(1, 4, 4096, 128), mk(1, 4, 4096, 128)

    def grads(dout):
        qq, kk, vv = (t.detach().requires_grad_(True) for t in (q, k, v))
        A.attention_pytorch_causal(qq, kk, vv).backward(dout)
        return qq.grad.float(), kk.grad.float(), vv.grad.float()

    q1, k1, v1 = grads(d1)
    q2, k2, v2 = grads(d2)
    q3, k3, v3 = grads((d1.float() + d2.float()).to(torch.bfloat16))
    # dout is rounded to bf16 once more in the third call; gradients are O(1)
    assert (v3 - (v1 + v2)).abs().max().item() < 6e-2 and (v3 - (v1 + v2)).abs().mean().item() < 4e-3
    lhs, rhs = (q1 * q.float()).sum().item(), (k1 * k.float()).sum().item()
    assert abs(lhs - rhs) <= 2e-2 * max(abs(lhs), abs(rhs), 1.0), (lhs, rhs)
    z = grads(torch.zeros_like(d1))
    assert all(float(t.abs().max()) == 0.0 for t in z)
    # row 0 attends only key 0, with weight 1 whatever q is: its dq is zero and dv[0] collects dout[0] in full
    assert float(q1[0, :, 0].abs().max()) < 1e-6


@pytest.mark.gpu
def test_gradients_under_torch_compile_equal_eager():
    # the differentiable operator carries its autograd rule into compiled graphs (forward and backward graphs hold
    # flashlight_amd::attn_fwd_lse and flashlight_amd::attn_bwd)
    q, k, v, dout = _inputs(2, 4, 2, 200, 64, seed=91)
    fn = lambda q, k, v: A.attention_pytorch_sliding_window(q, k, v, window_size=31, enable_gqa=True)  # noqa: E731
    eager = _grads(fn, q, k, v, dout, torch.bfloat16)
    torch._dynamo.reset()
    compiled = _grads(torch.compile(fn, backend="aot_eager", fullgraph=True), q, k, v, dout, torch.bfloat16)
    for a, b in zip(eager, compiled):
        assert torch.equal(a, b)
    torch.library.opcheck(torch.ops.flashlight_amd.attn_fwd_lse.default,
                          (q.detach().requires_grad_(True), k, v, -1.0, 1, 0, 0, None, 0, 0.0),
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))


# ---- gradients through bias operands, the gate and the two branches of differential attention ------------------------------

def _compare(name, got, want):
    for what, g_, w_ in zip(name[1], got, want):
        assert g_ is not None and tuple(g_.shape) == tuple(w_.shape), f"{name[0]}: {what}"
        scale = max(1.0, w_.abs().max().item())
        assert_parity(g_.float() / scale, w_.float() / scale, f"{name[0]}: {what}")


@pytest.mark.gpu
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("D", [64, 128])
def test_gradients_dense_score_mod(D, causal):
    """attention_pytorch_alibi with an arbitrary dense tensor (alibi.py:26-30): gradients reach q, k, v and the tensor."""
    B, Hq, Hkv, L = 2, 4, 2, 200
    q, k, v, dout = _inputs(B, Hq, Hkv, L, D, seed=300 + D)
    g = torch.Generator().manual_seed(9)
    dense = torch.randn(Hq, L, L, generator=g)
    outs = []
    for dev, dtype, mod in ((DEV, torch.bfloat16, A), ("cpu", torch.float32, None)):
        qq, kk, vv = (t.detach().to(dev).to(dtype).requires_grad_(True) for t in (q, k, v))
        dd = dense.to(dev).requires_grad_(True)
        if mod is not None:
            out = A.attention_pytorch_alibi(qq, kk, vv, score_mod=lambda L_, S_: dd, enable_gqa=True, is_causal=causal)
        else:
            out = O.attention_alibi(qq, kk, vv, score_mod=lambda L_, S_: dd, enable_gqa=True, is_causal=causal,
                                    honor_causal=True)
        out.backward(dout.to(dev).to(out.dtype).reshape(out.shape))
        outs.append((out.detach().reshape(B, Hq, L, D), qq.grad, kk.grad, vv.grad, dd.grad))
    torch.cuda.synchronize()
    _compare((f"dense score_mod D={D} causal={causal}", ("out", "dq", "dk", "dv", "dbias")), outs[0], outs[1])


@pytest.mark.gpu
@pytest.mark.parametrize("B,N,S,H,D", [(1, 6, 96, 2, 32), (2, 3, 70, 3, 64)])
def test_gradients_evoformer_biases_and_gate(B, N, S, H, D):
    """attention_reference with the benchmark's two biases (evoformer.py:46-47) and the gate: gradients of every operand."""
    g = torch.Generator().manual_seed(B + S)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)  # noqa: E731
    q, k, v, gate, dout = (mk(B, N, S, H, D) for _ in range(5))
    b1, b2 = mk(B, N, 1, 1, S), mk(B, 1, H, S, S)
    res = []
    for dev, dtype in ((DEV, torch.bfloat16), ("cpu", torch.float32)):
        ts = [t.detach().to(dev).to(dtype).requires_grad_(True) for t in (q, k, v, b1, b2, gate)]
        fn = A.attention_reference if dev == DEV else O.attention_evoformer
        out = fn(ts[0], ts[1], ts[2], [ts[3], ts[4]], gate=ts[5])
        out.backward(dout.to(dev).to(out.dtype))
        res.append([out.detach()] + [t.grad for t in ts])
    torch.cuda.synchronize()
    _compare((f"evoformer {B, N, S, H, D}", ("out", "dq", "dk", "dv", "dbias1", "dbias2", "dgate")), res[0], res[1])


@pytest.mark.gpu
@pytest.mark.parametrize("causal", [False, True])
def test_gradients_differential_attention(causal):
    B, H, S, d = 2, 2, 200, 64
    g = torch.Generator().manual_seed(17)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)  # noqa: E731
    q, k, v, dout = mk(B, 2 * H, S, d), mk(B, 2 * H, S, d), mk(B, H, S, 2 * d), mk(B, H, S, 2 * d)
    res = []
    for dev, dtype in ((DEV, torch.bfloat16), ("cpu", torch.float32)):
        ts = [t.detach().to(dev).to(dtype).requires_grad_(True) for t in (q, k, v)]
        fn = A.diffattn if dev == DEV else O.diff_attention
        out = fn(ts[0], ts[1], ts[2], lambda_full=0.8, is_causal=causal)
        out.backward(dout.to(dev).to(out.dtype))
        res.append([out.detach()] + [t.grad for t in ts])
    torch.cuda.synchronize()
    _compare((f"diffattn causal={causal}", ("out", "dq", "dk", "dv")), res[0], res[1])


@pytest.mark.gpu
@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("kind", ["alibi", "softcap", "document", "document+alibi+softcap"])
def test_gradients_bias_operands_with_other_score_modifications(D, kind):
    """Bias operands together with the in-kernel ALiBi term, the soft-cap and document ids: gradients of q, k, v always,
    of the operands too unless a soft-cap is on (the dense score_mod of alibi.py:26-30 with `softcap=`, and what the
    graph rewrite composes)."""
    from flashlight_amd import ops
    from oracle.attention import _softmax_attention, alibi_slopes
    B, Hq, Hkv, L = 2, 4, 2, 210
    q, k, v, dout = _inputs(B, Hq, Hkv, L, D, seed=400 + D)
    g = torch.Generator().manual_seed(D)
    table = torch.randn(1, Hq, L, L, generator=g)
    row = torch.randn(B, 1, 1, L, generator=g)
    ids = torch.sort(torch.randint(0, 4, (B, L), generator=g), dim=1).values
    alibi, cap, doc = "alibi" in kind, (9.0 if "softcap" in kind else None), "document" in kind
    bias_grads = cap is None
    # the kernels
    qq, kk, vv = (t.detach().to(DEV).requires_grad_(True) for t in (q, k, v))
    tb, rb = table.to(torch.bfloat16).to(DEV).requires_grad_(bias_grads), row.to(DEV).requires_grad_(bias_grads)
    out = ops.dispatch(qq, kk, vv, mask_kind=_ffi.MASK_DOCUMENT_CAUSAL if doc else _ffi.MASK_CAUSAL,
                       doc_ids=ids.to(DEV) if doc else None, alibi_heads=Hq if alibi else 0, softcap=cap or 0.0,
                       biases=[(tb, B), (rb, 1)])
    out.backward(dout.to(DEV))
    # the oracle
    qf, kf, vf = (t.detach().float().cpu().requires_grad_(True) for t in (q, k, v))
    tf, rf = table.to(torch.bfloat16).float().requires_grad_(True), row.clone().requires_grad_(True)
    slopes = alibi_slopes(Hq).float().view(1, Hq, 1, 1)

    def masked(qi, ki):
        m = ki > qi
        return (m | (ids[:, qi.view(-1)].view(B, 1, -1, 1) != ids[:, ki.view(-1)].view(B, 1, 1, -1))) if doc else m

    def bias(qi, ki):
        return ([slopes * (ki - qi).float()] if alibi else []) + [tf[..., qi.view(-1), :], rf]

    ref = _softmax_attention(qf, kf.repeat_interleave(Hq // Hkv, 1), vf.repeat_interleave(Hq // Hkv, 1), 1.0 / math.sqrt(D),
                             masked=masked, bias=bias, softcap=cap)
    ref.backward(dout.float().cpu())
    names, got, want = ["out", "dq", "dk", "dv"], [out.detach(), qq.grad, kk.grad, vv.grad], [ref.detach(), qf.grad, kf.grad, vf.grad]
    if bias_grads:
        names += ["dtable", "drow"]
        got += [tb.grad, rb.grad]
        want += [tf.grad, rf.grad]
    else:
        with pytest.raises(NotImplementedError, match="soft-cap"):
            ops.dispatch(qq, kk, vv, mask_kind=_ffi.MASK_CAUSAL, softcap=cap, biases=[(tb.detach().requires_grad_(True), B)])
    torch.cuda.synchronize()
    for what, g_, w_ in zip(names, got, want):
        assert g_ is not None and tuple(g_.shape) == tuple(w_.shape), what
        scale = max(1.0, w_.abs().max().item())
        # (a bias gradient is a sum of score gradients over everything the operand broadcasts over: the bound grows with
        # the square root of the number of summands)
        fan = math.sqrt(B) if what == "dtable" else math.sqrt(Hq * L / 8) if what == "drow" else 1.0
        assert_parity(g_.float() / scale, w_.float() / scale, f"{kind} D={D}: {what}", max_tol=2e-2 * fan, mean_tol=2e-3 * fan)


@pytest.mark.gpu
def test_plain_gradients_at_head_dim_32():
    q, k, v, dout = _inputs(2, 4, 2, 300, 32, seed=32)
    _check("causal D=32", *VARIANTS["causal"], q, k, v, dout)
    _check("sliding D=32", *VARIANTS["sliding"], q, k, v, dout)
    _check("alibi+softcap+causal D=32", *VARIANTS["alibi+softcap+causal"], q, k, v, dout)
    ids = torch.randint(0, 4, (2, 300), generator=torch.Generator().manual_seed(6)).sort(dim=1).values.to(DEV)
    _check("document causal D=32",
           lambda q, k, v: A.attention_pytorch_document_mask(q, k, v, ids, enable_gqa=True, is_causal=True),
           lambda q, k, v: O.attention_document_mask(q, k, v, ids, enable_gqa=True, is_causal=True), q, k, v, dout)
