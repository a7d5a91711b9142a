"""Dropout on the softmax weights.  The reference's variants accept `dropout_p` and ignore it (attention_variants/
causal.py:4-36, alibi.py:13-33, softcap.py:4-53), so there is no reference output to compare with.  What is pinned:

  * the semantics (oracle/dropout.py) against library routines: all weights kept == scaled_dot_product_attention; the
    1 / (1 - p) convention against torch.nn.functional.dropout; the mean over many seeds approaches the undropped result;
  * the decision function: a second restatement in plain Python integers, frozen known values, and its statistics
    (rate, uniformity, no correlation along rows, columns, diagonals, heads or seeds);
  * its gradients: autograd through the oracle against central differences in float64;
  * the kernels (GPU tests): forward and gradients, through the C ABI, against the oracle given the same seed.
"""
import ctypes as C

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import flashlight_amd.attention_variants as A
from flashlight_amd import _ffi, ops
from oracle import dropout as OD
from tests.conftest import assert_parity
from tests.test_abi import good_params

DEV = "cuda"


# ---- the decision function -------------------------------------------------------------------------------------------------

def _scalar_random16(seed, bh, q, k):
    """The same 16 bits in plain Python integers (no numpy), written from the description in oracle/dropout.py."""
    m = 0xFFFFFFFF

    def fmix(x):
        x &= m
        x ^= x >> 16
        x = (x * 0x85EBCA6B) & m
        x ^= x >> 13
        x = (x * 0xC2B2AE35) & m
        return x ^ (x >> 16)

    s0 = fmix((seed & m) ^ fmix(((seed >> 32) + 0x9E3779B9 * (bh + 1)) & m))
    x = (s0 + q * 0x9E3779B1 + (k // 2) * 0x85EBCA77) & m
    x ^= x >> 16
    x = ((x & 0xFFFFFF) * 0xCA6B35 + (x >> 8)) & m
    x ^= x >> 13
    x = (((x >> 8) & 0xFFFFFF) * 0xB2AE3D + x) & m
    x ^= x >> 16
    return (x >> 16) if k % 2 else (x & 0xFFFF)


def test_decision_bits_two_restatements_and_known_values():
    for seed, bh in ((0, 0), (1234, 3), (2 ** 63 + 12345, 63), (0xFFFFFFFFFFFFFFFF, 7)):
        r = OD.random16(seed, bh, 9, 14)
        for q in range(9):
            for k in range(14):
                assert r[q, k] == _scalar_random16(seed, bh, q, k), (seed, bh, q, k)
    # frozen values: a change of any constant, shift or operand order shows up here
    assert OD.head_seed(0, 0) == 2856213345 and OD.head_seed(1, 5) == 4171907236
    assert OD.random16(1234, 3, 2, 8).tolist() == [[12170, 21700, 45079, 30570, 41986, 25535, 54504, 33553],
                                                    [45153, 33049, 5915, 51856, 49463, 23721, 16504, 11248]]
    # positions far out (32-bit wrap-around of the products)
    r = OD.random16(99, 1, 70000, 6)[-1]
    assert [int(x) for x in r] == [_scalar_random16(99, 1, 69999, k) for k in range(6)]


def test_threshold_and_effective_rate():
    assert OD.threshold16(0.0) == 0 and OD.threshold16(0.5) == 32768 and OD.threshold16(0.1) == 6554
    assert OD.threshold16(0.9999999) == 65535
    assert _ffi.dropout_threshold(0.1) == OD.threshold16(0.1) and _ffi.dropout_threshold(0.25) == 16384
    for bad in (-0.1, 1.0, 2.0):
        with pytest.raises(ValueError):
            OD.threshold16(bad)
        with pytest.raises(ValueError):
            _ffi.dropout_threshold(bad)
    assert abs(OD.effective_rate(0.1) - 0.1) < 2 ** -16


def test_decision_bits_statistics():
    def corr(a, b):
        return abs(np.corrcoef(a.ravel(), b.ravel())[0, 1])

    n = 512
    noise = 5.0 / n  # five standard deviations of a sample correlation over n * n pairs
    for seed, bh in ((0, 0), (1, 5), (987654321987, 63)):
        u = OD.random16(seed, bh, n, n) / 65536.0
        assert abs(u.mean() - 0.5) < 0.003
        hist = np.bincount((u * 16).astype(int).ravel(), minlength=16) / u.size
        assert np.abs(hist - 1 / 16).max() < 0.002
        for a, b in ((u[:, :-1], u[:, 1:]), (u[:, :-2], u[:, 2:]), (u[:, :-4], u[:, 4:]), (u[:-1], u[1:]), (u[:-2], u[2:]),
                     (u[:-4], u[4:]), (u[:-1, :-1], u[1:, 1:]), (u[:-1, 1:], u[1:, :-1]), (u[:-1, :-2], u[1:, 2:])):
            assert corr(a, b) < noise
        assert corr(u, OD.random16(seed, bh + 1, n, n) / 65536.0) < noise
        assert corr(u, OD.random16(seed + 1, bh, n, n) / 65536.0) < noise
        for p in (0.1, 0.5):
            keep = u >= OD.effective_rate(p)
            assert abs(keep.mean() - (1 - p)) < 0.003
            sd = np.sqrt(p * (1 - p) / n)  # of a row's or column's keep rate
            assert 0.8 * sd < keep.mean(1).std() < 1.2 * sd and 0.8 * sd < keep.mean(0).std() < 1.2 * sd


# ---- the semantics ---------------------------------------------------------------------------------------------------------

def _rand(B, Hq, Hkv, L, S, E, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g, dtype=dtype)  # noqa: E731
    return mk(B, Hq, L, E), mk(B, Hkv, S, E), mk(B, Hkv, S, E)


def test_oracle_dropout_semantics_against_library_routines():
    q, k, v = _rand(2, 4, 2, 7, 9, 8)
    ones = torch.ones(2, 4, 7, 9, dtype=torch.bool)
    # nothing dropped: plain attention (p only sets the scale, 1 here)
    ref = F.scaled_dot_product_attention(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1))
    assert torch.allclose(OD.attention_dropout(q, k, v, ones, 0.0), ref, atol=1e-6)
    causal = torch.tril(torch.ones(7, 9, dtype=torch.bool))
    ref = F.scaled_dot_product_attention(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1), attn_mask=causal)
    assert torch.allclose(OD.attention_dropout(q, k, v, ones, 0.0, attend=causal), ref, atol=1e-6)
    # everything dropped: zeros; kept weights carry the factor torch's own dropout uses
    assert OD.attention_dropout(q, k, v, ~ones, 0.25).abs().max() == 0
    kept_value = F.dropout(torch.ones(1000), 0.25, training=True).max().item()
    assert abs(kept_value - 1 / (1 - OD.effective_rate(0.25))) < 1e-6
    # one key kept per row: that key's value times weight / (1 - p)
    keep = torch.zeros(2, 4, 7, 9, dtype=torch.bool)
    keep[..., 3] = True
    w = torch.softmax(q @ k.repeat_interleave(2, 1).transpose(-1, -2) / 8 ** 0.5, -1)[..., 3:4]
    want = w * v.repeat_interleave(2, 1)[:, :, 3:4, :] / (1 - OD.effective_rate(0.25))
    assert torch.allclose(OD.attention_dropout(q, k, v, keep, 0.25), want, atol=1e-6)
    # unbiased: the mean over seeds approaches the undropped result
    ref = OD.attention_dropout(q, k, v, ones, 0.0)
    acc = torch.zeros_like(ref)
    n = 400
    for seed in range(n):
        acc += OD.attention_dropout(q, k, v, OD.keep_mask(seed, 2, 4, 7, 9, 0.3), 0.3)
    assert (acc / n - ref).abs().max() < 0.15 and (acc / n - ref).abs().mean() < 0.03


def test_oracle_dropout_gradients_against_finite_differences():
    q, k, v = (t.requires_grad_(True) for t in _rand(1, 2, 1, 5, 6, 4, dtype=torch.float64))
    keep = OD.keep_mask(5, 1, 2, 5, 6, 0.4)
    causal = torch.tril(torch.ones(5, 6, dtype=torch.bool))
    assert 0.2 < keep.float().mean() < 0.9
    assert torch.autograd.gradcheck(lambda a, b, c: OD.attention_dropout(a, b, c, keep, 0.4, attend=causal), (q, k, v),
                                    eps=1e-6, atol=1e-5, rtol=1e-4)


# ---- the boundary ----------------------------------------------------------------------------------------------------------

def test_abi_validation_of_dropout_fields():
    lib = _ffi.load_library()
    rc = lambda p: lib.fl_attn_validate(C.byref(p))  # noqa: E731
    for D in (64, 128):
        p = good_params(D=D)
        p.dropout_threshold = 6554
        p.dropout_seed[0], p.dropout_seed[1] = 0xFFFFFFFF, 0x7FFFFFFF
        p.mask_kind = _ffi.MASK_CAUSAL
        assert rc(p) == 0, _ffi.last_error()
    p = good_params()
    p.dropout_threshold = 65536
    assert rc(p) == -5 and "dropout_threshold" in _ffi.last_error()
    for mutate in (lambda p: setattr(p, "alibi_heads", 4), lambda p: setattr(p, "softcap", 30.0),
                   lambda p: (setattr(p, "alibi_heads", 4), setattr(p, "softcap", 30.0))):
        p = good_params()
        p.dropout_threshold = 100
        mutate(p)
        assert rc(p) == 0, _ffi.last_error()
    for kind in (_ffi.MASK_DOCUMENT, _ffi.MASK_DOCUMENT_CAUSAL):  # a document mask alone goes with dropout
        p = good_params()
        p.dropout_threshold = 100
        p.mask_kind, p.doc_ids = kind, 0x50000
        p.workspace, p.workspace_bytes = 0x80000, lib.fl_workspace_bytes(C.byref(p))
        assert rc(p) == 0, _ffi.last_error()
    doc = lambda p: (setattr(p, "mask_kind", _ffi.MASK_DOCUMENT), setattr(p, "doc_ids", 0x50000),  # noqa: E731
                     setattr(p, "workspace", 0x80000), setattr(p, "workspace_bytes", lib.fl_workspace_bytes(C.byref(p))))
    def dense(p):
        p.bias[0], p.bias_batch_div[0] = 0x60000, 1
        p.bias_strides[0][:] = (0, 0, p.Lk, 1)

    for mutate in (dense, lambda p: (dense(p), setattr(p, "mask_kind", _ffi.MASK_CAUSAL)),
                   lambda p: (setattr(p, "gate", 0x70000), p.gate_strides.__setitem__(slice(0, 4), list(p.o_strides)))):
        p = good_params()
        p.dropout_threshold = 100
        mutate(p)
        assert rc(p) == 0, _ffi.last_error()
    # ... and so does every combination of them (the workspace size follows the kernel chosen: ids last)
    for mutate in (lambda p: (setattr(p, "alibi_heads", 4), doc(p)),
                   lambda p: (setattr(p, "softcap", 30.0), doc(p)),
                   lambda p: (dense(p), doc(p)),
                   lambda p: (dense(p), setattr(p, "softcap", 30.0))):
        p = good_params()
        p.dropout_threshold = 100
        mutate(p)
        assert rc(p) == 0, _ffi.last_error()
    for mutate in (lambda p: setattr(p, "diff", 1),
                   lambda p: (setattr(p, "score_fn", _ffi.SCORE_CLAMP), p.score_fn_params.__setitem__(slice(0, 4), [1.0, 0.0, -1.0, 1.0]))):
        p = good_params()
        p.dropout_threshold = 100
        mutate(p)
        assert rc(p) == -4, _ffi.last_error()
    p = good_params(D=32)  # no dropout kernel at head dim 32
    p.dropout_threshold = 100
    assert rc(p) == -4, _ffi.last_error()
    p = good_params()
    p.flags = 4
    assert rc(p) == -5 and "flags" in _ffi.last_error()


def test_front_end_switch_and_refusals():
    q = torch.zeros(1, 2, 8, 64)
    # default: dropout_p is ignored like the reference does, so a CPU call fails for the usual reason, not for dropout
    with pytest.raises(Exception) as e:
        A.attention_pytorch_causal(q, q, q, dropout_p=0.5)
    assert "dropout" not in str(e.value)
    with pytest.raises(NotImplementedError, match="dropout"):
        ops.dispatch(q, q, q, dropout_p=0.1, diff=True)
    with pytest.raises(NotImplementedError, match="dropout"):  # score functions take no dropout
        ops.dispatch(q, q, q, dropout_p=0.1, score_fn=(_ffi.SCORE_CLAMP, (1.0, 0.0, -1.0, 1.0)))
    with pytest.raises(ValueError, match="dropout_p"):
        ops.dispatch(q, q, q, dropout_p=1.5)
    with A.honor_dropout():
        from flashlight_amd.attention_variants import _common
        assert _common._honor_dropout
    assert not _common._honor_dropout


# ---- the kernels -----------------------------------------------------------------------------------------------------------

def _gpu_inputs(B, Hq, Hkv, L, S, D, seed):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(DEV)  # noqa: E731
    return mk(B, Hq, L, D), mk(B, Hkv, S, D), mk(B, Hkv, S, D), mk(B, Hq, L, D)


def _attend(mask_kind, L, S, window=0, prefix=0):
    qi = torch.arange(L)[:, None]
    ki = torch.arange(S)[None, :]
    if mask_kind == _ffi.MASK_CAUSAL:
        return ki <= qi
    if mask_kind == _ffi.MASK_SLIDING:
        return (ki <= qi) & (qi - ki <= window)
    if mask_kind == _ffi.MASK_PREFIX_LM:
        return (ki < prefix) | (ki <= qi)
    return None


CASES = [
    # B, Hq, Hkv, L, S, D, mask, window, prefix, p
    (2, 4, 2, 200, 200, 64, _ffi.MASK_NONE, 0, 0, 0.1),
    (1, 4, 1, 257, 257, 128, _ffi.MASK_CAUSAL, 0, 0, 0.25),
    (2, 2, 2, 130, 300, 128, _ffi.MASK_NONE, 0, 0, 0.5),
    (1, 2, 1, 300, 130, 64, _ffi.MASK_CAUSAL, 0, 0, 0.1),
    (1, 2, 2, 400, 400, 64, _ffi.MASK_SLIDING, 50, 0, 0.2),
    (1, 2, 2, 333, 333, 128, _ffi.MASK_PREFIX_LM, 0, 70, 0.3),
    (1, 1, 1, 1, 1, 64, _ffi.MASK_NONE, 0, 0, 0.1),
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(map(str, c)))
def test_forward_and_gradients_with_dropout_match_the_oracle(case):
    B, Hq, Hkv, L, S, D, mask_kind, window, prefix, p = case
    seed = 0x1234567 * (L + 1) + (S << 40)
    q, k, v, dout = _gpu_inputs(B, Hq, Hkv, L, S, D, seed=L + D)
    kw = dict(mask_kind=mask_kind, window=window, prefix=prefix, dropout_p=p, dropout_seed=seed)
    lse = torch.empty(B, Hq, L, dtype=torch.float32, device=DEV)
    out = _ffi.attn_fwd(q, k, v, lse=lse, **kw)
    dq, dk, dv = _ffi.attn_bwd(q, k, v, out, lse, dout, **kw)
    torch.cuda.synchronize()

    keep = OD.keep_mask(seed, B, Hq, L, S, p)
    qf, kf, vf = (t.float().cpu().requires_grad_(True) for t in (q, k, v))
    ref = OD.attention_dropout(qf, kf, vf, keep, p, attend=_attend(mask_kind, L, S, window, prefix))
    ref.backward(dout.float().cpu())
    assert_parity(out, ref, "forward with dropout")
    for what, got, want in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
        scale = max(1.0, want.abs().max().item())
        assert_parity(got.float() / scale, want / scale, f"{what} with dropout")
    # the row statistics do not see the dropout
    lse0 = torch.empty_like(lse)
    _ffi.attn_fwd(q, k, v, lse=lse0, mask_kind=mask_kind, window=window, prefix=prefix)
    assert torch.allclose(lse, lse0, atol=2e-2, rtol=0)  # sums of bf16-rounded weights over different tile sizes


@pytest.mark.gpu
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("alibi,softcap", [(True, None), (False, 3.0), (True, 5.0)])
def test_dropout_with_alibi_and_softcap(D, alibi, softcap):
    B, Hq, Hkv, L = 1, 4, 2, 230
    q, k, v, dout = _gpu_inputs(B, Hq, Hkv, L, L, D, seed=D + (7 if alibi else 0))
    p, seed = 0.2, 0xABCDEF0123
    kw = dict(mask_kind=_ffi.MASK_CAUSAL, alibi_heads=Hq if alibi else 0, softcap=softcap or 0.0, dropout_p=p, dropout_seed=seed)
    lse = torch.empty(B, Hq, L, dtype=torch.float32, device=DEV)
    out = _ffi.attn_fwd(q, k, v, lse=lse, **kw)
    dq, dk, dv = _ffi.attn_bwd(q, k, v, out, lse, dout, **kw)
    torch.cuda.synchronize()
    import oracle as O
    bias = None
    if alibi:
        rel = (torch.arange(L)[None, :] - torch.arange(L)[:, None]).float()
        bias = O.alibi_slopes(Hq)[:, None, None] * rel[None]
    qf, kf, vf = (t.float().cpu().requires_grad_(True) for t in (q, k, v))
    ref = OD.attention_dropout(qf, kf, vf, OD.keep_mask(seed, B, Hq, L, L, p), p, attend=_attend(_ffi.MASK_CAUSAL, L, L),
                               bias=bias, softcap=softcap)
    ref.backward(dout.float().cpu())
    assert_parity(out, ref, "forward with dropout and score modifications")
    for what, got, want in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
        scale = max(1.0, want.abs().max().item())
        assert_parity(got.float() / scale, want / scale, f"{what} with dropout and score modifications")


def _document_ids(B, L, lengths, shuffle_seed=None):
    ids = torch.repeat_interleave(torch.arange(len(lengths)), torch.tensor(lengths))[:L]
    ids = torch.cat([ids, ids.new_full((L - ids.numel(),), len(lengths))])
    rows = []
    for b in range(B):
        row = (ids + 3 * b) * 7 - 11  # any integers, not 0..n
        if shuffle_seed is not None:  # unsorted ids: same-document positions scattered over the sequence
            row = row[torch.randperm(L, generator=torch.Generator().manual_seed(shuffle_seed + b))]
        rows.append(row)
    return torch.stack(rows).to(torch.int64)


@pytest.mark.gpu
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("causal,shuffled", [(False, False), (True, False), (False, True)])
def test_dropout_under_a_document_mask(D, causal, shuffled):
    B, Hq, Hkv, L = 2, 4, 2, 391
    q, k, v, dout = _gpu_inputs(B, Hq, Hkv, L, L, D, seed=D + 31 * causal + 5 * shuffled)
    ids = _document_ids(B, L, [70, 1, 129, 64, 100], shuffle_seed=17 if shuffled else None)
    p, seed = 0.15, 0x5EED0000DEADBEEF >> 1
    kind = _ffi.MASK_DOCUMENT_CAUSAL if causal else _ffi.MASK_DOCUMENT
    kw = dict(mask_kind=kind, doc_ids=ids.to(DEV), dropout_p=p, dropout_seed=seed)
    lse = torch.empty(B, Hq, L, dtype=torch.float32, device=DEV)
    out = _ffi.attn_fwd(q, k, v, lse=lse, **kw)
    dq, dk, dv = _ffi.attn_bwd(q, k, v, out, lse, dout, **kw)
    torch.cuda.synchronize()
    attend = (ids[:, :, None] == ids[:, None, :])[:, None]  # [B, 1, L, L]
    if causal:
        attend = attend & (torch.arange(L)[None, :] <= torch.arange(L)[:, None])
    qf, kf, vf = (t.float().cpu().requires_grad_(True) for t in (q, k, v))
    ref = OD.attention_dropout(qf, kf, vf, OD.keep_mask(seed, B, Hq, L, L, p), p, attend=attend)
    ref.backward(dout.float().cpu())
    assert_parity(out, ref, "forward with dropout under a document mask")
    for what, got, want in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
        scale = max(1.0, want.abs().max().item())
        assert_parity(got.float() / scale, want / scale, f"{what} with dropout under a document mask")
    # the dropped weights are the ones the positional-mask kernels drop for the same seed: one document gives the
    # unmasked / causal call's result
    one = torch.zeros(B, L, dtype=torch.int64, device=DEV)
    a = _ffi.attn_fwd(q, k, v, mask_kind=kind, doc_ids=one, dropout_p=p, dropout_seed=seed)
    b = _ffi.attn_fwd(q, k, v, mask_kind=_ffi.MASK_CAUSAL if causal else _ffi.MASK_NONE, dropout_p=p, dropout_seed=seed)
    assert_parity(a, b.float().cpu(), "one document against the positional mask")
    # the variant function takes dropout_p once the switch is on
    with A.honor_dropout():
        torch.manual_seed(5)
        x = A.attention_pytorch_document_mask(q, k, v, ids.to(DEV), enable_gqa=True, is_causal=causal, dropout_p=p)
        torch.manual_seed(5)
        y = A.attention_pytorch_document_mask(q, k, v, ids.to(DEV), enable_gqa=True, is_causal=causal, dropout_p=p)
    z = A.attention_pytorch_document_mask(q, k, v, ids.to(DEV), enable_gqa=True, is_causal=causal, dropout_p=p)
    assert torch.equal(x, y) and not torch.equal(x, z)


@pytest.mark.gpu
@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("mask_kind", [_ffi.MASK_NONE, _ffi.MASK_CAUSAL])
def test_dropout_with_bias_operands_and_the_gate(D, mask_kind):
    """A dense additive term per head (shared by the batch: a relative-position table) and a row-broadcast fp32 term, with
    dropout: forward, gradients of q, k, v and the score gradient the bias gradients are summed from."""
    B, Hq, Hkv, L, S = 2, 4, 2, 210, 275
    q, k, v, dout = _gpu_inputs(B, Hq, Hkv, L, S, D, seed=D + mask_kind)
    g = torch.Generator().manual_seed(D)
    table = torch.randn(1, Hq, L, S, generator=g).to(torch.bfloat16).to(DEV)
    rowb = (torch.randn(B, 1, 1, S, generator=g) * 2).to(DEV)
    p, seed = 0.2, 0x0123456789ABCDE
    kw = dict(mask_kind=mask_kind, biases=[(table, 1), (rowb, 1)], dropout_p=p, dropout_seed=seed)
    lse = torch.empty(B, Hq, L, dtype=torch.float32, device=DEV)
    out = _ffi.attn_fwd(q, k, v, lse=lse, **kw)
    dscores = torch.zeros(B, Hq, L, S, dtype=torch.float32, device=DEV)
    dq, dk, dv = _ffi.attn_bwd(q, k, v, out, lse, dout, dscores=dscores, **kw)
    torch.cuda.synchronize()
    qf, kf, vf = (t.float().cpu().requires_grad_(True) for t in (q, k, v))
    bias = (table.float().cpu() + rowb.cpu()).requires_grad_(True)
    ref = OD.attention_dropout(qf, kf, vf, OD.keep_mask(seed, B, Hq, L, S, p), p, attend=_attend(mask_kind, L, S), bias=bias)
    ref.backward(dout.float().cpu())
    assert_parity(out, ref, "forward with bias operands and dropout")
    for what, got, want in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad), ("dscores", dscores, bias.grad)):
        scale = max(1.0, want.abs().max().item())
        assert_parity(got.float() / scale, want / scale, f"{what} with bias operands and dropout")
    # the gate multiplies the result, whatever was dropped
    gate = torch.randn(B, Hq, L, D, generator=g).to(torch.bfloat16).to(DEV)
    gated = _ffi.attn_fwd(q, k, v, gate=gate, **kw)
    assert_parity(gated, ref.detach() * torch.sigmoid(gate.float().cpu()), "gate with dropout")
    plain = _ffi.attn_fwd(q, k, v, gate=gate, mask_kind=mask_kind, dropout_p=p, dropout_seed=seed)
    ref0 = OD.attention_dropout(qf.detach(), kf.detach(), vf.detach(), OD.keep_mask(seed, B, Hq, L, S, p), p,
                                attend=_attend(mask_kind, L, S))
    assert_parity(plain, ref0 * torch.sigmoid(gate.float().cpu()), "gate with dropout, no bias")
    # through autograd: bias gradients are the score gradient summed over what the operand broadcasts over
    qg, kg, vg, tg, rg = (t.detach().clone().requires_grad_(True) for t in (q, k, v, table, rowb))
    o = ops.dispatch(qg, kg, vg, mask_kind=mask_kind, biases=[(tg, 1), (rg, 1)], gate=gate, dropout_p=p, dropout_seed=seed)
    o.backward(dout)
    sg = torch.sigmoid(gate.float().cpu())
    qf2, kf2, vf2 = (t.float().cpu().requires_grad_(True) for t in (q, k, v))
    tf, rf = table.float().cpu().requires_grad_(True), rowb.cpu().requires_grad_(True)
    r2 = OD.attention_dropout(qf2, kf2, vf2, OD.keep_mask(seed, B, Hq, L, S, p), p, attend=_attend(mask_kind, L, S),
                              bias=tf + rf) * sg
    r2.backward(dout.float().cpu())
    assert_parity(o, r2, "autograd forward with bias operands, gate and dropout")
    for what, got, want in (("dq", qg.grad, qf2.grad), ("dtable", tg.grad, tf.grad), ("drow", rg.grad, rf.grad)):
        scale = max(1.0, want.abs().max().item())
        assert_parity(got.float() / scale, want / scale, f"autograd {what} with bias operands, gate and dropout",
                      max_tol=3e-2)


def _random_dropout_case(seed):
    import random
    rnd = random.Random(seed)
    D = rnd.choice([64, 128])
    Hkv, G, B = rnd.choice([1, 2, 3]), rnd.choice([1, 2, 4]), rnd.choice([1, 2])
    L = rnd.choice([1, 33, 64, 100, 129, 200, 257, 384, 450])
    S = L if rnd.random() < 0.6 else rnd.choice([17, 64, 150, 300])
    family = rnd.choice(["plain", "mods", "document", "bias", "all", "all"])
    mask_kind = rnd.choice([_ffi.MASK_NONE, _ffi.MASK_CAUSAL, _ffi.MASK_SLIDING, _ffi.MASK_PREFIX_LM])
    if family == "all" and rnd.random() < 0.5:
        mask_kind = rnd.choice([_ffi.MASK_DOCUMENT, _ffi.MASK_DOCUMENT_CAUSAL])
    if mask_kind in (_ffi.MASK_SLIDING, _ffi.MASK_PREFIX_LM):
        S = L  # (as in the reference: these masks are defined for equal lengths)
    if family == "document":
        mask_kind = rnd.choice([_ffi.MASK_DOCUMENT, _ffi.MASK_DOCUMENT_CAUSAL])
    if mask_kind in (_ffi.MASK_DOCUMENT, _ffi.MASK_DOCUMENT_CAUSAL):
        S = L
    return dict(seed=seed, D=D, Hkv=Hkv, G=G, B=B, L=L, S=S, family=family, mask_kind=mask_kind,
                window=rnd.choice([1, 31, 70, 128]), prefix=rnd.choice([1, 32, 50, 129]), p=rnd.choice([0.05, 0.3, 0.7]),
                alibi=rnd.random() < 0.6, cap=rnd.choice([None, 4.0, 25.0]), ndocs=rnd.choice([1, 3, 7]),
                fp16=rnd.random() < 0.25)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(500, 580))
def test_random_dropout_cases(seed):
    """Seeded draws over what the dropout kernels cover (every mask kind; ALiBi, soft-cap, bias operands, alone and all
    together), ragged and unequal lengths, grouped heads, both element types: forward and gradients against autograd
    through the oracle with the same seed."""
    import oracle as O
    c = _random_dropout_case(seed)
    B, Hkv, Hq, L, S, D, p = c["B"], c["Hkv"], c["Hkv"] * c["G"], c["L"], c["S"], c["D"], c["p"]
    dt = torch.float16 if c["fp16"] else torch.bfloat16
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g).to(dt).to(DEV)  # noqa: E731
    q, k, v, dout = mk(B, Hq, L, D), mk(B, Hkv, S, D), mk(B, Hkv, S, D), mk(B, Hq, L, D)
    kw = dict(mask_kind=c["mask_kind"], window=c["window"], prefix=c["prefix"], dropout_p=p, dropout_seed=seed * 0x9E3779B97F4A7 + 1)
    attend = _attend(c["mask_kind"], L, S, c["window"], c["prefix"])
    bias, cap, operand = None, None, None
    fam = c["family"]
    if fam in ("mods", "all"):
        cap = c["cap"]
        if c["alibi"] or cap is None:
            rel = (torch.arange(S)[None, :] - torch.arange(L)[:, None]).float()
            bias = O.alibi_slopes(Hq)[:, None, None] * rel[None]
            kw["alibi_heads"] = Hq
        kw["softcap"] = cap or 0.0
    if c["mask_kind"] in (_ffi.MASK_DOCUMENT, _ffi.MASK_DOCUMENT_CAUSAL):
        ids = torch.sort(torch.randint(0, c["ndocs"], (B, L), generator=g), dim=1).values
        if seed % 3 == 0:
            ids = ids[:, torch.randperm(L, generator=g)]
        kw["doc_ids"] = ids.to(DEV)
        attend = (ids[:, :, None] == ids[:, None, :])[:, None]
        if c["mask_kind"] == _ffi.MASK_DOCUMENT_CAUSAL:
            attend = attend & (torch.arange(L)[None, :] <= torch.arange(L)[:, None])
    if fam in ("bias", "all"):
        operand = torch.randn(1, Hq, L, S, generator=g).to(dt).to(DEV)
        kw["biases"] = [(operand, 1)]
        bias = operand.float().cpu() if bias is None else bias + operand.float().cpu()
    lse = torch.empty(B, Hq, L, dtype=torch.float32, device=DEV)
    out = _ffi.attn_fwd(q, k, v, lse=lse, **kw)
    dq, dk, dv = _ffi.attn_bwd(q, k, v, out, lse, dout, **kw)
    torch.cuda.synchronize()
    qf, kf, vf = (t.float().cpu().requires_grad_(True) for t in (q, k, v))
    ref = OD.attention_dropout(qf, kf, vf, OD.keep_mask(kw["dropout_seed"], B, Hq, L, S, p), p, attend=attend, bias=bias,
                               softcap=cap)
    ref.backward(dout.float().cpu())
    # kept weights are scaled by 1 / (1 - p): the tolerances scale with it
    f = 1.0 / (1.0 - p)
    assert_parity(out.float() / f, ref / f, f"forward {c}")
    # With a single key the exact score gradient is 0 (dP / (1 - p) - Delta cancels), and what the kernels return is
    # the rounding of the bf16 forward result inside Delta times q or k: a few 1e-3 on every element, so such a case
    # is held to the max-abs bound alone.
    mean_tol = 2e-2 if S == 1 else 2e-3
    for what, got, want in (("dq", dq, qf.grad), ("dk", dk, kf.grad), ("dv", dv, vf.grad)):
        scale = max(1.0, want.abs().max().item()) * f
        assert_parity(got.float() / scale, want / scale, f"{what} {c}", mean_tol=mean_tol)


@pytest.mark.gpu
def test_dropout_fp16_forward_and_determinism():
    q, k, v, _ = _gpu_inputs(1, 2, 2, 192, 192, 128, seed=3)
    q, k, v = (t.to(torch.float16) for t in (q, k, v))
    a = _ffi.attn_fwd(q, k, v, mask_kind=_ffi.MASK_CAUSAL, dropout_p=0.2, dropout_seed=77)
    b = _ffi.attn_fwd(q, k, v, mask_kind=_ffi.MASK_CAUSAL, dropout_p=0.2, dropout_seed=77)
    c = _ffi.attn_fwd(q, k, v, mask_kind=_ffi.MASK_CAUSAL, dropout_p=0.2, dropout_seed=78)
    assert torch.equal(a, b) and not torch.equal(a, c)
    keep = OD.keep_mask(77, 1, 2, 192, 192, 0.2)
    ref = OD.attention_dropout(q.float().cpu(), k.float().cpu(), v.float().cpu(), keep, 0.2,
                               attend=_attend(_ffi.MASK_CAUSAL, 192, 192))
    assert_parity(a, ref, "fp16 forward with dropout")


@pytest.mark.gpu
def test_dropout_through_autograd_and_the_variant_switch():
    q, k, v, dout = _gpu_inputs(1, 4, 2, 160, 160, 64, seed=9)
    # default: the variant ignores dropout_p, as the reference does
    base = A.attention_pytorch_causal(q, k, v, enable_gqa=True)
    assert torch.equal(A.attention_pytorch_causal(q, k, v, dropout_p=0.5, enable_gqa=True), base)
    with A.honor_dropout():
        torch.manual_seed(11)
        a = A.attention_pytorch_causal(q, k, v, dropout_p=0.5, enable_gqa=True)
        torch.manual_seed(11)
        b = A.attention_pytorch_causal(q, k, v, dropout_p=0.5, enable_gqa=True)
        c = A.attention_pytorch_causal(q, k, v, dropout_p=0.5, enable_gqa=True)
        assert torch.equal(a, b) and not torch.equal(a, c) and not torch.equal(a, base)
        dense = lambda L, S: torch.zeros(4, L, S, device=DEV)  # noqa: E731  (a dense score_mod tensor: the bias path)
        torch.manual_seed(11)
        d = A.attention_pytorch_alibi(q, k, v, score_mod=dense, dropout_p=0.5, enable_gqa=True, is_causal=True)
        assert torch.equal(d, a)  # a zero bias and the same seed: the same weights are dropped
        e = A.attention_pytorch_alibi(q, k, v, score_mod=dense, dropout_p=0.5, enable_gqa=True, softcap=5.0)
        assert torch.isfinite(e).all() and not torch.equal(e, a)  # with a soft-cap too
    # autograd: the backward regenerates the forward's decisions from the seed
    qg, kg, vg = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    out = ops.dispatch(qg, kg, vg, mask_kind=_ffi.MASK_CAUSAL, dropout_p=0.3, dropout_seed=2024)
    out.backward(dout)
    keep = OD.keep_mask(2024, 1, 4, 160, 160, 0.3)
    qf, kf, vf = (t.float().cpu().requires_grad_(True) for t in (q, k, v))
    ref = OD.attention_dropout(qf, kf, vf, keep, 0.3, attend=_attend(_ffi.MASK_CAUSAL, 160, 160))
    ref.backward(dout.float().cpu())
    assert_parity(out, ref, "autograd forward with dropout")
    for what, got, want in (("dq", qg.grad, qf.grad), ("dk", kg.grad, kf.grad), ("dv", vg.grad, vf.grad)):
        scale = max(1.0, want.abs().max().item())
        assert_parity(got.float() / scale, want / scale, f"autograd {what} with dropout")


@pytest.mark.gpu
def test_dropout_rate_at_benchmark_size_through_a_ones_value():
    # with V = 1 every output element is (sum of kept weights) / (1 - p): its mean over rows is 1, its spread that of the
    # kept weight mass; keys attended uniformly (q = 0) make the weights 1 / S, so out = kept fraction / (1 - p)
    B, H, S, D = 1, 4, 4096, 128
    q = torch.zeros(B, H, S, D, dtype=torch.bfloat16, device=DEV)
    k = torch.randn(B, H, S, D, device=DEV).to(torch.bfloat16)
    v = torch.ones(B, H, S, D, dtype=torch.bfloat16, device=DEV)
    for p in (0.1, 0.5):
        out = _ffi.attn_fwd(q, k, v, dropout_p=p, dropout_seed=31337).float()
        assert (out[..., 0:1] - out).abs().max() < 1e-2           # every column of a row sees the same decisions
        frac = out[..., 0] * (1 - OD.effective_rate(p))             # kept fraction per row
        assert abs(frac.mean().item() - (1 - p)) < 2e-3
        sd = (p * (1 - p) / S) ** 0.5
        assert 0.7 * sd < frac.std().item() < 1.4 * sd + 2e-3       # binomial spread (plus bf16 rounding of the weights)
