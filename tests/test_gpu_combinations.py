"""Head dim 256 and feature combinations beyond the benchmark's (document mask + ALiBi / soft-cap, dense bias +
soft-cap, score_mod callables of the soft-cap signature), HIP kernels through the C ABI against the CPU oracle.
Tolerance: bf16 kernel against the fp32 oracle, max-abs 2e-2 and mean-abs 2e-3.

The reference's generated kernel takes any head dim up to 256 in one block (monkeypatch/fusion/_common.py:4) and
whatever composition of mask and score modification the eager function writes."""
import math

import pytest
import torch

import flashlight_amd.attention_variants as A
import oracle as O
from flashlight_amd import _ffi, ops
from oracle.attention import _softmax_attention, alibi_slopes
from tests.conftest import assert_parity

pytestmark = pytest.mark.gpu
DEV = "cuda"


def f32(*ts):
    return tuple(t.float().cpu() for t in ts)


def qkv(B, Hq, Hkv, S, D, Dv=None, seed=0, amp=1.0):
    g = torch.Generator().manual_seed(seed)
    shapes = [(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, Dv or D)]
    ts = [torch.randn(s, generator=g) for s in shapes]
    ts[0] = ts[0] * amp
    return tuple(t.to(torch.bfloat16).to(DEV) for t in ts)


@pytest.mark.parametrize("S", [1, 65, 300, 1024])
@pytest.mark.parametrize("Dv", [128, 256])
def test_head_dim_256_masks(S, Dv):
    q, k, v = qkv(2, 4, 2, S, 256, Dv, seed=S + Dv)
    qf, kf, vf = f32(q, k, v)
    assert_parity(A.attention_pytorch(q, k, v, enable_gqa=True), O.attention_vanilla(qf, kf, vf, enable_gqa=True), "vanilla")
    assert_parity(A.attention_pytorch_causal(q, k, v, enable_gqa=True), O.attention_causal(qf, kf, vf, enable_gqa=True),
                  "causal")
    assert_parity(A.attention_pytorch_sliding_window(q, k, v, window_size=70, enable_gqa=True),
                  O.attention_sliding_window(qf, kf, vf, window_size=70, enable_gqa=True), "sliding")
    assert_parity(A.attention_pytorch_prefix_lm(q, k, v, prefix_lengths=100, enable_gqa=True),
                  O.attention_prefix_lm(qf, kf, vf, prefix_lengths=100, enable_gqa=True), "prefix")


def test_head_dim_256_score_mods_and_documents():
    S = 700
    q, k, v = qkv(2, 4, 4, S, 256, 256, seed=5, amp=3.0)
    qf, kf, vf = f32(q, k, v)
    assert_parity(A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(4)),
                  O.attention_alibi(qf, kf, vf, score_mod=4), "alibi")
    assert_parity(A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(20.0)),
                  O.attention_softcapped(qf, kf, vf, score_mod=20.0), "softcap")
    assert_parity(A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(4), is_causal=True, softcap=15.0),
                  O.attention_alibi(qf, kf, vf, score_mod=4, is_causal=True, honor_causal=True, softcap=15.0),
                  "alibi+softcap+causal")
    g = torch.Generator().manual_seed(6)
    ids = torch.sort(torch.randint(0, 5, (2, S), generator=g), dim=1).values
    for causal in (False, True):
        assert_parity(A.attention_pytorch_document_mask(q, k, v, ids.to(DEV), is_causal=causal),
                      O.attention_document_mask(qf, kf, vf, ids, is_causal=causal), f"document causal={causal}")


def test_head_dim_256_row_statistics_come_from_the_first_slab():
    """Values wider than 128 columns go in slabs; lse depends on q and k only and is written once."""
    q, k, v = qkv(1, 2, 2, 200, 256, 256, seed=8)
    lse = torch.empty(1, 2, 200, dtype=torch.float32, device=DEV)
    _ffi.attn_fwd(q, k, v, mask_kind=_ffi.MASK_CAUSAL, lse=lse)
    qf, kf, _ = f32(q, k, v)
    s = torch.matmul(qf, kf.transpose(-1, -2)) / math.sqrt(256)
    s = s.masked_fill(torch.ones(200, 200, dtype=torch.bool).triu(1), float("-inf"))
    ref = torch.logsumexp(s, dim=-1) / math.log(2.0)  # the kernels keep row statistics in log2 units
    assert (lse.cpu() - ref).abs().max().item() < 2e-2


@pytest.mark.parametrize("D,Dv,S", [(512, 128, 1), (512, 512, 333), (320, 320, 200), (384, 64, 1024), (512, 256, 97)])
def test_head_dims_up_to_512(D, Dv, S):
    """Head dims above 256 run on the 512-wide instances (one wave per SIMD); widths in between are zero-padded.  The
    reference's generated kernel loops over the head dim there (monkeypatch/fusion/reduction_kernel_fusion.py:1102)."""
    q, k, v = qkv(2, 4, 2, S, D, Dv, seed=S + D + Dv)
    qf, kf, vf = f32(q, k, v)
    assert_parity(A.attention_pytorch(q, k, v, enable_gqa=True), O.attention_vanilla(qf, kf, vf, enable_gqa=True), "vanilla")
    assert_parity(A.attention_pytorch_causal(q, k, v, enable_gqa=True), O.attention_causal(qf, kf, vf, enable_gqa=True),
                  "causal")
    assert_parity(A.attention_pytorch_sliding_window(q, k, v, window_size=33, enable_gqa=True),
                  O.attention_sliding_window(qf, kf, vf, window_size=33, enable_gqa=True), "sliding")
    assert_parity(A.attention_pytorch_prefix_lm(q, k, v, prefix_lengths=50, enable_gqa=True),
                  O.attention_prefix_lm(qf, kf, vf, prefix_lengths=50, enable_gqa=True), "prefix")


def test_head_dim_512_score_mods_documents_and_fp16():
    S = 450
    q, k, v = qkv(2, 4, 4, S, 512, 256, seed=15, amp=3.0)
    qf, kf, vf = f32(q, k, v)
    assert_parity(A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(4)),
                  O.attention_alibi(qf, kf, vf, score_mod=4), "alibi")
    assert_parity(A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(20.0)),
                  O.attention_softcapped(qf, kf, vf, score_mod=20.0), "softcap")
    assert_parity(A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(4), is_causal=True, softcap=15.0),
                  O.attention_alibi(qf, kf, vf, score_mod=4, is_causal=True, honor_causal=True, softcap=15.0),
                  "alibi+softcap+causal")
    g = torch.Generator().manual_seed(16)
    ids = torch.sort(torch.randint(0, 5, (2, S), generator=g), dim=1).values
    for causal in (False, True):
        assert_parity(A.attention_pytorch_document_mask(q, k, v, ids.to(DEV), is_causal=causal),
                      O.attention_document_mask(qf, kf, vf, ids, is_causal=causal), f"document causal={causal}")
    h = tuple(t.to(torch.float16) for t in (q / 3.0, k, v))
    assert_parity(A.attention_pytorch_causal(*h), O.attention_causal(*f32(*h)), "fp16 causal")
    with pytest.raises(_ffi.FlashlightError, match="no kernel instance"):
        big = torch.zeros(1, 1, 8, 520, dtype=torch.bfloat16, device=DEV)
        A.attention_pytorch(big, big, big)


def _doc_alibi_oracle(qf, kf, vf, ids, nheads, cap, causal):
    """Eager fp32 composition: cap * tanh(q k^T s / cap) + slope_h (k - q), masked where the ids differ (or k > q)."""
    slopes = alibi_slopes(nheads).float().view(1, nheads, 1, 1)

    def masked(qi, ki):
        m = ids[:, qi.view(-1)].view(ids.size(0), 1, -1, 1) != ids[:, ki.view(-1)].view(ids.size(0), 1, 1, -1)
        return (m | (ki > qi)) if causal else m

    return _softmax_attention(qf, kf, vf, 1.0 / math.sqrt(qf.size(-1)), masked=masked, softcap=cap,
                              bias=lambda qi, ki: slopes * (ki - qi).float())


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("cap", [None, 12.0])
@pytest.mark.parametrize("causal", [False, True])
def test_document_mask_with_alibi_and_softcap(D, cap, causal):
    B, H, S = 2, 4, 600
    q, k, v = qkv(B, H, H, S, D, seed=D + 3, amp=3.0)
    g = torch.Generator().manual_seed(21)
    ids = torch.sort(torch.randint(0, 6, (B, S), generator=g), dim=1).values
    out = ops.dispatch(q, k, v, mask_kind=_ffi.MASK_DOCUMENT_CAUSAL if causal else _ffi.MASK_DOCUMENT, doc_ids=ids.to(DEV),
                       alibi_heads=H, softcap=cap or 0.0)
    assert_parity(out, _doc_alibi_oracle(*f32(q, k, v), ids, H, cap, causal), f"D={D} cap={cap} causal={causal}")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("cap", [None, 12.0])
@pytest.mark.parametrize("causal", [False, True])
def test_document_mask_with_dense_bias_and_gate(D, cap, causal):
    """Documents + a dense additive term per head (bf16, shared by the batch) + a row-broadcast fp32 term + the gate."""
    B, H, S = 2, 4, 520
    q, k, v = qkv(B, H, H, S, D, seed=D + 11, amp=2.0)
    g = torch.Generator().manual_seed(23)
    ids = torch.sort(torch.randint(0, 5, (B, S), generator=g), dim=1).values
    if causal:
        ids = ids[:, torch.randperm(S, generator=g)]  # ids in no order: the tile lists have holes
    dense = (torch.randn(1, H, S, S, generator=g) * 1.5).to(torch.bfloat16)
    row = torch.randn(B, 1, 1, S, generator=g)
    gate = torch.randn(B, H, S, D, generator=g).to(torch.bfloat16)
    out = ops.dispatch(q, k, v, mask_kind=_ffi.MASK_DOCUMENT_CAUSAL if causal else _ffi.MASK_DOCUMENT, doc_ids=ids.to(DEV),
                       softcap=cap or 0.0, biases=[(dense.to(DEV), B), (row.to(DEV), 1)], gate=gate.to(DEV))

    def masked(qi, ki):
        m = ids[:, qi.view(-1)].view(B, 1, -1, 1) != ids[:, ki.view(-1)].view(B, 1, 1, -1)
        return (m | (ki > qi)) if causal else m

    qf, kf, vf = f32(q, k, v)
    ref = _softmax_attention(qf, kf, vf, 1.0 / math.sqrt(D), masked=masked, softcap=cap,
                             bias=lambda qi, ki: (dense.float()[..., qi.view(-1), :], row))
    assert_parity(out, ref * torch.sigmoid(gate.float()), f"D={D} cap={cap} causal={causal}")


@pytest.mark.parametrize("D,Dv", [(32, 32), (64, 64), (128, 128), (256, 128), (512, 128), (64, 128), (32, 64), (96, 256)])
@pytest.mark.parametrize("kind", [_ffi.MASK_SLIDING, _ffi.MASK_DOCUMENT_CAUSAL])
@pytest.mark.parametrize("cap", [None, 12.0])
def test_all_score_modifications_together_at_every_head_dim(D, Dv, kind, cap):
    """The in-kernel ALiBi term, the soft-cap (or none), a dense bf16 operand, a row-broadcast fp32 operand and the gate
    under a sliding window or causal documents: at every compiled head dim, at the rectangular pairs (which go to the
    square instances for this) and at a padded one."""
    B, Hq, Hkv, S, window = 2, 4, 2, 290, 77
    q, k, v = qkv(B, Hq, Hkv, S, D, Dv, seed=D + Dv + kind, amp=2.0)
    g = torch.Generator().manual_seed(29)
    ids = torch.sort(torch.randint(0, 4, (B, S), generator=g), dim=1).values
    dense = (torch.randn(1, Hq, S, S, generator=g) * 1.5).to(torch.bfloat16)
    row = torch.randn(B, 1, 1, S, generator=g)
    gate = torch.randn(B, Hq, S, Dv, generator=g).to(torch.bfloat16)
    doc = kind == _ffi.MASK_DOCUMENT_CAUSAL
    out = ops.dispatch(q, k, v, mask_kind=kind, window=window, doc_ids=ids.to(DEV) if doc else None, alibi_heads=Hq,
                       softcap=cap or 0.0, biases=[(dense.to(DEV), B), (row.to(DEV), 1)], gate=gate.to(DEV))
    slopes = alibi_slopes(Hq).float().view(1, Hq, 1, 1)

    def masked(qi, ki):
        if doc:
            return (ids[:, qi.view(-1)].view(B, 1, -1, 1) != ids[:, ki.view(-1)].view(B, 1, 1, -1)) | (ki > qi)
        return (ki > qi) | (qi - ki > window)

    qf, kf, vf = f32(q, k, v)
    ref = _softmax_attention(qf, kf.repeat_interleave(Hq // Hkv, 1), vf.repeat_interleave(Hq // Hkv, 1), 1.0 / math.sqrt(D),
                             masked=masked, softcap=cap,
                             bias=lambda qi, ki: (slopes * (ki - qi).float(), dense.float()[..., qi.view(-1), :], row))
    assert_parity(out, ref * torch.sigmoid(gate.float()), f"D={D}/{Dv} kind={kind} cap={cap}")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("gqa", [False, True])
def test_dense_score_mod_with_softcap(D, gqa):
    """attention_pytorch_alibi(score_mod=<any callable>, softcap=...): cap first, then the dense tensor (alibi.py:26-30)."""
    B, Hq, Hkv, S = 2, 4, (2 if gqa else 4), 333
    q, k, v = qkv(B, Hq, Hkv, S, D, seed=D + 9, amp=4.0)
    g = torch.Generator().manual_seed(31)
    dense = torch.randn(Hq, S, S, generator=g) * 2.0

    out = A.attention_pytorch_alibi(q, k, v, score_mod=lambda L, S_: dense.to(DEV), enable_gqa=gqa, softcap=9.0, is_causal=True)
    ref = O.attention_alibi(*f32(q, k, v), score_mod=lambda L, S_: dense, enable_gqa=gqa, softcap=9.0, is_causal=True,
                            honor_causal=True)
    assert_parity(out, ref, f"D={D} gqa={gqa}")


def _eager_softcapped(qf, kf, vf, fn, causal=False):
    """softcap.py:40-53 in fp32 on the CPU: the callable is applied to the whole scaled score matrix."""
    s = torch.matmul(qf, kf.transpose(-1, -2)) / math.sqrt(qf.size(-1))
    s = fn(s, 0, 0, None, None)
    if causal:
        L, S = s.shape[-2:]
        s = s.masked_fill(torch.ones(L, S, dtype=torch.bool).triu(1), float("-inf"))
    return torch.matmul(torch.softmax(s, dim=-1), vf)


@pytest.mark.parametrize("D", [64, 128])
def test_score_mod_callables_of_the_softcap_signature(D):
    """softcap.py:49 calls score_mod(attn_weight, N, Hq, query, key) with any callable; the ones the kernel can apply
    in registers are recognised by tracing them."""
    B, H, S = 2, 4, 400
    q, k, v = qkv(B, H, H, S, D, seed=D + 40, amp=5.0)
    qf, kf, vf = f32(q, k, v)
    g = torch.Generator().manual_seed(41)
    rel = torch.randn(H, S, S, generator=g)

    def gym_softcap(score, b, h, q_idx, kv_idx):  # attn_gym.mods.generate_tanh_softcap(30, approx=False), as published
        return 30 * torch.tanh(score / 30)

    def other_spelling(score, b, h, q_idx, kv_idx):
        return torch.tanh(score * 0.125).mul(8.0)

    def temperature(score, b, h, q_idx, kv_idx):
        return score / 2.5

    def capped_then_shifted(score, b, h, q_idx, kv_idx):
        return 10.0 * torch.tanh(score / 10.0) + rel_dev - 3.0

    def scaled_cap(score, b, h, q_idx, kv_idx):  # post != 1 / pre
        return 6.0 * torch.tanh(0.5 * score)

    for fn in (gym_softcap, other_spelling, temperature, scaled_cap):
        assert_parity(A.attention_softcapped(q, k, v, score_mod=fn), _eager_softcapped(qf, kf, vf, fn), fn.__name__)
    rel_dev = rel.to(DEV)
    out = A.attention_softcapped(q, k, v, score_mod=capped_then_shifted, is_causal=True)
    rel_dev = rel
    assert_parity(out, _eager_softcapped(qf, kf, vf, capped_then_shifted, causal=True), "capped_then_shifted")


def test_head_dim_32_score_functions_and_dropout_run_on_the_64_wide_kernels():
    """Score functions other than the soft-cap and dropout are compiled from head dim 64 up; narrower calls are padded."""
    import oracle.dropout as OD
    q, k, v = qkv(2, 4, 4, 150, 32, seed=60, amp=3.0)
    qf, kf, vf = f32(q, k, v)
    relu = lambda s, b, h, qi, ki: torch.relu(s)  # noqa: E731
    assert_parity(A.attention_softcapped(q, k, v, score_mod=relu, is_causal=True),
                  _eager_softcapped(qf, kf, vf, relu, causal=True), "relu at head dim 32")
    out = ops.dispatch(q, k, v, mask_kind=_ffi.MASK_CAUSAL, dropout_p=0.25, dropout_seed=99)
    keep = OD.keep_mask(99, 2, 4, 150, 150, 0.25)
    causal = torch.arange(150)[None, :] <= torch.arange(150)[:, None]
    assert_parity(out, OD.attention_dropout(qf, kf, vf, keep, 0.25, attend=causal), "dropout at head dim 32")


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("fill", [-1e9, -30000.0, float("-inf")])
def test_additive_padding_mask_over_a_ragged_last_tile(D, dtype, fill):
    """Key padding written as an additive term (a large finite negative number, as model code does, or -inf) that covers
    the whole ragged last tile of every sequence: the softmax reference must not follow such a tile down (it once did
    when nothing had moved it yet, and scaled what was accumulated past the largest float: NaN)."""
    B, Hq, Hkv = 3, 4, 2
    for S, valid in ((100, (90, 37, 96)), (200, (150, 190, 64)), (333, (320, 100, 288))):
        q, k, v = (t.to(dtype) for t in qkv(B, Hq, Hkv, S, D, seed=S + D))
        pad = torch.zeros(B, 1, 1, S)
        for b, n in enumerate(valid):
            pad[b, ..., n:] = fill
        for operand in (pad, pad.to(dtype)):  # fp32, and the element type (fp16 turns -1e9 into -inf)
            out = ops.dispatch(q, k, v, biases=[(operand.to(DEV), 1)])
            qf, kf, vf = f32(q, k, v)
            ref = _softmax_attention(qf, kf.repeat_interleave(Hq // Hkv, 1), vf.repeat_interleave(Hq // Hkv, 1),
                                     1.0 / math.sqrt(D), bias=lambda qi, ki: operand.float())
            assert_parity(out, ref, f"D={D} S={S} {dtype} fill={fill} operand {operand.dtype}")
            # the same under the causal mask (the first tile of early rows is then the masked diagonal one)
            out = ops.dispatch(q, k, v, mask_kind=_ffi.MASK_CAUSAL, biases=[(operand.to(DEV), 1)])
            ref = _softmax_attention(qf, kf.repeat_interleave(Hq // Hkv, 1), vf.repeat_interleave(Hq // Hkv, 1),
                                     1.0 / math.sqrt(D), masked=lambda qi, ki: ki > qi, bias=lambda qi, ki: operand.float())
            assert_parity(out, ref, f"causal D={D} S={S} {dtype} fill={fill} operand {operand.dtype}")


def test_score_mod_the_kernel_cannot_apply_is_refused():
    q, k, v = qkv(1, 2, 2, 64, 64, seed=50)
    for fn in (lambda s, b, h, qi, ki: torch.exp(s),
               lambda s, b, h, qi, ki: torch.tanh(torch.tanh(s)),
               lambda s, b, h, qi, ki: s ** 4,
               lambda s, b, h, qi, ki: torch.sigmoid(s) * s):
        with pytest.raises(NotImplementedError):
            A.attention_softcapped(q, k, v, score_mod=fn)


@pytest.mark.parametrize("D,Dv", [(16, 16), (48, 48), (80, 80), (96, 96), (112, 64), (40, 100), (192, 192), (128, 256), (72, 160)])
def test_head_dims_between_the_compiled_ones(D, Dv):
    """Any head dim up to 256 (the reference's generated kernel takes them in one block, monkeypatch/fusion/_common.py:4):
    q, k and v are zero-padded to a compiled head dim and the result is cut back; the default scale is that of the
    unpadded head dim."""
    q, k, v = qkv(2, 4, 2, 260, D, Dv, seed=D + Dv)
    qf, kf, vf = f32(q, k, v)
    assert_parity(A.attention_pytorch(q, k, v, enable_gqa=True), O.attention_vanilla(qf, kf, vf, enable_gqa=True), "vanilla")
    assert_parity(A.attention_pytorch_causal(q, k, v, enable_gqa=True), O.attention_causal(qf, kf, vf, enable_gqa=True),
                  "causal")
    assert_parity(A.attention_pytorch_sliding_window(q, k, v, window_size=50, enable_gqa=True),
                  O.attention_sliding_window(qf, kf, vf, window_size=50, enable_gqa=True), "sliding")


def test_gradients_at_a_head_dim_between_the_compiled_ones():
    D = 96
    g = torch.Generator().manual_seed(96)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)  # noqa: E731
    q, k, v, dout = mk(2, 4, 150, D), mk(2, 2, 150, D), mk(2, 2, 150, D), mk(2, 4, 150, D)
    res = []
    for dev, dtype in ((DEV, torch.bfloat16), ("cpu", torch.float32)):
        ts = [t.detach().to(dev).to(dtype).requires_grad_(True) for t in (q, k, v)]
        fn = A.attention_pytorch_causal if dev == DEV else O.attention_causal
        out = fn(ts[0], ts[1], ts[2], enable_gqa=True)
        out.backward(dout.to(dev).to(out.dtype).reshape(out.shape))
        res.append([out.detach().reshape(2, 4, 150, D)] + [t.grad for t in ts])
    for what, got, want in zip(("out", "dq", "dk", "dv"), res[0], res[1]):
        scale = max(1.0, want.abs().max().item())
        assert_parity(got.float() / scale, want / scale, what)


def test_differential_attention_at_head_dim_48():
    g = torch.Generator().manual_seed(48)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)  # noqa: E731
    q, k, v = mk(2, 4, 200, 48), mk(2, 4, 200, 48), mk(2, 2, 200, 96)
    out = A.diffattn(q.to(DEV), k.to(DEV), v.to(DEV), lambda_full=0.5, is_causal=True)
    assert_parity(out, O.diff_attention(q.float(), k.float(), v.float(), lambda_full=0.5, is_causal=True), "diff d=48")
