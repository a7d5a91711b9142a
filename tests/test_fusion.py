"""`flashlight_amd.fusion`: eager attention captured by `torch.compile` is rewritten into one fused launch per region
(the reference reaches the same end by patching TorchInductor: `from monkeypatch.fusion import ...`,
tests/test_causal.py:14-17,33).  The CPU tests check what the rewrite recognises; the GPU tests check that the
rewritten function returns what the eager one returns."""
import functools
import math

import pytest
import torch

from flashlight_amd import _ffi, fusion
from tests import eager_idioms as E
from tests.conftest import assert_parity

BF = torch.bfloat16


def _rewrite(fn, *args):
    """Captures `fn` with Dynamo, rewrites the graph and returns (graph module, fused call nodes) without running it."""
    got = []

    class _Stop(Exception):
        pass

    def be(gm, example_inputs):
        fusion.fuse_attention(gm)
        got.append(gm)

        def run(*a):
            raise _Stop
        return run

    torch._dynamo.reset()
    with pytest.raises(_Stop):
        torch.compile(fn, backend=be, dynamic=False, fullgraph=True)(*args)
    assert len(got) == 1
    gm = got[0]
    return gm, [n for n in gm.graph.nodes if n.op == "call_function" and n.target is fusion.fused_attention]


def _leftover(gm):
    names = {fusion._name(n) for n in gm.graph.nodes}
    return names & {"matmul", "softmax", "where", "masked_fill", "tanh"}


def _qkv(N=2, Hq=4, Hkv=4, L=48, E=32, dev="cpu", seed=0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g).to(BF).to(dev)  # noqa: E731
    return mk(N, Hq, L, E), mk(N, Hkv, L, E), mk(N, Hkv, L, E)


def _ids(N, L, dev="cpu"):
    g = torch.Generator().manual_seed(3)
    return torch.randint(0, 4, (N, L), generator=g).sort(dim=1).values.to(dev)


# name -> (function of (q, k, v, *extra), extra-input builder, expected kwargs of the fused call, Hkv)
CASES = {
    "plain": (E.plain, None, dict(mask_kind=_ffi.MASK_NONE, gqa=False), 4),
    "plain gqa": (functools.partial(E.plain, enable_gqa=True), None, dict(mask_kind=_ffi.MASK_NONE, gqa=True), 2),
    "div by sqrt(d), .mT": (E.divided_by_sqrt_d, None, dict(mask_kind=_ffi.MASK_NONE), 4),
    "causal triu/where": (E.causal_triu, None, dict(mask_kind=_ffi.MASK_CAUSAL), 4),
    "causal gqa": (functools.partial(E.causal_triu, enable_gqa=True), None, dict(mask_kind=_ffi.MASK_CAUSAL, gqa=True), 2),
    "causal tril/keep": (E.causal_tril_keep, None, dict(mask_kind=_ffi.MASK_CAUSAL, scale=0.2), 4),
    "sliding": (functools.partial(E.sliding, window=5), None, dict(mask_kind=_ffi.MASK_SLIDING, window=5), 4),
    "sliding gqa": (functools.partial(E.sliding, window=17, enable_gqa=True), None,
                    dict(mask_kind=_ffi.MASK_SLIDING, window=17, gqa=True), 1),
    "sliding wider than L": (functools.partial(E.sliding, window=1000), None, dict(mask_kind=_ffi.MASK_CAUSAL), 4),
    "prefix": (functools.partial(E.prefix_lm, prefix=9), None, dict(mask_kind=_ffi.MASK_PREFIX_LM, prefix=9), 4),
    "prefix gqa": (functools.partial(E.prefix_lm, prefix=20, enable_gqa=True), None,
                   dict(mask_kind=_ffi.MASK_PREFIX_LM, prefix=20, gqa=True), 2),
    "alibi": (E.alibi, None, dict(alibi_heads=4, mask_kind=_ffi.MASK_NONE), 4),
    "alibi gqa": (functools.partial(E.alibi, enable_gqa=True), None, dict(alibi_heads=4, gqa=True), 2),
    "softcap": (functools.partial(E.softcap, cap=30.0), None, dict(softcap=30.0, mask_kind=_ffi.MASK_NONE), 4),
    "softcap causal": (functools.partial(E.softcap, cap=50.0, causal=True), None,
                       dict(softcap=50.0, mask_kind=_ffi.MASK_CAUSAL), 4),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_rewrite_recognises(name):
    fn, _, want, hkv = CASES[name]
    q, k, v = _qkv(Hkv=hkv)
    gm, calls = _rewrite(fn, q, k, v)
    assert len(calls) == 1 and not _leftover(gm), gm.graph
    kw = calls[0].kwargs
    for key, val in want.items():
        assert kw[key] == pytest.approx(val), (key, kw)
    if "scale" not in want:
        assert kw["scale"] == pytest.approx(32 ** -0.5)
    # nothing dense survives: no bias operand, no run-time mask
    assert list(calls[0].args[4]) == [] and list(calls[0].args[5]) == [] and calls[0].args[3] is None


# name -> (function, number of extra tensor inputs, expected score_fn kind and constants, other expected kwargs)
FN_CASES = {
    "relu": (E.relu_scores, 0, (_ffi.SCORE_CLAMP, (1.0, 0.0, 0.0, float("inf"))), dict(mask_kind=_ffi.MASK_NONE)),
    "relu causal": (functools.partial(E.relu_scores, causal=True), 0, (_ffi.SCORE_CLAMP, (1.0, 0.0, 0.0, float("inf"))),
                    dict(mask_kind=_ffi.MASK_CAUSAL)),
    "sigmoid + bias": (E.sigmoid_scores, 1, (_ffi.SCORE_SIGMOID, (0.5, -1.0, 8.0, 0.0)), dict(scale=0.25)),
    "clamp": (E.clamped_scores, 0, (_ffi.SCORE_CLAMP, (2.0, 0.0, -4.0, 6.0)), dict()),
    "polynomial": (E.squared_scores, 0, (_ffi.SCORE_POLY, (0.0, 1.0, -0.5, 0.0)), dict(scale=0.125)),
}


def _fn_extra(n, q, dev="cpu"):
    g = torch.Generator().manual_seed(5)
    return [torch.randn(q.size(1), q.size(2), q.size(2), generator=g).to(BF).to(dev) for _ in range(n)]


@pytest.mark.parametrize("name", sorted(FN_CASES))
def test_rewrite_recognises_score_functions(name):
    # a ReLU, sigmoid, clamp or polynomial between the first matmul and the softmax becomes the kernel's score_fn: the
    # chain is analysed like a caller's score_mod (the scale stays with the kernel's `scale` where it is a plain factor)
    fn, n_extra, (kind, consts), want = FN_CASES[name]
    q, k, v = _qkv()
    gm, calls = _rewrite(fn, q, k, v, *_fn_extra(n_extra, q))
    assert len(calls) == 1 and not _leftover(gm), gm.graph
    kw = calls[0].kwargs
    got_kind, got_consts = kw["score_fn"]
    scale = kw["scale"]
    assert got_kind == kind and kw["softcap"] == 0.0
    # the analysis may leave the scale inside the function (scale 1) or outside: compare the composition on a grid
    x = torch.linspace(-6, 6, 25, dtype=torch.float64)
    want_scale = want.get("scale", 32 ** -0.5)

    def apply(kind, c, z):
        if kind == _ffi.SCORE_SIGMOID:
            return c[2] * torch.sigmoid(c[0] * z + c[1]) + c[3]
        if kind == _ffi.SCORE_CLAMP:
            return torch.clamp(c[0] * z + c[1], min=c[2], max=c[3])
        return c[0] + c[1] * z + c[2] * z ** 2 + c[3] * z ** 3
    assert torch.allclose(apply(got_kind, got_consts, x * scale), apply(kind, consts, x * want_scale), atol=1e-9)
    if "mask_kind" in want:
        assert kw["mask_kind"] == want["mask_kind"]
    assert len(calls[0].args[4]) == n_extra and list(calls[0].args[5]) == []


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(FN_CASES))
def test_rewritten_score_functions_equal_eager_on_gpu(name):
    fn, n_extra, _, _ = FN_CASES[name]
    q, k, v = _qkv(N=2, Hq=4, Hkv=4, L=200, E=64, dev="cuda", seed=13)
    _check_on_gpu(fn, (q, k, v, *_fn_extra(n_extra, q, "cuda")), name)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("gqa", [False, True])
def test_rewrite_recognises_document_masks_by_probing(causal, gqa):
    q, k, v = _qkv(Hkv=2 if gqa else 4)
    ids = _ids(2, 48)
    gm, calls = _rewrite(functools.partial(E.documents, causal=causal, enable_gqa=gqa), q, k, v, ids)
    assert len(calls) == 1 and not _leftover(gm)
    assert calls[0].kwargs["mask_kind"] == (_ffi.MASK_DOCUMENT_CAUSAL if causal else _ffi.MASK_DOCUMENT)
    ids_node = calls[0].args[3]
    assert ids_node.op == "placeholder" and list(calls[0].args[4]) == [] and list(calls[0].args[5]) == []


def test_rewrite_keeps_what_it_cannot_name_as_dense_operands():
    q, k, v = _qkv()
    # constant mask without a closed form -> one constant additive operand
    gm, calls = _rewrite(E.checkerboard, q, k, v)
    assert len(calls) == 1 and not _leftover(gm)
    (b,) = calls[0].args[4]
    buf = getattr(gm, b.target)
    assert b.op == "get_attr" and buf.dtype == BF and tuple(buf.shape) == (48, 48)
    assert bool(torch.isinf(buf[0, 1])) and float(buf[0, 2]) == 0.0
    # run-time bias and run-time boolean mask stay graph inputs
    bias = torch.randn(2, 4, 48, 48)
    pad = torch.zeros(2, 48, dtype=torch.bool)
    gm, calls = _rewrite(E.learned_bias, q, k, v, bias, pad)
    assert len(calls) == 1 and not _leftover(gm)
    assert [n.op for n in calls[0].args[4]] == ["placeholder"] and len(calls[0].args[5]) == 1
    assert calls[0].kwargs["mask_kind"] == _ffi.MASK_NONE


def test_rewrite_differential_and_msa_row():
    q, k, _ = _qkv(Hq=8, Hkv=8)
    v = torch.randn(2, 4, 48, 64).to(BF)
    gm, calls = _rewrite(functools.partial(E.differential, lam=0.3), q, k, v)
    assert not _leftover(gm)
    assert len(calls) == 1 and calls[0].kwargs["diff_lambda"] == pytest.approx(0.3)
    assert calls[0].args[0].op == "placeholder" and calls[0].args[1].op == "placeholder"
    Q, K, V = (torch.randn(1, 3, 40, 2, 32).to(BF) for _ in range(3))
    mask, pair = torch.randn(1, 3, 1, 1, 40).to(BF), torch.randn(1, 1, 2, 40, 40).to(BF)
    gm, calls = _rewrite(lambda Q, K, V, m, p: E.msa_row(Q, K, V, [m, p]), Q, K, V, mask, pair)
    assert len(calls) == 1 and not _leftover(gm) and len(calls[0].args[4]) == 2


def test_rewrite_maps_training_mode_dropout_to_the_kernel():
    q, k, v = _qkv(E=64)
    gm, calls = _rewrite(E.causal_with_dropout, q, k, v)
    assert len(calls) == 1 and not _leftover(gm) and "dropout" not in {fusion._name(n) for n in gm.graph.nodes}
    assert calls[0].kwargs["dropout_p"] == 0.1 and calls[0].kwargs["mask_kind"] == _ffi.MASK_CAUSAL
    # evaluation mode: the dropout is the identity and leaves no trace
    gm, calls = _rewrite(functools.partial(E.causal_with_dropout, training=False), q, k, v)
    assert len(calls) == 1 and not calls[0].kwargs.get("dropout_p") and not _leftover(gm)
    gm, calls = _rewrite(E.learned_bias_with_dropout, q, k, v, torch.randn(4, 48, 48))
    assert len(calls) == 1 and calls[0].kwargs["dropout_p"] == 0.2 and len(calls[0].args[4]) == 1
    gm, calls = _rewrite(E.documents_with_dropout, q, k, v, _ids(2, 48))
    assert len(calls) == 1 and calls[0].kwargs["dropout_p"] == 0.1 and calls[0].kwargs["mask_kind"] == _ffi.MASK_DOCUMENT
    # outside what the dropout kernels cover the region stays eager: head dims above 128, score functions
    q256, k256, v256 = _qkv(E=256)
    gm, calls = _rewrite(E.causal_with_dropout, q256, k256, v256)
    assert calls == [] and "dropout" in {fusion._name(n) for n in gm.graph.nodes}
    q32, k32, v32 = _qkv(E=32)  # (head dim 32 is padded to 64 at run time)
    gm, calls = _rewrite(E.causal_with_dropout, q32, k32, v32)
    assert len(calls) == 1 and calls[0].kwargs["dropout_p"] == 0.1
    # a fill written as a one-element constant tensor is a fill like any number
    def tensor_fill(q, k, v):
        future = torch.ones(q.size(-2), k.size(-2), dtype=torch.bool).triu(1)
        s = torch.where(future, torch.tensor(float("-inf")), q @ k.transpose(-2, -1) * 0.125)
        s = s.masked_fill(future, torch.full((), -1e10))
        return torch.softmax(s, dim=-1) @ v
    gm, calls = _rewrite(tensor_fill, q, k, v)
    assert len(calls) == 1 and not _leftover(gm) and calls[0].kwargs["mask_kind"] == _ffi.MASK_CAUSAL

    def capped_bias_dropout(q, k, v, b):
        w = torch.softmax(20.0 * torch.tanh(q @ k.transpose(-2, -1) * 0.125 / 20.0) + b, dim=-1)
        return torch.nn.functional.dropout(w, 0.1) @ v
    gm, calls = _rewrite(capped_bias_dropout, q, k, v, torch.randn(4, 48, 48))
    assert len(calls) == 1 and calls[0].kwargs["dropout_p"] == 0.1 and calls[0].kwargs["softcap"] == 20.0

    def relu_dropout(q, k, v):  # score functions have no dropout kernels: left eager
        return torch.nn.functional.dropout(torch.softmax(torch.relu(q @ k.transpose(-2, -1) * 0.125), dim=-1), 0.1) @ v
    gm, calls = _rewrite(relu_dropout, q, k, v)
    assert calls == []


def _decoder_mask(B, L, dtype, dev="cpu", pad=(5, 0)):
    """[B, 1, L, L]: causal, and the first pad[b] keys of batch entry b padded (left padding), as the dtype's minimum."""
    m = torch.zeros(B, 1, L, L, dtype=dtype, device=dev)
    m.masked_fill_(torch.ones(L, L, dtype=torch.bool, device=dev).triu(1), torch.finfo(dtype).min)
    for b, n in enumerate(pad[:B]):
        m[b, :, :, :n] = torch.finfo(dtype).min
    return m


def test_rewrite_recognises_decoder_layer_attention_with_repeated_heads():
    q, k, v = _qkv(Hq=8, Hkv=2, E=64)
    mask = _decoder_mask(2, 48, BF)
    for fn in (E.decoder_layer_attention, E.decoder_layer_attention_softcapped):
        gm, calls = _rewrite(fn, q, k, v, mask)
        names = {fusion._name(n) for n in gm.graph.nodes}
        assert len(calls) == 1 and not _leftover(gm) and not names & {"expand", "reshape", "repeat_interleave"}, names
        # key and value reach the kernel with their own two heads
        assert fusion._val(calls[0].args[1]).size(1) == 2 and fusion._val(calls[0].args[2]).size(1) == 2
        assert len(calls[0].args[4]) == 1  # the additive mask, as a run-time bias operand
    assert calls[0].kwargs["softcap"] == 50.0
    # heads repeated in another order (the whole block of heads tiled) are not grouped-query attention: kept as they are
    def tiled(q, k, v):
        kk, vv = k.repeat(1, 4, 1, 1), v.repeat(1, 4, 1, 1)
        return torch.softmax(q @ kk.transpose(-2, -1) * 0.125, dim=-1) @ vv
    gm, calls = _rewrite(tiled, q, k, v)
    assert len(calls) == 1 and fusion._val(calls[0].args[1]).size(1) == 8


def test_rewrite_maps_scaled_dot_product_attention_calls():
    import torch.nn.functional as F
    q, k, v = _qkv(Hq=8, Hkv=2, E=64)
    keep, add = torch.rand(2, 1, 48, 48) > 0.2, torch.randn(2, 8, 48, 48)
    gm, calls = _rewrite(lambda q, k, v: F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True), q, k, v)
    assert len(calls) == 1 and calls[0].kwargs["mask_kind"] == _ffi.MASK_CAUSAL and calls[0].kwargs["scale"] == 0.125
    assert "scaled_dot_product_attention" not in {fusion._name(n) for n in gm.graph.nodes}
    # a boolean mask is True where a key takes part; heads repeated by the caller are grouped again
    gm, calls = _rewrite(lambda q, k, v, m: F.scaled_dot_product_attention(q, k.repeat_interleave(4, 1), v.repeat_interleave(4, 1),
                                                                        attn_mask=m), q, k, v, keep)
    assert len(calls) == 1 and calls[0].kwargs["mask_invert"] == (True,) and fusion._val(calls[0].args[1]).size(1) == 2
    # a float mask is a bias; dropout_p and scale carry over
    gm, calls = _rewrite(lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m, dropout_p=0.1, scale=0.2,
                                                                        enable_gqa=True), q, k, v, add)
    assert len(calls) == 1 and len(calls[0].args[4]) == 1 and calls[0].kwargs["dropout_p"] == 0.1 and calls[0].kwargs["scale"] == 0.2
    # a constant lower-triangular mask is the causal mask
    gm, calls = _rewrite(lambda q, k, v: F.scaled_dot_product_attention(q, k, v, enable_gqa=True,
                                                                     attn_mask=torch.ones(48, 48, dtype=torch.bool).tril()), q, k, v)
    assert len(calls) == 1 and calls[0].kwargs["mask_kind"] == _ffi.MASK_CAUSAL and not calls[0].args[4] and not calls[0].args[5]
    # operands without a head axis, [N, L, E], are one head
    q3 = torch.randn(3, 48, 64, dtype=BF)
    gm, calls = _rewrite(lambda q, m: F.scaled_dot_product_attention(q, q, q, attn_mask=m), q3, torch.randn(3, 48, 48))
    assert len(calls) == 1 and len(calls[0].args[4]) == 1
    # left alone: head dims without a kernel, dropout beyond head dim 128
    big = torch.randn(1, 2, 16, 640, dtype=BF)
    gm, calls = _rewrite(lambda q: F.scaled_dot_product_attention(q, q, q), big)
    assert calls == []
    wide = torch.randn(1, 2, 16, 256, dtype=BF)
    gm, calls = _rewrite(lambda q: F.scaled_dot_product_attention(q, q, q, dropout_p=0.1), wide)
    assert calls == []
    gm, calls = _rewrite(lambda q: F.scaled_dot_product_attention(q, q, q), wide)
    assert len(calls) == 1


def test_rewrite_follows_casts_of_the_weights():
    """Model code casts the fp32 softmax back in several spellings (`.to(dtype)`, `.type(dtype)`, `.type_as(v)`,
    `.bfloat16()`): all are passed through on the way to the second matmul."""
    q, k, v = _qkv()
    for cast in (lambda w, v: w.to(v.dtype), lambda w, v: w.type(v.dtype), lambda w, v: w.type_as(v), lambda w, v: w.bfloat16()):
        fn = lambda q, k, v: cast(torch.softmax((q @ k.transpose(-2, -1) * 0.1).float(), dim=-1), v) @ v
        gm, calls = _rewrite(fn, q, k, v)
        assert len(calls) == 1 and "softmax" not in _leftover(gm)


def test_rewrite_takes_16_bit_operands_that_the_region_upcast():
    """GPT-J / GPT-Neo multiply in fp32: `query.to(torch.float32) @ key.to(torch.float32).transpose(-1, -2)`.  The kernel
    gets the 16-bit tensors themselves (exact products, fp32 accumulation either way); a region whose result was fp32
    keeps that type through a cast behind the fused node."""
    q, k, v = _qkv()

    def gptj(q, k, v):
        w = torch.softmax(q.to(torch.float32) @ k.to(torch.float32).transpose(-1, -2) / 8.0, dim=-1)
        return w.to(v.dtype) @ v

    gm, calls = _rewrite(gptj, q, k, v)
    assert len(calls) == 1 and all(fusion._val(a).dtype == BF for a in calls[0].args[:3])
    assert not any(fusion._name(n) == "to" for n in calls[0].users)

    def all_fp32(q, k, v):
        return torch.softmax(q.float() @ k.float().transpose(-1, -2) / 8.0, dim=-1) @ v.float()

    gm, calls = _rewrite(all_fp32, q, k, v)
    assert len(calls) == 1 and all(fusion._val(a).dtype == BF for a in calls[0].args[:3])
    (cast,) = calls[0].users
    assert fusion._name(cast) == "to" and cast.args[1] == torch.float32


def test_rewrite_takes_attention_spelled_with_einsum():
    """einsum calls that are batched matrix products become permute / matmul nodes first, so the matcher sees them; an
    einsum of another kind stays."""
    q, k, v = _qkv(Hq=4, Hkv=4)
    keep = torch.rand(2, 1, 48, 48) > 0.2
    gm, calls = _rewrite(E.einsum_attention, q, k, v, keep)
    assert len(calls) == 1 and "einsum" not in {fusion._name(n) for n in gm.graph.nodes}
    qs, ks, vs = (t.transpose(1, 2).contiguous() for t in (q, k, v))   # [N, L, H, E]
    gm, calls = _rewrite(E.einsum_attention_seq_major, qs, ks, vs)
    assert len(calls) == 1 and calls[0].kwargs["mask_kind"] == _ffi.MASK_CAUSAL
    assert tuple(fusion._val(calls[0].args[0]).shape) == tuple(q.shape)   # handed over as [N, H, L, E] views
    # an outer product and a trace are not matrix products of this kind
    gm, calls = _rewrite(lambda a, b: torch.einsum("bhid,bhjd->bhijd", a, b).sum(-1), q, k)
    assert calls == [] and "einsum" in {fusion._name(n) for n in gm.graph.nodes}


def test_rewrite_reads_constant_additive_masks_as_positional_masks():
    """Model code that gets no padding mask builds its causal (or sliding-window) mask as a constant additive tensor, zeros
    and the dtype's most negative number: it becomes the kernel's positional mask, not a dense bias operand."""
    q, k, v = _qkv()
    L = q.size(2)

    def causal_additive(q, k, v):
        mask = torch.full((L, L), torch.finfo(q.dtype).min, dtype=q.dtype).triu(1)[None, None]
        return torch.softmax(q @ k.transpose(-2, -1) * 0.125 + mask, dim=-1) @ v

    gm, calls = _rewrite(causal_additive, q, k, v)
    assert len(calls) == 1 and calls[0].kwargs["mask_kind"] == _ffi.MASK_CAUSAL and not calls[0].args[4]

    def window_additive(q, k, v):
        i = torch.arange(L)
        out = (i[None, :] > i[:, None]) | (i[:, None] - i[None, :] > 7)
        mask = torch.zeros(L, L).masked_fill(out, float("-inf"))
        return torch.softmax(q @ k.transpose(-2, -1) * 0.125 + mask, dim=-1) @ v

    gm, calls = _rewrite(window_additive, q, k, v)
    assert len(calls) == 1 and calls[0].kwargs["mask_kind"] == _ffi.MASK_SLIDING and calls[0].kwargs["window"] == 7
    # a constant bias with other values stays a dense operand
    gm, calls = _rewrite(lambda q, k, v: torch.softmax(q @ k.transpose(-2, -1) * 0.125 + torch.ones(L, L).tril() * -3.0, dim=-1) @ v, q, k, v)
    assert len(calls) == 1 and calls[0].kwargs["mask_kind"] == _ffi.MASK_NONE and len(calls[0].args[4]) == 1


def test_rewrite_leaves_other_graphs_alone():
    q, k, v = _qkv()
    gm, calls = _rewrite(E.returns_weights, q, k, v)
    assert calls == [] and _leftover(gm) >= {"matmul", "softmax"}
    gm, calls = _rewrite(lambda a, b: torch.softmax(a @ b, dim=-1), q, k.transpose(-2, -1))
    assert calls == []
    # softmax over the query axis is not attention
    gm, calls = _rewrite(lambda q, k, v: torch.softmax(q @ k.transpose(-2, -1), dim=-2) @ v, q, k, v)
    assert calls == []
    # a bias added before the scale cannot be expressed
    gm, calls = _rewrite(lambda q, k, v, b: torch.softmax((q @ k.transpose(-2, -1) + b) * 0.1, dim=-1) @ v, q, k, v,
                         torch.randn(48, 48))
    assert calls == []


def test_rewritten_function_fails_loudly_without_a_gpu():
    q, k, v = _qkv()
    torch._dynamo.reset()
    with pytest.raises(NotImplementedError, match="no CPU path"):
        torch.compile(E.causal_triu, backend=fusion.backend, dynamic=False)(q, k, v)
    torch._dynamo.reset()
    with pytest.raises(NotImplementedError, match="no CPU path"):  # registered under a name as well
        torch.compile(E.plain, backend="flashlight_amd", dynamic=False)(q, k, v)


def test_mask_classifier_closed_forms():
    L = 37
    q, k = torch.arange(L).view(L, 1), torch.arange(L).view(1, L)
    C = fusion._classify_constant_mask
    assert C(torch.zeros(L, L, dtype=torch.bool), L, L) == (_ffi.MASK_NONE, 0, 0)
    assert C((k > q), L, L) == (_ffi.MASK_CAUSAL, 0, 0)
    assert C((k > q).expand(3, 2, L, L), L, L) == (_ffi.MASK_CAUSAL, 0, 0)
    for w in (0, 1, 7, 35):
        assert C((q < k) | (q - k > w), L, L) == (_ffi.MASK_SLIDING, w, 0)
    assert C((q < k) | (q - k > 36), L, L) == (_ffi.MASK_CAUSAL, 0, 0)          # the window reaches every key
    for p in (2, 9, 36):
        assert C(k > torch.clamp(q, min=p - 1), L, L) == (_ffi.MASK_PREFIX_LM, 0, p)
    assert C(k > torch.clamp(q, min=L - 1), L, L) == (_ffi.MASK_NONE, 0, 0)      # prefix covers everything
    assert C((q + k) % 2 == 1, L, L) is None
    assert C((k >= q), L, L) is None                                             # strictly-lower: row 0 attends nothing
    per_batch = torch.stack([(k > q), (k > q + 1)])
    assert C(per_batch, L, L) is None
    # rectangular scores: causal is defined (upper-left aligned), the window forms are not
    assert C(torch.arange(50).view(1, 50) > q, L, 50) == (_ffi.MASK_CAUSAL, 0, 0)


# ---- on the GPU: rewritten == eager ------------------------------------------------------------------------------------------

def _check_on_gpu(fn, args, what):
    torch._dynamo.reset()
    got = torch.compile(fn, backend=fusion.backend, dynamic=False, fullgraph=True)(*args)
    want = fn(*[a.float() if isinstance(a, torch.Tensor) and a.is_floating_point() else
                [x.float() for x in a] if isinstance(a, list) else a for a in args])
    assert got.shape == want.shape and got.dtype == BF, what
    assert_parity(got, want, what)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_rewritten_equals_eager_on_gpu(name):
    fn, _, _, hkv = CASES[name]
    q, k, v = _qkv(N=2, Hq=4, Hkv=hkv, L=200, E=64, dev="cuda", seed=11)
    _check_on_gpu(fn, (q, k, v), name)


@pytest.mark.gpu
def test_rewritten_dense_document_differential_and_msa_on_gpu():
    dev = "cuda"
    q, k, v = _qkv(N=2, Hq=4, Hkv=4, L=136, E=64, dev=dev, seed=12)
    _check_on_gpu(E.checkerboard, (q, k, v), "checkerboard")
    g = torch.Generator().manual_seed(5)
    bias = torch.randn(2, 4, 136, 136, generator=g).to(dev)
    pad = torch.zeros(2, 136, dtype=torch.bool)
    pad[0, 100:] = True
    _check_on_gpu(E.learned_bias, (q, k, v, bias, pad.to(dev)), "bias + padding mask")
    for causal in (False, True):
        for gqa in (False, True):
            qq, kk, vv = _qkv(N=2, Hq=4, Hkv=2 if gqa else 4, L=136, E=64, dev=dev, seed=13)
            _check_on_gpu(functools.partial(E.documents, causal=causal, enable_gqa=gqa), (qq, kk, vv, _ids(2, 136, dev)),
                          f"documents causal={causal} gqa={gqa}")
    qd, kd, _ = _qkv(N=2, Hq=8, Hkv=8, L=136, E=64, dev=dev, seed=14)
    vd = torch.randn(2, 4, 136, 128, generator=g).to(BF).to(dev)
    _check_on_gpu(functools.partial(E.differential, lam=0.3), (qd, kd, vd), "differential")
    Q, K, V = (torch.randn(1, 3, 104, 2, 32, generator=g).to(BF).to(dev) for _ in range(3))
    mask, pair = torch.randn(1, 3, 1, 1, 104, generator=g).to(BF).to(dev), torch.randn(1, 1, 2, 104, 104, generator=g).to(BF).to(dev)
    _check_on_gpu(lambda Q, K, V, m, p: E.msa_row(Q, K, V, [m, p]), (Q, K, V, mask, pair), "msa row")


@pytest.mark.gpu
def test_rewritten_dropout_regions_on_gpu():
    """The kernel's random stream is not torch's, so the rewritten function is compared with the kernel called directly
    for the same seed (itself checked against the oracle in tests/test_dropout.py), and with the eager function through
    what does not depend on the stream: the kept fraction, and p = 0 in evaluation mode."""
    from flashlight_amd import ops
    q, k, v = _qkv(N=2, Hq=4, Hkv=4, L=300, E=64, dev="cuda", seed=21)
    torch._dynamo.reset()
    fn = torch.compile(E.causal_with_dropout, backend=fusion.backend, dynamic=False, fullgraph=True)
    torch.manual_seed(5)
    a = fn(q, k, v)
    torch.manual_seed(5)
    b = fn(q, k, v)
    c = fn(q, k, v)
    torch.manual_seed(5)
    direct = ops.dispatch(q, k, v, mask_kind=_ffi.MASK_CAUSAL, dropout_p=0.1)
    assert torch.equal(a, b) and not torch.equal(a, c) and torch.equal(a, direct)
    # with value = 1 every output element is (kept weight mass) / (1 - p): mean 1 over rows with many keys
    ones = torch.ones_like(v)
    mass = fn(q * 0, k, ones).float()[:, :, 150:, 0]  # uniform weights over >= 151 keys
    assert abs(mass.mean().item() - 1.0) < 0.01 and 0.02 < mass.std().item() < 0.06
    torch._dynamo.reset()
    ev = torch.compile(functools.partial(E.causal_with_dropout, training=False), backend=fusion.backend, dynamic=False,
                       fullgraph=True)(q, k, v)
    assert_parity(ev, E.causal_with_dropout(q.float(), k.float(), v.float(), training=False), "evaluation mode")
    # gradients flow through the rewritten region (the backward regenerates the forward's decisions)
    qg = q.detach().clone().requires_grad_(True)
    torch.manual_seed(9)
    fn(qg, k, v).float().sum().backward()
    q2 = q.detach().clone().requires_grad_(True)
    torch.manual_seed(9)
    ops.dispatch(q2, k, v, mask_kind=_ffi.MASK_CAUSAL, dropout_p=0.1).float().sum().backward()
    assert torch.equal(qg.grad, q2.grad) and qg.grad.abs().max().item() > 0
    # documents and a learned bias
    ids = _ids(2, 300, "cuda")
    torch._dynamo.reset()
    fd = torch.compile(E.documents_with_dropout, backend=fusion.backend, dynamic=False, fullgraph=True)
    torch.manual_seed(3)
    x = fd(q, k, v, ids)
    torch.manual_seed(3)
    y = ops.dispatch(q, k, v, mask_kind=_ffi.MASK_DOCUMENT, doc_ids=ids, dropout_p=0.1)
    assert torch.equal(x, y)
    bias = torch.randn(4, 300, 300, device="cuda")
    torch._dynamo.reset()
    fb = torch.compile(E.learned_bias_with_dropout, backend=fusion.backend, dynamic=False, fullgraph=True)
    torch.manual_seed(4)
    x = fb(q, k, v, bias)
    torch.manual_seed(4)
    y = ops.dispatch(q, k, v, scale=0.125, biases=[(bias.unsqueeze(0), 1)], dropout_p=0.2)
    assert torch.equal(x, y)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rewritten_decoder_layer_attention_on_gpu(dtype):
    g = torch.Generator().manual_seed(77)
    B, Hq, Hkv, L, D = 2, 8, 2, 230, 64
    q, k, v = (torch.randn(B, h, L, D, generator=g).to(dtype).to("cuda") for h in (Hq, Hkv, Hkv))
    mask = _decoder_mask(B, L, dtype, "cuda", pad=(37, 0))
    for fn in (E.decoder_layer_attention, E.decoder_layer_attention_softcapped):
        torch._dynamo.reset()
        got = torch.compile(fn, backend=fusion.backend, dynamic=False, fullgraph=True)(q, k, v, mask)
        want = fn(q.float(), k.float(), v.float(), mask.float())
        assert got.shape == want.shape and got.dtype == dtype and torch.isfinite(got).all()
        # the first 37 query positions of batch entry 0 are padding themselves: every key they may see is padded, eager
        # averages over all keys there (the fills are equal) and the kernels return zeros; such rows are not compared
        rows = slice(37, None)
        a, b = (x if x.size(1) == L else x.transpose(1, 2) for x in (got, want))  # [B, L, H, E] either way
        assert_parity(a[0, rows], b[0, rows], fn.__name__ + ", padded entry")
        assert_parity(a[1], b[1], fn.__name__ + ", full entry")
    # training mode: the kernel's dropout, reproducible from torch's seed
    import functools
    torch._dynamo.reset()
    tr = torch.compile(functools.partial(E.decoder_layer_attention, dropout=0.1, training=True), backend=fusion.backend,
                       dynamic=False, fullgraph=True)
    torch.manual_seed(3)
    a = tr(q, k, v, mask)
    torch.manual_seed(3)
    b = tr(q, k, v, mask)
    assert torch.equal(a, b) and torch.isfinite(a).all() and not torch.equal(a, got)


@pytest.mark.gpu
def test_rewritten_scaled_dot_product_attention_on_gpu():
    import torch.nn.functional as F
    g = torch.Generator().manual_seed(91)
    B, Hq, Hkv, L, S, D = 2, 8, 2, 200, 264, 128
    q = torch.randn(B, Hq, L, D, generator=g).to(BF).to("cuda")
    k, v = (torch.randn(B, Hkv, S, D, generator=g).to(BF).to("cuda") for _ in range(2))
    keep = (torch.rand(B, 1, L, S, generator=g) > 0.3).to("cuda")
    keep[..., 0] = True
    add = torch.randn(1, Hq, L, S, generator=g).to("cuda")
    cases = {
        "plain gqa": (lambda q, k, v: F.scaled_dot_product_attention(q, k, v, enable_gqa=True), ()),
        "causal, unequal lengths": (lambda q, k, v: F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True), ()),
        "boolean mask": (lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m, enable_gqa=True), (keep,)),
        "float mask, scale": (lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m, scale=0.05, enable_gqa=True), (add,)),
    }
    for name, (fn, extra) in cases.items():
        torch._dynamo.reset()
        got = torch.compile(fn, backend=fusion.backend, dynamic=False, fullgraph=True)(q, k, v, *extra)
        want = fn(q.float().cpu(), k.float().cpu(), v.float().cpu(), *(e.cpu() for e in extra))
        assert_parity(got, want, name)
    # [N, L, E] operands (no head axis) with a mask / bias that has a batch axis of its own, as a call and spelled out
    q3, k3, v3 = q[:, 0], k[:, 0], v[:, 0]
    keep3, add3 = keep[:, 0], torch.randn(B, L, S, generator=g).to("cuda")
    cases3 = {
        "3-D, boolean mask": (lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m), keep3),
        "3-D, float mask": (lambda q, k, v, m: F.scaled_dot_product_attention(q, k, v, attn_mask=m), add3),
        "3-D, spelled out": (lambda q, k, v, m: torch.softmax(q @ k.transpose(-2, -1) * 0.08 + m, dim=-1) @ v, add3),
    }
    for name, (fn, m) in cases3.items():
        torch._dynamo.reset()
        got = torch.compile(fn, backend=fusion.backend, dynamic=False, fullgraph=True)(q3, k3, v3, m)
        assert got.shape == (B, L, D)
        assert_parity(got, fn(q3.float().cpu(), k3.float().cpu(), v3.float().cpu(), m.cpu()), name)


@pytest.mark.gpu
def test_a_fully_masked_row_comes_out_as_zeros():
    """A row whose keys a run-time mask all removes: eager PyTorch averages the values uniformly under a finite fill
    (every score equals the fill) and returns NaN under -inf; the rewritten graph treats any fill <= -1e9 as "not
    attended" and returns zeros for such a row, like every entry of the package.  Rows with a key left are unaffected."""
    dev = "cuda"
    q, k, v = _qkv(N=1, Hq=2, Hkv=2, L=72, E=64, dev=dev, seed=21)
    bias = torch.zeros(1, 2, 72, 72, device=dev)
    pad = torch.ones(1, 72, dtype=torch.bool, device=dev)   # every key padded away: all rows fully masked
    torch._dynamo.reset()
    got = torch.compile(E.learned_bias, backend=fusion.backend, dynamic=False, fullgraph=True)(q, k, v, bias, pad)
    assert torch.count_nonzero(got).item() == 0
    pad[0, :5] = False                                         # five keys left: ordinary attention over them
    torch._dynamo.reset()
    got = torch.compile(E.learned_bias, backend=fusion.backend, dynamic=False, fullgraph=True)(q, k, v, bias, pad)
    assert_parity(got, E.learned_bias(q.float(), k.float(), v.float(), bias, pad), "five keys left")


def test_rewrite_takes_multi_head_attention_modules():
    """torch.nn.MultiheadAttention calls torch.nn.functional.multi_head_attention_forward, which Dynamo keeps as one
    node: the rewrite replaces that node when no weights are returned, and leaves it alone otherwise."""
    import torch.nn as nn
    x = torch.randn(2, 40, 128, dtype=BF)
    pad = torch.zeros(2, 40, dtype=torch.bool)

    def targets(mod, *args, **kwargs):
        got = []

        def be(gm, example_inputs):
            fusion.fuse_attention(gm)
            got.extend(n.target for n in gm.graph.nodes if n.op == "call_function")

            def run(*a):
                raise _Done
            return run

        class _Done(Exception):
            pass

        torch._dynamo.reset()
        with pytest.raises(_Done):
            torch.compile(mod, backend=be, dynamic=False)(*args, **kwargs)
        return got

    mha = nn.MultiheadAttention(128, 4, batch_first=True).to(BF).train()
    got = targets(mha, x, x, x, need_weights=False, key_padding_mask=pad)
    assert fusion.fused_multi_head_attention in got and torch.nn.functional.multi_head_attention_forward not in got
    got = targets(mha, x, x, x, need_weights=True)
    assert fusion.fused_multi_head_attention not in got and torch.nn.functional.multi_head_attention_forward in got
    layer = nn.TransformerEncoderLayer(128, 4, 256, dropout=0.1, batch_first=True).to(BF).train()
    got = targets(layer, x, src_key_padding_mask=pad)
    assert fusion.fused_multi_head_attention in got
    # head dim 256 in training mode has no backward kernel: left alone; in evaluation mode it is taken
    wide = nn.MultiheadAttention(512, 2, batch_first=True).to(BF)
    xw = torch.randn(2, 40, 512, dtype=BF)
    assert fusion.fused_multi_head_attention not in targets(wide.train(), xw, xw, xw, need_weights=False)
    assert fusion.fused_multi_head_attention in targets(wide.eval(), xw, xw, xw, need_weights=False)
    # bias_k / bias_v and add_zero_attn append keys: left alone
    odd = nn.MultiheadAttention(128, 4, batch_first=True, add_bias_kv=True).to(BF).train()
    assert fusion.fused_multi_head_attention not in targets(odd, x, x, x, need_weights=False)


@pytest.mark.gpu
def test_multi_head_attention_modules_on_gpu():
    """torch.nn.MultiheadAttention and Transformer layers through the rewrite: the module in bf16 on the GPU against a
    copy of it in fp32 on the CPU; results, and for the attention module the gradients of every parameter."""
    import copy
    import torch.nn as nn
    from flashlight_amd import ops
    torch.manual_seed(0)
    B, L, E, H = 2, 200, 256, 4
    x = torch.randn(B, L, E).to(BF)
    pad = torch.zeros(B, L, dtype=torch.bool)
    pad[0, 150:] = True
    pad[1, 77:] = True
    causal = nn.Transformer.generate_square_subsequent_mask(L)
    launches = [0]
    real = ops.dispatch

    def counting(*a, **k):
        launches[0] += 1
        return real(*a, **k)

    def check(name, mod, args, kwargs, n_launches, grads=True, tol=(2e-2, 2e-3)):
        ref = copy.deepcopy(mod).float().train()
        m = mod.to(BF).to("cuda").train()
        dev = lambda t: t.to("cuda") if torch.is_tensor(t) else t
        launches[0] = 0
        torch._dynamo.reset()
        ops.dispatch = counting
        try:
            got = torch.compile(m, backend=fusion.backend, dynamic=False)(*map(dev, args), **{k: dev(v) for k, v in kwargs.items()})
        finally:
            ops.dispatch = real
        want = ref(*(a.float() if torch.is_tensor(a) and a.is_floating_point() else a for a in args), **kwargs)
        got, want = (t[0] if isinstance(t, tuple) else t for t in (got, want))
        assert launches[0] == n_launches, name
        assert_parity(got, want, name, max_tol=tol[0] * max(1.0, want.abs().max().item()), mean_tol=tol[1] * max(1.0, want.abs().max().item()))
        if not grads:
            return
        w = torch.randn(want.shape, generator=torch.Generator().manual_seed(5))
        (want * w).sum().backward()
        (got.float() * w.to("cuda")).sum().backward()
        for (pn, p32), (_, p16) in zip(ref.named_parameters(), m.named_parameters()):
            assert (p32.grad is None) == (p16.grad is None), f"{name}: {pn}"
            if p32.grad is not None:
                err = (p16.grad.float().cpu() - p32.grad).abs().max().item()
                assert err <= 2e-2 * p32.grad.abs().max().item() + 1e-4, f"{name}: gradient of {pn} off by {err}"

    mha = lambda **kw: nn.MultiheadAttention(E, H, **kw)
    nw = dict(need_weights=False)
    xt = x.transpose(0, 1)
    check("self-attention", mha(batch_first=True), (x, x, x), nw, 1)
    check("padding mask", mha(batch_first=True), (x, x, x), dict(nw, key_padding_mask=pad), 1)
    check("causal mask tensor", mha(batch_first=True), (x, x, x), dict(nw, attn_mask=causal), 1)
    check("causal hint", mha(batch_first=True), (x, x, x), dict(nw, attn_mask=causal, is_causal=True), 1)
    check("sequence first", mha(), (xt, xt, xt), nw, 1)
    check("unbatched", mha(), (x[0], x[0], x[0]), dict(nw, key_padding_mask=pad[0]), 1)
    check("key / value widths of their own", mha(batch_first=True, kdim=128, vdim=64), (x, x[:, :120, :128], x[:, :120, :64]), nw, 1)
    check("float masks", mha(batch_first=True), (x, x, x),
          dict(nw, attn_mask=torch.randn(L, L), key_padding_mask=torch.zeros(B, L).masked_fill(pad, float("-inf"))), 1)
    check("a mask per head", mha(batch_first=True), (x, x, x), dict(nw, attn_mask=torch.randn(B * H, L, L)), 1)
    check("head dim 16", nn.MultiheadAttention(E, 16, batch_first=True), (x, x, x), dict(nw, key_padding_mask=pad), 2)  # padded: 2 calls
    check("returns weights: left alone", mha(batch_first=True), (x, x, x), dict(need_weights=True), 0)
    # whole layers: bf16 rounding of the feed-forward part dominates, so results only
    check("encoder layer", nn.TransformerEncoderLayer(E, H, 512, dropout=0.0, batch_first=True), (x,),
          dict(src_key_padding_mask=pad), 1, grads=False)
    check("decoder layer", nn.TransformerDecoderLayer(E, H, 512, dropout=0.0, batch_first=True), (x, x[:, :120]),
          dict(tgt_mask=causal, tgt_is_causal=True, memory_key_padding_mask=pad[:, :120]), 2, grads=False)
    check("three encoder layers", nn.TransformerEncoder(nn.TransformerEncoderLayer(E, H, 512, dropout=0.0, batch_first=True), 3,
                                                        enable_nested_tensor=False), (x,), dict(src_key_padding_mask=pad), 3, grads=False)


def test_inductor_backend_keeps_graphs_with_dropout_out_of_the_tracer(monkeypatch):
    """`backend="flashlight_amd_inductor"` hands the rewritten graph to Inductor, except when a region drops weights:
    its seed is drawn per call, which a tracer would freeze."""
    import torch._inductor.compile_fx as cfx
    handed = []
    monkeypatch.setattr(cfx, "compile_fx", lambda gm, ex: handed.append(gm) or gm.forward)
    q, k, v = _qkv()

    def capture(fn, *args):
        got = []

        class _Done(Exception):
            pass

        def be(gm, example_inputs):
            got.append(fusion.backend_inductor(gm, example_inputs))

            def run(*a):
                raise _Done
            return run

        torch._dynamo.reset()
        with pytest.raises(_Done):
            torch.compile(fn, backend=be, dynamic=False, fullgraph=True)(*args)
        return got[0]

    capture(E.causal_triu, q, k, v)
    assert len(handed) == 1
    drop = lambda q, k, v: torch.nn.functional.dropout(torch.softmax(q @ k.transpose(-2, -1) * 0.1, dim=-1), 0.1, True) @ v
    capture(drop, q, k, v)
    assert len(handed) == 1
    assert "flashlight_amd_inductor" in torch._dynamo.list_backends(exclude_tags=())


@pytest.mark.gpu
def test_rewrite_followed_by_inductor_on_gpu():
    """A pre-norm transformer block (eager attention spelled out, causal) and a torch.nn encoder layer under
    `backend="flashlight_amd_inductor"`: the attention on the fused kernel, everything else compiled by Inductor; results
    and parameter gradients against the same module in fp32 on the CPU."""
    import copy
    import torch.nn as nn

    class Block(nn.Module):
        def __init__(self, E=256, H=4):
            super().__init__()
            self.H = H
            self.qkv, self.o = nn.Linear(E, 3 * E), nn.Linear(E, E)
            self.n1, self.n2 = nn.LayerNorm(E), nn.LayerNorm(E)
            self.f1, self.f2 = nn.Linear(E, 2 * E), nn.Linear(2 * E, E)

        def forward(self, x):
            B, L, E = x.shape
            q, k, v = self.qkv(self.n1(x)).view(B, L, 3, self.H, E // self.H).permute(2, 0, 3, 1, 4)
            s = q @ k.transpose(-2, -1) / math.sqrt(E // self.H)
            s = s.masked_fill(torch.ones(L, L, dtype=torch.bool, device=x.device).triu(1), float("-inf"))
            a = torch.softmax(s, dim=-1) @ v
            x = x + self.o(a.transpose(1, 2).reshape(B, L, E))
            return x + self.f2(torch.tanh(self.f1(self.n2(x))))

    torch.manual_seed(0)
    x = torch.randn(2, 200, 256).to(BF)
    pad = torch.zeros(2, 200, dtype=torch.bool)
    pad[1, 120:] = True
    # a constant mask of no positional form is a dense operand the rewrite made: it reaches Inductor as a graph input
    pattern = torch.rand(200, 200, generator=torch.Generator().manual_seed(9)) > 0.4
    pattern[:, 0] = True

    def patterned(q, k, v):
        s = (q @ k.transpose(-2, -1)) * 0.125
        return torch.softmax(s.masked_fill(~pattern.to(q.device), float("-inf")), dim=-1) @ v

    q, k, v = (torch.randn(2, 4, 200, 64).to(BF).to("cuda") for _ in range(3))
    torch._dynamo.reset()
    got = torch.compile(patterned, backend="flashlight_amd_inductor", dynamic=False)(q, k, v)
    assert_parity(got, patterned(q.float().cpu(), k.float().cpu(), v.float().cpu()), "constant pattern")
    for name, mod, kwargs in (("block", Block(), {}),
                              ("encoder layer", nn.TransformerEncoderLayer(256, 4, 512, dropout=0.0, batch_first=True, activation=torch.tanh),
                               dict(src_key_padding_mask=pad))):
        ref = copy.deepcopy(mod).float().train()
        m = mod.to(BF).to("cuda").train()
        torch._dynamo.reset()
        regions = []
        real = fusion.fuse_attention
        fusion.fuse_attention = lambda gm: regions.append(real(gm)) or regions[-1]
        try:
            got = torch.compile(m, backend="flashlight_amd_inductor", dynamic=False)(x.to("cuda"), **{k: v.to("cuda") for k, v in kwargs.items()})
        finally:
            fusion.fuse_attention = real
        assert sum(regions) == 1, name   # (after the rewrite nothing but the fused kernel computes the attention)
        want = ref(x.float(), **kwargs)
        top = max(1.0, want.abs().max().item())
        assert_parity(got, want, name, max_tol=3e-2 * top, mean_tol=3e-3 * top)
        w = torch.randn(want.shape, generator=torch.Generator().manual_seed(5))
        (want * w).sum().backward()
        (got.float() * w.to("cuda")).sum().backward()
        for (pn, p32), (_, p16) in zip(ref.named_parameters(), m.named_parameters()):
            assert p16.grad is not None, f"{name}: {pn}"
            err = (p16.grad.float().cpu() - p32.grad).abs().max().item()
            assert err <= 4e-2 * p32.grad.abs().max().item() + 1e-3, f"{name}: gradient of {pn} off by {err}"


@pytest.mark.gpu
def test_rewritten_einsum_attention_on_gpu():
    g = torch.Generator().manual_seed(17)
    B, H, L, S, D = 2, 4, 150, 210, 64
    q = torch.randn(B, H, L, D, generator=g).to(BF).to("cuda")
    k, v = (torch.randn(B, H, S, D, generator=g).to(BF).to("cuda") for _ in range(2))
    keep = (torch.rand(B, 1, L, S, generator=g) > 0.3).to("cuda")
    keep[..., 0] = True
    torch._dynamo.reset()
    got = torch.compile(E.einsum_attention, backend=fusion.backend, dynamic=False, fullgraph=True)(q, k, v, keep)
    assert_parity(got, E.einsum_attention(q.float().cpu(), k.float().cpu(), v.float().cpu(), keep.cpu()), "einsum, mask")
    qs, ks, vs = (t.transpose(1, 2).contiguous() for t in (q, k, v))   # [B, L, H, E]
    torch._dynamo.reset()
    got = torch.compile(E.einsum_attention_seq_major, backend=fusion.backend, dynamic=False, fullgraph=True)(qs, ks, vs)
    assert got.shape == (B, L, H, D)
    assert_parity(got, E.einsum_attention_seq_major(qs.float().cpu(), ks.float().cpu(), vs.float().cpu()), "einsum, sequence-major")
    # gradients through the lowered graph
    torch._dynamo.reset()
    leaves = [t.clone().requires_grad_(True) for t in (qs, ks, vs)]
    out = torch.compile(E.einsum_attention_seq_major, backend=fusion.backend, dynamic=False, fullgraph=True)(*leaves)
    w = torch.randn(out.shape, generator=g)
    (out.float() * w.to("cuda")).sum().backward()
    refs = [t.float().cpu().requires_grad_(True) for t in (qs, ks, vs)]
    (E.einsum_attention_seq_major(*refs) * w).sum().backward()
    for name, a, b in zip(("dq", "dk", "dv"), leaves, refs):
        scale = max(1.0, b.grad.abs().max().item())
        assert_parity(a.grad / scale, b.grad / scale, name)
