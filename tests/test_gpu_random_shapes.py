"""Seeded random shapes and mask parameters against the CPU oracle: every mask kind, ragged and unequal lengths,
grouped heads, the in-kernel ALiBi term (whose kernels walk the key tiles from the last one down) and the soft-cap.
The shapes are chosen to put windows, prefixes, diagonals and document boundaries at every position relative to the
32-row blocks of a wave and the key tiles, so that waves of one workgroup start and end their runs of tiles at different
steps.  Tolerance: bf16 kernel against the fp32 oracle, max-abs 2e-2 and mean-abs 2e-3."""
import random

import pytest
import torch

import flashlight_amd.attention_variants as A
import oracle as O
from tests.conftest import assert_parity

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _case(seed):
    rnd = random.Random(seed)
    D = rnd.choice([32, 64, 128])
    Hkv = rnd.choice([1, 2, 3])
    G = rnd.choice([1, 2, 4])
    B = rnd.choice([1, 2])
    L = rnd.choice([1, 17, 33, 64, 100, 129, 200, 257, 384, 450, 641])
    kind = rnd.choice(["vanilla", "causal", "sliding", "prefix", "document", "document_causal", "alibi", "softcap_causal",
                       "alibi_softcap_causal"])
    return dict(seed=seed, D=D, Hkv=Hkv, G=G, B=B, L=L, kind=kind, window=rnd.choice([0, 1, 31, 32, 33, 70, 128, 300]),
                prefix=rnd.choice([0, 1, 32, 50, 64, 127, 128, 129, 1000]), ndocs=rnd.choice([1, 2, 5, 9]),
                cap=rnd.choice([5.0, 30.0]), amp=rnd.choice([1.0, 3.0]))


@pytest.mark.parametrize("seed", range(96))
def test_random_shape(seed):
    _run_case(seed, torch.bfloat16)


@pytest.mark.parametrize("seed", range(200, 248))
def test_random_shape_fp16(seed):
    """The same draw with fp16 elements (every instance is compiled once per element type)."""
    _run_case(seed, torch.float16)


def _functions(c, seed, g):
    """(HIP front-end, oracle) as functions of (q, k, v) for the drawn case; `g` supplies the document ids."""
    B, Hq, L = c["B"], c["Hkv"] * c["G"], c["L"]
    kind = c["kind"]
    if kind == "vanilla":
        return (lambda q, k, v: A.attention_pytorch(q, k, v, enable_gqa=True),
                lambda q, k, v: O.attention_vanilla(q, k, v, enable_gqa=True))
    if kind == "causal":
        return (lambda q, k, v: A.attention_pytorch_causal(q, k, v, enable_gqa=True),
                lambda q, k, v: O.attention_causal(q, k, v, enable_gqa=True))
    if kind == "sliding":
        return (lambda q, k, v: A.attention_pytorch_sliding_window(q, k, v, window_size=c["window"], enable_gqa=True),
                lambda q, k, v: O.attention_sliding_window(q, k, v, window_size=c["window"], enable_gqa=True))
    if kind == "prefix":
        return (lambda q, k, v: A.attention_pytorch_prefix_lm(q, k, v, prefix_lengths=c["prefix"], enable_gqa=True),
                lambda q, k, v: O.attention_prefix_lm(q, k, v, prefix_lengths=c["prefix"], enable_gqa=True))
    if kind in ("document", "document_causal"):
        ids = torch.sort(torch.randint(0, c["ndocs"], (B, L), generator=g), dim=1).values
        if seed % 3 == 0:
            ids = ids[:, torch.randperm(L, generator=g)]  # ids in no order: tiles of one document lie scattered
        causal = kind == "document_causal"
        return (lambda q, k, v: A.attention_pytorch_document_mask(q, k, v, ids.to(q.device), enable_gqa=True, is_causal=causal),
                lambda q, k, v: O.attention_document_mask(q, k, v, ids.to(q.device), enable_gqa=True, is_causal=causal))
    if kind == "alibi":
        return (lambda q, k, v: A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(Hq), enable_gqa=True),
                lambda q, k, v: O.attention_alibi(q, k, v, score_mod=Hq, enable_gqa=True))
    if kind == "softcap_causal":
        return (lambda q, k, v: A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(c["cap"]), enable_gqa=True,
                                                       is_causal=True),
                lambda q, k, v: O.attention_softcapped(q, k, v, score_mod=c["cap"], enable_gqa=True, is_causal=True,
                                                       honor_causal=True))
    return (lambda q, k, v: A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(Hq), enable_gqa=True,
                                                      is_causal=True, softcap=c["cap"]),
            lambda q, k, v: O.attention_alibi(q, k, v, score_mod=Hq, enable_gqa=True, is_causal=True, honor_causal=True,
                                              softcap=c["cap"]))


def _draw(seed, dtype):
    c = _case(seed)
    g = torch.Generator().manual_seed(1000 + seed)
    B, Hq, Hkv, L, D = c["B"], c["Hkv"] * c["G"], c["Hkv"], c["L"], c["D"]
    q = (torch.randn(B, Hq, L, D, generator=g) * c["amp"]).to(dtype)
    k = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    return c, g, q, k, v


def _run_case(seed, dtype):
    c, g, q, k, v = _draw(seed, dtype)
    hip_fn, oracle_fn = _functions(c, seed, g)
    got, want = hip_fn(q.to(DEV), k.to(DEV), v.to(DEV)), oracle_fn(q.float(), k.float(), v.float())
    assert_parity(got.reshape(want.shape), want, str(c))


@pytest.mark.parametrize("seed", range(300, 348))
def test_random_shape_gradients(seed):
    """dq, dk, dv of the same draws from the HIP backward kernels (the reference has no backward) against autograd through
    the fp32 oracle, each scaled by its largest reference entry so that the forward's tolerance applies."""
    c, g, q, k, v = _draw(seed, torch.bfloat16)
    hip_fn, oracle_fn = _functions(c, seed, g)
    dout = torch.randn(q.shape, generator=g).to(torch.bfloat16)

    def grads(fn, dtype, device):
        a, b, w = (t.to(device=device, dtype=dtype).requires_grad_(True) for t in (q, k, v))
        out = fn(a, b, w)
        out.backward(dout.to(device=device, dtype=out.dtype).reshape(out.shape))
        return a.grad, b.grad, w.grad

    got = grads(hip_fn, torch.bfloat16, DEV)
    want = grads(oracle_fn, torch.float32, "cpu")
    for name, x, y in zip(("dq", "dk", "dv"), got, want):
        scale = max(1.0, y.abs().max().item())
        assert_parity(x.float() / scale, y / scale, f"{name} {c}")
