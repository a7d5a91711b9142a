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


def _run_case(seed, dtype):
    c = _case(seed)
    g = torch.Generator().manual_seed(1000 + seed)
    B, Hq, Hkv, L, D = c["B"], c["Hkv"] * c["G"], c["Hkv"], c["L"], c["D"]
    q = (torch.randn(B, Hq, L, D, generator=g) * c["amp"]).to(dtype)
    k = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    qf, kf, vf = q.float(), k.float(), v.float()
    kind = c["kind"]
    if kind == "vanilla":
        got, want = A.attention_pytorch(qd, kd, vd, enable_gqa=True), O.attention_vanilla(qf, kf, vf, enable_gqa=True)
    elif kind == "causal":
        got, want = A.attention_pytorch_causal(qd, kd, vd, enable_gqa=True), O.attention_causal(qf, kf, vf, enable_gqa=True)
    elif kind == "sliding":
        got = A.attention_pytorch_sliding_window(qd, kd, vd, window_size=c["window"], enable_gqa=True)
        want = O.attention_sliding_window(qf, kf, vf, window_size=c["window"], enable_gqa=True)
    elif kind == "prefix":
        got = A.attention_pytorch_prefix_lm(qd, kd, vd, prefix_lengths=c["prefix"], enable_gqa=True)
        want = O.attention_prefix_lm(qf, kf, vf, prefix_lengths=c["prefix"], enable_gqa=True)
    elif kind in ("document", "document_causal"):
        ids = torch.sort(torch.randint(0, c["ndocs"], (B, L), generator=g), dim=1).values
        if seed % 3 == 0:
            ids = ids[:, torch.randperm(L, generator=g)]  # ids in no order: tiles of one document lie scattered
        causal = kind == "document_causal"
        got = A.attention_pytorch_document_mask(qd, kd, vd, ids.to(DEV), enable_gqa=True, is_causal=causal)
        want = O.attention_document_mask(qf, kf, vf, ids, enable_gqa=True, is_causal=causal)
    elif kind == "alibi":
        got = A.attention_pytorch_alibi(qd, kd, vd, score_mod=A.generate_alibi_bias_pytorch(Hq), enable_gqa=True)
        want = O.attention_alibi(qf, kf, vf, score_mod=Hq, enable_gqa=True)
    elif kind == "softcap_causal":
        got = A.attention_softcapped(qd, kd, vd, score_mod=A.generate_tanh_softcap(c["cap"]), enable_gqa=True, is_causal=True)
        want = O.attention_softcapped(qf, kf, vf, score_mod=c["cap"], enable_gqa=True, is_causal=True, honor_causal=True)
    else:
        got = A.attention_pytorch_alibi(qd, kd, vd, score_mod=A.generate_alibi_bias_pytorch(Hq), enable_gqa=True,
                                        is_causal=True, softcap=c["cap"])
        want = O.attention_alibi(qf, kf, vf, score_mod=Hq, enable_gqa=True, is_causal=True, honor_causal=True,
                                 softcap=c["cap"])
    assert_parity(got.reshape(want.shape), want, str(c))
