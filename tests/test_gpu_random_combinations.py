"""Seeded random draws over everything `ops.dispatch` composes: head dims 32 .. 512 (padded ones included), unequal
lengths, every mask kind, the in-kernel ALiBi term, the soft-cap, up to two bias operands of either element type and any
broadcast shape, the gate, both element types, against the oracle's generic attention (the reference's variants are
plain PyTorch compositions of exactly these pieces, attention_variants/*.py).  A draw the library refuses fails the
test: every such combination has a kernel.  Tolerance: max-abs 2e-2 and mean-abs 2e-3, times the query amplitude."""
import math
import random

import pytest
import torch

from flashlight_amd import _ffi, ops
from oracle.attention import _softmax_attention, alibi_slopes

pytestmark = pytest.mark.gpu
DEV = "cuda"
KINDS = {"none": _ffi.MASK_NONE, "causal": _ffi.MASK_CAUSAL, "sliding": _ffi.MASK_SLIDING, "prefix": _ffi.MASK_PREFIX_LM,
         "doc": _ffi.MASK_DOCUMENT, "doc_causal": _ffi.MASK_DOCUMENT_CAUSAL}


def _draw(seed):
    rnd = random.Random(seed)
    D = rnd.choice([32, 64, 128, 128, 64, 48, 96, 160, 256, 320, 512])
    c = dict(seed=seed, D=D, Dv=D if rnd.random() < 0.7 else rnd.choice([32, 64, 128, 256]),
             Hkv=rnd.choice([1, 2, 3]), G=rnd.choice([1, 2, 4]), B=rnd.choice([1, 2, 3]),
             L=rnd.choice([1, 2, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 511, 513, 700]))
    c["S"] = c["L"] if rnd.random() < 0.6 else rnd.choice([1, 8, 17, 40, 64, 96, 150, 264, 300, 520])
    c["mask"] = rnd.choice(sorted(KINDS))
    if c["mask"] != "none" and c["mask"] != "causal":
        c["S"] = c["L"]  # (as in the reference: these masks are written for equal lengths)
    c.update(alibi=rnd.random() < 0.3, cap=rnd.choice([None, None, 5.0, 30.0]), nbias=rnd.choice([0, 0, 0, 1, 2]),
             gate=rnd.random() < 0.2, fp16=rnd.random() < 0.3, amp=rnd.choice([1.0, 3.0]),
             window=rnd.choice([0, 1, 31, 32, 33, 70, 128, 300]), prefix=rnd.choice([0, 1, 32, 50, 64, 127, 128, 129, 1000]),
             ndocs=rnd.choice([1, 2, 5, 9]))
    c["bias_shapes"] = [rnd.choice(["1HLS", "B11S", "BHLS", "11LS", "1H1S"]) for _ in range(c["nbias"])]
    c["bias_f32"] = [rnd.random() < 0.5 for _ in range(c["nbias"])]
    return c


@pytest.mark.parametrize("seed", range(240))
def test_random_combination(seed):
    c = _draw(seed)
    B, Hkv, G, L, S, D, Dv = c["B"], c["Hkv"], c["G"], c["L"], c["S"], c["D"], c["Dv"]
    Hq = Hkv * G
    dt = torch.float16 if c["fp16"] else torch.bfloat16
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Hq, L, D, generator=g) * c["amp"]).to(dt)
    k = torch.randn(B, Hkv, S, D, generator=g).to(dt)
    v = torch.randn(B, Hkv, S, Dv, generator=g).to(dt)
    ids = None
    if c["mask"].startswith("doc"):
        ids = torch.sort(torch.randint(0, c["ndocs"], (B, L), generator=g), dim=1).values
        if seed % 3 == 0:
            ids = ids[:, torch.randperm(L, generator=g)]
    shapes = {"1HLS": (1, Hq, L, S), "B11S": (B, 1, 1, S), "BHLS": (B, Hq, L, S), "11LS": (1, 1, L, S), "1H1S": (1, Hq, 1, S)}
    biases = [torch.randn(shapes[s], generator=g).to(torch.float32 if f32 else dt)
              for s, f32 in zip(c["bias_shapes"], c["bias_f32"])]
    gate = torch.randn(B, Hq, L, Dv, generator=g).to(dt) if c["gate"] else None

    out = ops.dispatch(q.to(DEV), k.to(DEV), v.to(DEV), mask_kind=KINDS[c["mask"]], window=c["window"], prefix=c["prefix"],
                       doc_ids=None if ids is None else ids.to(DEV), alibi_heads=Hq if c["alibi"] else 0,
                       softcap=c["cap"] or 0.0, biases=[(b.to(DEV), 1) for b in biases],
                       gate=None if gate is None else gate.to(DEV))

    def masked(qi, ki):
        if c["mask"] == "causal":
            return ki > qi
        if c["mask"] == "sliding":
            return (ki > qi) | (qi - ki > c["window"])
        if c["mask"] == "prefix":
            return (ki > qi) & (ki >= c["prefix"])
        m = ids[:, qi.view(-1)].view(B, 1, -1, 1) != ids[:, ki.view(-1)].view(B, 1, 1, -1)
        return (m | (ki > qi)) if c["mask"] == "doc_causal" else m

    def bias(qi, ki):
        terms = [alibi_slopes(Hq).float().view(1, Hq, 1, 1) * (ki - qi).float()] if c["alibi"] else []
        terms += [b.float()[..., qi.view(-1) if b.size(2) > 1 else slice(None), :] for b in biases]
        return terms if terms else torch.zeros(())

    ref = _softmax_attention(q.float(), k.float().repeat_interleave(G, dim=1), v.float().repeat_interleave(G, dim=1),
                             1.0 / math.sqrt(D), masked=None if c["mask"] == "none" else masked, bias=bias, softcap=c["cap"])
    if gate is not None:
        ref = ref * torch.sigmoid(gate.float())
    o = out.float().cpu()
    d = (o - ref).abs()
    assert torch.isfinite(o).all(), c
    assert d.max().item() <= 2e-2 * c["amp"] and d.mean().item() <= 2e-3 * c["amp"], (c, d.max().item(), d.mean().item())
