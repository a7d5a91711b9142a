"""Key padding written as an additive mask, the way model code writes it: a fill of -1e9, -1e4, the most negative number
of fp32 or of the element type, or -inf; padding on the left (generation), on the right, on both sides or in runs;
one row per batch entry or a dense [.., L, S] tensor; fp32 or the element type; with or without the causal mask.  Seeded
draws through `ops.dispatch` against eager fp32.  Fully padded leading tiles, and ragged last tiles that are all padding,
are what these masks produce as a matter of course; finite fills of such magnitude once became the softmax reference
(their own rounding in the exponent, inf - inf at -3e38) and gave NaN.  Rows whose every permitted key is padded are left
out of the comparison (eager averages over the padded keys under a finite fill and returns NaN under -inf; the kernels
return that average or zeros) but must stay finite.  Tolerance: max-abs 2e-2, mean-abs 2e-3, times the query amplitude."""
import math
import random

import pytest
import torch

from flashlight_amd import _ffi, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _draw(seed):
    rnd = random.Random(seed)
    c = dict(seed=seed, D=rnd.choice([32, 64, 128, 96]), Hkv=rnd.choice([1, 2]), G=rnd.choice([1, 2, 4]), B=rnd.choice([1, 2, 3]),
             L=rnd.choice([1, 17, 33, 64, 100, 128, 129, 200, 256, 300, 333, 512, 700]), fp16=rnd.random() < 0.4,
             fill=rnd.choice(["1e9", "1e4", "min_f32", "min_elem", "inf", "min_elem_as_f32"]),
             side=rnd.choice(["right", "left", "runs", "both"]), shape=rnd.choice(["B11S", "B1LS", "BHLS"]),
             mask_f32=rnd.random() < 0.5, causal=rnd.random() < 0.5, amp=rnd.choice([1.0, 3.0]))
    keep = torch.ones(c["B"], c["L"], dtype=torch.bool)
    L = c["L"]
    for b in range(c["B"]):
        n = rnd.randint(1, L)
        if c["side"] == "right":
            keep[b, n:] = False
        elif c["side"] == "left":
            keep[b, :L - n] = False
        elif c["side"] == "both":
            a = rnd.randint(0, L - 1)
            keep[b, :a] = False
            keep[b, min(L, a + n):] = False
        else:
            for _ in range(rnd.randint(1, 4)):
                a = rnd.randint(0, L - 1)
                keep[b, a:a + rnd.randint(1, 80)] = False
        if not keep[b].any():
            keep[b, rnd.randint(0, L - 1)] = True
    return c, keep


@pytest.mark.parametrize("seed", range(160))
def test_additive_padding_mask(seed):
    c, keep = _draw(seed)
    B, Hkv, G, L, D = c["B"], c["Hkv"], c["G"], c["L"], c["D"]
    Hq = Hkv * G
    dt = torch.float16 if c["fp16"] else torch.bfloat16
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, Hq, L, D, generator=g) * c["amp"]).to(dt)
    k, v = torch.randn(B, Hkv, L, D, generator=g).to(dt), torch.randn(B, Hkv, L, D, generator=g).to(dt)
    fill = {"1e9": -1e9, "1e4": -1e4, "min_f32": torch.finfo(torch.float32).min, "min_elem": torch.finfo(dt).min,
            "inf": float("-inf"), "min_elem_as_f32": torch.finfo(dt).min}[c["fill"]]
    mdt = dt if c["fill"] == "min_elem" else torch.float32 if c["fill"] == "min_f32" or c["mask_f32"] else dt
    m = torch.zeros(B, 1, 1, L).masked_fill(~keep.view(B, 1, 1, L), fill)
    if c["shape"] != "B11S":
        m = m.expand(B, Hq if c["shape"] == "BHLS" else 1, L, L).contiguous()
    m = m.to(mdt)
    out = ops.dispatch(q.to(DEV), k.to(DEV), v.to(DEV), mask_kind=_ffi.MASK_CAUSAL if c["causal"] else _ffi.MASK_NONE,
                       biases=[(m.to(DEV), 1)]).float().cpu()
    future = torch.ones(L, L, dtype=torch.bool).triu(1)
    s = (q.float() @ k.float().repeat_interleave(G, 1).transpose(-1, -2)) / math.sqrt(D) + m.float()
    if c["causal"]:
        s = s.masked_fill(future, float("-inf"))
    ref = torch.softmax(s, -1) @ v.float().repeat_interleave(G, 1)
    permitted = keep.view(B, 1, 1, L).expand(B, 1, L, L)
    if c["causal"]:
        permitted = permitted & ~future
    rows = permitted.any(-1).unsqueeze(-1).expand_as(out)  # rows with at least one key that is neither padded nor masked
    assert torch.isfinite(out[rows]).all(), c
    if fill != float("-inf"):
        assert torch.isfinite(out).all(), c
    d = ((out - ref).abs() * rows).nan_to_num(0.0)
    assert d.max().item() <= 2e-2 * c["amp"] and d.mean().item() <= 2e-3 * c["amp"], (c, d.max().item(), d.mean().item())
