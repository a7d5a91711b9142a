"""analyse_score_mod: what a traced callable of the soft-cap signature (softcap.py:49) does to the scores.  CPU only."""
import math

import pytest
import torch

from flashlight_amd import _ffi
from flashlight_amd.attention_variants.softcap import analyse_score_mod


def _apply(mult, cap, bias, x, fn=None):
    y = x * mult
    if cap:
        y = cap * torch.tanh(y / cap)
    if fn is not None:  # the forms of fl_attn_params.score_fn, restated from the header
        kind, (p0, p1, p2, p3) = fn
        if kind == _ffi.SCORE_SIGMOID:
            y = p2 * torch.sigmoid(p0 * y + p1) + p3
        elif kind == _ffi.SCORE_CLAMP:
            y = torch.clamp(p0 * y + p1, min=p2, max=p3)
        else:
            y = p0 + p1 * y + p2 * y ** 2 + p3 * y ** 3
    return y if bias is None else y + bias


@pytest.mark.parametrize("fn", [
    lambda s, b, h, q, k: 30 * torch.tanh(s / 30),
    lambda s, b, h, q, k: torch.tanh(s * 0.125).mul(8.0),
    lambda s, b, h, q, k: s / 2.5,
    lambda s, b, h, q, k: 6.0 * torch.tanh(0.5 * s),
    lambda s, b, h, q, k: (s * 2.0 + 1.0) * 0.5,
    lambda s, b, h, q, k: 4.0 * (torch.tanh(s / 7.0) * 3.0) - 2.0,
    # the compiled-in score functions: sigmoid, clamp / ReLU, polynomials up to the cube
    lambda s, b, h, q, k: torch.relu(s),
    lambda s, b, h, q, k: 3 * torch.sigmoid(0.5 * s - 1) + 2,
    lambda s, b, h, q, k: torch.clamp(2 * s + 1, min=-3, max=5) * -2 + 1,
    lambda s, b, h, q, k: s.clamp_max(4.0) / 2,
    lambda s, b, h, q, k: torch.clamp(s, min=-1.5),
    lambda s, b, h, q, k: 0.01 * s ** 3 - s + 4,
    lambda s, b, h, q, k: s * s / 10,
    lambda s, b, h, q, k: (s + 1) * (2 - s) * 0.1,
    lambda s, b, h, q, k: -s,
    lambda s, b, h, q, k: 1.0 - torch.nn.functional.relu(0.5 * s),
    lambda s, b, h, q, k: torch.square(s - 2.0) * 0.05,
])
def test_analysis_reproduces_the_callable(fn):
    x = torch.linspace(-40, 40, 161, dtype=torch.float64)
    mult, cap, bias, score_fn = analyse_score_mod(fn)
    assert score_fn is None or (mult == 1.0 and cap == 0.0)
    got = _apply(mult, cap, bias, x, score_fn)
    want = fn(x, 0, 0, None, None)
    shift = (want - got)[0]  # a number added to every score changes no softmax and is dropped
    assert torch.allclose(got + shift, want, atol=1e-12)


def test_tensor_addends_are_returned_as_bias():
    t = torch.arange(6.0).view(2, 3)
    mult, cap, bias, _ = analyse_score_mod(lambda s, b, h, q, k: 5 * torch.tanh(s / 5) + t - 1.0)
    assert mult == pytest.approx(1.0) and cap == 5 and torch.equal(bias, t - 1.0)
    mult, cap, bias, _ = analyse_score_mod(lambda s, b, h, q, k: (s + t) * 2.0)
    assert mult == 2.0 and cap == 0.0 and torch.equal(bias, t * 2.0)


@pytest.mark.parametrize("fn", [
    lambda s, b, h, q, k: torch.tanh(torch.tanh(s)),
    lambda s, b, h, q, k: s ** 4,
    lambda s, b, h, q, k: torch.relu(s * s),
    lambda s, b, h, q, k: torch.sigmoid(s) * s,
    lambda s, b, h, q, k: torch.exp(s),
    lambda s, b, h, q, k: torch.tanh(s + 1.0),
    lambda s, b, h, q, k: -3.0 * torch.tanh(s),
    lambda s, b, h, q, k: s if s.sum() > 0 else -s,
    lambda s, b, h, q, k: 2.0,
])
def test_what_the_kernel_cannot_apply_is_refused(fn):
    with pytest.raises(NotImplementedError):
        analyse_score_mod(fn)
