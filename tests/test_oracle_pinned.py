"""Pins the CPU oracle from outside: committed known-answer vectors (made from library routines by
tests/golden/make_golden.py), pure-Python brute force, and identities each variant must satisfy."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle as O
from tests.variant_calls import GOLDEN_NAMES, oracle_call

torch.manual_seed(7)


@pytest.mark.parametrize("name", GOLDEN_NAMES)
def test_oracle_matches_golden_fp64(golden, name):
    case = golden[name]
    out = oracle_call(name, case.to("cpu", torch.float64), case.meta)
    assert tuple(out.shape) == tuple(case.expected.shape)
    err = (out.float() - case.expected).abs().max().item()
    assert err < 2e-6, f"{name}: {err}"


@pytest.mark.parametrize("name", GOLDEN_NAMES)
def test_oracle_fp32_close_to_golden(golden, name):
    case = golden[name]
    out = oracle_call(name, case.to("cpu", torch.float32), case.meta)
    err = (out - case.expected).abs().max().item()
    assert err < 5e-5, f"{name}: {err}"


def brute_force(q, k, v, scale, attend=None, logit=None):
    """Triple Python loop, floats only: softmax over attended keys of logit(q.k*scale, h, i, j)."""
    N, H, L, E = q.shape
    S, Ev = k.shape[2], v.shape[3]
    out = torch.zeros(N, H, L, Ev, dtype=torch.float64)
    for n in range(N):
        for h in range(H):
            for i in range(L):
                logits = []
                for j in range(S):
                    if attend is not None and not attend(n, i, j):
                        continue
                    s = sum(float(q[n, h, i, e]) * float(k[n, h, j, e]) for e in range(E)) * scale
                    logits.append((j, s if logit is None else logit(s, h, i, j)))
                m = max(s for _, s in logits)
                w = [(j, math.exp(s - m)) for j, s in logits]
                z = sum(x for _, x in w)
                for j, x in w:
                    for e in range(Ev):
                        out[n, h, i, e] += x / z * float(v[n, h, j, e])
    return out


def small(N=1, H=2, L=9, E=4):
    return (torch.randn(N, H, L, E, dtype=torch.float64) for _ in range(3))


def test_bruteforce_vanilla_causal_sliding_prefix():
    q, k, v = small()
    sc = 1 / math.sqrt(4)
    assert torch.allclose(O.attention_vanilla_nogqa(q, k, v), brute_force(q, k, v, sc), atol=1e-12)
    assert torch.allclose(O.attention_causal(q, k, v), brute_force(q, k, v, sc, lambda n, i, j: j <= i), atol=1e-12)
    assert torch.allclose(O.attention_sliding_window(q, k, v, window_size=3),
                          brute_force(q, k, v, sc, lambda n, i, j: 0 <= i - j <= 3), atol=1e-12)
    assert torch.allclose(O.attention_prefix_lm(q, k, v, prefix_lengths=4),
                          brute_force(q, k, v, sc, lambda n, i, j: j < 4 or j <= i), atol=1e-12)


def test_bruteforce_document_alibi_softcap():
    q, k, v = small(N=2)
    sc = 1 / math.sqrt(4)
    ids = torch.tensor([[0, 0, 3, 3, 3, 1, 1, 0, 0], [5, 5, 5, 5, 5, 5, 5, 5, 5]])
    assert torch.allclose(O.attention_document_mask(q, k, v, ids),
                          brute_force(q, k, v, sc, lambda n, i, j: ids[n, i] == ids[n, j]), atol=1e-12)
    assert torch.allclose(O.attention_document_mask(q, k, v, ids, is_causal=True),
                          brute_force(q, k, v, sc, lambda n, i, j: ids[n, i] == ids[n, j] and j <= i), atol=1e-12)
    H = q.size(1)
    # alibi.py builds the bias in float32 and casts it to the score dtype: compare at float32 resolution
    alibi = O.attention_alibi(q, k, v, score_mod=H)
    ref = brute_force(q, k, v, sc, logit=lambda s, h, i, j: s + 2.0 ** (-8.0 * (h + 1) / H) * (j - i))
    assert torch.allclose(alibi, ref, atol=1e-6)
    cap = 0.7
    assert torch.allclose(O.attention_softcapped(q, k, v, score_mod=cap),
                          brute_force(q, k, v, sc, logit=lambda s, h, i, j: cap * math.tanh(s / cap)), atol=1e-12)
    assert torch.allclose(O.tanh_softcap(torch.tensor([0.3, -2.0, 9.0], dtype=torch.float64), 1.5),
                          torch.tensor([1.5 * math.tanh(0.2), 1.5 * math.tanh(-2 / 1.5), 1.5 * math.tanh(6.0)],
                                       dtype=torch.float64), atol=1e-14)


def test_gqa_head_mapping_against_sdpa():
    q = torch.randn(2, 6, 11, 8, dtype=torch.float64)
    k, v = torch.randn(2, 2, 11, 8, dtype=torch.float64), torch.randn(2, 2, 11, 8, dtype=torch.float64)
    ref = F.scaled_dot_product_attention(q, k.repeat_interleave(3, 1), v.repeat_interleave(3, 1))
    assert torch.allclose(O.attention_vanilla(q, k, v, enable_gqa=True), ref, atol=1e-12)
    # every other variant keeps the grouped 5-D layout
    out = O.attention_causal(q, k, v, enable_gqa=True)
    assert out.shape == (2, 2, 3, 11, 8)
    ref = F.scaled_dot_product_attention(q, k.repeat_interleave(3, 1), v.repeat_interleave(3, 1), is_causal=True)
    assert torch.allclose(out.flatten(1, 2), ref, atol=1e-12)


def test_identities():
    q, k, v = (torch.randn(1, 2, 33, 8, dtype=torch.float64) for _ in range(3))
    S = 33
    van, cau = O.attention_vanilla_nogqa(q, k, v), O.attention_causal(q, k, v)
    assert torch.allclose(cau[..., 0, :], v[..., 0, :])                                   # row 0 sees only key 0
    assert torch.allclose(O.attention_sliding_window(q, k, v, window_size=S - 1), cau)     # window covers all
    assert torch.allclose(O.attention_sliding_window(q, k, v, window_size=0), v)           # only the diagonal
    assert torch.allclose(O.attention_prefix_lm(q, k, v, prefix_lengths=1), cau)
    assert torch.allclose(O.attention_prefix_lm(q, k, v, prefix_lengths=0), cau)
    assert torch.allclose(O.attention_prefix_lm(q, k, v, prefix_lengths=S), van)
    one_doc = torch.zeros(1, S, dtype=torch.int64)
    assert torch.allclose(O.attention_document_mask(q, k, v, one_doc), van)
    assert torch.allclose(O.attention_document_mask(q, k, v, one_doc, is_causal=True), cau)
    assert torch.allclose(O.attention_softcapped(q, k, v, score_mod=1e9), van, atol=1e-9)  # cap -> inf
    # is_causal is accepted and ignored unless the extension switch is on (alibi.py:15, softcap.py:11)
    assert torch.allclose(O.attention_softcapped(q, k, v, score_mod=2.0, is_causal=True),
                          O.attention_softcapped(q, k, v, score_mod=2.0))
    # document attention == independent attention per document
    lens = [5, 17, 11]
    ids = O.document_ids_from_lengths(lens)
    doc = O.attention_document_mask(q, k, v, torch.from_numpy(ids)[None])
    a = 0
    for n in lens:
        sl = slice(a, a + n)
        assert torch.allclose(doc[..., sl, :], O.attention_vanilla_nogqa(q[..., sl, :], k[..., sl, :], v[..., sl, :]))
        a += n
    # differential attention
    q2, k2 = torch.cat([q, q], 1), torch.cat([k, k], 1)
    v2 = torch.randn(1, 2, S, 16, dtype=torch.float64)
    base = O.attention_vanilla_nogqa(q, k, v2)
    assert torch.allclose(O.diff_attention(q2, k2, v2, lambda_full=0.0), base)
    assert torch.allclose(O.diff_attention(q2, k2, v2, lambda_full=0.3), 0.7 * base)
    assert torch.allclose(O.diff_attention(q2, k2, v2), 0.8 * base)                       # default lambda 0.2
    # evoformer with zero biases == vanilla on transposed layout
    qe, ke, ve = (torch.randn(2, 3, 10, 2, 4, dtype=torch.float64) for _ in range(3))
    z = torch.zeros(2, 1, 2, 10, 10, dtype=torch.float64)
    ref = O.attention_vanilla_nogqa(qe.transpose(2, 3), ke.transpose(2, 3), ve.transpose(2, 3)).transpose(2, 3)
    assert torch.allclose(O.attention_evoformer(qe, ke, ve, [z]), ref)
    assert torch.allclose(O.attention_evoformer(qe, ke, ve, []), ref)
    big = torch.full_like(qe, 50.0)
    assert torch.allclose(O.attention_evoformer(qe, ke, ve, [z], gate=big), ref)          # sigmoid(50) == 1


def test_row_blocks_do_not_change_results():
    q, k, v = (torch.randn(1, 2, 50, 8) for _ in range(3))
    ids = torch.from_numpy(O.document_ids_from_lengths([20, 30]))[None]
    for fn in (lambda **kw: O.attention_causal(q, k, v, **kw),
               lambda **kw: O.attention_document_mask(q, k, v, ids, is_causal=True, **kw),
               lambda **kw: O.attention_alibi(q, k, v, score_mod=2, softcap=3.0, **kw)):
        assert torch.equal(fn(), fn(q_block=50))
        assert torch.allclose(fn(), fn(q_block=16), atol=1e-6)
