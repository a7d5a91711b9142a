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


def test_callable_score_mod_against_pure_python_loops_and_identities():
    # softcap.py:49 hands the scaled score matrix to whatever callable it was given: the oracle's callable path against
    # the triple loops with math.* functions on single logits, and the identities that tie it to the pinned variants
    q, k, v = small()
    sc = 1 / math.sqrt(4)
    cases = [
        (lambda s, *_: torch.relu(s), lambda s, h, i, j: max(s, 0.0)),
        (lambda s, *_: 6.0 * torch.sigmoid(0.5 * s - 1.0) + 2.0, lambda s, h, i, j: 6.0 / (1.0 + math.exp(-(0.5 * s - 1.0))) + 2.0),
        (lambda s, *_: torch.clamp(2.0 * s + 1.0, min=-0.5, max=0.75), lambda s, h, i, j: min(max(2.0 * s + 1.0, -0.5), 0.75)),
        (lambda s, *_: 0.5 * s ** 3 - s + 4.0, lambda s, h, i, j: 0.5 * s * s * s - s + 4.0),
    ]
    for fn, logit in cases:
        assert torch.allclose(O.attention_softcapped(q, k, v, score_mod=fn), brute_force(q, k, v, sc, logit=logit), atol=1e-12)
        assert torch.allclose(O.attention_softcapped(q, k, v, score_mod=fn, is_causal=True, honor_causal=True),
                              brute_force(q, k, v, sc, lambda n, i, j: j <= i, logit=logit), atol=1e-12)
    assert torch.allclose(O.attention_softcapped(q, k, v, score_mod=lambda s, *_: s), O.attention_vanilla_nogqa(q, k, v))
    assert torch.allclose(O.attention_softcapped(q, k, v, score_mod=lambda s, *_: 2.5 * torch.tanh(s / 2.5)),
                          O.attention_softcapped(q, k, v, score_mod=2.5))
    # the callable sees the score times `scale`, nothing else
    assert torch.allclose(O.attention_softcapped(q, k, v, score_mod=lambda s, *_: torch.relu(s), scale=0.3),
                          brute_force(q, k, v, 0.3, logit=lambda s, h, i, j: max(s, 0.0)), atol=1e-12)


def test_row_blocks_do_not_change_results():
    q, k, v = (torch.randn(1, 2, 50, 8) for _ in range(3))
    ids = torch.from_numpy(O.document_ids_from_lengths([20, 30]))[None]
    for fn in (lambda **kw: O.attention_causal(q, k, v, **kw),
               lambda **kw: O.attention_document_mask(q, k, v, ids, is_causal=True, **kw),
               lambda **kw: O.attention_alibi(q, k, v, score_mod=2, softcap=3.0, **kw)):
        assert torch.equal(fn(), fn(q_block=50))
        assert torch.allclose(fn(), fn(q_block=16), atol=1e-6)


# ---- dense score_mod (alibi.py:26-29 with an arbitrary callable) -----------------------------------------------------------

@pytest.mark.parametrize("gqa", [False, True])
def test_dense_score_mod_against_sdpa(gqa):
    g = torch.Generator().manual_seed(31)
    N, Hq, Hkv, L, E = 2, 4, (2 if gqa else 4), 9, 8
    q = torch.randn(N, Hq, L, E, generator=g, dtype=torch.float64)
    k = torch.randn(N, Hkv, L, E, generator=g, dtype=torch.float64)
    v = torch.randn(N, Hkv, L, E, generator=g, dtype=torch.float64)
    dense = torch.randn(Hq, L, L, generator=g, dtype=torch.float64)
    out = O.attention_alibi(q, k, v, score_mod=lambda l, s: dense, enable_gqa=gqa)
    ref = F.scaled_dot_product_attention(q, k, v, attn_mask=dense, enable_gqa=gqa)
    if gqa:
        assert tuple(out.shape) == (N, Hkv, Hq // Hkv, L, E)
    assert (out.reshape(N, Hq, L, E) - ref).abs().max().item() < 1e-12


# ---- invariant point attention (tests/test_ipa.py:57-125) ------------------------------------------------------------------

def _ipa_inputs(seed, B=1, H=2, N=5, C=4, P=3, Pv=2, X=3, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=dtype)  # noqa: E731
    return dict(q_scalar=r(B, H, N, C), k_scalar=r(B, H, N, C), v_scalar=r(B, H, N, C), q_points=r(B, H, N, P, X),
                k_points=r(B, H, N, P, X), v_points=r(B, H, N, Pv, X), pair_bias=r(B, H, N, N))


def test_ipa_bruteforce_loops():
    a = _ipa_inputs(41, B=2, H=2, N=6, C=4, P=3, Pv=2, X=3)
    c_hidden, P = 4, 3
    o_s, o_p = O.invariant_point_attention(**a, c_hidden=c_hidden, no_qk_points=P)
    B, H, N, C = a["q_scalar"].shape
    Pv, X = a["v_points"].shape[-2:]
    assert tuple(o_s.shape) == (B, H, N, C) and tuple(o_p.shape) == (B, N, H, Pv, X)
    for b in range(B):
        for h in range(H):
            for i in range(N):
                logits = []
                for j in range(N):
                    dot = sum(float(a["q_scalar"][b, h, i, c]) * float(a["k_scalar"][b, h, j, c]) for c in range(C))
                    d2 = 0.0
                    for p in range(P):
                        for x in range(X):
                            d2 += (float(a["q_points"][b, h, i, p, x]) - float(a["k_points"][b, h, j, p, x])) ** 2
                    logits.append(dot / math.sqrt(c_hidden) - 0.5 * math.sqrt(9.0 / (2 * P)) * d2 +
                                  float(a["pair_bias"][b, h, i, j]))
                m = max(logits)
                wts = [math.exp(x - m) for x in logits]
                z = sum(wts)
                for c in range(C):
                    want = sum(wts[j] / z * float(a["v_scalar"][b, h, j, c]) for j in range(N))
                    assert abs(float(o_s[b, h, i, c]) - want) < 1e-10
                for p in range(Pv):
                    for x in range(X):
                        want = sum(wts[j] / z * float(a["v_points"][b, h, j, p, x]) for j in range(N))
                        assert abs(float(o_p[b, i, h, p, x]) - want) < 1e-10


def test_ipa_identities():
    a = _ipa_inputs(43, B=2, H=3, N=7, C=8, P=4, Pv=3, X=4)
    # no points: plain attention with the pair bias as float mask and scale 1/sqrt(c_hidden)
    z = dict(a, q_points=torch.zeros_like(a["q_points"]), k_points=torch.zeros_like(a["k_points"]))
    o_s, o_p = O.invariant_point_attention(**z, c_hidden=16, no_qk_points=4)
    ref = F.scaled_dot_product_attention(a["q_scalar"], a["k_scalar"], a["v_scalar"], attn_mask=a["pair_bias"],
                                         scale=1 / 4.0)
    assert (o_s - ref).abs().max().item() < 1e-12
    vp = a["v_points"].flatten(-2)
    refp = F.scaled_dot_product_attention(a["q_scalar"], a["k_scalar"], vp, attn_mask=a["pair_bias"], scale=1 / 4.0)
    assert (o_p.transpose(1, 2).flatten(-2) - refp).abs().max().item() < 1e-12
    # distances only see differences: moving every query and key point by the same vector changes nothing
    shift = torch.tensor([0.7, -1.3, 2.1, 0.4], dtype=torch.float64)
    s = dict(a, q_points=a["q_points"] + shift, k_points=a["k_points"] + shift)
    o1 = O.invariant_point_attention(**a, c_hidden=16, no_qk_points=4)
    o2 = O.invariant_point_attention(**s, c_hidden=16, no_qk_points=4)
    assert (o1[0] - o2[0]).abs().max().item() < 1e-10 and (o1[1] - o2[1]).abs().max().item() < 1e-10
    # one query at the origin, two keys at distances d1 and d2, nothing else: weights in the ratio exp(w (d1^2 - d2^2))
    for P in (1, 4, 8):
        w = -0.5 * math.sqrt(9.0 / (2 * P))
        d1, d2 = 0.5, 1.25
        qp = torch.zeros(1, 1, 1, 1, 3, dtype=torch.float64)
        kp = torch.zeros(1, 1, 2, 1, 3, dtype=torch.float64)
        kp[0, 0, 0, 0, 0], kp[0, 0, 1, 0, 2] = d1, d2
        zero = torch.zeros(1, 1, 1, 2, dtype=torch.float64)
        vs = torch.tensor([[1.0, 0.0], [0.0, 1.0]], dtype=torch.float64).view(1, 1, 2, 2)
        o_s, _ = O.invariant_point_attention(zero[..., :1, :], torch.zeros(1, 1, 2, 2, dtype=torch.float64), vs, qp, kp,
                                             torch.zeros(1, 1, 2, 1, 3, dtype=torch.float64), None, c_hidden=2,
                                             no_qk_points=P)
        assert abs(float(o_s[0, 0, 0, 0] / o_s[0, 0, 0, 1]) - math.exp(w * (d1 * d1 - d2 * d2))) < 1e-12
