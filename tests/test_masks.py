"""Mask predicates, attended-pair closed forms and the workload generators (CPU only)."""
import itertools

import numpy as np
import pytest

from flashlight_amd import workloads as W
from oracle import masks as M


def loop_matrix(L, fn):
    return np.array([[bool(fn(q, k)) for k in range(L)] for q in range(L)])


@pytest.mark.parametrize("L", [1, 2, 7, 33])
def test_predicates_against_loops(L):
    assert (M.attend_matrix("none", L, L) == loop_matrix(L, lambda q, k: True)).all()
    assert (M.attend_matrix("causal", L, L) == loop_matrix(L, lambda q, k: k <= q)).all()
    for w in (0, 1, 5, L, 2 * L):
        assert (M.attend_matrix("sliding", L, L, window=w) == loop_matrix(L, lambda q, k: 0 <= q - k <= w)).all()
    for p in (0, 1, 3, L, L + 4):
        assert (M.attend_matrix("prefix", L, L, prefix=p) == loop_matrix(L, lambda q, k: k < p or k <= q)).all()
    ids = [(i * 5) % 3 for i in range(L)]
    assert (M.attend_matrix("document", L, L, doc_ids=ids) == loop_matrix(L, lambda q, k: ids[q] == ids[k])).all()
    assert (M.attend_matrix("document_causal", L, L, doc_ids=ids) ==
            loop_matrix(L, lambda q, k: ids[q] == ids[k] and k <= q)).all()


def test_sliding_window_attends_window_plus_one_keys():
    m = M.attend_matrix("sliding", 40, 40, window=4)
    assert m[20].sum() == 5 and m[2].sum() == 3


@pytest.mark.parametrize("S", [1, 5, 64, 257])
def test_pair_counts_closed_forms(S):
    for fn_o, fn_w in ((lambda: M.attended_pairs("none", S), lambda: W.pairs_none(S)),
                       (lambda: M.attended_pairs("causal", S), lambda: W.pairs_causal(S))):
        assert fn_o() == fn_w()
    assert M.attended_pairs("none", S) == M.attend_matrix("none", S, S).sum()
    assert M.attended_pairs("causal", S) == M.attend_matrix("causal", S, S).sum()
    for w in (0, 3, S - 1, S + 10):
        n = M.attend_matrix("sliding", S, S, window=w).sum()
        assert M.attended_pairs("sliding", S, window=w) == n == W.pairs_sliding(S, w)
    for p in (0, 1, S // 2, S, S + 3):
        n = M.attend_matrix("prefix", S, S, prefix=p).sum()
        assert M.attended_pairs("prefix", S, prefix=p) == n == W.pairs_prefix(S, p)


def test_document_pair_counts_and_generators():
    lens = [3, 10, 1, 6]
    ids = M.document_ids_from_lengths(lens)
    assert ids.tolist() == [0] * 3 + [1] * 10 + [2] + [3] * 6
    S = sum(lens)
    assert M.attended_pairs("document", S, doc_lengths=lens) == M.attend_matrix("document", S, S, doc_ids=ids).sum()
    assert M.attended_pairs("document_causal", S, doc_lengths=lens) == \
        M.attend_matrix("document_causal", S, S, doc_ids=ids).sum() == W.pairs_documents(lens, True)
    # the benchmark's document lengths: product-side generator and the oracle's restatement agree, and are valid
    for seed in (0, 1003):
        a, b = W.document_lengths(16384, seed), M.document_lengths_cfg3(16384, seed)
        assert a == b and sum(a) == 16384 and all(512 <= n <= 4096 for n in a[:-1]) and 1 <= a[-1] <= 4096


def test_benchmark_flop_table():
    """Algorithmic FLOPs of the benchmark configurations (2 * (Dqk + Dv) per attended pair per branch)."""
    w = {x.name: x for x in W.build_workloads()}
    assert w["cfg1/vanilla"].flops == 4 * 128 * 4096 * 4096 * 64
    assert w["cfg1/causal"].pairs_per_head == 8390656
    assert w["cfg1/sliding_window"].pairs_per_head == 1019776
    assert w["cfg2/gqa_alibi_softcap_causal"].pairs_per_head == 33558528
    assert w["cfg3/prefix_lm"].pairs_per_head == 8914432
    assert w["cfg4/diff_attn_causal"].flops == 2 * (128 + 256) * 8390656 * 32
    assert w["cfg4/evoformer_bias_gate"].flops == 4 * 32 * 384 * 384 * 256 * 8
