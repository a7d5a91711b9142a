"""Bit-exactness of the attended-key sets: the kernel's own bitmap of the pairs it attended (after tile skipping and
the element predicate) against the dense predicate matrices, at sizes straddling tile edges; and size-independent
properties of the outputs at full benchmark size."""
import numpy as np
import pytest
import torch

import flashlight_amd.attention_variants as A
from flashlight_amd import _ffi
from oracle import masks as M

pytestmark = pytest.mark.gpu
DEV = "cuda"

KIND = {"none": _ffi.MASK_NONE, "causal": _ffi.MASK_CAUSAL, "sliding": _ffi.MASK_SLIDING, "prefix": _ffi.MASK_PREFIX_LM,
        "document": _ffi.MASK_DOCUMENT, "document_causal": _ffi.MASK_DOCUMENT_CAUSAL}


def attended_bitmap(kind, S, D=64, H=2, **kw):
    g = torch.Generator().manual_seed(S)
    q, k, v = (torch.randn(1, H, S, D, generator=g).bfloat16().to(DEV) for _ in range(3))
    dump = torch.zeros(1, H, S, S, dtype=torch.uint8, device=DEV)
    args = {}
    if "doc_ids" in kw:
        args["doc_ids"] = torch.as_tensor(np.asarray(kw["doc_ids"]), dtype=torch.int64, device=DEV)[None]
    _ffi.attn_fwd(q, k, v, mask_kind=KIND[kind], window=kw.get("window", 0), prefix=kw.get("prefix", 0),
                  attended_dump=dump, **args)
    torch.cuda.synchronize()
    return dump.cpu().numpy().astype(bool)


SIZES = [1, 63, 64, 65, 127, 128, 129, 255, 256, 257, 1000]


@pytest.mark.parametrize("S", SIZES)
def test_positional_masks_bit_exact(S):
    for kind, kws in (("none", [{}]), ("causal", [{}]),
                      ("sliding", [{"window": w} for w in (0, 1, 63, 64, 65, 200, S + 5)]),
                      ("prefix", [{"prefix": p} for p in (0, 1, 64, 65, 100, S, S + 9)])):
        for kw in kws:
            got = attended_bitmap(kind, S, **kw)
            want = M.attend_matrix(kind, S, S, **kw)
            for h in range(got.shape[1]):
                assert np.array_equal(got[0, h], want), f"{kind} {kw} S={S}: {np.argwhere(got[0, h] != want)[:5]}"


@pytest.mark.parametrize("S", [65, 256, 257, 1000])
def test_document_masks_bit_exact(S):
    rng = np.random.default_rng(S)
    cuts = np.sort(rng.choice(np.arange(1, S), size=min(5, S - 1), replace=False))
    sorted_ids = np.searchsorted(cuts, np.arange(S), side="right") * 3 - 4
    layouts = {"sorted": sorted_ids, "unsorted": rng.integers(-2, 2, size=S) * (2 ** 40), "single": np.zeros(S, np.int64),
               "edges at 64": (np.arange(S) // 64)}
    for tag, ids in layouts.items():
        for kind in ("document", "document_causal"):
            got = attended_bitmap(kind, S, doc_ids=ids)
            want = M.attend_matrix(kind, S, S, doc_ids=ids)
            assert np.array_equal(got[0, 0], want) and np.array_equal(got[0, 1], want), f"{kind}/{tag} S={S}"


@pytest.mark.parametrize("Lq,Lk", [(100, 300), (300, 100), (129, 64), (64, 129), (1, 200), (513, 190)])
def test_unmasked_and_causal_bit_exact_with_unequal_lengths(Lq, Lk):
    # the causal mask is top-left aligned (query i and key j compare as positions i and j): rows past the last key see
    # all keys
    g = torch.Generator().manual_seed(Lq * 1000 + Lk)
    q = torch.randn(1, 2, Lq, 64, generator=g).bfloat16().to(DEV)
    k, v = (torch.randn(1, 2, Lk, 64, generator=g).bfloat16().to(DEV) for _ in range(2))
    # (the sliding-window and prefix-LM masks are defined for Lq == Lk only, like the reference's mask builders)
    for kind, kws in (("none", [{}]), ("causal", [{}])):
        for kw in kws:
            dump = torch.zeros(1, 2, Lq, Lk, dtype=torch.uint8, device=DEV)
            _ffi.attn_fwd(q, k, v, mask_kind=KIND[kind], window=kw.get("window", 0), prefix=kw.get("prefix", 0),
                          attended_dump=dump)
            torch.cuda.synchronize()
            got = dump.cpu().numpy().astype(bool)
            want = M.attend_matrix(kind, Lq, Lk, **kw)
            for h in range(2):
                assert np.array_equal(got[0, h], want), f"{kind} {kw} Lq={Lq} Lk={Lk}: {np.argwhere(got[0, h] != want)[:5]}"


def test_d128_instance_bit_exact():
    for kind, kw in (("causal", {}), ("sliding", {"window": 100}), ("prefix", {"prefix": 70})):
        got = attended_bitmap(kind, 300, D=128, **kw)
        assert np.array_equal(got[0, 0], M.attend_matrix(kind, 300, 300, **kw))


def _dump_call(q, k, v, S, **kw):
    """Attended-pair bitmap of one call, after checking that the instance chosen with the dump hook has the tile shape
    (query rows per workgroup, keys per tile, threads) of the instance the same call runs without it."""
    Hq = q.shape[1] // (2 if kw.get("diff") else 1)
    dump = torch.zeros(1, Hq, S, S, dtype=torch.uint8, device=DEV)
    shapes = []
    for d in (None, dump):
        out = torch.empty(1, Hq, S, v.shape[-1], dtype=q.dtype, device=DEV)
        fk = dict(scale=None, mask_kind=kw.get("mask_kind", _ffi.MASK_NONE), window=kw.get("window", 0), prefix=0,
                  doc_ids=kw.get("doc_ids"), alibi_heads=0, softcap=0.0, biases=[], gate=None, diff=kw.get("diff", False),
                  lambda_full=kw.get("lambda_full", 0.0), attended_dump=d)
        p, _keep = _ffi._fill_params(_ffi.load_library(), q, k, v, out, Hq, k.shape[1] // (2 if kw.get("diff") else 1),
                                     fk["scale"], fk["mask_kind"], fk["window"], fk["prefix"], fk["doc_ids"], 0, 0.0, [],
                                     None, fk["diff"], fk["lambda_full"], d)
        plan = _ffi.plan(p)
        shapes.append((plan["rows_per_workgroup"], plan["keys_per_tile"], plan["threads"]))
    assert shapes[0] == shapes[1], f"dump instance {shapes[1]} differs from the production instance {shapes[0]}"
    _ffi.attn_fwd(q, k, v, attended_dump=dump, **kw)
    torch.cuda.synchronize()
    return dump.cpu().numpy().astype(bool), shapes[0]


@pytest.mark.parametrize("S", [63, 65, 129, 257, 300, 1000])
def test_production_tile_shapes_bit_exact(S):
    # The tile shapes the benchmark configurations launch under a mask, other than the default 128 rows x 64 keys:
    # head dim 128 with a short sliding window (two-wave workgroups, 64 rows x 32 keys), document masks at head dim 128
    # (128 rows x 32 keys), causal differential attention (32-key tiles, two softmax branches).
    g = torch.Generator().manual_seed(7000 + S)
    mk = lambda h, d: torch.randn(1, h, S, d, generator=g).bfloat16().to(DEV)  # noqa: E731
    q, k, v = mk(2, 128), mk(2, 128), mk(2, 128)
    for w in (0, 31, 32, 33, 100, 255, 256):
        got, shape = _dump_call(q, k, v, S, mask_kind=_ffi.MASK_SLIDING, window=w)
        # (two-wave workgroups below a window of 256 keys, the default 128 x 64 tile from there on; shorter sequences
        # than window + 128 count as short too)
        assert shape == ((64, 32, 128) if min(S, w + 128) < 384 else (128, 64, 256)), shape
        want = M.attend_matrix("sliding", S, S, window=w)
        assert np.array_equal(got[0, 0], want) and np.array_equal(got[0, 1], want), f"sliding {w} S={S}"
    rng = np.random.default_rng(S)
    cuts = np.sort(rng.choice(np.arange(1, S), size=min(4, S - 1), replace=False))
    for tag, ids in (("sorted", np.searchsorted(cuts, np.arange(S), side="right")),
                     ("unsorted", rng.integers(-1, 2, size=S) * (2 ** 35)), ("edges at 32", np.arange(S) // 32)):
        for kind in ("document", "document_causal"):
            got, shape = _dump_call(q, k, v, S, mask_kind=KIND[kind],
                                    doc_ids=torch.as_tensor(ids, dtype=torch.int64, device=DEV)[None])
            assert shape == (128, 32, 256), shape
            want = M.attend_matrix(kind, S, S, doc_ids=ids)
            assert np.array_equal(got[0, 0], want) and np.array_equal(got[0, 1], want), f"{kind}/{tag} S={S}"
    q2, k2, v2 = mk(4, 64), mk(4, 64), mk(2, 128)
    for kind in ("none", "causal"):
        got, shape = _dump_call(q2, k2, v2, S, mask_kind=KIND[kind], diff=True, lambda_full=0.8)
        assert shape == (128, 32, 256), shape
        want = M.attend_matrix(kind, S, S)
        assert np.array_equal(got[0, 0], want) and np.array_equal(got[0, 1], want), f"diff {kind} S={S}"


# ---- properties that hold at any size: checked at the full benchmark shapes -----------------------------------------------

def test_rows_sum_to_one_and_value_linearity_full_size():
    B, H, S, D = 4, 16, 4096, 128
    g = torch.Generator().manual_seed(21)
    q, k, v = (torch.randn(B, H, S, D, generator=g).bfloat16().to(DEV) for _ in range(3))
    ones = torch.ones_like(v)
    for fn in (A.attention_pytorch, A.attention_pytorch_causal,
               lambda *a: A.attention_pytorch_sliding_window(*a, window_size=256)):
        out = fn(q, k, ones).float()
        assert (out - 1).abs().max().item() <= 8e-3      # softmax weights sum to 1 (bf16 rounding of P and out)
    # causal: the first query attends only key 0, so its output is value row 0 exactly
    assert torch.equal(A.attention_pytorch_causal(q, k, v)[:, :, 0], v[:, :, 0])
    # window 0 attends only the diagonal: output equals the values
    assert torch.equal(A.attention_pytorch_sliding_window(q, k, v, window_size=0), v)
    # linearity in V: f(2v) = 2 f(v) exactly (power-of-two scaling commutes with every rounding step)
    assert torch.equal(A.attention_pytorch_causal(q, k, (v.float() * 2).bfloat16()).float(),
                       A.attention_pytorch_causal(q, k, v).float() * 2)


def test_key_permutation_invariance_full_size():
    B, H, S, D = 1, 4, 4096, 128
    g = torch.Generator().manual_seed(22)
    q, k, v = (torch.randn(B, H, S, D, generator=g).bfloat16().to(DEV) for _ in range(3))
    perm = torch.randperm(S, generator=g).to(DEV)
    a = A.attention_pytorch(q, k, v).float()
    b = A.attention_pytorch(q, k[:, :, perm].contiguous(), v[:, :, perm].contiguous()).float()
    torch.testing.assert_close(a, b, rtol=2 ** -7, atol=4e-3)   # one bf16 ulp: the summation order differs


def test_documents_equal_independent_attention_full_size():
    from flashlight_amd import workloads as W
    w = W.workload_by_name("cfg3/document_mask_causal")
    t = w.make(DEV)
    out = w.call(t)
    lengths = W.document_lengths(16384, 1003)
    a = 0
    for n in lengths:
        sl = slice(a, a + n)
        alone = A.attention_pytorch_causal(t["q"][:, :, sl].contiguous(), t["k"][:, :, sl].contiguous(),
                                           t["v"][:, :, sl].contiguous())
        # the two launches tile the keys differently: allow one bf16 ulp (2^-7 relative) of the result
        torch.testing.assert_close(out[:, :, sl].float(), alone.float(), rtol=2 ** -7, atol=4e-3)
        a += n
