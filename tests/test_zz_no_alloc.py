"""The entry point that allocates nothing (fl_attn_bwd_static) against fl_attn_bwd, through the C ABI.

Two calls in a row on one GPU, the second with a smaller input: the static scratch keeps the first call's contents (row
sums, document table), and the second call must not be disturbed by them.  Results must be bit-identical to
fl_attn_bwd's (same kernels, same order of operations)."""
import ctypes as C

import pytest
import torch

from flashlight_amd import _ffi

DEV = "cuda"


def _doc_case(B, H, S, D, n_docs, seed):
    g = torch.Generator().manual_seed(seed)
    q, k, v, dout = (torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(DEV) for _ in range(4))
    cuts = torch.sort(torch.randperm(S - 1, generator=g)[: n_docs - 1] + 1).values
    ids = torch.bucketize(torch.arange(S), cuts, right=True).to(torch.int64)
    ids = (ids * 7 - 3).unsqueeze(0).expand(B, S).contiguous().to(DEV)  # arbitrary integers, one id per document
    return q, k, v, dout, ids


@pytest.mark.gpu
def test_static_scratch_matches_the_allocating_entry_point_twice_in_a_row():
    lib = _ffi.load_library()
    assert lib.fl_static_scratch_bytes() >= 1 << 20
    for (B, H, S, D, n_docs, seed) in ((2, 4, 4096, 64, 9, 1), (1, 2, 1000, 128, 4, 2)):  # the second call is smaller
        q, k, v, dout, ids = _doc_case(B, H, S, D, n_docs, seed)
        for kind, doc in ((_ffi.MASK_DOCUMENT_CAUSAL, ids), (_ffi.MASK_DOCUMENT, ids), (_ffi.MASK_CAUSAL, None)):
            lse = torch.empty(B, H, S, dtype=torch.float32, device=DEV)
            out = _ffi.attn_fwd(q, k, v, mask_kind=kind, doc_ids=doc, lse=lse)
            want = _ffi.attn_bwd(q, k, v, out, lse, dout, mask_kind=kind, doc_ids=doc)
            grads = tuple(torch.empty_like(t) for t in (q, k, v))
            n_alloc = torch.cuda.memory_stats()["allocation.all.allocated"]
            got = _ffi.attn_bwd(q, k, v, out, lse, dout, mask_kind=kind, doc_ids=doc, static_scratch=True, grads=grads)
            # the binding asked torch's allocator for nothing either (no row-sum tensor, no workspace)
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == n_alloc
            torch.cuda.synchronize()
            for name, a, b in zip(("dq", "dk", "dv"), got, want):
                assert torch.equal(a, b), (name, B, H, S, D, kind)


@pytest.mark.gpu
def test_static_scratch_refuses_a_call_that_would_overlap_on_another_stream():
    """All calls on a GPU share the static array.  A call on a second stream while the first call's kernels are still
    running is refused (FL_ERR_WORKSPACE) instead of racing; the same stream, or the other stream once the first call
    has finished, passes and gives the same gradients."""
    B, H, S, D = 8, 16, 4096, 128   # a backward of a few milliseconds, 2 MiB of row sums
    g = torch.Generator().manual_seed(3)
    q, k, v, dout = (torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(DEV) for _ in range(4))
    lse = torch.empty(B, H, S, dtype=torch.float32, device=DEV)
    out = _ffi.attn_fwd(q, k, v, mask_kind=_ffi.MASK_CAUSAL, lse=lse)
    want = _ffi.attn_bwd(q, k, v, out, lse, dout, mask_kind=_ffi.MASK_CAUSAL)
    g1, g2 = (tuple(torch.empty_like(t) for t in (q, k, v)) for _ in range(2))
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    call = lambda grads: _ffi.attn_bwd(q, k, v, out, lse, dout, mask_kind=_ffi.MASK_CAUSAL, static_scratch=True, grads=grads)
    with torch.cuda.stream(s1):
        call(g1)
    with torch.cuda.stream(s2):
        with pytest.raises(_ffi.FlashlightError, match="still in use") as err:
            call(g2)
    assert err.value.code == -6
    with torch.cuda.stream(s1):     # behind the first call on its own stream: ordered, accepted
        call(g1)
    torch.cuda.synchronize()
    with torch.cuda.stream(s2):     # the first stream has drained
        call(g2)
    torch.cuda.synchronize()
    for name, a, b, c in zip(("dq", "dk", "dv"), g1, g2, want):
        assert torch.equal(a, c) and torch.equal(b, c), name


def test_static_scratch_rejects_what_does_not_fit():
    lib = _ffi.load_library()
    b = _ffi.FlAttnBwdParams()
    b.fwd.B, b.fwd.Hq, b.fwd.Lq = 8, 64, 8192  # 16 MiB of row sums
    assert 8 * 64 * 8192 * 4 > lib.fl_static_scratch_bytes()
    assert lib.fl_attn_bwd_static(C.byref(b), None) == -6  # FL_ERR_WORKSPACE, before anything else is looked at
    assert b"static scratch" in lib.fl_last_error()
