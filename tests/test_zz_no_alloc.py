"""The entry point that allocates nothing (fl_attn_fwd_static) against fl_attn_fwd, through the C ABI.

Two calls in a row on one GPU, the second with a smaller input: the static scratch keeps the first call's contents, and
the second call must not be disturbed by them.  Results must be bit-identical to fl_attn_fwd's (same kernels)."""
import ctypes as C

import pytest
import torch

from flashlight_amd import _ffi

DEV = "cuda"


def _doc_case(B, H, S, D, n_docs, seed):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(DEV) for _ in range(3))
    cuts = torch.sort(torch.randperm(S - 1, generator=g)[: n_docs - 1] + 1).values
    ids = torch.bucketize(torch.arange(S), cuts, right=True).to(torch.int64)
    ids = (ids * 7 - 3).unsqueeze(0).expand(B, S).contiguous().to(DEV)  # arbitrary integers, one id per document
    return q, k, v, ids


@pytest.mark.gpu
def test_static_scratch_matches_the_allocating_entry_point_twice_in_a_row():
    lib = _ffi.load_library()
    assert lib.fl_static_scratch_bytes() >= 1 << 20
    for (B, H, S, D, n_docs, seed) in ((2, 4, 4096, 64, 9, 1), (1, 2, 1000, 128, 4, 2)):  # the second call is smaller
        q, k, v, ids = _doc_case(B, H, S, D, n_docs, seed)
        for kind in (_ffi.MASK_DOCUMENT_CAUSAL, _ffi.MASK_DOCUMENT):
            want = _ffi.attn_fwd(q, k, v, mask_kind=kind, doc_ids=ids)
            out = torch.empty_like(want)
            n_alloc = torch.cuda.memory_stats()["allocation.all.allocated"]
            got = _ffi.attn_fwd(q, k, v, mask_kind=kind, doc_ids=ids, out=out, static_scratch=True)
            # the binding asked torch's allocator for nothing either (no workspace tensor)
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == n_alloc
            torch.cuda.synchronize()
            assert torch.equal(got, want), (B, H, S, D, kind)
    # a mask that needs no scratch goes through the same entry point
    q, k, v, _ = _doc_case(1, 2, 512, 64, 2, 3)
    assert torch.equal(_ffi.attn_fwd(q, k, v, mask_kind=_ffi.MASK_CAUSAL, static_scratch=True),
                       _ffi.attn_fwd(q, k, v, mask_kind=_ffi.MASK_CAUSAL))


def test_static_scratch_rejects_what_does_not_fit():
    lib = _ffi.load_library()
    p = _ffi.FlAttnParams()
    p.mask_kind, p.B, p.Lk = _ffi.MASK_DOCUMENT, 64, 1 << 20  # 64 * 32768 blocks * 16 bytes = 32 MiB
    assert lib.fl_workspace_bytes(C.byref(p)) > lib.fl_static_scratch_bytes()
    assert lib.fl_attn_fwd_static(C.byref(p), None) == -6  # FL_ERR_WORKSPACE
    assert b"static scratch" in lib.fl_last_error()
