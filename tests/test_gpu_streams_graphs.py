"""The library launches on the caller's current stream, allocates nothing and never synchronises, so a call can sit on a
side stream or inside a captured HIP graph.  Every replay of a graph is compared with the eager call on the same
operands (bit-exact: the same kernels on the same data), with eager work and synchronisations between the replays."""
import pytest
import torch

import flashlight_amd.attention_variants as A

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _qkv(B, H, S, D, seed):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(B, H, S, D, generator=g).to(torch.bfloat16).to(DEV) for _ in range(3))


def test_launches_on_the_callers_stream():
    q_old, k, v = _qkv(2, 4, 300, 64, 1)
    q_new = _qkv(2, 4, 300, 64, 2)[0]
    want = A.attention_pytorch_causal(q_new, k, v)
    torch.cuda.synchronize()
    q = q_old.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        torch.cuda._sleep(40_000_000)  # the side stream is busy for a while; the default stream is idle
        q.copy_(q_new)                 # queued behind the sleep
        out = A.attention_pytorch_causal(q, k, v)  # on the side stream it sees the new q; on any other, the old one
    side.synchronize()
    assert torch.equal(out, want)


def _replay_against_eager(make_call, operands, fresh):
    """Captures make_call(*operands) once, then replays it on three fresh sets of operand values."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up outside the capture, as torch.cuda.graph asks
        make_call(*operands)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = make_call(*operands)
    for i in range(3):
        for dst, src in zip(operands, fresh(i)):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        eager = make_call(*operands)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i}"


def test_forward_in_a_captured_graph_causal_gqa():
    g = torch.Generator().manual_seed(3)
    q = torch.randn(2, 8, 257, 128, generator=g).to(torch.bfloat16).to(DEV)
    k, v = (torch.randn(2, 2, 257, 128, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))

    def fresh(i):
        gi = torch.Generator().manual_seed(100 + i)
        return (torch.randn(q.shape, generator=gi).to(torch.bfloat16).to(DEV),
                torch.randn(k.shape, generator=gi).to(torch.bfloat16).to(DEV),
                torch.randn(v.shape, generator=gi).to(torch.bfloat16).to(DEV))

    _replay_against_eager(lambda a, b, c: A.attention_pytorch_causal(a, b, c, enable_gqa=True), (q, k, v), fresh)


def test_forward_in_a_captured_graph_document_mask():
    """Three kernels per call (the two pre-pass kernels and the forward) and a workspace from torch's allocator."""
    q, k, v = _qkv(2, 4, 700, 64, 5)
    ids = torch.sort(torch.randint(0, 6, (2, 700), generator=torch.Generator().manual_seed(6)), dim=1).values.to(DEV)

    def fresh(i):
        gi = torch.Generator().manual_seed(200 + i)
        new_ids = torch.sort(torch.randint(0, 3 + 4 * i, (2, 700), generator=gi), dim=1).values.to(DEV)
        return (*_qkv(2, 4, 700, 64, 300 + i), new_ids)

    _replay_against_eager(lambda a, b, c, d: A.attention_pytorch_document_mask(a, b, c, d, is_causal=True),
                          (q, k, v, ids), fresh)


def test_forward_in_a_captured_graph_shared_bias_kernel():
    g = torch.Generator().manual_seed(7)
    shape = (1, 16, 256, 4, 32)
    q, k, v, gate = (torch.randn(shape, generator=g).to(torch.bfloat16).to(DEV) for _ in range(4))
    bias = torch.randn(1, 1, 4, 256, 256, generator=g).to(torch.bfloat16).to(DEV)

    def fresh(i):
        gi = torch.Generator().manual_seed(400 + i)
        return (*(torch.randn(shape, generator=gi).to(torch.bfloat16).to(DEV) for _ in range(4)),
                torch.randn(bias.shape, generator=gi).to(torch.bfloat16).to(DEV))

    _replay_against_eager(lambda a, b, c, d, e: A.attention_reference(a, b, c, [e], gate=d), (q, k, v, gate, bias), fresh)


def test_training_step_in_a_captured_graph_with_the_static_scratch_backward():
    """Forward with row statistics, then the backward that allocates nothing (`static_scratch`: the library's own
    device array is its scratch), results into tensors made beforehand: the whole step is captured and replayed."""
    from flashlight_amd import _ffi
    B, Hq, Hkv, L, D = 2, 4, 2, 333, 64
    g = torch.Generator().manual_seed(11)
    q = torch.randn(B, Hq, L, D, generator=g).to(torch.bfloat16).to(DEV)
    k, v = (torch.randn(B, Hkv, L, D, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    dout = torch.randn(B, Hq, L, D, generator=g).to(torch.bfloat16).to(DEV)
    out, lse = torch.empty_like(q), torch.empty(B, Hq, L, dtype=torch.float32, device=DEV)
    grads = (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v))

    def step(q_, k_, v_, dout_):
        _ffi.attn_fwd(q_, k_, v_, mask_kind=_ffi.MASK_CAUSAL, out=out, lse=lse)
        _ffi.attn_bwd(q_, k_, v_, out, lse, dout_, mask_kind=_ffi.MASK_CAUSAL, static_scratch=True, grads=grads)
        return torch.cat([t.reshape(-1) for t in (out, *grads)])

    def eager(q_, k_, v_, dout_):
        o = torch.empty_like(q_)
        s = torch.empty_like(lse)
        _ffi.attn_fwd(q_, k_, v_, mask_kind=_ffi.MASK_CAUSAL, out=o, lse=s)
        return torch.cat([t.reshape(-1) for t in (o, *_ffi.attn_bwd(q_, k_, v_, o, s, dout_, mask_kind=_ffi.MASK_CAUSAL))])

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(q, k, v, dout)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        flat = step(q, k, v, dout)
    for i in range(3):
        gi = torch.Generator().manual_seed(500 + i)
        for t in (q, k, v, dout):
            t.copy_(torch.randn(t.shape, generator=gi).to(torch.bfloat16))
        graph.replay()
        torch.cuda.synchronize()
        want = eager(q, k, v, dout)
        torch.cuda.synchronize()
        assert torch.equal(flat, want), f"replay {i}"


def test_results_repeat_bit_for_bit():
    """No atomics and a fixed order of accumulation: the same call twice gives the same bits, forward and backward,
    whatever else ran in between (here: the other call's launches, queued on the same stream)."""
    from flashlight_amd import _ffi
    g = torch.Generator().manual_seed(13)
    q = torch.randn(2, 8, 700, 64, generator=g).to(torch.bfloat16).to(DEV)
    k, v = (torch.randn(2, 2, 700, 64, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    dout = torch.randn(2, 8, 700, 64, generator=g).to(torch.bfloat16).to(DEV)
    ids = torch.sort(torch.randint(0, 7, (2, 700), generator=g), dim=1).values.to(DEV)

    def once():
        outs = []
        for kw in (dict(mask_kind=_ffi.MASK_CAUSAL), dict(mask_kind=_ffi.MASK_DOCUMENT_CAUSAL, doc_ids=ids),
                   dict(mask_kind=_ffi.MASK_SLIDING, window=100, alibi_heads=8, softcap=20.0)):
            lse = torch.empty(2, 8, 700, dtype=torch.float32, device=DEV)
            out = _ffi.attn_fwd(q, k, v, lse=lse, **kw)
            outs += [out, lse, *_ffi.attn_bwd(q, k, v, out, lse, dout, **kw)]
        return outs

    first, second = once(), once()
    torch.cuda.synchronize()
    for a, b in zip(first, second):
        assert torch.equal(a, b)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 32, 8, 1, 32768, 128), (1, 8, 2, 2, 8201, 64), (4, 16, 4, 1, 8192, 128), (16, 32, 8, 1, 1024, 128)])
def test_decoding_steps_replay_from_a_graph(shape):
    """A serving loop replays its decoding step from a graph.  The front end's reshapes for such calls (query heads as
    rows; key chunks as batch entries or heads, a shorter last chunk, the merge launch) allocate their buffers inside the
    capture and record plain launches only: every replay, on new cache contents, equals the eager call."""
    B, Hq, Hkv, Lq, Lk, D = shape
    g = torch.Generator().manual_seed(Lk)
    q = torch.randn(B, Hq, Lq, D, generator=g).to(torch.bfloat16).to(DEV)
    k, v = (torch.randn(B, Hkv, Lk, D, generator=g).to(torch.bfloat16).to(DEV) for _ in range(2))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            A.attention_pytorch(q, k, v, enable_gqa=True)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = A.attention_pytorch(q, k, v, enable_gqa=True)
    for step in range(3):
        q.copy_(torch.randn(q.shape, generator=g).to(torch.bfloat16))
        k[:, :, step::3].mul_(-0.5)
        v.copy_(torch.randn(v.shape, generator=g).to(torch.bfloat16))
        graph.replay()
        torch.cuda.synchronize()
        eager = A.attention_pytorch(q, k, v, enable_gqa=True)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), (shape, step)
