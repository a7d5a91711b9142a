"""The variant functions under `torch.compile`: one `flashlight_amd::attn_fwd` node per call, no graph break
(the reference's callers wrap the same functions in `torch.compile`, benchmarks/run_flex_variants.py:118-124)."""
import pytest
import torch

import flashlight_amd.attention_variants as A
import flashlight_amd.ops  # noqa: F401  (registers the operator)
import oracle as O
from tests.conftest import assert_parity

BF = torch.bfloat16


class _Stop(Exception):
    pass


def _trace(fn, *args, **kwargs):
    """Compiles `fn` with a backend that records the FX graph and refuses to run it (tracing needs no GPU)."""
    graphs = []

    def backend(gm, example_inputs):
        graphs.append(gm)

        def run(*a):
            raise _Stop
        return run

    torch._dynamo.reset()
    with pytest.raises(_Stop):
        torch.compile(fn, backend=backend, fullgraph=True)(*args, **kwargs)
    assert len(graphs) == 1, "one graph, no break"
    return [n for n in graphs[0].graph.nodes if n.op == "call_function" and n.target is torch.ops.flashlight_amd.attn_fwd.default]


def _qkv(B=1, Hq=4, Hkv=2, S=64, D=64):
    g = torch.Generator().manual_seed(0)
    return (torch.randn(B, Hq, S, D, generator=g).to(BF), torch.randn(B, Hkv, S, D, generator=g).to(BF),
            torch.randn(B, Hkv, S, D, generator=g).to(BF))


ORACLE = {
    "vanilla": lambda q, k, v: O.attention_vanilla(q, k, v, enable_gqa=True),
    "causal": lambda q, k, v: O.attention_causal(q, k, v, enable_gqa=True),
    "sliding": lambda q, k, v: O.attention_sliding_window(q, k, v, window_size=16, enable_gqa=True),
    "prefix": lambda q, k, v: O.attention_prefix_lm(q, k, v, prefix_lengths=8, enable_gqa=True),
    "alibi": lambda q, k, v: O.attention_alibi(q, k, v, score_mod=q.size(-3), enable_gqa=True),
    "softcap": lambda q, k, v: O.attention_softcapped(q, k, v, score_mod=30.0, enable_gqa=True),
}
CASES = {
    "vanilla": lambda q, k, v: A.attention_pytorch(q, k, v, enable_gqa=True),
    "causal": lambda q, k, v: A.attention_pytorch_causal(q, k, v, enable_gqa=True),
    "sliding": lambda q, k, v: A.attention_pytorch_sliding_window(q, k, v, window_size=16, enable_gqa=True),
    "prefix": lambda q, k, v: A.attention_pytorch_prefix_lm(q, k, v, prefix_lengths=8, enable_gqa=True),
    "alibi": lambda q, k, v: A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(q.size(-3)), enable_gqa=True),
    "softcap": lambda q, k, v: A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(30.0), enable_gqa=True),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_variant_traces_into_one_operator(name):
    nodes = _trace(CASES[name], *_qkv())
    assert len(nodes) == 1
    # (unmasked grouped heads with so few queries reach the operator packed: the 2 query heads of a key / value head as
    # 128 rows of that head)
    assert tuple(nodes[0].meta["example_value"].shape) == ((1, 2, 128, 64) if name in ("vanilla", "softcap") else (1, 4, 64, 64))


def test_document_diff_and_evoformer_trace():
    q, k, v = _qkv()
    ids = torch.arange(64).div(20, rounding_mode="floor")[None]
    assert len(_trace(lambda q, k, v, ids: A.attention_pytorch_document_mask(q, k, v, ids, enable_gqa=True), q, k, v, ids)) == 1
    qd, kd, _ = _qkv(Hq=4, Hkv=4)
    vd = torch.randn(1, 2, 64, 128).to(BF)
    nodes = _trace(lambda q, k, v: A.diffattn(q, k, v, lambda_full=0.5, is_causal=True), qd, kd, vd)
    assert len(nodes) == 1 and tuple(nodes[0].meta["example_value"].shape) == (1, 2, 64, 128)
    Q, K, V, G = (torch.randn(1, 3, 40, 2, 32).to(BF) for _ in range(4))
    pair, mask = torch.randn(1, 1, 2, 40, 40).to(BF), torch.randn(1, 3, 1, 1, 40).to(BF)
    nodes = _trace(lambda Q, K, V, m, p, G: A.attention_reference(Q, K, V, [m, p], gate=G), Q, K, V, mask, pair, G)
    assert len(nodes) == 1
    # [prod(*), H, S, D] view of a [prod(*), S, H, D] buffer
    val = nodes[0].meta["example_value"]
    assert tuple(val.shape) == (3, 2, 40, 32) and val.stride() == (40 * 2 * 32, 32, 2 * 32, 1)


def test_dense_score_mod_and_ipa_trace():
    q, k, v = _qkv(Hq=4, Hkv=4)
    dense = torch.randn(4, 64, 64)
    nodes = _trace(lambda q, k, v, d: A.attention_pytorch_alibi(q, k, v, score_mod=lambda l, s: d, is_causal=True), q, k, v, dense)
    assert len(nodes) == 1 and nodes[0].args[10].meta["example_value"].dtype == torch.float32  # bias0 stays fp32
    r = lambda *s: torch.randn(*s).to(BF)  # noqa: E731
    args = (r(2, 4, 48, 16), r(2, 4, 48, 16), r(2, 4, 48, 16), r(2, 4, 48, 4, 3), r(2, 4, 48, 4, 3), r(2, 4, 48, 8, 3),
            r(2, 4, 48, 48))
    nodes = _trace(lambda *a: A.invariant_point_attention(*a, c_hidden=16, no_qk_points=4), *args)
    assert len(nodes) == 1
    # scalar and point channels of q/k padded from 28 to 32, of v from 40 to 64
    assert tuple(nodes[0].args[0].meta["example_value"].shape) == (2, 4, 48, 32)
    assert tuple(nodes[0].meta["example_value"].shape) == (2, 4, 48, 64)


@pytest.mark.gpu
def test_compiled_equals_eager_on_gpu():
    dev = "cuda"
    q, k, v = (t.to(dev) for t in _qkv(B=2, Hq=8, Hkv=2, S=300, D=64))
    for name, fn in CASES.items():
        torch._dynamo.reset()
        got = torch.compile(fn, backend="aot_eager", fullgraph=True)(q, k, v)
        assert torch.equal(got, fn(q, k, v)), name
        # and against the CPU oracle: the compiled graph computes the right thing, not merely the same thing
        want = ORACLE[name](q.float().cpu(), k.float().cpu(), v.float().cpu())
        assert_parity(got.reshape(want.shape), want, f"compiled {name}")
    Q, K, V, G = (torch.randn(1, 3, 104, 2, 32, device=dev).to(BF) for _ in range(4))
    pair, mask = torch.randn(1, 1, 2, 104, 104, device=dev).to(BF), torch.randn(1, 3, 1, 1, 104, device=dev).to(BF)
    fn = lambda Q, K, V, m, p, G: A.attention_reference(Q, K, V, [m, p], gate=G)
    torch._dynamo.reset()
    got = torch.compile(fn, backend="aot_eager", fullgraph=True)(Q, K, V, mask, pair, G)
    want = fn(Q, K, V, mask, pair, G)
    assert got.shape == want.shape and torch.equal(got, want)
    torch.library.opcheck(torch.ops.flashlight_amd.attn_fwd.default,
                          (q, k, v, -1.0, 1, 0, 0, None, 0, 0.0, None, 1, None, 1, None, False, 0.0, False))


@pytest.mark.gpu
def test_compiled_gradients_with_bias_gate_and_differential_attention():
    """Gradients through `torch.compile` (aot_eager: forward and backward graphs are traced, the fused calls stay opaque
    operators) for the calls whose backward is a composition: Evoformer attention with two bias operands and the
    gate, and differential attention.  Each must give what differentiating the eager call gives."""
    dev = "cuda"
    g = torch.Generator().manual_seed(3)
    mk = lambda *s: torch.randn(*s, generator=g).to(BF).to(dev)  # noqa: E731

    def grads(fn, args):
        leaves = [a.detach().clone().requires_grad_(True) for a in args]
        out = fn(*leaves)
        out.float().square().sum().backward()
        return [out.detach()] + [leaf.grad for leaf in leaves]

    Q, K, V, G = (mk(1, 3, 104, 2, 32) for _ in range(4))
    pair, mask = mk(1, 1, 2, 104, 104), mk(1, 3, 1, 1, 104)
    evo = lambda Q, K, V, m, p, G: A.attention_reference(Q, K, V, [m, p], gate=G)  # noqa: E731
    q, k, v = mk(2, 8, 200, 64), mk(2, 8, 200, 64), mk(2, 4, 200, 128)
    diff = lambda q, k, v: A.diffattn(q, k, v, lambda_full=0.3, is_causal=True)  # noqa: E731
    for name, fn, args in (("evoformer", evo, (Q, K, V, mask, pair, G)), ("diffattn", diff, (q, k, v))):
        torch._dynamo.reset()
        want = grads(fn, args)
        got = grads(torch.compile(fn, backend="aot_eager", fullgraph=True), args)
        for i, (a, b) in enumerate(zip(got, want)):
            assert a.shape == b.shape, f"{name}: output {i}"
            scale = max(1.0, b.float().abs().max().item())
            assert (a.float() - b.float()).abs().max().item() <= 2e-2 * scale, f"{name}: output {i}"
    torch.library.opcheck(torch.ops.flashlight_amd.attn_fwd_bias_lse.default,
                          (mk(2, 2, 64, 32), mk(2, 2, 64, 32), mk(2, 2, 64, 32), -1.0, 0, 0, 0, mk(1, 2, 64, 64), 2, None, 1))


@pytest.mark.gpu
def test_variants_under_the_default_backend():
    """`torch.compile(dynamic=False)(fn)` with no backend named (Inductor) is how the reference's scripts call these
    functions (tests/test_causal.py:33, benchmarks/run_flex_variants.py:118-124): the operator goes through as an
    external kernel, forward and backward."""
    g = torch.Generator().manual_seed(0)
    B, Hq, Hkv, S, D = 2, 8, 2, 300, 64
    q, k, v = (torch.randn(B, h, S, D, generator=g).to(BF) for h in (Hq, Hkv, Hkv))
    ids = torch.sort(torch.randint(0, 4, (B, S), generator=g), dim=1).values
    f = lambda t: t.float()
    dev = lambda *ts: tuple(t.to("cuda") for t in ts)
    cases = {
        "vanilla": (lambda q, k, v: A.attention_pytorch(q, k, v, enable_gqa=True),
                    lambda: O.attention_vanilla(f(q), f(k), f(v), enable_gqa=True)),
        "sliding": (lambda q, k, v: A.attention_pytorch_sliding_window(q, k, v, window_size=50, enable_gqa=True),
                    lambda: O.attention_sliding_window(f(q), f(k), f(v), window_size=50, enable_gqa=True)),
        "softcap": (lambda q, k, v: A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(30.0), enable_gqa=True),
                    lambda: O.attention_softcapped(f(q), f(k), f(v), score_mod=30.0, enable_gqa=True)),
        "document": (lambda q, k, v: A.attention_pytorch_document_mask(q, k, v, ids.to("cuda"), enable_gqa=True),
                     lambda: O.attention_document_mask(f(q), f(k), f(v), ids, enable_gqa=True)),
    }
    for name, (fn, ref) in cases.items():
        torch._dynamo.reset()
        got = torch.compile(fn, dynamic=False, fullgraph=True)(*dev(q, k, v))
        want = ref()
        assert_parity(got.reshape(want.shape), want, name)
    # a training step: causal, gradients against autograd through the oracle
    torch._dynamo.reset()
    leaves = [t.requires_grad_(True) for t in dev(q, k, v)]
    out = torch.compile(lambda q, k, v: A.attention_pytorch_causal(q, k, v, enable_gqa=True), dynamic=False, fullgraph=True)(*leaves)
    w = torch.randn(out.shape, generator=g)
    (out.float() * w.to("cuda")).sum().backward()
    refs = [f(t).requires_grad_(True) for t in (q, k, v)]
    want = O.attention_causal(*refs, enable_gqa=True)
    (want * w.reshape(want.shape)).sum().backward()
    assert_parity(out.reshape(want.shape), want, "causal")
    for name, a, b in zip(("dq", "dk", "dv"), leaves, refs):
        scale = max(1.0, b.grad.abs().max().item())
        assert_parity(a.grad / scale, b.grad / scale, name)
    # the two variants with layouts of their own
    torch._dynamo.reset()
    qd, kd = (torch.randn(2, 8, 200, 64, generator=g).to(BF) for _ in range(2))
    vd = torch.randn(2, 4, 200, 128, generator=g).to(BF)
    got = torch.compile(lambda q, k, v: A.diffattn(q, k, v, lambda_full=0.8), dynamic=False, fullgraph=True)(*dev(qd, kd, vd))
    want = O.diff_attention(f(qd), f(kd), f(vd), lambda_full=0.8)
    assert_parity(got.reshape(want.shape), want, "diffattn")
    torch._dynamo.reset()
    Q, K, V = (torch.randn(1, 8, 96, 4, 32, generator=g).to(BF) for _ in range(3))
    mb, pb = torch.randn(1, 8, 1, 1, 96, generator=g).to(BF), torch.randn(1, 1, 4, 96, 96, generator=g).to(BF)
    got = torch.compile(lambda Q, K, V, a, b: A.attention_reference(Q, K, V, [a, b]), dynamic=False, fullgraph=True)(*dev(Q, K, V, mb, pb))
    want = O.attention_evoformer(f(Q), f(K), f(V), [f(mb), f(pb)])
    assert_parity(got.reshape(want.shape), want, "evoformer")
