"""Parity of the HIP kernels (through the C ABI) with the CPU oracle and the committed known-answer vectors.
Tolerance: bf16 kernel against an fp32/fp64 reference, max-abs 2e-2 and mean-abs 2e-3."""
import math
import random

import pytest
import torch

import flashlight_amd.attention_variants as A
import oracle as O
from flashlight_amd import _ffi
from flashlight_amd import workloads as W
from tests.conftest import assert_parity
from tests.variant_calls import GOLDEN_NAMES, hip_call

pytestmark = pytest.mark.gpu
DEV = "cuda"


def f32(*ts):
    return tuple(t.float() for t in ts)


def qkv(B, Hq, Hkv, S, D, Dv=None, seed=0, lo_hi=None):
    g = torch.Generator().manual_seed(seed)
    shapes = [(B, Hq, S, D), (B, Hkv, S, D), (B, Hkv, S, Dv or D)]
    if lo_hi is None:
        ts = [torch.randn(s, generator=g) for s in shapes]
    else:  # the reference's tests draw uniformly in [-9, 9] (torch.testing.make_tensor defaults)
        ts = [torch.rand(s, generator=g) * (lo_hi[1] - lo_hi[0]) + lo_hi[0] for s in shapes]
    return tuple(t.to(torch.bfloat16).to(DEV) for t in ts)


@pytest.mark.parametrize("name", GOLDEN_NAMES)
def test_known_answer_vectors(golden, name):
    case = golden[name]
    out = hip_call(name, case.to(DEV), case.meta)
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16
    assert_parity(out, case.expected, name)


def oracle_for(w: W.Workload, t: dict, q_block):
    """fp32 oracle evaluation of a benchmark workload, on the tensors' device (plain eager PyTorch either way)."""
    from oracle.benchmark_cases import evaluate
    return evaluate(w.name, {k: (v.float() if v.is_floating_point() else v) for k, v in t.items()}, w.params, q_block)


WORKLOAD_NAMES = [w.name for w in W.build_workloads()]


@pytest.mark.parametrize("name", WORKLOAD_NAMES)
def test_benchmark_configs_reduced(name):
    """Every benchmark configuration at 1/4 sequence length, oracle on the host CPU."""
    w = W.workload_by_name(name, scale_down=4)
    t = w.make(DEV)
    out = w.call(t)
    torch.cuda.synchronize()
    ref = oracle_for(w, {k: v.cpu() for k, v in t.items()}, q_block=512)
    assert_parity(out, ref, name)


@pytest.mark.parametrize("name", WORKLOAD_NAMES)
def test_benchmark_configs_full_size(name):
    """Full benchmark sizes.  The oracle (same eager fp32 code) is evaluated on the GPU tensors, in blocks of
    query rows, because the dense score matrices do not fit a CPU run of a few seconds."""
    w = W.workload_by_name(name)
    t = w.make(DEV)
    out = w.call(t)
    torch.cuda.synchronize()
    ref = oracle_for(w, t, q_block=512)
    assert_parity(out, ref, name)
    del ref, out, t
    torch.cuda.empty_cache()


# ---- shapes and input distribution of the reference's own test scripts (tests/test_*.py there), sequence lengths
# ---- kept, batch reduced where the fp32 oracle would not fit; inputs uniform in [-9, 9] like make_tensor.
# ---- Outputs reach magnitude 9 there, where one bf16 ulp is 0.03, so these use the tolerance those scripts state:
# ---- assert_close(atol=2e-2, rtol=1e-2) (e.g. tests/test_causal.py:36 of the reference).

def assert_script_tolerance(out, ref, what=""):
    """The reference scripts' own check, every element: |out - ref| <= 2e-2 + 1e-2 |ref|
    (torch.testing.assert_close(atol=2e-2, rtol=1e-2), e.g. tests/test_causal.py:36, tests/test_alibi.py:40 there).
    On failure the message carries the worst excess over the bound and how many elements are past it."""
    assert tuple(out.shape) == tuple(ref.shape), what
    o, r = out.float(), ref.float().to(out.device)
    assert torch.isfinite(o).all(), what
    excess = (o - r).abs() / (2e-2 + 1e-2 * r.abs())
    n_over = int((excess > 1).sum().item())
    print(f"[script tolerance] {what}: worst {excess.max().item():.3f} x bound, {n_over} of {excess.numel()} over")
    assert n_over == 0, f"{what}: worst {excess.max().item():.3f} x bound, {n_over} of {excess.numel()} elements over"


@pytest.mark.parametrize("D", [64, 128])
def test_sequences_of_65536_through_size_independent_properties(D):
    """Too long for the CPU oracle: (1) the unmasked result equals the merge, through the row statistics, of four calls
    that each see a quarter of the keys; (2) a document mask over sorted ids equals separate calls per document, with and
    without the causal term.  Both sides are 16-bit results of the same kernels on different tilings and list lengths,
    so the bound is the suite's (max-abs 2e-2, mean-abs 2e-3)."""
    L, H = 65536, 2
    g = torch.Generator().manual_seed(65 + D)
    q, k, v = (torch.randn(1, H, L, D, generator=g).to(torch.bfloat16).to(DEV) for _ in range(3))
    lse = torch.empty(1, H, L, dtype=torch.float32, device=DEV)
    full = _ffi.attn_fwd(q, k, v, lse=lse).float()
    parts, stats = [], []
    for c in range(4):
        ks = slice(c * L // 4, (c + 1) * L // 4)
        st = torch.empty(1, H, L, dtype=torch.float32, device=DEV)
        parts.append(_ffi.attn_fwd(q, k[:, :, ks], v[:, :, ks], lse=st, scale=1.0 / math.sqrt(D)).float())
        stats.append(st)
    stats = torch.stack(stats)                                   # log2 of the row sums
    total = torch.logsumexp(stats * math.log(2.0), dim=0) / math.log(2.0)
    merged = sum(p * torch.exp2(st - total).unsqueeze(-1) for p, st in zip(parts, stats))
    assert_parity(full, merged, "65536 keys against four quarters")
    assert (lse - total).abs().max().item() < 2e-2
    lengths = [20000, 1, 30001, 15534]
    ids = torch.repeat_interleave(torch.arange(4), torch.tensor(lengths)).view(1, L).to(DEV)
    for causal in (False, True):
        got = A.attention_pytorch_document_mask(q, k, v, ids, is_causal=causal)
        a = 0
        for n in lengths:
            sl = slice(a, a + n)
            fn = A.attention_pytorch_causal if causal else A.attention_pytorch
            want = fn(q[:, :, sl], k[:, :, sl], v[:, :, sl], scale=1.0 / math.sqrt(D))
            assert_parity(got[:, :, sl], want, f"document of {n} positions at {a}, causal={causal}")
            a += n


def test_reference_script_vanilla_and_causal():   # tests/test_vanilla.py:21-36, tests/test_causal.py:21-36
    q, k, v = qkv(2, 1, 1, 16384, 128, seed=1, lo_hi=(-9, 9))
    assert_script_tolerance(A.attention_pytorch(q, k, v), O.attention_vanilla(*f32(q, k, v), q_block=1024), "vanilla")
    assert_script_tolerance(A.attention_pytorch_causal(q, k, v), O.attention_causal(*f32(q, k, v), q_block=1024), "causal")


def test_reference_script_alibi():                 # tests/test_alibi.py:20-40
    q, k, v = qkv(4, 16, 2, 1024, 64, seed=2, lo_hi=(-9, 9))
    out = A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(q.size(-3)), enable_gqa=True)
    assert out.shape == (4, 2, 8, 1024, 64)
    assert_script_tolerance(out, O.attention_alibi(*f32(q, k, v), score_mod=16, enable_gqa=True), "alibi")


def test_reference_script_sliding_window():        # tests/test_sliding_window.py:13-33
    q, k, v = qkv(4, 16, 2, 1024, 64, seed=3, lo_hi=(-9, 9))
    out = A.attention_pytorch_sliding_window(q, k, v, window_size=256, enable_gqa=True)
    assert_script_tolerance(out, O.attention_sliding_window(*f32(q, k, v), window_size=256, enable_gqa=True), "sliding")


def test_reference_script_prefix_lm():             # tests/test_prefix_lm.py:14-34 (batch 32 -> 4)
    q, k, v = qkv(4, 16, 2, 1024, 64, seed=4, lo_hi=(-9, 9))
    out = A.attention_pytorch_prefix_lm(q, k, v, prefix_lengths=256, enable_gqa=True)
    assert_script_tolerance(out, O.attention_prefix_lm(*f32(q, k, v), prefix_lengths=256, enable_gqa=True), "prefix")


def test_reference_script_document_mask():         # tests/test_document_mask.py:15-35
    q, k, v = qkv(1, 16, 2, 16384, 64, seed=5, lo_hi=(-9, 9))
    random.seed(0)
    ids = A.create_document_id(1, 16384, 12, device=DEV)
    assert ids.shape == (1, 16384) and ids.dtype == torch.int64 and int(ids.max()) == 11
    out = A.attention_pytorch_document_mask(q, k, v, ids, enable_gqa=True)
    assert_script_tolerance(out, O.attention_document_mask(*f32(q, k, v), ids, enable_gqa=True, q_block=1024), "document")


def test_reference_script_gqa():                   # tests/test_gqa.py:69-96 (batch 32 -> 2), tolerance 1e-2 there
    q, k, v = qkv(2, 16, 2, 4096, 64, seed=6, lo_hi=(-9, 9))
    out = A.attention_pytorch(q, k, v, enable_gqa=True)
    assert out.shape == (2, 16, 4096, 64)
    assert_script_tolerance(out, O.attention_vanilla(*f32(q, k, v), enable_gqa=True, q_block=1024), "gqa")


def test_reference_script_diffattn():              # tests/test_diffattn.py:20-41: head_dim 128, value dim 256
    # (batch 4 instead of 16 to keep the fp32 oracle small); the 256 value columns go through two launches
    q, k, v = qkv(4, 16, 16, 1024, 128, Dv=256, seed=7, lo_hi=(-9, 9))
    v = v[:, :8].contiguous()
    assert_script_tolerance(A.diffattn(q, k, v), O.diff_attention(*f32(q, k, v)), "diffattn 128/256")
    # the benchmark's other shape: head_dim 64, value dim 128 (diff_attn.py:33-38 with nheads = 32)
    q, k, v = qkv(4, 16, 16, 1024, 64, Dv=128, seed=7, lo_hi=(-9, 9))
    v = v[:, :8].contiguous()
    assert_script_tolerance(A.diffattn(q, k, v), O.diff_attention(*f32(q, k, v)), "diffattn 64/128")


def test_reference_script_evoformer():             # tests/test_evoattn.py:21-71 (randn inputs, batch 2)
    g = torch.Generator().manual_seed(8)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(DEV)
    B, N, S, H, D = 2, 256, 256, 4, 32
    Q, K, V = mk(B, N, S, H, D), mk(B, N, S, H, D), mk(B, N, S, H, D)
    b1, b2 = mk(B, N, 1, 1, S), mk(B, 1, H, S, S)
    out = A.attention_reference(Q, K, V, [b1, b2], 1 / math.sqrt(D))
    assert out.shape == (B, N, S, H, D)
    ref = O.attention_evoformer(*f32(Q, K, V), [b1.float(), b2.float()], 1 / math.sqrt(D))
    assert_script_tolerance(out, ref, "evoformer")


# ---- edge cases ----------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("S", [1, 2, 31, 63, 64, 65, 255, 256, 257, 1000])
@pytest.mark.parametrize("D", [32, 64, 128])
def test_ragged_lengths(S, D):
    q, k, v = qkv(1, 2, 1, S, D, seed=S + D)
    qf, kf, vf = f32(q, k, v)
    assert_parity(A.attention_pytorch(q, k, v, enable_gqa=True), O.attention_vanilla(qf, kf, vf, enable_gqa=True))
    assert_parity(A.attention_pytorch_causal(q, k, v, enable_gqa=True).flatten(1, 2),
                  O.attention_causal(qf, kf, vf, enable_gqa=True).flatten(1, 2))
    assert_parity(A.attention_pytorch_sliding_window(q, k, v, window_size=40, enable_gqa=True),
                  O.attention_sliding_window(qf, kf, vf, window_size=40, enable_gqa=True))


def test_cross_attention_lengths_differ():
    g = torch.Generator().manual_seed(11)
    q = torch.randn(2, 2, 300, 64, generator=g).bfloat16().to(DEV)
    k = torch.randn(2, 2, 77, 64, generator=g).bfloat16().to(DEV)
    v = torch.randn(2, 2, 77, 64, generator=g).bfloat16().to(DEV)
    assert_parity(A.attention_pytorch(q, k, v), O.attention_vanilla(*f32(q, k, v)))
    # causal is top-left aligned (causal.py:32): query rows beyond the keys see every key
    assert_parity(A.attention_pytorch_causal(q, k, v), O.attention_causal(*f32(q, k, v)))
    assert_parity(A.attention_pytorch_causal(k, q, q), O.attention_causal(*f32(k, q, q)))


def test_strided_inputs_and_explicit_scale():
    g = torch.Generator().manual_seed(12)
    packed = torch.randn(2, 200, 3, 4, 64, generator=g).bfloat16().to(DEV)   # [B, S, 3, H, D] as benchmarks/_utils.py:221-240
    q, k, v = (packed[:, :, i].transpose(1, 2) for i in range(3))            # non-contiguous [B, H, S, D] views
    assert not q.is_contiguous()
    assert_parity(A.attention_pytorch(q, k, v, scale=0.3), O.attention_vanilla(*f32(q, k, v), scale=0.3))
    assert_parity(A.attention_pytorch_causal(q, k, v, scale=0.05), O.attention_causal(*f32(q, k, v), scale=0.05))


def test_document_ids_arbitrary_values_and_per_batch():
    q, k, v = qkv(2, 2, 2, 500, 64, seed=13)
    g = torch.Generator().manual_seed(14)
    ids = torch.randint(-3, 3, (2, 500), generator=g).to(DEV) * 1_000_000_007   # large, unsorted, negative
    for causal in (False, True):
        out = A.attention_pytorch_document_mask(q, k, v, ids, is_causal=causal)
        assert_parity(out, O.attention_document_mask(*f32(q, k, v), ids, is_causal=causal), f"causal={causal}")


def test_large_logits_and_masked_neighbours_stay_finite():
    q, k, v = qkv(1, 2, 2, 512, 128, seed=15)
    q = (q.float() * 30).bfloat16()
    out = A.attention_pytorch_causal(q, k, v)
    assert_parity(out, O.attention_causal(*f32(q, k, v)))


def test_softcap_default_threshold_and_causal_extension():
    q, k, v = qkv(1, 4, 4, 300, 64, seed=16)
    q = (q.float() * 6).bfloat16()
    assert_parity(A.attention_softcapped(q, k, v), O.attention_softcapped(*f32(q, k, v), score_mod=30.0))
    assert_parity(A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(10.0), is_causal=True),
                  O.attention_softcapped(*f32(q, k, v), score_mod=10.0, is_causal=True, honor_causal=True))


def test_evoformer_bias_layouts():
    g = torch.Generator().manual_seed(17)
    mk = lambda *s: torch.randn(*s, generator=g).bfloat16().to(DEV)
    B, N, S, H, D = 2, 5, 100, 4, 32
    Q, K, V = mk(B, N, S, H, D), mk(B, N, S, H, D), mk(B, N, S, H, D)
    cases = {
        "pair only": [mk(B, 1, H, S, S)],
        "mask only": [mk(B, N, 1, 1, S)],
        "shared pair": [mk(1, 1, H, S, S)],
        "three biases": [mk(B, N, 1, 1, S), mk(B, 1, H, S, S), mk(1, 1, 1, S, S)],
        "full": [mk(B, N, H, S, S)],
        "none": [],
    }
    for name, biases in cases.items():
        out = A.attention_reference(Q, K, V, biases)
        ref = O.attention_evoformer(*f32(Q, K, V), [b.float() for b in biases])
        assert_parity(out, ref, name)


@pytest.mark.parametrize("D", [32, 64, 128])
def test_evoformer_bias_staged_and_direct_paths(D):
    # S = 104: the key count is a multiple of 8 (bias rows travel through LDS) but not of any key tile or query block,
    # so the last staged tile is ragged in both directions.  Operand pairs cover: row-broadcast + dense, two dense
    # (the second one is read directly), two row-broadcast, and a dense operand whose rows start 2 bytes off a 16-byte
    # boundary (read directly), each with the sigmoid gate.
    g = torch.Generator().manual_seed(170 + D)
    mk = lambda *s: torch.randn(*s, generator=g).bfloat16().to(DEV)
    mk32 = lambda *s: torch.randn(*s, generator=g).to(DEV)
    B, N, S, H = 1, 3, 104, 2
    Q, K, V, G = mk(B, N, S, H, D), mk(B, N, S, H, D), mk(B, N, S, H, D), mk(B, N, S, H, D)
    wide = mk(B, 1, H, S, S + 8)
    cases = {
        "mask + pair": [mk(B, N, 1, 1, S), mk(B, 1, H, S, S)],
        "two dense": [mk(B, 1, H, S, S), mk(B, N, H, S, S)],
        "two masks": [mk(B, N, 1, 1, S), mk(B, 1, 1, 1, S)],
        # fp32 rows: the first is staged as the row operand, a second one is read directly (the staged tiles hold
        # 16-bit elements)
        "two fp32 masks": [mk32(B, N, 1, 1, S), mk32(B, 1, 1, 1, S)],
        "mask + fp32 mask": [mk(B, N, 1, 1, S), mk32(B, 1, H, 1, S)],
        "fp32 mask + pair": [mk32(B, N, 1, 1, S), mk(B, 1, H, S, S)],
        "misaligned rows": [wide[..., 1:S + 1]],
        "padded rows": [wide[..., 8:S + 8]],
    }
    for name, biases in cases.items():
        out = A.attention_reference(Q, K, V, biases, gate=G)
        ref = O.attention_evoformer(*f32(Q, K, V), [b.float() for b in biases], gate=G.float())
        assert_parity(out, ref, f"D={D} {name}")


def test_empty_problems_return_what_eager_returns():
    """No queries, no batch entries or no heads: an empty tensor; queries without keys: zeros.  Gradients are zeros."""
    mk = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device=DEV)  # noqa: E731
    assert A.attention_pytorch_causal(mk(2, 4, 0, 64), mk(2, 4, 0, 64), mk(2, 4, 0, 64)).shape == (2, 4, 0, 64)
    assert A.attention_pytorch(mk(0, 4, 16, 64), mk(0, 4, 16, 64), mk(0, 4, 16, 64)).shape == (0, 4, 16, 64)
    q = torch.randn(2, 4, 16, 64, device=DEV).to(torch.bfloat16).requires_grad_(True)
    k = mk(2, 4, 0, 64).requires_grad_(True)
    out = A.attention_pytorch(q, k, mk(2, 4, 0, 128))
    ref = torch.softmax(q.float() @ k.float().transpose(-1, -2), -1) @ torch.zeros(2, 4, 0, 128, device=DEV)
    assert out.shape == ref.shape == (2, 4, 16, 128) and torch.equal(out.float(), ref)
    out.sum().backward()
    assert q.grad is not None and not q.grad.any() and k.grad.shape == (2, 4, 0, 64)


def test_front_end_errors_on_gpu_tensors():
    q, k, v = qkv(1, 4, 2, 64, 64)
    with pytest.raises(ValueError, match="enable_gqa"):
        A.attention_pytorch_causal(q, k, v)
    with pytest.raises(NotImplementedError, match="bfloat16"):
        A.attention_pytorch(q.float(), k.float(), v.float(), enable_gqa=True)
    with pytest.raises(AssertionError):
        A.attention_pytorch_sliding_window(q, k[:, :, :32], v[:, :, :32], enable_gqa=True)
    with pytest.raises(ValueError, match="generated for"):
        A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(8), enable_gqa=True)
    q48 = torch.randn(1, 2, 64, 48, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(_ffi.FlashlightError, match="no kernel instance"):
        _ffi.attn_fwd(q48, q48, q48)  # the C ABI takes compiled head dims only (the front-ends pad others)
    q640 = torch.randn(1, 2, 64, 640, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(_ffi.FlashlightError, match="no kernel instance"):
        A.attention_pytorch(q640, q640, q640)  # beyond 512


def test_mfma_rate_probe_runs_and_sums_products():
    # 8 x 4 fragment pairs of ones: every accumulator element ends at 16 (k) * 8 (A fragments) * iters per B fragment
    iters, wgs = 3, 2
    ones = torch.ones(1 << 12, dtype=torch.bfloat16, device=DEV)
    sink = torch.zeros(wgs * 512, dtype=torch.float32, device=DEV)
    flops = _ffi.probe_mfma_rate(ones, iters, wgs, sink)
    torch.cuda.synchronize()
    assert flops == wgs * 8 * iters * 32 * 32768
    assert torch.all(sink == 16.0 * 8 * iters * 4 * 16)


@pytest.mark.parametrize("D,offsets", [
    (128, [-2600.0, -2000.0, 400.0, 2600.0, -800.0, 3000.0, -3000.0, 0.0]),   # logits jump by hundreds of nats per tile
    (128, [-3000.0] * 8),                                                       # every logit far below zero
    (64, [0.0, 1500.0, -1500.0, 30.0, -30.0, 2500.0, 2500.0, -2500.0]),
])
def test_reference_free_weights_survive_extreme_logit_ranges(D, offsets):
    # Unmasked tiles form their weights against the running reference without looking at the row maximum first and
    # fall back to the exact path when a row sum overflows or underflows.  Keys of the j-th block of 64 carry the
    # offset offsets[j] along the direction every query points in, so whole tiles sit hundreds of nats above or below
    # whatever came before; the result must still match the fp32 oracle.
    S = 64 * len(offsets)
    g = torch.Generator().manual_seed(18)
    q = torch.randn(1, 2, S, D, generator=g)
    k = torch.randn(1, 2, S, D, generator=g)
    v = torch.randn(1, 2, S, D, generator=g)
    q[..., 0] = 16.0
    k[..., 0] = torch.tensor(offsets).repeat_interleave(64) / 16.0
    q, k, v = (t.bfloat16().to(DEV) for t in (q, k, v))
    assert_parity(A.attention_pytorch(q, k, v), O.attention_vanilla(*f32(q, k, v)), "vanilla")
    assert_parity(A.attention_pytorch_causal(q, k, v, enable_gqa=True), O.attention_causal(*f32(q, k, v), enable_gqa=True), "causal")
    # soft-cap kernels subtract the running reference while they modify the scores, one step before the weights are
    # formed; with a cap this wide the capped logits still jump by hundreds of nats, so the recomputing path runs on
    # scores that are relative to a reference which then moves
    cap = 1500.0
    assert_parity(A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(cap)),
                  O.attention_softcapped(*f32(q, k, v), score_mod=cap), "softcap")
    assert_parity(A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(2), is_causal=True, softcap=cap),
                  O.attention_alibi(*f32(q, k, v), score_mod=2, is_causal=True, honor_causal=True, softcap=cap), "alibi+softcap+causal")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_256_row_workgroups_ragged_and_cross_lengths(dtype):
    # enough (batch, head) pairs that the unmasked head-dim-128 call takes the 8-wave tile; 300 query rows leave the
    # second workgroup of every head 44 rows (six of its eight waves have none), 333 keys a ragged last tile; GQA 4:1
    B, Hq, Hkv, Lq, Lk, D = 4, 64, 16, 300, 333, 128
    g = torch.Generator().manual_seed(52)
    q = torch.randn(B, Hq, Lq, D, generator=g).to(dtype).to(DEV)
    k = torch.randn(B, Hkv, Lk, D, generator=g).to(dtype).to(DEV)
    v = torch.randn(B, Hkv, Lk, D, generator=g).to(dtype).to(DEV)
    p, _keep = _ffi._fill_params(_ffi.load_library(), q, k, v, torch.empty_like(q), Hq, Hkv, None, _ffi.MASK_NONE, 0, 0, None,
                                 0, 0.0, [], None, False, 0.0, None)
    assert _ffi.plan(p)["rows_per_workgroup"] == 256
    out = A.attention_pytorch(q, k, v, enable_gqa=True)
    assert_parity(out, O.attention_vanilla(*f32(q, k, v), enable_gqa=True), f"8-wave tile {dtype}")


@pytest.mark.parametrize("D,mask", [(128, "none"), (64, "causal"), (32, "none")])
def test_results_written_to_an_8_byte_aligned_view_match_the_16_byte_path(D, mask):
    # a result tensor that is 16-byte aligned with strides that are multiples of 8 elements is written in 16-byte stores
    # (the two lanes of a query trade register halves first); any other placement the ABI admits (8-byte alignment,
    # strides that are multiples of 4) takes 8-byte stores.  Both give the same bits.  S = 333: rows past the end.
    B, H, S = 2, 3, 333
    q, k, v = qkv(B, H, H, S, D, seed=44)
    kind = _ffi.MASK_CAUSAL if mask == "causal" else _ffi.MASK_NONE
    wide = _ffi.attn_fwd(q, k, v, mask_kind=kind)
    big = torch.full((B, H, S, D + 12), 7.0, dtype=q.dtype, device=DEV)
    view = big[..., 4:4 + D]
    assert view.data_ptr() % 16 == 8 and view.stride(2) % 8 == 4
    out = _ffi.attn_fwd(q, k, v, mask_kind=kind, out=view)
    assert out.data_ptr() == view.data_ptr()
    assert torch.equal(view, wide)
    assert torch.all(big[..., :4] == 7.0) and torch.all(big[..., 4 + D:] == 7.0)  # nothing written beside the view


SCORE_MODS = {
    "relu": lambda s, *_: torch.relu(s),
    "sigmoid": lambda s, *_: 6.0 * torch.sigmoid(0.5 * s - 1.0) + 2.0,
    "clamp": lambda s, *_: torch.clamp(2.0 * s + 1.0, min=-3.0, max=5.0),
    "negated clamp": lambda s, *_: 1.0 - torch.clamp(s, min=-2.0) * 1.5,
    "cubic": lambda s, *_: 0.02 * s ** 3 - 0.5 * s + 4.0,
    "square": lambda s, *_: -0.25 * s * s,
}


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("name", sorted(SCORE_MODS))
def test_score_mod_callables_beyond_the_soft_cap(name, D):
    # softcap.py:49 applies whatever score_mod it is handed to the scaled score matrix; callables that trace to a
    # sigmoid, ReLU / clamp or polynomial (up to the cube) of the score run in the kernel's registers like the tanh
    fn = SCORE_MODS[name]
    B, Hq, Hkv, S = 2, 8, 2, 333
    q, k, v = qkv(B, Hq, Hkv, S, D, seed=61)
    q = (q.float() * 2.0).to(q.dtype)  # logits of a few units, so that every branch of the functions is exercised
    for causal in (False, True):
        out = A.attention_softcapped(q, k, v, score_mod=fn, enable_gqa=True, is_causal=causal)
        ref = O.attention_softcapped(*f32(q, k, v), score_mod=fn, enable_gqa=True, is_causal=causal, honor_causal=True)
        assert_parity(out, ref, f"{name} D={D} causal={causal}")
    # with a tensor addend (a dense bias operand rides along) and a caller's scale
    t = torch.randn(Hq, S, S, generator=torch.Generator().manual_seed(7)).to(DEV)  # (under GQA the reference views it as [Hkv, G, L, S])
    fn_t = lambda s, *a: fn(s) + t  # noqa: E731
    out = A.attention_softcapped(q, k, v, score_mod=fn_t, enable_gqa=True, scale=0.2)
    ref = O.attention_softcapped(*f32(q, k, v), score_mod=lambda s, *a: fn(s) + t.float().view(Hkv, Hq // Hkv, S, S), enable_gqa=True, scale=0.2)
    assert_parity(out, ref, f"{name} D={D} + tensor")


def test_score_functions_are_forward_only():
    q, k, v = qkv(1, 2, 2, 64, 64, seed=3)
    q.requires_grad_(True)
    with pytest.raises(NotImplementedError, match="forward-only"):
        A.attention_softcapped(q, k, v, score_mod=lambda s, *_: torch.relu(s))


# ---- dense score_mod and invariant point attention -------------------------------------------------------------------------

@pytest.mark.parametrize("gqa", [False, True])
@pytest.mark.parametrize("D", [64, 128])
def test_dense_score_mod_matches_the_in_kernel_alibi_and_the_oracle(D, gqa):
    # an untagged callable that returns the reference's dense fp32 ALiBi tensor (alibi.py:5-9) must give what the
    # in-kernel ALiBi term gives; S = 333 leaves the fp32 rows unaligned for vector loads on odd rows
    B, Hq, Hkv, S = 2, 8, (2 if gqa else 8), 333
    q, k, v = qkv(B, Hq, Hkv, S, D, seed=5)
    dense = lambda l, s: A.alibi_bias(Hq, l, s, device=DEV)  # noqa: E731
    out = A.attention_pytorch_alibi(q, k, v, score_mod=dense, enable_gqa=gqa)
    tagged = A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(Hq), enable_gqa=gqa)
    ref = O.attention_alibi(*f32(q, k, v), score_mod=Hq, enable_gqa=gqa)
    assert out.shape == tagged.shape == ref.shape
    assert_parity(out, ref, "dense fp32")
    assert (out.float() - tagged.float()).abs().max().item() <= 2e-2  # one bf16 step of an output near 2
    # 16-byte aligned fp32 rows (vector loads), bf16 tensor through the staged path, and is_causal
    S = 256
    q, k, v = qkv(B, Hq, Hkv, S, D, seed=6)
    g = torch.Generator().manual_seed(8)
    t32 = torch.randn(Hq, S, S, generator=g).to(DEV)
    for t in (t32, t32.bfloat16(), t32[:, :1], t32[:, :1].bfloat16(), t32[:1]):
        full = t.expand(Hq, S, S).contiguous()
        # under GQA the reference views the tensor as [Hkv, G, L, S], which needs every element; without GQA the
        # size-1 axes broadcast
        given = full if gqa else t
        out = A.attention_pytorch_alibi(q, k, v, score_mod=lambda l, s: given, enable_gqa=gqa, is_causal=True)
        ref = O.attention_alibi(*f32(q, k, v), score_mod=lambda l, s: full.float(), enable_gqa=gqa, is_causal=True,
                                honor_causal=True)
        assert_parity(out, ref, f"dense {t.dtype} {tuple(t.shape)}")


def _ipa_inputs(B, H, N, C, P, Pv, X, seed, spread=1.0, centre=0.0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(*s, generator=g)  # noqa: E731
    t = dict(q_scalar=mk(B, H, N, C), k_scalar=mk(B, H, N, C), v_scalar=mk(B, H, N, C),
             q_points=mk(B, H, N, P, X) * spread + centre, k_points=mk(B, H, N, P, X) * spread + centre,
             v_points=mk(B, H, N, Pv, X), pair_bias=mk(B, H, N, N))
    return {n: x.bfloat16().to(DEV) for n, x in t.items()}


@pytest.mark.parametrize("shape", [
    dict(B=2, H=8, N=64, C=16, P=4, Pv=8, X=4),    # tests/test_ipa.py:141-157: Dqk = 32, Dv = 48 -> 64
    dict(B=1, H=12, N=384, C=16, P=4, Pv=8, X=3),  # AlphaFold's structure module: Dqk = 28 -> 32, Dv = 40 -> 64
    dict(B=2, H=4, N=203, C=32, P=8, Pv=12, X=3),  # Dqk = 56 -> 64, Dv = 68 -> 128, ragged length
    dict(B=1, H=2, N=130, C=64, P=8, Pv=8, X=3),   # Dqk = 88 -> 128, Dv = 88 -> 128
])
def test_invariant_point_attention(shape):
    t = _ipa_inputs(**shape, seed=61)
    o_s, o_p = A.invariant_point_attention(**t, c_hidden=shape["C"], no_qk_points=shape["P"])
    r_s, r_p = O.invariant_point_attention(**{n: x.float() for n, x in t.items()}, c_hidden=shape["C"],
                                           no_qk_points=shape["P"])
    assert o_s.shape == r_s.shape and o_p.shape == r_p.shape
    # the reference's own bar (tests/test_ipa.py:195) and this suite's
    torch.testing.assert_close(o_s.float(), r_s, atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(o_p.float(), r_p, atol=1e-2, rtol=1e-2)
    assert_parity(o_s, r_s, "scalar")
    assert_parity(o_p, r_p, "points")


def test_invariant_point_attention_far_from_the_origin_and_broadcast_bias():
    # point clouds centred 40 units from the origin: |q|^2 + |k|^2 - 2 q.k loses nothing as long as the inputs enter
    # the product unrounded and the key term stays fp32; pair bias shared by the batch; extra leading axis; no bias
    t = _ipa_inputs(B=2, H=4, N=96, C=16, P=4, Pv=8, X=3, seed=67, spread=0.5, centre=40.0)
    t["pair_bias"] = t["pair_bias"][:1]
    o_s, o_p = A.invariant_point_attention(**t, c_hidden=16, no_qk_points=4)
    r_s, r_p = O.invariant_point_attention(**{n: x.double() for n, x in t.items()}, c_hidden=16, no_qk_points=4)
    assert_parity(o_s, r_s, "scalar, far")
    assert_parity(o_p, r_p, "points, far")
    t5 = {n: x.unsqueeze(0) for n, x in _ipa_inputs(B=2, H=2, N=40, C=16, P=4, Pv=8, X=3, seed=68).items()}
    t5["pair_bias"] = None
    o_s, o_p = A.invariant_point_attention(**t5, c_hidden=16, no_qk_points=4)
    r_s, r_p = O.invariant_point_attention(**{n: None if x is None else x.float() for n, x in t5.items()}, c_hidden=16,
                                           no_qk_points=4)
    assert o_s.shape == r_s.shape == (1, 2, 2, 40, 16) and o_p.shape == r_p.shape == (1, 2, 40, 2, 8, 3)
    assert_parity(o_s, r_s, "scalar, 5-D")
    assert_parity(o_p, r_p, "points, 5-D")


# ---- fp16 elements (the reference's typing admits them: monkeypatch/fusion/_reduction.py:55-57) ------------------------------

def _half(*ts):
    return tuple(t.to(torch.float16) for t in ts)


@pytest.mark.parametrize("D", [32, 64, 128])
def test_fp16_variants(D):
    q, k, v = _half(*qkv(2, 4, 2, 333, D, seed=40 + D))
    ref32 = f32(q, k, v)
    cases = {
        "vanilla": (A.attention_pytorch(q, k, v, enable_gqa=True), O.attention_vanilla(*ref32, enable_gqa=True)),
        "causal": (A.attention_pytorch_causal(q, k, v, enable_gqa=True), O.attention_causal(*ref32, enable_gqa=True)),
        "sliding": (A.attention_pytorch_sliding_window(q, k, v, window_size=50, enable_gqa=True),
                    O.attention_sliding_window(*ref32, window_size=50, enable_gqa=True)),
        "prefix": (A.attention_pytorch_prefix_lm(q, k, v, prefix_lengths=77, enable_gqa=True),
                   O.attention_prefix_lm(*ref32, prefix_lengths=77, enable_gqa=True)),
    }
    if D != 32:  # the score-modification and document kernels are compiled for head dims 64 and 128
        ids = torch.arange(333).div(100, rounding_mode="floor")[None].expand(2, -1).to(DEV)
        cases.update({
            "alibi+softcap+causal": (
                A.attention_pytorch_alibi(q, k, v, score_mod=A.generate_alibi_bias_pytorch(4), enable_gqa=True,
                                          is_causal=True, softcap=20.0),
                O.attention_alibi(*ref32, score_mod=4, enable_gqa=True, is_causal=True, honor_causal=True, softcap=20.0)),
            "document": (A.attention_pytorch_document_mask(q, k, v, ids, enable_gqa=True, is_causal=True),
                         O.attention_document_mask(*ref32, ids, enable_gqa=True, is_causal=True)),
        })
    for name, (out, ref) in cases.items():
        assert out.dtype == torch.float16
        assert_parity(out, ref, f"fp16 D={D} {name}")


def test_fp16_differential_evoformer_and_mixed_types():
    qd, kd, _ = _half(*qkv(2, 8, 8, 200, 64, seed=50))
    vd = _half(qkv(2, 4, 4, 200, 128, seed=51)[2])[0]
    assert_parity(A.diffattn(qd, kd, vd, lambda_full=0.7, is_causal=True),
                  O.diff_attention(*f32(qd, kd, vd), lambda_full=0.7, is_causal=True), "fp16 diff")
    g = torch.Generator().manual_seed(52)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.float16).to(DEV)  # noqa: E731
    Q, K, V, G = mk(1, 3, 104, 2, 32), mk(1, 3, 104, 2, 32), mk(1, 3, 104, 2, 32), mk(1, 3, 104, 2, 32)
    pair, mask = mk(1, 1, 2, 104, 104), mk(1, 3, 1, 1, 104)
    out = A.attention_reference(Q, K, V, [mask, pair.float()], gate=G)  # one fp16 operand, one fp32 operand
    assert out.dtype == torch.float16
    assert_parity(out, O.attention_evoformer(*f32(Q, K, V), [mask.float(), pair.float()], gate=G.float()), "fp16 evoformer")
    # element types do not mix
    qb, kb, vb = qkv(1, 2, 2, 64, 64, seed=53)
    with pytest.raises(NotImplementedError, match="mixed element types"):
        A.attention_pytorch(qb, kb.to(torch.float16), vb)
    with pytest.raises(NotImplementedError, match="mixed element types"):
        A.attention_reference(Q, K, V, [pair.bfloat16()])


def test_fp16_large_weights_take_the_exact_path():
    # logits that climb by hundreds per tile: weights formed against a stale reference overflow fp16 (65504), the row
    # sums see it, and the exact path recomputes them
    g = torch.Generator().manual_seed(54)
    S, D = 512, 64
    q = torch.randn(1, 1, S, D, generator=g)
    k = torch.randn(1, 1, S, D, generator=g)
    k[0, 0] += torch.linspace(0, 3, S).unsqueeze(1) * q[0, 0].mean(0, keepdim=True).sign()
    v = torch.randn(1, 1, S, D, generator=g)
    q, k, v = (t.to(torch.float16).to(DEV) for t in (q * 4, k * 4, v))
    out = A.attention_pytorch(q, k, v, scale=1.0)
    assert_parity(out, O.attention_vanilla(*f32(q, k, v), scale=1.0), "fp16 large logits")


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("via_bias", [False, True])
def test_fp16_weights_in_the_subnormal_band(D, via_bias):
    # every logit sits 12 to 18 nats below zero, the reference a row starts with: weights formed against it are fp16
    # subnormals (2^-17 .. 2^-26, a few bits or none), so the kernel has to notice the small row sums and settle a
    # reference from the row maxima before it trusts them.  Driven once through q.k itself (plain instances) and once
    # through a dense fp32 score_mod (bias instances).
    g = torch.Generator().manual_seed(77)
    S = 1024
    q = torch.randn(1, 2, S, D, generator=g) * 0.5
    k = torch.randn(1, 2, S, D, generator=g) * 0.5
    v = torch.randn(1, 2, S, D, generator=g)
    low = -(12.0 + 5.0 * torch.rand(S, generator=g))  # per key, natural units
    if not via_bias:
        q[..., 0] = math.sqrt(D)
        k[..., 0] = low  # q0 * k0 / sqrt(D) = low
    q, k, v = (t.to(torch.float16).to(DEV) for t in (q, k, v))
    qf, kf, vf = f32(q, k, v)
    if via_bias:
        bias = low.view(1, 1, 1, S).expand(1, 2, S, S).contiguous().to(DEV)
        out = A.attention_pytorch_alibi(q, k, v, score_mod=lambda l, s: bias)
        ref = O.attention_alibi(qf, kf, vf, score_mod=lambda l, s: bias)
        assert_parity(out, ref, "dense score_mod")
        return
    assert_parity(A.attention_pytorch(q, k, v), O.attention_vanilla(qf, kf, vf), "vanilla")
    assert_parity(A.attention_pytorch_causal(q, k, v), O.attention_causal(qf, kf, vf), "causal")


def test_config0_shape_causal():
    # configuration 0 of the baseline file (the reference's CPU-sized case): causal, B=2 H=8 S=512 D=64, fp32 N(0,1)
    # inputs from seed 1000; the kernel takes their bf16 rounding, the oracle the fp32 originals
    g = torch.Generator().manual_seed(1000)
    q, k, v = (torch.randn(2, 8, 512, 64, generator=g) for _ in range(3))
    out = A.attention_pytorch_causal(*(t.to(torch.bfloat16).to(DEV) for t in (q, k, v)))
    assert out.shape == (2, 8, 512, 64)
    assert_parity(out, O.attention_causal(q, k, v), "config 0")


# ---- the shared-bias streaming kernel (head dim 32, one dense bias shared by the rows of an MSA, 256 / 320 / 384 keys) ----

@pytest.mark.parametrize("B,N,S,H,gate,dtype,inf", [
    (1, 64, 384, 8, True, torch.bfloat16, False),    # the benchmark's shape class
    (1, 37, 256, 4, False, torch.bfloat16, False),   # no gate; a row count that leaves a short last chunk
    (2, 19, 320, 3, True, torch.bfloat16, False),    # two bias groups, odd head count
    (1, 5, 256, 8, True, torch.float16, False),      # fp16 elements
    (1, 33, 384, 2, True, torch.bfloat16, True),     # -inf entries in the bias (an additive mask)
    (1, 2, 256, 8, False, torch.bfloat16, False),    # two rows: chunks of one entry
    (1, 21, 320, 2, False, torch.bfloat16, False),   # five tiles per entry without a gate
    (1, 40, 384, 4, False, torch.float16, False),    # six tiles per entry without a gate, fp16
    (2, 11, 128, 4, True, torch.bfloat16, False),    # two tiles per entry: the ring runs three entries ahead
    (1, 23, 128, 2, False, torch.float16, True),
    (1, 17, 192, 8, True, torch.bfloat16, True),     # three tiles per entry
    (3, 6, 192, 1, False, torch.bfloat16, False),
])
def test_shared_bias_streaming_kernel(B, N, S, H, gate, dtype, inf):
    g = torch.Generator().manual_seed(31)
    mk = lambda *s: torch.randn(*s, generator=g).to(dtype).to(DEV)  # noqa: E731
    q, k, v = mk(B, N, S, H, 32), mk(B, N, S, H, 32), mk(B, N, S, H, 32)
    bias = mk(B, 1, H, S, S)
    if inf:
        bias[..., ::7] = float("-inf")
        bias[..., 3::14] = -1e9 if dtype == torch.bfloat16 else -6e4  # finite masks beyond fp16's range saturate in the kernel
        bias[..., 5::31] *= 40.0                                       # and ordinary values of some size
    gt = mk(B, N, S, H, 32) if gate else None
    # the call must be one the streaming kernel takes (the plan says so), not the general one
    p, _keep = _ffi._fill_params(_ffi.load_library(), *(t.reshape(-1, S, H, 32).transpose(1, 2) for t in (q, k, v)),
                                 torch.empty(B * N, H, S, 32, dtype=dtype, device=DEV), H, H, None, _ffi.MASK_NONE, 0, 0,
                                 None, 0, 0.0, [(bias.reshape(B, H, S, S), N)], None, False, 0.0, None)
    assert _ffi.plan(p)["streaming"] == 1
    out = A.attention_reference(q, k, v, [bias], gate=gt) if gate else A.attention_reference(q, k, v, [bias])
    ref = O.attention_evoformer(*f32(q, k, v), [bias.float()], gate=None if gt is None else gt.float())
    assert_parity(out, ref, f"B{B} N{N} S{S} H{H}")


@pytest.mark.parametrize("dtype,drop", [(torch.bfloat16, float("-inf")), (torch.float16, -21.0)])
def test_shared_bias_streaming_kernel_half_masked_lanes(dtype, drop):
    # The two lanes of a query hold alternate runs of 8 keys.  Here one lane's keys of the first 64 positions carry no
    # weight (-inf in bf16; 30 log2 units down in fp16, whose weights underflow there) while the other lane's do, and
    # the second 32-key block's maximum lies below the first's: both lanes must still agree on one softmax reference.
    g = torch.Generator().manual_seed(33)
    mk = lambda *s: torch.randn(*s, generator=g).to(dtype).to(DEV)  # noqa: E731
    B, N, S, H = 1, 9, 256, 2
    q, k, v = mk(B, N, S, H, 32), mk(B, N, S, H, 32), mk(B, N, S, H, 32)
    bias = mk(B, 1, H, S, S).float()
    keys = torch.arange(S, device=DEV)
    stripe = (keys < 64) & (keys % 16 < 8)
    bias[..., stripe] = float("-inf") if drop == float("-inf") else bias[..., stripe] + drop
    bias[..., 8:16] += 6.0
    bias = bias.to(dtype)
    p, _keep = _ffi._fill_params(_ffi.load_library(), *(t.reshape(-1, S, H, 32).transpose(1, 2) for t in (q, k, v)),
                                 torch.empty(B * N, H, S, 32, dtype=dtype, device=DEV), H, H, None, _ffi.MASK_NONE, 0, 0,
                                 None, 0, 0.0, [(bias.reshape(B, H, S, S), N)], None, False, 0.0, None)
    assert _ffi.plan(p)["streaming"] == 1
    out = A.attention_reference(q, k, v, [bias])
    assert_parity(out, O.attention_evoformer(*f32(q, k, v), [bias.float()]), f"half-masked lanes {dtype}")


@pytest.mark.parametrize("D,B,N,S,H,gate,dtype,mask,scale", [
    (64, 2, 8, 256, 4, False, torch.bfloat16, "1e9", None),      # the reference benchmark's inputs (evoformer.py:41-49)
    (64, 1, 5, 256, 2, False, torch.bfloat16, "randn", None),    # an odd number of entries: the last chunk is short
    (64, 1, 9, 256, 4, False, torch.bfloat16, "inf", 0.1),       # 1 / scale inexact in bf16: both selector terms
    (64, 1, 6, 256, 2, False, torch.float16, "randn", None),
    (32, 1, 13, 384, 8, True, torch.bfloat16, "1e9", None),      # head dim 32 with mask bias, pair bias and gate
    (32, 2, 7, 256, 4, False, torch.bfloat16, "inf", None),
    (32, 1, 10, 320, 2, True, torch.float16, "randn", None),
    (32, 2, 9, 128, 4, True, torch.bfloat16, "inf", None),       # 128 and 192 keys, both head dims
    (32, 1, 14, 192, 2, False, torch.float16, "1e9", 0.2),
    (64, 1, 12, 128, 4, False, torch.bfloat16, "1e9", None),
    (64, 2, 7, 192, 2, False, torch.bfloat16, "randn", 0.1),
    (64, 1, 3, 192, 8, False, torch.float16, "inf", None),
])
def test_shared_bias_streaming_kernel_with_a_row_bias(D, B, N, S, H, gate, dtype, mask, scale):
    # two operands: a row of keys per batch entry (the reference's mask bias [B, N, 1, 1, S]) and the shared pair bias
    # [B, 1, H, S, S]; the streaming kernel adds both on the matrix pipe.  Either order of the operands.
    g = torch.Generator().manual_seed(35)
    mk = lambda *s: torch.randn(*s, generator=g).to(dtype).to(DEV)  # noqa: E731
    q, k, v = mk(B, N, S, H, D), mk(B, N, S, H, D), mk(B, N, S, H, D)
    pair = mk(B, 1, H, S, S)
    if mask == "randn":
        row = mk(B, N, 1, 1, S)
    else:
        keep = (torch.rand(B, N, 1, 1, S, generator=g) > 0.25).to(DEV)
        keep[..., 0] = True
        low = float("-inf") if mask == "inf" else (-1e9 if dtype == torch.bfloat16 else -6e4)
        row = torch.where(keep, 0.0, low).to(dtype)
    gt = mk(B, N, S, H, D) if gate else None
    ops4 = [t.reshape(-1, S, H, D).transpose(1, 2) for t in (q, k, v)]
    p, _keep = _ffi._fill_params(_ffi.load_library(), *ops4, torch.empty(B * N, H, S, D, dtype=dtype, device=DEV), H, H, None,
                                 _ffi.MASK_NONE, 0, 0, None, 0, 0.0,
                                 [(row.reshape(B * N, 1, 1, S), 1), (pair.reshape(B, H, S, S), N)], None, False, 0.0, None)
    assert _ffi.plan(p)["streaming"] == 1
    kw = {} if scale is None else {"sm_scale": scale}
    ref = O.attention_evoformer(*f32(q, k, v), [row.float(), pair.float()], gate=None if gt is None else gt.float(), **kw)
    for biases in ([row, pair], [pair, row]):
        out = A.attention_reference(q, k, v, biases, gate=gt, **kw) if gate else A.attention_reference(q, k, v, biases, **kw)
        assert_parity(out, ref, f"D{D} B{B} N{N} S{S} H{H} {mask}")


def test_shared_bias_streaming_kernel_matches_the_general_kernel():
    # same call through both kernels: a second bias operand that differs by head (all zeros) makes the library take the
    # general one
    g = torch.Generator().manual_seed(32)
    mk = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(DEV)  # noqa: E731
    B, N, S, H = 1, 24, 384, 4
    q, k, v, gt = mk(B, N, S, H, 32), mk(B, N, S, H, 32), mk(B, N, S, H, 32), mk(B, N, S, H, 32)
    bias = mk(B, 1, H, S, S)
    zero = torch.zeros(B, N, H, 1, S, dtype=torch.bfloat16, device=DEV)
    fast = A.attention_reference(q, k, v, [bias], gate=gt)
    general = A.attention_reference(q, k, v, [zero, bias], gate=gt)
    assert (fast.float() - general.float()).abs().max().item() <= 2e-2
    assert_parity(fast, O.attention_evoformer(*f32(q, k, v), [bias.float()], gate=gt.float()), "streaming")


def test_document_mask_prepared_workspace_skips_the_prepass_and_matches():
    # A workspace handle keeps the key-tile lists across calls on the same ids (FL_FLAG_DOC_PREPARED); other ids, or ids
    # modified in place, refill it.  Every result equals the plain call's bit for bit.
    g = torch.Generator().manual_seed(41)
    B, H, S, D = 2, 3, 700, 64
    q, k, v = (torch.randn(B, H, S, D, generator=g).bfloat16().to(DEV) for _ in range(3))
    ids = torch.sort(torch.randint(0, 5, (B, S), generator=g), dim=1).values.to(DEV)
    ws = A.DocumentMaskWorkspace()
    for causal in (False, True):
        plain = A.attention_pytorch_document_mask(q, k, v, ids, is_causal=causal)
        first = A.attention_pytorch_document_mask(q, k, v, ids, is_causal=causal, workspace=ws)
        key = ws.key
        again = A.attention_pytorch_document_mask(q * 2, k, v, ids, is_causal=causal, workspace=ws)  # other q, same ids
        assert ws.key == key
        assert torch.equal(plain, first)
        assert torch.equal(again, A.attention_pytorch_document_mask(q * 2, k, v, ids, is_causal=causal))
    ids[:, S // 2:] += 7  # in place: the handle notices the new version and runs the pre-pass again
    out = A.attention_pytorch_document_mask(q, k, v, ids, is_causal=True, workspace=ws)
    assert torch.equal(out, A.attention_pytorch_document_mask(q, k, v, ids, is_causal=True))
    ref = O.attention_document_mask(*f32(q, k, v), ids, is_causal=True)
    assert_parity(out, ref, "prepared workspace")


@pytest.mark.gpu
def test_operands_of_more_than_two_to_the_31_elements():
    """[16, 64, 16384, 128] in bf16 is 4 GiB per operand: element offsets pass 2^31 and byte offsets 2^32.  Slices of the
    forward's and the backward's results against runs on the slices alone, which launch the same kernels: bit-equal."""
    from flashlight_amd import _ffi
    B, H, L, D = 16, 64, 16384, 128

    def fill(seed):
        t = torch.empty(B, H, L, D, dtype=torch.bfloat16, device="cuda")
        gen = torch.Generator(device="cuda").manual_seed(seed)
        flat, step = t.view(-1), 1 << 28
        for i in range(0, flat.numel(), step):
            flat[i:i + step].copy_(torch.randn(step, generator=gen, device="cuda"))
        return t
    q, k, v, do = (fill(s) for s in (1, 2, 3, 4))
    assert q.numel() == 1 << 31
    lse = torch.empty(B, H, L, dtype=torch.float32, device="cuda")
    out = _ffi.attn_fwd(q, k, v, mask_kind=_ffi.MASK_CAUSAL, lse=lse)
    grads = _ffi.attn_bwd(q, k, v, out, lse, do, mask_kind=_ffi.MASK_CAUSAL)
    for b, h in ((0, 0), (8, 0), (15, 63)):
        one = lambda t: t[b:b + 1, h:h + 1].contiguous()
        lse1 = torch.empty(1, 1, L, dtype=torch.float32, device="cuda")
        out1 = _ffi.attn_fwd(one(q), one(k), one(v), mask_kind=_ffi.MASK_CAUSAL, lse=lse1)
        grads1 = _ffi.attn_bwd(one(q), one(k), one(v), out1, lse1, one(do), mask_kind=_ffi.MASK_CAUSAL)
        assert torch.equal(out[b, h], out1[0, 0]) and torch.equal(lse[b, h], lse1[0, 0]), (b, h)
        for name, a, c in zip(("dq", "dk", "dv"), grads, grads1):
            assert torch.equal(a[b, h], c[0, 0]), (name, b, h)
    assert torch.isfinite(out[15, 63].float()).all() and out[15, 63].float().abs().max() > 0
    del q, k, v, do, out, grads, lse
    torch.cuda.empty_cache()


@pytest.mark.gpu
def test_calls_from_several_threads_on_streams_of_their_own():
    """The library is re-entrant: no state is shared between calls but a thread-local error text and the lazily set kernel
    attributes.  Eight threads, each on its own stream, run different variants (document masks with their pre-pass and
    workspace, a staged bias, a refused call in between, whose message must be the thread's own) 20 times over; every
    result must be bit-equal to the same call made alone."""
    import threading
    g = torch.Generator().manual_seed(77)

    def rnd(*shape):
        return torch.randn(*shape, generator=g).to(torch.bfloat16).to("cuda")

    ids = torch.sort(torch.randint(0, 5, (2, 777), generator=g), dim=1).values.to("cuda")
    jobs = [
        ("vanilla", lambda: _ffi.attn_fwd(*qkv128)),
        ("causal", lambda: _ffi.attn_fwd(*qkv128, mask_kind=_ffi.MASK_CAUSAL)),
        ("sliding", lambda: _ffi.attn_fwd(*qkv64, mask_kind=_ffi.MASK_SLIDING, window=100)),
        ("document", lambda: _ffi.attn_fwd(*qkv64, mask_kind=_ffi.MASK_DOCUMENT_CAUSAL, doc_ids=ids)),
        ("alibi + soft-cap", lambda: _ffi.attn_fwd(*qkv128, alibi_heads=4, softcap=20.0, mask_kind=_ffi.MASK_CAUSAL)),
        ("bias", lambda: _ffi.attn_fwd(*qkv64, biases=[(bias, 1)])),
        ("prefix", lambda: _ffi.attn_fwd(*qkv64, mask_kind=_ffi.MASK_PREFIX_LM, prefix=300)),
        ("document, not causal", lambda: _ffi.attn_fwd(*qkv64, mask_kind=_ffi.MASK_DOCUMENT, doc_ids=ids)),
    ]
    qkv128 = (rnd(2, 4, 777, 128), rnd(2, 2, 777, 128), rnd(2, 2, 777, 128))
    qkv64 = (rnd(2, 4, 777, 64), rnd(2, 4, 777, 64), rnd(2, 4, 777, 64))
    bias = rnd(2, 4, 777, 784)[..., :777]
    alone = [fn().clone() for _, fn in jobs]
    torch.cuda.synchronize()
    errors = []
    start = threading.Barrier(len(jobs))

    def worker(i):
        name, fn = jobs[i]
        try:
            stream = torch.cuda.Stream()
            start.wait()
            with torch.cuda.stream(stream):
                for it in range(20):
                    out = fn()
                    if it % 5 == i % 5:   # a refused call: the message is this thread's
                        try:
                            _ffi.attn_fwd(qkv64[0], qkv64[1], qkv64[2], mask_kind=_ffi.MASK_SLIDING, window=-(i + 1))
                            errors.append((name, "a negative window was accepted"))
                        except _ffi.FlashlightError as e:
                            if "window" not in str(e):
                                errors.append((name, f"foreign error text: {e}"))
                    stream.synchronize()
                    if not torch.equal(out, alone[i]):
                        errors.append((name, f"iteration {it} differs from the call made alone"))
                        return
        except Exception as e:  # noqa: BLE001 - reported below
            errors.append((name, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not any(t.is_alive() for t in threads), "a worker did not finish"
    assert errors == [], errors


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 32, 8, 1, 32768, 128), (2, 8, 8, 7, 8192, 64), (1, 4, 1, 130, 12288, 128), (1, 16, 4, 1, 65536, 128),
                                   (3, 4, 4, 2, 4096, 32), (1, 6, 2, 3, 8201, 64), (2, 6, 2, 3, 8200, 64)])
def test_few_queries_against_a_long_cache_are_split_over_the_keys(shape):
    """A decoding step: B * Hq workgroups cannot fill the chip, so the front end runs the key chunks as extra heads of one
    launch and merges the partial results by their row statistics.  Against eager fp32; the last two shapes' key lengths
    have no usable divisor: with one batch entry the rest is a shorter last chunk, with more the ordinary launch runs."""
    import torch.nn.functional as F
    from flashlight_amd import ops
    B, Hq, Hkv, Lq, Lk, D = shape
    g = torch.Generator().manual_seed(Lk + Lq)
    q = torch.randn(B, Hq, Lq, D, generator=g).to(torch.bfloat16)
    k, v = (torch.randn(B, Hkv, Lk, D, generator=g).to(torch.bfloat16) for _ in range(2))
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    # (a key length without a usable divisor is cut all the same when there is one batch entry: a shorter last chunk)
    assert (ops._split_over_keys(qd, kd, vd, None, 0.0) is not None) == (Lk % 16 == 0 or B == 1)
    got = A.attention_pytorch(qd, kd, vd, enable_gqa=True)
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), enable_gqa=True)
    assert_parity(got, want, str(shape), max_tol=2e-3, mean_tol=2e-4)
    # a soft-cap goes along; a cache whose heads are not contiguous (a slice of a longer buffer) is not split
    got = A.attention_softcapped(qd, kd, vd, score_mod=A.generate_tanh_softcap(20.0), enable_gqa=True)
    want = O.attention_softcapped(q.float(), k.float(), v.float(), score_mod=20.0, enable_gqa=True)
    assert_parity(got.reshape(want.shape), want, str(shape) + " soft-cap", max_tol=2e-3, mean_tol=2e-4)
    if Lk % 16 == 0:
        # a padding mask is cut with the keys; a chunk it removes entirely, and a row it removes entirely, come out as zeros
        pad = torch.zeros(B, 1, 1, Lk)
        pad[:, :, :, Lk // 64:Lk // 3] = float("-inf")
        pad[0, :, :, Lk // 2:] = -1e9
        got = ops.dispatch(qd, kd, vd, biases=[(pad.to(torch.bfloat16).cuda(), 1)])
        want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=pad, enable_gqa=True)
        assert_parity(got, want, str(shape) + " padding mask", max_tol=2e-3, mean_tol=2e-4)
        got = ops.dispatch(qd, kd, vd, biases=[(torch.full((B, 1, 1, Lk), float("-inf")).to(torch.bfloat16).cuda(), 1)])
        assert torch.count_nonzero(got).item() == 0
    longer = torch.randn(B, Hkv, Lk + 64, D, generator=g).to(torch.bfloat16).cuda()
    ks, vs = longer[:, :, :Lk], torch.flip(longer, dims=(1,))[:, :, 64:]
    if B > 1:   # (heads further apart than their rows: only one batch entry can be cut, its chunks as batch entries)
        assert ops._split_over_keys(qd, ks, vs, None, 0.0) is None
    else:
        assert ops._split_over_keys(qd, ks, vs, None, 0.0) is not None
        pad = torch.zeros(1, 1, 1, Lk)
        pad[..., 5:Lk // 2 + 3] = float("-inf")
        got = ops.dispatch(qd, ks, vs, biases=[(pad.to(torch.bfloat16).cuda(), 1)])
        want = F.scaled_dot_product_attention(q.float(), ks.float().cpu(), vs.float().cpu(), attn_mask=pad, enable_gqa=True)
        assert_parity(got, want, str(shape) + " cache slice", max_tol=2e-3, mean_tol=2e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(4, 32, 8, 1, 2048, 128), (3, 12, 2, 5, 333, 64), (2, 8, 1, 16, 1000, 32), (1, 64, 8, 2, 8192, 128),
                                   (2, 6, 3, 40, 77, 64)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_grouped_heads_with_few_queries_are_packed_as_rows(shape, dtype):
    """Unmasked grouped-query attention with few queries per head (decoding): the front end hands the kernel the G query
    heads of a key / value head as G times as many rows of that head.  Same results as eager fp32, through every variant
    that has no mask; a causal call is not packed and stays right."""
    import torch.nn.functional as F
    B, Hq, Hkv, Lq, Lk, D = shape
    g = torch.Generator().manual_seed(Lk * 7 + Lq)
    q = torch.randn(B, Hq, Lq, D, generator=g).to(dtype)
    k, v = (torch.randn(B, Hkv, Lk, D, generator=g).to(dtype) for _ in range(2))
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), enable_gqa=True)
    assert_parity(A.attention_pytorch(qd, kd, vd, enable_gqa=True), want, f"{shape} vanilla")
    want = O.attention_softcapped(q.float(), k.float(), v.float(), score_mod=20.0, enable_gqa=True)
    got = A.attention_softcapped(qd, kd, vd, score_mod=A.generate_tanh_softcap(20.0), enable_gqa=True)
    assert_parity(got.reshape(want.shape), want, f"{shape} soft-cap")
    want = O.attention_causal(q.float(), k.float(), v.float(), enable_gqa=True)
    got = A.attention_pytorch_causal(qd, kd, vd, enable_gqa=True)
    assert_parity(got.reshape(want.shape), want, f"{shape} causal")
    # a padding mask (one row of keys per batch entry, added to every head and row) goes along with the packed rows
    pad = torch.zeros(B, 1, 1, Lk)
    pad[:, :, :, Lk // 3:Lk // 2] = float("-inf")
    pad[0, :, :, :Lk // 4] = -1e9
    from flashlight_amd import ops
    got = ops.dispatch(qd, kd, vd, biases=[(pad.to(dtype).cuda(), 1)])
    want = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=pad, enable_gqa=True)
    assert_parity(got, want, f"{shape} padding mask")
    # a query tensor that is a strided view is not packed (no view of it has the rows adjacent) and stays right
    wide = torch.randn(B, Hq, Lq, D + 8, generator=g).to(dtype).cuda()
    want = F.scaled_dot_product_attention(wide[..., :D].float().cpu(), k.float(), v.float(), enable_gqa=True)
    assert_parity(A.attention_pytorch(wide[..., :D], kd, vd, enable_gqa=True), want, f"{shape} strided q")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_merge_of_key_chunks_through_the_abi(dtype):
    """fl_attn_merge_chunks against the same sum in fp32 tensor operations: random statistics, chunks marked as holding no
    keys for some rows (+inf), rows without keys in any chunk (zeros), value widths from 2 to 512."""
    g = torch.Generator().manual_seed(5)
    for outer, chunks, inner, dv in ((3, 4, 5, 128), (1, 64, 1, 512), (7, 2, 130, 2), (2, 9, 3, 96)):
        part = torch.randn(outer, chunks, inner, dv, generator=g).to(dtype).cuda()
        lse = (torch.randn(outer, chunks, inner, generator=g) * 6 + 10).cuda()
        lse[torch.rand(outer, chunks, inner, generator=g).cuda() < 0.2] = float("inf")
        lse[0, :, 0] = float("inf")
        got = _ffi.merge_chunks(part, lse)
        l = torch.where(lse == float("inf"), torch.full_like(lse, float("-inf")), lse)
        top = l.amax(dim=1, keepdim=True)
        w = torch.exp2(l - torch.where(top == float("-inf"), torch.zeros_like(top), top))
        want = (w.unsqueeze(-1) * part.float()).sum(dim=1) / w.sum(dim=1).clamp_min(1e-30).unsqueeze(-1)
        assert torch.count_nonzero(got[0, 0]).item() == 0
        assert_parity(got, want, f"{(outer, chunks, inner, dv)}", max_tol=2e-2 if dtype == torch.bfloat16 else 4e-3, mean_tol=2e-3)
