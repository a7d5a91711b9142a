#!/usr/bin/env python3
"""Sweep of the attention variants in the format of the reference's benchmark harness.

    python -m flashlight_amd.benchmarks.run_variants [--batch_size ...] [--seqlen ...] [--dim D] [--headdim ...]
                                                     [--group_size ...] [--filter KEYWORD ...] [--output NAME]

Mirrors benchmarks/run_flex_variants.py:126-147,159-216,230-246 and benchmarks/_utils.py of the reference: the same
variant names and hyper-parameters (soft-cap 30, window 256, prefix 256, 12 documents), the same default sweep
(batch sizes 32..1 zipped with sequence lengths 512..16384, model dim 1024, head dim 64, group sizes 1 and 8), the same
timing recipe (10 warm-up calls, 20 timed calls, a 256 MB buffer zeroed before each to flush the caches, one event pair
per call, mean), the same FLOP accounting (4 B S^2 H D, times the share of non-empty 128 x 128 blocks of the variant's
mask; causal counts half) and the same CSV columns, so the tables line up with the reference's plots.
"""
from __future__ import annotations

import argparse
import os
import random
from typing import Callable, Dict, List, Optional

import numpy as np

CSV_COLUMNS = ("Implementation", "FW_Time_ms", "FW_TFLOPS", "batch_size", "seqlen", "nheads", "headdim", "group_size",
               "dropout_p")
BLOCK = 128  # block size of the reference's mask-sparsity accounting (flex_attention's default sparse block size)
DEFAULTS = {"batch_sizes": [32, 16, 8, 4, 2, 1], "seq_lengths": [512, 1024, 2048, 4096, 8192, 16384], "head_dims": [64],
            "group_size": [1, 8], "model_dim": 1024}


def attention_nflop(batch: int, seqlen: int, nheads: int, headdim: int, causal: bool = False) -> float:
    """benchmarks/_utils.py:16-21, forward only."""
    return 4 * batch * seqlen ** 2 * nheads * headdim // (2 if causal else 1)


def benchmark_document_lengths(seqlen: int, num_docs: int = 12) -> List[int]:
    """Document lengths of the reference's mask for the FLOP accounting (run_flex_variants.py:58-77): seed 0, every
    position beyond one per document goes to a uniformly drawn document."""
    rng = random.Random(0)
    lengths = [1] * num_docs
    for _ in range(seqlen - num_docs):
        lengths[rng.randint(0, num_docs - 1)] += 1
    return lengths


def nonempty_block_share(name: str, seqlen: int) -> Optional[float]:
    """Share of the 128 x 128 (query, key) blocks in which the variant's accounting mask attends at least one pair
    (1 - BlockMask.sparsity() / 100 in the reference); None for variants that are accounted dense."""
    nb = (seqlen + BLOCK - 1) // BLOCK
    lo = np.arange(nb) * BLOCK                     # first position of a block
    hi = np.minimum(lo + BLOCK, seqlen) - 1        # last position of a block
    q_lo, q_hi, k_lo, k_hi = lo[:, None], hi[:, None], lo[None, :], hi[None, :]
    causal = k_lo <= q_hi                          # some k <= q
    if name == "full_with_causal":
        occ = causal
    elif name == "full_with_sliding_window":       # 0 <= q - k <= 256 for some pair: [q_lo - k_hi, q_hi - k_lo] meets [0, 256]
        occ = causal & (q_lo - k_hi <= 256)
    elif name == "full_with_prefix_lm":            # k < 256 or k <= q
        occ = causal | (k_lo < 256)
    elif name == "full_with_document_mask":        # same document and k <= q (the accounting mask is the causal one)
        ends = np.cumsum(benchmark_document_lengths(seqlen))
        doc = np.searchsorted(ends, np.arange(seqlen), side="right")
        d_lo, d_hi = doc[lo], doc[hi]              # ids are non-decreasing: a block spans ids d_lo..d_hi
        share = (d_lo[:, None] <= d_hi[None, :]) & (d_lo[None, :] <= d_hi[:, None])
        # a shared document that lies entirely above the diagonal inside a diagonal block still has k <= q pairs only
        # if the block pair is causal-occupied; off-diagonal blocks are either fully below or fully above
        occ = share & causal
    else:
        return None
    return float(occ.sum()) / float(nb * nb)


def variant_flops(name: str, batch: int, seqlen: int, nheads: int, headdim: int) -> float:
    share = nonempty_block_share(name, seqlen)
    if share is not None:
        return share * attention_nflop(batch, seqlen, nheads, headdim)
    return attention_nflop(batch, seqlen, nheads, headdim, causal="causal" in name)


def registry() -> Dict[str, Callable]:
    """Variant name -> callable(q, k, v, enable_gqa=...), run_flex_variants.py:126-147.  The document ids of
    "full_with_document_mask" are drawn once per (batch, seqlen) rather than inside every call: the reference's
    callable runs under torch.compile, where the Python loop that draws them is traced once."""
    from flashlight_amd import attention_variants as A

    ids_cache: dict = {}

    def document_ids(q):
        key = (q.size(0), q.size(2))
        if key not in ids_cache:
            ids_cache[key] = A.create_document_id(q.size(0), q.size(2), num_docs=12)
        return ids_cache[key]

    return {
        "full": lambda q, k, v, **kw: A.attention_pytorch(q, k, v, **kw),
        "full_with_alibi": lambda q, k, v, **kw: A.attention_pytorch_alibi(
            q, k, v, score_mod=A.generate_alibi_bias_pytorch(q.size(-3)), **kw),
        "full_with_softcap": lambda q, k, v, **kw: A.attention_softcapped(q, k, v, score_mod=A.generate_tanh_softcap(30), **kw),
        "full_with_causal": lambda q, k, v, **kw: A.attention_pytorch_causal(q, k, v, **kw),
        "full_with_sliding_window": lambda q, k, v, **kw: A.attention_pytorch_sliding_window(q, k, v, window_size=256, **kw),
        "full_with_prefix_lm": lambda q, k, v, **kw: A.attention_pytorch_prefix_lm(q, k, v, prefix_lengths=256, **kw),
        "full_with_document_mask": lambda q, k, v, **kw: A.attention_pytorch_document_mask(
            q, k, v, document_id=document_ids(q), **kw),
    }


def dropout_registry(dropout_p: float) -> Dict[str, Callable]:
    """The variants that have a dropout kernel (positional masks), with `--dropout_p` applied.  The reference records
    the flag in its CSV and never applies it (benchmarks/_utils.py:231-233); its own variants are timed with
    `--dropout_p 0`.  One fixed seed: the decisions cost the same whatever it is."""
    from flashlight_amd import _ffi, ops

    def variant(**kw):
        return lambda q, k, v, enable_gqa=False: ops.dispatch(q, k, v, dropout_p=dropout_p, dropout_seed=1, **kw)

    return {
        "full": variant(),
        "full_with_causal": variant(mask_kind=_ffi.MASK_CAUSAL),
        "full_with_sliding_window": variant(mask_kind=_ffi.MASK_SLIDING, window=256),
        "full_with_prefix_lm": variant(mask_kind=_ffi.MASK_PREFIX_LM, prefix=256),
    }


def make_qkv(batch: int, seqlen: int, nheads: int, headdim: int, group_size: int):
    """benchmarks/_utils.py:226-247: bf16 N(0,1); without GQA the three tensors are unbound from one packed
    [B, S, 3, H, D] draw and made contiguous in [B, H, S, D] order."""
    import torch

    if nheads % group_size or group_size > nheads:
        raise ValueError(f"cannot divide Hq={nheads} into groups of {group_size}")
    if group_size == 1:
        qkv = torch.randn(batch, seqlen, 3, nheads, headdim, device="cuda", dtype=torch.bfloat16)
        return tuple(t.transpose(1, 2).contiguous() for t in qkv.unbind(dim=2))
    return (torch.randn(batch, nheads, seqlen, headdim, device="cuda", dtype=torch.bfloat16),
            torch.randn(batch, nheads // group_size, seqlen, headdim, device="cuda", dtype=torch.bfloat16),
            torch.randn(batch, nheads // group_size, seqlen, headdim, device="cuda", dtype=torch.bfloat16))


def time_forward(fn: Callable[[], object], n_warmup: int = 10, n_repeat: int = 20) -> float:
    """Mean milliseconds per call, benchmarks/_utils.py:147-199 without the clock-heating loop."""
    import torch

    fn()
    torch.cuda.synchronize()
    cache = torch.empty(int(256e6 // 4), dtype=torch.int, device="cuda")
    for _ in range(n_warmup):
        fn()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for s, e in zip(starts, ends):
        cache.zero_()
        s.record()
        fn()
        e.record()
    torch.cuda.synchronize()
    return sum(s.elapsed_time(e) for s, e in zip(starts, ends)) / n_repeat


def write_results_csv(rows: List[tuple], path: str) -> None:
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "w") as f:
        f.write(",".join(CSV_COLUMNS) + "\n")
        for r in rows:
            f.write(",".join(str(x) for x in r) + "\n")


def parse_args(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--suite", choices=("variants", "diffattn", "evoformer", "ipa", "backward", "decode"), default="variants",
                    help="variants: run_flex_variants.py; diffattn: run_diff_attn.py (model dim 2048, head dims 64 and "
                         "128, published FLOP estimate 8 B S^2 H D); evoformer: run_evoformer.py (N_seq = S = 256, 4 "
                         "heads, mask bias + pair bias, FLOPs 4 B 256 S^2 H D); ipa: invariant point attention of "
                         "tests/test_ipa.py at 12 heads x (16 scalar + 4 query/key points + 8 value points); backward: the "
                         "gradient kernels alone (dq, dk, dv from saved output and row statistics), FLOPs = 2.5 x the "
                         "forward's as in benchmarks/_utils.py:16-21")
    ap.add_argument("--filter", type=str, nargs="+", default=[], help="keywords of variants to benchmark")
    ap.add_argument("--batch_size", type=int, nargs="+", default=DEFAULTS["batch_sizes"])
    ap.add_argument("--seqlen", type=int, nargs="+", default=DEFAULTS["seq_lengths"])
    ap.add_argument("--dim", type=int, default=None, help="model dimension = heads x head dim (1024; 2048 for --suite diffattn)")
    ap.add_argument("--headdim", type=int, nargs="+", default=None, help="head dims (64; 64 and 128 for the other suites)")
    ap.add_argument("--group_size", type=int, nargs="+", default=DEFAULTS["group_size"], help="query heads per key/value head")
    ap.add_argument("--dropout_p", type=float, default=0.0)
    ap.add_argument("--output", type=str, default="benchmark", help="output file name, `.csv` is appended")
    a = ap.parse_args(argv)
    if a.dim is None:
        a.dim = DEFAULTS["model_dim"] if a.suite in ("variants", "backward") else 2048
    if a.headdim is None:
        a.headdim = DEFAULTS["head_dims"] if a.suite in ("variants", "backward") else [16] if a.suite == "ipa" else [64, 128]
    return a


def main(argv=None) -> List[tuple]:
    import torch

    args = parse_args(argv)
    if not torch.cuda.is_available():
        raise SystemExit("run_variants needs an MI355X: there is no CPU execution path")
    torch.manual_seed(0)
    rows: List[tuple] = []
    if args.suite != "variants":
        rows = _run_backward_suite(args) if args.suite == "backward" else _run_decode_suite(args) if args.suite == "decode" \
            else _run_other_suite(args)
        write_results_csv(rows, f"{args.output}.csv")
        return rows
    variants = registry() if args.dropout_p == 0.0 else dropout_registry(args.dropout_p)
    for group_size in args.group_size:
        for headdim in args.headdim:
            for batch, seqlen in zip(args.batch_size, args.seqlen):
                nheads = args.dim // headdim
                config = (batch, seqlen, nheads, headdim, group_size, args.dropout_p)
                print(f"### Config: {config} ###")
                q, k, v = make_qkv(batch, seqlen, nheads, headdim, group_size)
                for name, fn in variants.items():
                    if args.filter and all(key not in name for key in args.filter):
                        continue
                    ms = time_forward(lambda: fn(q, k, v, enable_gqa=group_size != 1))
                    tflops = variant_flops(name, batch, seqlen, nheads, headdim) / ms / 1e9
                    rows.append((name, ms, tflops, *config))
                    print(f"{name:28s} {ms:9.4f} ms {tflops:8.1f} TFLOP/s")
    write_results_csv(rows, f"{args.output}.csv")
    return rows


DECODE_SHAPES = (  # batch, query heads, key / value heads, queries, keys, head dim
    (1, 32, 8, 1, 32768, 128), (8, 32, 8, 1, 8192, 128), (32, 32, 8, 1, 2048, 128), (128, 32, 8, 1, 512, 128),
    (16, 64, 8, 1, 4096, 128), (8, 32, 8, 16, 8192, 128), (4, 32, 32, 1, 4096, 64), (1, 32, 8, 1, 40001, 128))


def _run_decode_suite(args) -> List[tuple]:
    """Decoding steps (no counterpart in the reference's sweeps): a few queries per sequence against a long key / value
    cache, unmasked, grouped heads.  Times `attention_pytorch` (the front end packs the query heads of a key / value head
    as rows and splits long key sequences into chunks) and, as `torch_sdpa`, torch's scaled_dot_product_attention on the
    same operands (warm caches: a cache that was just written).  The TFLOP/s column is replaced by the rate at which the
    keys and values are read, in TB/s."""
    import torch
    import torch.nn.functional as F
    from ..attention_variants import attention_pytorch

    def warm(fn, n=50):
        for _ in range(10):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(n):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / n

    rows: List[tuple] = []
    for B, Hq, Hkv, Lq, Lk, D in DECODE_SHAPES:
        q = torch.randn(B, Hq, Lq, D, device="cuda", dtype=torch.bfloat16)
        k, v = (torch.randn(B, Hkv, Lk, D, device="cuda", dtype=torch.bfloat16) for _ in range(2))
        print(f"### Config: B={B} Hq={Hq} Hkv={Hkv} Lq={Lq} Lk={Lk} D={D} ###")
        for name, fn in (("decode", lambda: attention_pytorch(q, k, v, enable_gqa=True)),
                         ("torch_sdpa", lambda: F.scaled_dot_product_attention(q, k, v, enable_gqa=True))):
            ms = warm(fn)
            tbs = 2 * k.numel() * 2 / ms / 1e9
            rows.append((name, ms, tbs, B, Lk, Hq, D, Hq // Hkv, 0.0))
            print(f"{name:28s} {ms:9.4f} ms {tbs:8.2f} TB/s of keys and values")
    return rows


def _run_backward_suite(args) -> List[tuple]:
    """Times fl_attn_bwd alone for the variants that have a backward, on the sweep's shapes.  The reference has no
    backward to compare with; its FLOP helper's "bwd" mode (2.5 x forward, benchmarks/_utils.py:16-21) and the same
    128-block accounting as the forward sweep give the TFLOP/s column."""
    import torch

    from flashlight_amd import _ffi
    from flashlight_amd.attention_variants.document_mask import create_document_id

    rows: List[tuple] = []
    for group_size in args.group_size:
        for headdim in args.headdim:
            for batch, seqlen in zip(args.batch_size, args.seqlen):
                nheads = args.dim // headdim
                config = (batch, seqlen, nheads, headdim, group_size, args.dropout_p)
                print(f"### Config: {config} ###")
                q, k, v = make_qkv(batch, seqlen, nheads, headdim, group_size)
                dout = torch.randn_like(q)
                cases = {  # the forward sweep's names and parameters (registry() above)
                    "full": {},
                    "full_with_alibi": dict(alibi_heads=nheads),
                    "full_with_softcap": dict(softcap=30.0),
                    "full_with_causal": dict(mask_kind=_ffi.MASK_CAUSAL),
                    "full_with_sliding_window": dict(mask_kind=_ffi.MASK_SLIDING, window=256),
                    "full_with_prefix_lm": dict(mask_kind=_ffi.MASK_PREFIX_LM, prefix=256),
                    "full_with_document_mask": dict(mask_kind=_ffi.MASK_DOCUMENT,
                                                    doc_ids=create_document_id(batch, seqlen, num_docs=12)),
                }
                if args.dropout_p > 0.0:  # the positional-mask cases have a dropout kernel
                    cases = {n: dict(kw, dropout_p=args.dropout_p, dropout_seed=1) for n, kw in cases.items()
                             if not ({"alibi_heads", "softcap", "doc_ids"} & set(kw))}
                for name, kw in cases.items():
                    if args.filter and all(key not in name for key in args.filter):
                        continue
                    lse = torch.empty(batch, nheads, seqlen, dtype=torch.float32, device="cuda")
                    out = _ffi.attn_fwd(q, k, v, lse=lse, **kw)
                    ms = time_forward(lambda: _ffi.attn_bwd(q, k, v, out, lse, dout, **kw))
                    tflops = 2.5 * variant_flops(name, batch, seqlen, nheads, headdim) / ms / 1e9
                    rows.append((name + "_bwd", ms, tflops, *config))
                    print(f"{name + '_bwd':28s} {ms:9.4f} ms {tflops:8.1f} TFLOP/s")
    return rows


def _run_other_suite(args) -> List[tuple]:
    """run_diff_attn.py:42-82 / run_evoformer.py:40-82 with this package's kernels as the only implementation."""
    import torch

    from flashlight_amd import attention_variants as A
    from flashlight_amd._ffi import FlashlightError

    rows: List[tuple] = []
    for headdim in args.headdim:
        for batch, seqlen in zip(args.batch_size, args.seqlen):
            if args.suite == "diffattn":
                nheads = args.dim // headdim
                config = (batch, seqlen, nheads, headdim, 1, args.dropout_p)
                flops = 8 * batch * seqlen ** 2 * nheads * headdim  # the reference's estimate ("double vanilla"); 6 is exact
                inputs = A.diff_attn.make_input(config)
                name, fn = "diffattn", lambda: A.diffattn(*inputs)
            elif args.suite == "ipa":
                # not swept by the reference (tests/test_ipa.py runs one shape once): AlphaFold's structure-module head
                # layout, 12 heads of 16 scalar channels, 4 query/key points and 8 value points, `seqlen` residues;
                # FLOPs count both products over the channels that carry data (16 + 12 and 16 + 24), launch and the
                # concatenation of scalar and point channels included in the time
                nheads, c, pq, pv = 12, 16, 4, 8
                config = (batch, seqlen, nheads, c, 1, args.dropout_p)
                flops = 2 * batch * nheads * seqlen ** 2 * ((c + 3 * pq) + (c + 3 * pv))
                mk = lambda *shape: torch.randn(*shape, dtype=torch.bfloat16, device="cuda")  # noqa: E731
                inputs = (mk(batch, nheads, seqlen, c), mk(batch, nheads, seqlen, c), mk(batch, nheads, seqlen, c),
                          mk(batch, nheads, seqlen, pq, 3), mk(batch, nheads, seqlen, pq, 3),
                          mk(batch, nheads, seqlen, pv, 3), mk(batch, nheads, seqlen, seqlen))
                name, fn = "ipa", lambda: A.invariant_point_attention(*inputs, c_hidden=c, no_qk_points=pq)
            else:
                seqlen, nheads = 256, 4
                config = (batch, seqlen, nheads, headdim, 1, args.dropout_p)
                flops = 4 * batch * 256 * seqlen ** 2 * nheads * headdim
                inputs = A.evoformer.make_input(config)
                name, fn = "evoformer", lambda: A.attention_reference(*inputs)
            print(f"### Config: {config} ###")
            try:
                ms = time_forward(fn)
            except FlashlightError as e:  # a head-dim combination without a kernel instance
                print(f"{name:28s} skipped: {e}")
                continue
            rows.append((name, ms, flops / ms / 1e9, *config))
            print(f"{name:28s} {ms:9.4f} ms {flops / ms / 1e9:8.1f} TFLOP/s")
    return rows


if __name__ == "__main__":
    main()
