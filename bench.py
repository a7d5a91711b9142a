#!/usr/bin/env python3
"""Benchmark of the fused attention forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-other-configs] [--calibrate-copy]

A step is one pass of the hot path over the headline benchmark batch (configuration 1: B=4, H=16, S=4096, D=128, bf16,
seeded N(0,1) inputs already resident in HBM): one vanilla, one causal and one sliding-window (window 256) forward,
three kernel launches.  `value` is the unmasked (algorithmic) FLOPs of the step divided by its wall time.  Prints one
JSON line; per-variant numbers, the roofline of the dominant kernel, the other configurations (measured outside the
timed region) and the CPU baseline ride along in it.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the eager CPU timing (about 20 s)")
    ap.add_argument("--no-other-configs", action="store_true", help="only run the configuration the metric is quoted on")
    ap.add_argument("--only", metavar="WORKLOAD", default=None,
                    help="profiling aid: launch just this workload (e.g. cfg3/document_mask_causal) --warmup + --steps times "
                         "and print its event-timed duration; nothing else runs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one 256 MiB device-to-device copy (known traffic, for scaling rocprofv3 counters)")
    return ap.parse_args()


def measured_hbm_bytes() -> dict:
    """HBM bytes per launch of each workload as rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE measured them (scaled by a
    256 MiB copy's readings): profiles/hbm_traffic.json, written from the same profiler runs as the per-workload
    summaries beside it (which give the commands and raw values).  Empty if the file is missing."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            return {k: float(v) for k, v in json.load(f)["bytes_per_launch"].items()}
    except (OSError, KeyError, ValueError):
        return {}

FLUSH_BYTES = 512 << 20  # twice the 256 MB memory-side cache: zeroing it evicts the operands of the previous launch
CPU_CAP_S = 12.0         # wall-clock cap per configuration for the eager CPU timing


def event_pair():
    return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)


def time_launches(fn, iters: int, warmup: int = 20, flush=None, flush_by: str = "zero"):
    """Trimmed mean / median / plain mean duration (ms) of single launches of `fn`, each bracketed by its own pair of events on the
    current stream (the stream the kernels are launched on).  With `flush` (a device buffer larger than the caches)
    the buffer is zeroed before every bracketed launch, like the reference's harness does (benchmarks/_utils.py:145-151
    there): the launch then reads its operands from HBM.  Zeroing leaves the memory-side cache full of modified lines,
    whose write-back shares the HBM with the launch that follows (a plain copy of 268 MB takes 0.072 ms after it, 0.049
    ms after a flush that only reads); `flush_by="read"` sums the buffer instead: cold operands, clean cache."""
    for _ in range(warmup):
        fn()
    pairs = [event_pair() for _ in range(iters)]
    for a, b in pairs:
        if flush is not None:
            if flush_by == "zero":
                flush.zero_()
            else:
                flush.view(torch.int32).sum()
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in pairs)
    keep = ts[: max(1, int(len(ts) * 0.9))]  # drop the slowest tenth: one-off host hiccups land inside an event pair
    return statistics.fmean(keep), statistics.median(ts), statistics.fmean(ts)


def time_back_to_back(fn, iters: int, warmup: int = 10) -> float:
    """Average duration (ms) of `iters` launches of `fn` queued back to back between one pair of events."""
    for _ in range(warmup):
        fn()
    a, b = event_pair()
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def roofline_entry(w, ms: float, W) -> dict:
    """Fraction of the roofline that bounds workload `w` at a launch duration of `ms`: unmasked FLOPs against the bf16
    MFMA peak, or algorithmic bytes (every operand and the result touched once) against the HBM peak."""
    if w.bound == "hbm":
        gbps = w.min_bytes / ms / 1e6
        return {"bound": "hbm", "achieved": gbps, "peak": W.PEAK_HBM_GBPS, "unit": "GB/s", "frac": gbps / W.PEAK_HBM_GBPS}
    tf = w.flops / ms / 1e9
    return {"bound": "mfma", "achieved": tf, "peak": W.PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tf / W.PEAK_BF16_TFLOPS}


def _cpu_chunks(t: dict):
    """Independent slices of a workload's CPU tensors: one per batch element, or per 32 N_seq rows of the 5-D
    Evoformer layout [B, N_seq, S, H, D] (whose pair bias [B, 1, H, S, S] is shared by all of them)."""
    q = t["q"]
    if q.dim() == 5:
        for a in range(0, q.size(1), 32):
            yield {k: (v if k == "pair_bias" else v[:, a:a + 32]) for k, v in t.items()}
    else:
        for b in range(q.size(0)):
            yield {k: v[b:b + 1] for k, v in t.items()}


def cpu_baseline() -> dict:
    """The eager fp32 restatement of the reference's CPU-runnable path (oracle/), timed on this host's cores: once over
    every benchmark configuration, in independent slices (one batch element at a time) and query blocks of 512 rows so
    that the dense score matrices fit, under a wall-clock cap per configuration.  `value` is the headline step
    (configuration 1: vanilla + causal + sliding window); a configuration that hits the cap reports the rate of the
    slices it finished and says so."""
    from oracle.benchmark_cases import evaluate  # the checker, imported here only to be timed as the CPU baseline
    import oracle as O
    from flashlight_amd import workloads as W

    cpu = torch.device("cpu")
    per = {}
    for w in W.build_workloads():
        t = {k: (v.float() if v.is_floating_point() else v) for k, v in w.make(cpu).items()}
        chunks = list(_cpu_chunks(t))
        done, elapsed = 0, 0.0
        for c in chunks:
            t0 = time.perf_counter()
            evaluate(w.name, c, w.params, q_block=512)
            elapsed += time.perf_counter() - t0
            done += 1
            if elapsed > CPU_CAP_S:
                break
        full_s = elapsed * len(chunks) / done
        per[w.name] = {"ms": 1e3 * full_s, "unmasked_TFLOPs": w.flops / full_s / 1e12, "slices_timed": done,
                       "slices_total": len(chunks)}
        if done < len(chunks):
            per[w.name]["note"] = (f"skipped: over cap ({CPU_CAP_S:.0f} s) after {done} of {len(chunks)} slices; ms is "
                                   "extrapolated from the slices timed")
        del t, chunks
    cfg1 = [w for w in W.build_workloads() if w.config == 1]
    step_s = sum(per[w.name]["ms"] for w in cfg1) / 1e3
    # configuration 0 of the baseline file: causal, B=2 H=8 S=512 D=64 fp32, the reference's own CPU-sized case
    g0 = torch.Generator().manual_seed(1000)
    q0, k0, v0 = (torch.randn(2, 8, 512, 64, generator=g0) for _ in range(3))
    O.attention_causal(q0, k0, v0)
    t0s = []
    for _ in range(10):
        t0 = time.perf_counter()
        O.attention_causal(q0, k0, v0)
        t0s.append(time.perf_counter() - t0)
    cfg0_flops = 4 * 64 * W.pairs_causal(512) * 16
    return {
        "value": sum(w.flops for w in cfg1) / step_s / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "eager fp32 oracle (dense scores like the reference, 512 query rows at a time), one pass over the "
                  "whole of configuration 1 (vanilla + causal + sliding window 256 at B=4 H=16 S=4096 D=128), "
                  f"{step_s:.1f} s; unmasked FLOPs.  per_config holds one pass over each other configuration",
        "per_config": per, "cap_s_per_config": CPU_CAP_S, "host_cpus": os.cpu_count(),
        "cfg0_causal_fp32_B2_H8_S512_D64": {"ms": 1e3 * statistics.median(t0s),
                                              "unmasked_GFLOPs": cfg0_flops / statistics.median(t0s) / 1e9},
    }


PREWARM_S = 0.5  # untimed run-in before the warm-up steps


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the fused forward is a single-device kernel and this build has no "
                 "multi-GPU path; run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X: no GPU is visible and there is no CPU execution path")
    from flashlight_amd import _ffi
    from flashlight_amd import workloads as W

    _ffi.load_library()  # fail loudly if the HIP extension is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.only:
        w = W.workload_by_name(args.only)
        t = w.make(dev)
        ms = time_back_to_back(lambda: w.call(t), iters=args.steps, warmup=args.warmup)
        if args.calibrate_copy:
            src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
            dst = torch.empty_like(src)
            dst.copy_(src)
            torch.cuda.synchronize()
        print(json.dumps({"workload": w.name, "ms": ms, "launches": args.steps, "warmup": args.warmup,
                          "unmasked_flops": w.flops, "min_bytes": w.min_bytes, "roofline": roofline_entry(w, ms, W)}))
        return
    all_w = W.build_workloads()
    cfg1 = [w for w in all_w if w.config == 1]
    tens = cfg1[0].make(dev)  # the three variants share q, k, v (same seed)
    step_flops = sum(w.flops for w in cfg1)

    def step():
        for w in cfg1:
            w.call(tens)

    # An idle part takes a few hundred milliseconds of load to reach its running clocks (30 steps, 25 ms, measured
    # 20 % slow on a fresh box): untimed steps for PREWARM_S seconds first, then the W warm-up steps that were asked for.
    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < PREWARM_S:
        step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # per-launch durations of each variant, HIP events on the launch stream: warm (the same operands launch after
    # launch, partly served by the 256 MB memory-side cache) and flushed (a 512 MB buffer zeroed before each launch)
    flush = torch.empty(FLUSH_BYTES, dtype=torch.uint8, device=dev)
    variants = {}
    for w in cfg1:
        mean_ms, med_ms, all_ms = time_launches(lambda w=w: w.call(tens), iters=max(50, args.steps))
        cold_ms, cold_med, _ = time_launches(lambda w=w: w.call(tens), iters=50, warmup=5, flush=flush)
        clean_ms, _, _ = time_launches(lambda w=w: w.call(tens), iters=50, warmup=5, flush=flush, flush_by="read")
        tf = w.flops / mean_ms / 1e9
        variants[w.name] = {"ms": mean_ms, "ms_median": med_ms, "ms_mean_untrimmed": all_ms,
                            "timing": "ms: mean of single event-bracketed launches without the slowest tenth; "
                                      "ms_mean_untrimmed: all of them; ms_back_to_back: launches queued between one pair of events",
                            "tflops": tf, "pct_mfma_peak": 100 * tf / W.PEAK_BF16_TFLOPS,
                            "ms_back_to_back": time_back_to_back(lambda w=w: w.call(tens), iters=max(50, args.steps), warmup=20),
                            "ms_flushed": cold_ms, "ms_flushed_median": cold_med, "tflops_flushed": w.flops / cold_ms / 1e9,
                            "ms_cold": clean_ms, "unmasked_flops": w.flops, "min_bytes": w.min_bytes,
                            "roofline": roofline_entry(w, mean_ms, W), "roofline_flushed": roofline_entry(w, cold_ms, W),
                            "roofline_cold": roofline_entry(w, clean_ms, W)}
    dom = max(cfg1, key=lambda w: variants[w.name]["ms"])  # the launch that dominates the step
    dv = variants[dom.name]
    roofline = {"bound": "mfma", "kernel": f"fl::fwd_kernel ({dom.name})", "achieved": dv["tflops"],
                "peak": W.PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": dv["tflops"] / W.PEAK_BF16_TFLOPS,
                "frac_flushed": dv["tflops_flushed"] / W.PEAK_BF16_TFLOPS,
                "traffic": measured_hbm_bytes().get(dom.name), "traffic_unit": "bytes/launch (rocprofv3, see profiles/)",
                "launch_ms": dv["ms"], "flops_per_launch": dom.flops}
    step_flushed_ms = sum(v["ms_flushed"] for v in variants.values())

    others = {}
    if not args.no_other_configs:
        del tens
        for w in all_w:
            if w.config == 1:
                continue
            t = w.make(dev)
            t_ramp = time.perf_counter()  # (the same run-in as the headline step gets: the clocks follow the load)
            while time.perf_counter() - t_ramp < PREWARM_S / 2:
                w.call(t)
                torch.cuda.synchronize()
            runs = [time_back_to_back(lambda: w.call(t), iters=100, warmup=50) for _ in range(3)]
            mean_ms = min(runs)
            cold_ms, _, _ = time_launches(lambda: w.call(t), iters=50, warmup=5, flush=flush)
            clean_ms, _, _ = time_launches(lambda: w.call(t), iters=50, warmup=5, flush=flush, flush_by="read")
            tf = w.flops / mean_ms / 1e9
            others[w.name] = {"ms": mean_ms, "ms_mean_of_runs": statistics.fmean(runs),
                              "timing": "ms: BEST of three runs of 100 launches back to back, each after 50 warm-up launches "
                                        "(ms_mean_of_runs: their mean); flushed: 50 launches, 512 MB zeroed before each",
                              "ms_flushed": cold_ms, "tflops": tf, "tflops_flushed": w.flops / cold_ms / 1e9,
                              "pct_mfma_peak": 100 * tf / W.PEAK_BF16_TFLOPS, "unmasked_flops": w.flops,
                              "ms_cold": clean_ms, "min_bytes": w.min_bytes, "roofline": roofline_entry(w, mean_ms, W),
                              "roofline_flushed": roofline_entry(w, cold_ms, W), "roofline_cold": roofline_entry(w, clean_ms, W)}
            if w.name == "cfg3/document_mask_causal":
                # the same call with a workspace handle that keeps the pre-pass's result (the key tiles every query tile
                # visits) across calls on one id tensor, as a model that runs many layers over one packed batch would:
                # reported beside the headline, which pays the pre-pass on every call
                from flashlight_amd.attention_variants import DocumentMaskWorkspace, attention_pytorch_document_mask
                ws = DocumentMaskWorkspace()
                prepared = lambda: attention_pytorch_document_mask(t["q"], t["k"], t["v"], t["document_id"], is_causal=True,  # noqa: E731
                                                                   workspace=ws)
                ms_p = min(time_back_to_back(prepared, iters=100, warmup=50) for _ in range(3))
                others[w.name]["prepared_workspace"] = {"ms": ms_p, "tflops": w.flops / ms_p / 1e9,
                                                        "roofline": roofline_entry(w, ms_p, W),
                                                        "note": "pre-pass skipped (FL_FLAG_DOC_PREPARED); best of three runs"}
            del t
            torch.cuda.empty_cache()
    # What a plain device-to-device copy with the headline configuration's traffic (268 MB read + written) takes under the
    # same three cache states: the practical HBM roofline of this part for the launches that are bound by it.
    src = torch.empty(128 << 20, dtype=torch.uint8, device=dev).random_()
    dst = torch.empty_like(src)
    copy_bytes = 2 * src.numel()
    hbm_cal = {"bytes": copy_bytes,
               "ms_warm": time_launches(lambda: dst.copy_(src), iters=50)[1],
               "ms_flushed": time_launches(lambda: dst.copy_(src), iters=50, warmup=5, flush=flush)[1],
               "ms_cold": time_launches(lambda: dst.copy_(src), iters=50, warmup=5, flush=flush, flush_by="read")[1]}
    for entry, w in [(variants[w.name], w) for w in cfg1] + [(others[w.name], w) for w in all_w if w.name in others]:
        if w.bound == "hbm":  # fraction of the plain copy's rate on the same number of bytes in the same cache state
            entry["vs_copy"] = {st: hbm_cal["ms_" + st] * w.min_bytes / copy_bytes / entry[key]
                                for st, key in (("warm", "ms"), ("flushed", "ms_flushed"), ("cold", "ms_cold"))}
    del flush, src, dst

    # What the matrix pipe alone sustains on this part (same MFMA instruction, operands in registers, nothing else
    # running), on N(0,1) operands like the benchmark's and on zeros, and the forward itself on all-zero inputs: the
    # part lowers its clock under data-dependent power, so these put the roofline fraction in context.
    context = {}
    if not args.no_other_configs:
        n_cu = torch.cuda.get_device_properties(0).multi_processor_count
        sink = torch.empty(n_cu * 512, dtype=torch.float32, device=dev)
        g = torch.Generator().manual_seed(7)
        ops = {"randn_operands": torch.randn(1 << 23, generator=g).to(torch.bfloat16).to(dev),
               "zero_operands": torch.zeros(1 << 23, dtype=torch.bfloat16, device=dev)}
        for tag, x in ops.items():
            flops = [0.0]

            def run(x=x):
                flops[0] = _ffi.probe_mfma_rate(x, 600, n_cu, sink)
            ms = time_back_to_back(run, iters=100, warmup=30)
            context["mfma_only_" + tag + "_TFLOPs"] = flops[0] / ms / 1e9
        tens = cfg1[0].make(dev)
        zeros = {k: torch.zeros_like(v) for k, v in tens.items()}
        ms = time_back_to_back(lambda: cfg1[0].call(zeros), iters=100, warmup=30)
        context["vanilla_on_zero_inputs_TFLOPs"] = cfg1[0].flops / ms / 1e9
        # the dominant launch against what the matrix pipe alone sustains on the same kind of data in this run
        context["roofline_frac_vs_mfma_only_randn"] = roofline["achieved"] / context["mfma_only_randn_operands_TFLOPs"]
        del tens, zeros, ops
        # The forward's step as a register-only probe (zero operands): nominal-clock cycles per 32 x 32 block of scores
        # and SIMD for the MFMAs alone, for the step as the forward has it (softmax vector work, data dependences), and
        # with the K / V fragments read from LDS; last, the forward itself on zero inputs.  The three-stage order of the
        # step (second product on the previous block's weights, both MFMA groups under the vector work) is the rung
        # the forward was built and measured on and does not use: its gain shows on zero operands only.
        sink2 = torch.empty(2 * n_cu * 256, dtype=torch.float32, device=dev)
        ladder = {}
        for D in (64, 128):
            for level, tag in ((0, "mfma_only"), (2, "step_in_registers"), (4, "three_stage_step_in_registers"),
                               (3, "plus_lds_operand_reads")):
                blocks = [0]

                def run(D=D, level=level):
                    blocks[0] = _ffi.probe_step(D, level, 1000, 2 * n_cu, sink2)
                ms = time_back_to_back(run, iters=20, warmup=5)
                # two workgroups of four waves per compute unit: every SIMD hosts two waves
                ladder[f"d{D}_{tag}"] = ms * 1e-3 * 2.4e9 / (2 * blocks[0])
        ladder["d128_forward_zero_inputs"] = 16 * 32 / (context["vanilla_on_zero_inputs_TFLOPs"] / W.PEAK_BF16_TFLOPS)
        context["cycles_per_block_at_2p4GHz"] = ladder
        # How much vector work fits under a matrix instruction (shader cycles per 32x32x16 MFMA, or per two 16x16x32, per
        # SIMD, two waves per SIMD; k = vector instructions of that kind after every unit of matrix work): the bare loop
        # takes 33-34; multiply-adds ride free up to 4 per MFMA (half of its 32 cycles) and cost their own time beyond;
        # the shorter MFMA leaves no more room; a lone v_dot2c_f32_bf16 waits for the matrix pipe to drain.
        co = {}
        for rows, kind, ks in ((32, "fma", (0, 2, 4, 6, 8)), (16, "fma", (0, 2, 4, 8)), (32, "exp", (1, 2, 4)),
                               (32, "dot2c", (1, 2, 4)), (32, "add", (2, 4)), (32, "cvt_pk_bf16", (2, 4))):
            co[f"mfma{rows}_{kind}"] = {f"k{k}": round(_ffi.probe_coissue(rows, kind, k, 2)["slowest_wave"], 1) for k in ks}
        context["coissue_cycles_per_mfma"] = co

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    line = {
        "metric": "fwd TFLOP/s (unmasked FLOPs)", "value": step_flops / wall_ms / 1e9, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "prewarm_s": PREWARM_S, "ms_per_step": wall_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: vanilla + causal + sliding-window(256, causal) forward, "
                               "B=4 H=16 S=4096 D=128, one launch each per step",
                   "seed": cfg1[0].seed, "unmasked_flops_per_step": step_flops},
        "pct_mfma_peak": 100 * step_flops / wall_ms / 1e9 / W.PEAK_BF16_TFLOPS,
        "cache_state": "value and ms_per_step: warm (steps back to back on the same operands); *_flushed: 512 MB zeroed "
                       "before each launch (the reference harness's recipe; the cache is then full of modified lines); "
                       "*_cold: 512 MB read before each launch (cold operands, clean cache)",
        "hbm_calibration": hbm_cal,
        "ms_per_step_flushed": step_flushed_ms, "value_flushed": step_flops / step_flushed_ms / 1e9,
        "peak_used_TFLOPs": W.PEAK_BF16_TFLOPS,
        "variants": variants, "roofline": roofline, "other_configs": others, "power_context": context,
        "device": torch.cuda.get_device_name(0),
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
