"""The harness-compatible sweep (flashlight_amd/benchmarks/run_variants.py): its FLOP accounting against dense masks,
its CSV layout against the reference's columns (benchmarks/_utils.py:24-28,362-373), and a tiny sweep on the GPU."""
import csv

import numpy as np
import pytest

from flashlight_amd.benchmarks import run_variants as R
from oracle import masks as M


def brute_block_share(attend: np.ndarray, block: int = 128) -> float:
    S = attend.shape[0]
    nb = (S + block - 1) // block
    occ = sum(bool(attend[i * block:(i + 1) * block, j * block:(j + 1) * block].any()) for i in range(nb) for j in range(nb))
    return occ / (nb * nb)


@pytest.mark.parametrize("S", [512, 1000, 2048])
def test_block_share_matches_dense_masks(S):
    assert R.nonempty_block_share("full_with_causal", S) == brute_block_share(M.attend_matrix("causal", S, S))
    assert R.nonempty_block_share("full_with_sliding_window", S) == brute_block_share(M.attend_matrix("sliding", S, S, window=256))
    assert R.nonempty_block_share("full_with_prefix_lm", S) == brute_block_share(M.attend_matrix("prefix", S, S, prefix=256))
    lengths = R.benchmark_document_lengths(S)
    assert sum(lengths) == S and len(lengths) == 12 and min(lengths) >= 1
    ids = np.repeat(np.arange(12), lengths)
    assert R.nonempty_block_share("full_with_document_mask", S) == brute_block_share(M.attend_matrix("document_causal", S, S, doc_ids=ids))
    for dense in ("full", "full_with_alibi", "full_with_softcap"):
        assert R.nonempty_block_share(dense, S) is None


def test_flop_accounting_and_defaults():
    assert R.attention_nflop(2, 1024, 16, 64) == 4 * 2 * 1024 ** 2 * 16 * 64
    assert R.variant_flops("full", 2, 1024, 16, 64) == R.attention_nflop(2, 1024, 16, 64)
    # 8 x 8 blocks, 36 on or below the diagonal
    assert R.variant_flops("full_with_causal", 2, 1024, 16, 64) == pytest.approx(36 / 64 * R.attention_nflop(2, 1024, 16, 64))
    a = R.parse_args([])
    assert a.batch_size == [32, 16, 8, 4, 2, 1] and a.seqlen == [512, 1024, 2048, 4096, 8192, 16384]
    assert a.dim == 1024 and a.headdim == [64] and a.group_size == [1, 8] and a.output == "benchmark"


def test_csv_layout(tmp_path):
    path = tmp_path / "out.csv"
    R.write_results_csv([("full", 0.5, 100.0, 1, 512, 16, 64, 1, 0.0)], str(path))
    rows = list(csv.reader(open(path)))
    assert rows[0] == ["Implementation", "FW_Time_ms", "FW_TFLOPS", "batch_size", "seqlen", "nheads", "headdim",
                       "group_size", "dropout_p"]
    assert rows[1][0] == "full" and len(rows[1]) == 9


@pytest.mark.gpu
def test_tiny_sweep_on_gpu(tmp_path):
    rows = R.main(["--batch_size", "2", "--seqlen", "512", "--group_size", "1", "8", "--output", str(tmp_path / "b")])
    assert len(rows) == 14 and {r[0] for r in rows} == set(R.registry())
    assert all(r[1] > 0 and r[2] > 0 for r in rows)
    assert (tmp_path / "b.csv").exists()


def test_dropout_registry_is_a_subset_with_the_same_names():
    # --dropout_p > 0 times the variants that have a dropout kernel, under the forward sweep's names
    assert set(R.dropout_registry(0.1)) == {"full", "full_with_causal", "full_with_sliding_window", "full_with_prefix_lm"}
    assert set(R.dropout_registry(0.1)) <= set(R.registry())


@pytest.mark.gpu
def test_tiny_sweep_with_dropout_on_gpu(tmp_path):
    rows = R.main(["--batch_size", "2", "--seqlen", "512", "--group_size", "1", "--dropout_p", "0.1", "--output",
                   str(tmp_path / "d")])
    assert {r[0] for r in rows} == set(R.dropout_registry(0.1)) and all(r[-1] == 0.1 and r[1] > 0 for r in rows)
    rows = R.main(["--suite", "backward", "--batch_size", "2", "--seqlen", "512", "--group_size", "1", "--dropout_p", "0.1",
                   "--output", str(tmp_path / "e")])
    assert {r[0] for r in rows} == {n + "_bwd" for n in R.dropout_registry(0.1)}


def test_measured_traffic_file_covers_every_workload_and_agrees_with_the_summaries():
    # bench.py reports roofline.traffic from profiles/hbm_traffic.json; the figure has to be the one the per-workload
    # profiler summary beside it states, for every benchmark workload
    import glob
    import json
    import os
    import re
    from flashlight_amd import workloads as W
    root = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "profiles")
    table = json.load(open(os.path.join(root, "hbm_traffic.json")))["bytes_per_launch"]
    assert set(table) == {w.name for w in W.build_workloads()}
    seen = {}
    for path in glob.glob(os.path.join(root, "*_cfg*.md")):
        text = open(path).read()
        name = re.match(r"# (\S+) ", text).group(1)
        seen[name] = float(re.search(r"^Total ([\d.]+) MB against", text, re.M).group(1)) * 1e6
    assert set(seen) == set(table)
    for name, measured in seen.items():
        assert abs(table[name] - measured) <= 0.5e5, name
