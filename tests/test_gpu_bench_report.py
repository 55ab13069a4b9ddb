"""The sweep benchmark (attention_amd/host/bench_report.cpp) writes a results file with the field names of the
reference's SaveResultsToJSON, benchmarks/benchmark_attention.cpp:625-669, and its derived figures follow
the reference's formulas (:241-246), backward pass timed as there (:215-235); --csv writes the table of
examples/performance_comparison.cpp:431-463."""
import csv
import json
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "attention_amd", "lib", "ahpc_bench_report")

pytestmark = pytest.mark.gpu

REFERENCE_FIELDS = ["backend", "batch_size", "sequence_length", "num_heads", "head_dimension", "total_elements", "success",
                    "forward_time_ms", "backward_time_ms", "total_time_ms", "memory_usage_bytes", "peak_memory_bytes", "gflops",
                    "throughput_tokens_per_sec", "theoretical_flops"]


@pytest.mark.parametrize("args", [["--device", "--dtype", "bf16", "--causal"], []])
def test_quick_sweep_writes_reference_shaped_results(tmp_path, args):
    assert os.path.exists(BIN), f"{BIN} missing: run __graft_entry__.build()"
    out = tmp_path / "benchmark_results.json"
    table = tmp_path / "performance_results.csv"
    r = subprocess.run([BIN, "--quick", "--json", str(out), "--csv", str(table)] + args, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "=== Performance Report ===" in r.stdout and "Best GFLOPS" in r.stdout
    rows = json.loads(out.read_text())["benchmark_results"]
    assert len(rows) == 2 * 3 * 2 * 2
    for row in rows:
        for f in REFERENCE_FIELDS:
            assert f in row, f
        assert row["success"] is True and row["backend"] == "HIP"
        B, N, H, d = (row[k] for k in ("batch_size", "sequence_length", "num_heads", "head_dimension"))
        assert row["total_elements"] == B * N * H * d
        assert row["backward_time_ms"] > 0
        assert row["total_time_ms"] == pytest.approx(row["forward_time_ms"] + row["backward_time_ms"], rel=1e-4)
        assert row["gflops"] == pytest.approx(B * H * N * N * d * 2 / 1e9 / (row["total_time_ms"] / 1e3), rel=1e-3)
        assert row["throughput_tokens_per_sec"] == pytest.approx(B * N / (row["forward_time_ms"] / 1e3), rel=1e-3)
        assert row["theoretical_flops"] == pytest.approx(B * H * N * N * (2 * d + 4), rel=1e-5)
        assert row["tensors_resident_on_device"] is ("--device" in args)
    # PagedAttention rows: the configurations BM_PagedAttention is registered for (benchmarks/benchmark_attention.cpp:436-457)
    assert "=== PagedAttention" in r.stdout
    paged = json.loads(out.read_text())["paged_results"]
    assert [(p["batch_size"], p["sequence_length"], p["num_heads"], p["head_dimension"]) for p in paged] == [
        (2, N, H, d) for N in (256, 512, 1024) for H in (4, 8) for d in (64, 128)]
    es = 4 if "--dtype" not in args else 2
    for p in paged:
        assert p["success"] is True and p["page_size"] == 16 and p["forward_time_ms"] > 0 and 0 < p["decode_time_ms"] < p["forward_time_ms"]
        n = p["batch_size"] * p["sequence_length"] * p["num_heads"] * p["head_dimension"]
        assert p["bytes_per_second"] == pytest.approx(n * es * 4 / (p["forward_time_ms"] / 1e3), rel=1e-3)
        assert p["decode_kv_bytes_per_second"] == pytest.approx(2 * n * es / (p["decode_time_ms"] / 1e3), rel=1e-3)
    # the CSV: the reference's header, one row per configuration, the same figures
    with open(table) as f:
        lines = list(csv.reader(f))
    assert lines[0] == ["Backend", "BatchSize", "SequenceLength", "NumHeads", "HeadDimension", "ForwardTimeMs", "BackwardTimeMs",
                        "TotalTimeMs", "MemoryUsageMB", "PeakMemoryMB", "ThroughputTokensPerSec", "GFLOPS", "Success", "ErrorMessage"]
    assert len(lines) == 1 + len(rows)
    for line, row in zip(lines[1:], rows):
        assert line[0] == "HIP" and [int(x) for x in line[1:5]] == [row[k] for k in ("batch_size", "sequence_length", "num_heads", "head_dimension")]
        assert float(line[5]) == pytest.approx(row["forward_time_ms"], rel=1e-4, abs=1e-5) and float(line[6]) == pytest.approx(row["backward_time_ms"], rel=1e-4, abs=1e-5)
        assert float(line[7]) == pytest.approx(row["total_time_ms"], rel=1e-4, abs=1e-5) and float(line[11]) == pytest.approx(row["gflops"], rel=1e-3, abs=1e-3)
        assert line[12] == "true" and line[13] == ""
