"""bench.py's contract at the edges that no measurement run shows: more than one GPU is refused
with one line and exit status 2, and the burst phase (the workload of the reference's own serving
benchmark, benchmarks/BENCHMARK_REPORT.md:30-36) gives one JSON line with its figures."""

from __future__ import annotations

import json
import sys

import pytest

import bench


def run_main(monkeypatch, capsys, *argv):
    monkeypatch.setattr(sys, "argv", ["bench.py", *argv])
    code = bench.main()
    return code, capsys.readouterr().out.strip().splitlines()


def test_more_than_one_gpu_is_refused(monkeypatch, capsys):
    code, lines = run_main(monkeypatch, capsys, "--gpus", "2")
    assert code == 2 and len(lines) == 1 and "one GPU" in lines[0]


def test_the_small_preset_goes_with_the_burst_phase(monkeypatch, capsys):
    code, lines = run_main(monkeypatch, capsys, "--preset", "small")
    assert code == 2 and len(lines) == 1


@pytest.mark.gpu
def test_burst_phase_reports_the_serving_figures(monkeypatch, capsys):
    code, lines = run_main(monkeypatch, capsys, "--phase", "burst", "--preset", "small")
    assert code == 0
    rec = json.loads(lines[-1])
    assert rec["phase"] == "burst" and rec["requests"] == 48
    assert rec["generated_tokens"] > 48 * 8 and rec["output_tok_s"] > 0
    assert rec["ttft_p50_ms"] > 0 and rec["ttft_p99_ms"] >= rec["ttft_p50_ms"] and rec["tpot_p50_ms"] > 0
    assert rec["forward_passes"] >= 128            # the longest request alone decodes up to 128 tokens
