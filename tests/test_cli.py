"""The serving process and its client: the wire format on the CPU, a whole run on the GPU."""
import json
import os
import subprocess
import sys

import pytest

from kv_cache_optimization_for_llm_amd.cli.client import checksum
from kv_cache_optimization_for_llm_amd.cli.serve import parse_request_line

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_request_lines(capsys):
    assert parse_request_line("7 16 1 5 6 7\n") == (7, 16, 1, [5, 6, 7])
    assert parse_request_line("7 16 8 5") == (7, 16, 8, [5])
    assert parse_request_line("") is None
    for bad, word in (("x 1 1 5", "no request id"), ("7 0 1 5", "output budget"), ("7", "output budget"),
                      ("7 16 9 5", "n_seqs"), ("7 16 0 5", "n_seqs"), ("7 16 1", "no tokens")):
        assert parse_request_line(bad) is None
        assert word in capsys.readouterr().err


def test_checksum_is_order_sensitive():
    assert checksum([1, 2, 3]) != checksum([3, 2, 1])
    assert checksum([]) == 0 and checksum([5]) == 5
    assert checksum([1, 2]) == (1 * 1000003 + 2) & 0xFFFFFFFF


@pytest.mark.gpu
def test_served_tokens_are_the_same_in_both_cache_modes(model_dirs, tmp_path, gpu):
    """The reference's cross-build gate (bench.py:226-237): the paged and the contiguous engine
    emit the same ids, and every sequence emits exactly its budget."""
    results = {}
    for mode, extra in (("paged", []), ("contiguous", [])):
        out = tmp_path / f"{mode}.json"
        env = dict(os.environ, IGNORE_EOS="1", ORCA_POLICY="oracle", REPETITION_PENALTY="1.15",
                   PYTHONPATH=ROOT)
        cmd = [sys.executable, "-m", "kv_cache_optimization_for_llm_amd.cli.client", model_dirs["C"], "5",
               "--prompt-len", "21", "--max-new-tokens", "12", "--num-seqs", "2", "--out", str(out), "--",
               "--dtype", "float32", "--cache-mode", mode, "--max-seqs", "6", "--max-seq-len", "64",
               "--cache-tokens", "512", "--chunk-size", "8", "--max-batch-tokens", "24"]
        proc = subprocess.run(cmd, env=env, cwd=ROOT, capture_output=True, text=True, timeout=280)
        assert proc.returncode == 0, proc.stdout + proc.stderr
        results[mode] = json.load(open(out))
    for r in results.values():
        assert r["status"] == "ok" and r["sequences_done"] == 10 and r["tokens"] == 120
        assert r["count_mismatches"] == 0 and r["budget_mismatches"] == 0 and r["errors"] == []
    assert results["paged"]["checksums"] == results["contiguous"]["checksums"]
    assert results["paged"]["engine_config"]["mechanism"] == "paged"
    assert results["contiguous"]["engine_config"]["reserve_policy"] == "oracle"


@pytest.mark.gpu
def test_sweep_reports_both_cache_modes_on_a_small_shape(model_dirs, tmp_path, gpu, capsys):
    """The sweep command on a tiny configuration: every request finishes with its budget, the
    contiguous cache reserves more than it holds (whole reservations), the paged cache about what
    it holds, and with a small pool pages are used again."""
    from kv_cache_optimization_for_llm_amd.cli import sweep
    cfg = os.path.join(model_dirs["A"], "config.json")
    out = tmp_path / "sweep.jsonl"
    assert sweep.main(["--shapes", cfg, "--batches", "3,6", "--cache-modes", "paged,contiguous", "--prompt-len", "40",
                       "--prompt-min", "5", "--workload", "mixed", "--new-tokens", "12", "--max-seqs", "3",
                       "--reserve-policy", "pow2", "--out", str(out)]) == 0
    lines = [json.loads(l) for l in out.read_text().splitlines()]
    assert [(l["cache_mode"], l["batch"]) for l in lines] == [("paged", 3), ("paged", 6), ("contiguous", 3), ("contiguous", 6)]
    for l in lines:
        assert l["requests_done"] == l["batch"] and l["tokens_emitted"] == 12 * l["batch"]
        assert l["finish_reasons"] == {"length": l["batch"]} and l["decode_tok_s"] > 0
        assert l["peak_kv_tokens_reserved"] >= l["peak_kv_tokens_live"] > 0
    paged, contiguous = lines[1], lines[3]
    assert paged["reserved_over_live"] < contiguous["reserved_over_live"]
    assert paged["pages_reused"] > 0                  # six requests through three seats
