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
