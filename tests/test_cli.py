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
    for bad, word in (("x 1 1 5", "integer id"), ("7 0 1 5", "max_tokens"), ("7", "max_tokens"),
                      ("7 16 9 5", "n_seqs"), ("7 16 0 5", "n_seqs"), ("7 16 1", "no prompt token")):
        assert parse_request_line(bad) is None
        assert word in capsys.readouterr().err


def test_a_server_times_the_vendor_products_for_its_decode_batches_and_its_portion_size():
    from kv_cache_optimization_for_llm_amd.cli.serve import serve_tune_rows
    assert serve_tune_rows(64, None, 3072) == [32, 64, 3072]
    assert serve_tune_rows(64, 512, 3072) == [32, 64, 512]
    assert serve_tune_rows(64, 4096, 3072) == [32, 64, 3072]      # a portion never exceeds a step
    assert serve_tune_rows(8, 8, 8) == []                          # the few-rows kernels take all of it


def test_checksum_is_order_sensitive():
    assert checksum([1, 2, 3]) != checksum([3, 2, 1])
    assert checksum([]) == 0 and checksum([5]) == 5
    assert checksum([1, 2]) == (1 * 1000003 + 2) & 0xFFFFFFFF


def test_a_sweep_knows_which_of_its_runs_a_results_file_already_holds(tmp_path):
    """Resuming (reference sweep.py:270-288): a run is identified by its parameters; a finished
    run's line in the --out file stands for it, a cut-off line or another run's line does not."""
    from kv_cache_optimization_for_llm_amd.cli import sweep
    out = tmp_path / "runs.jsonl"
    args = sweep.build_parser().parse_args(["--out", str(out), "--prompt-len", "64", "--new-tokens", "8"])
    key = sweep.run_key(args, "1b", 8, "paged")
    assert sweep.finished_runs(str(out)) == []                      # no file yet
    out.write_text(json.dumps({**key, "requests_done": 8, "decode_tok_s": 1.0}) + "\n"
                   + json.dumps({**sweep.run_key(args, "1b", 64, "paged"), "requests_done": 64})[:40] + "\n")
    done = sweep.finished_runs(str(out))
    assert key in done and len(done) == 1                           # the cut-off line does not count
    assert sweep.run_key(args, "1b", 64, "paged") not in done
    assert sweep.run_key(args, "1b", 8, "contiguous") not in done   # the same batch in the other mode is another run
    other = sweep.build_parser().parse_args(["--out", str(out), "--prompt-len", "128", "--new-tokens", "8"])
    assert sweep.run_key(other, "1b", 8, "paged") not in done       # and so is another prompt length


@pytest.mark.gpu
def test_served_tokens_are_the_same_in_both_cache_modes(sharp_model_dirs, tmp_path, gpu):
    """The reference's cross-build gate (bench.py:226-237): the paged and the contiguous engine
    emit the same ids, and every sequence emits exactly its budget."""
    results = {}
    for mode, extra in (("paged", []), ("contiguous", [])):
        out = tmp_path / f"{mode}.json"
        env = dict(os.environ, IGNORE_EOS="1", ORCA_POLICY="oracle", REPETITION_PENALTY="1.15",
                   PYTHONPATH=ROOT)
        cmd = [sys.executable, "-m", "kv_cache_optimization_for_llm_amd.cli.client", sharp_model_dirs["C"], "5",
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
def test_sweep_reports_both_cache_modes_on_a_small_shape(sharp_model_dirs, tmp_path, gpu, capsys):
    """The sweep command on a tiny configuration: every request finishes with its budget, the
    contiguous cache reserves more than it holds (whole reservations), the paged cache about what
    it holds, and with a small pool pages are used again."""
    from kv_cache_optimization_for_llm_amd.cli import sweep
    cfg = os.path.join(sharp_model_dirs["A"], "config.json")
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
    # started again with the same file, nothing is run again: every run's line is there already
    assert sweep.main(["--shapes", cfg, "--batches", "3,6", "--cache-modes", "paged,contiguous", "--prompt-len", "40",
                       "--prompt-min", "5", "--workload", "mixed", "--new-tokens", "12", "--max-seqs", "3",
                       "--reserve-policy", "pow2", "--out", str(out)]) == 0
    assert len(out.read_text().splitlines()) == 4


@pytest.mark.gpu
def test_plain_serve_command_starts_on_a_config_with_131072_positions(tmp_path, gpu):
    """``serve MODEL_DIR`` with nothing else given: 64 seats and a config.json that allows 131,072
    positions.  Every seat at its longest is far more cache than a served model leaves room
    for; the pool is made from what is free instead (the reference sizes its pool last, from
    leftover memory, paged_attention/src/engine.cu:186-215) and says how large it is."""
    from conftest import MID_E
    from kv_cache_optimization_for_llm_amd.weights.random_init import write_random_model
    cfg = dict(MID_E, max_position_embeddings=131072, num_hidden_layers=4)
    model_dir = write_random_model(str(tmp_path / "m"), cfg, 3, gain=1.0)
    env = dict(os.environ, IGNORE_EOS="1", PYTHONPATH=ROOT)
    proc = subprocess.run([sys.executable, "-m", "kv_cache_optimization_for_llm_amd.cli.serve", model_dir,
                           "--gemm-tune-rows", ""],
                          input="1 6 1 5 6 7 8 9\n2 4 2 11 12 13\n", env=env, cwd=ROOT, capture_output=True,
                          text=True, timeout=280)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    lines = [json.loads(l) for l in proc.stdout.splitlines()]
    conf = lines[0]
    assert conf["type"] == "engine_config" and conf["batch_size"] == 64 and conf["max_seq_len"] == 131072
    page_bytes = 4 * 2 * 2 * 64 * 16 * 2                       # layers x (K, V) x kv heads x head size x tokens x bf16
    assert 0 < conf["kv_pool_tokens"] <= 64 * 131072
    assert conf["kv_pool_tokens"] // 16 * page_bytes < 280 * 2 ** 30
    done = {(l["id"], l["seq"]): l for l in lines if l.get("done")}
    assert {k: v["tokens"] for k, v in done.items()} == {(1, 0): 6, (2, 0): 4, (2, 1): 4}
    assert not any("error" in v for v in done.values())
