"""The engine as a process, in the reference's manner: requests come in on standard input, one
per line, and per-token progress and statistics go out on standard output as JSON lines.

    python -m kv_cache_optimization_for_llm_amd.cli.serve [MODEL_DIR] [options]

Names and meanings follow the reference (``base/src/main.cu:42-105``,
``paged_attention/src/main.cu:67-92``, ``base/src/request_queue.cpp:11-61``):

* the model folder is ``argv[1]``, else ``$MODEL_DIR``;
* ``IGNORE_EOS=1`` runs every request to its full budget; ``TEMPERATURE`` (unset or <= 0 is
  greedy) and ``SAMPLING_SEED`` choose the sampler; ``ORCA_POLICY=max|pow2|oracle`` is the
  contiguous mode's reservation policy; ``PREEMPTION_POLICY=recompute`` (``swap`` is refused:
  this engine recomputes); ``REPETITION_PENALTY`` (the reference fixes 1.15);
* a request line is ``<request_id> <max_tokens> <n_seqs> <token> <token> ...``; a malformed
  line is reported on standard error and ignored;
* output lines: ``{"type":"engine_config",...}`` once, ``{"id","slot","seq","tok"}`` per
  token, ``{"type":"prefill_stats",...}`` when a prompt is in the cache, ``{"id","slot","seq",
  "done":true,"tokens","decode_time","decode_speed"[,"error"]}`` per finished sequence,
  ``{"type":"preempted",...}``, and ``{"type":"step",...}`` every 8 decode steps with the
  occupancy counters (reserved against live tokens).

What the reference fixes at build time is an option here (``--page-size``, ``--max-seqs``,
``--max-batch-tokens``, ...), and ``--cache-mode paged|contiguous`` chooses between what the
reference ships as two programs.  The process ends when standard input is closed and all
requests are done.
"""
from __future__ import annotations

import argparse
import json
import os
import queue
import sys
import threading
import time
from typing import Dict, Optional, Tuple

from ..engine.runner import MAX_PARALLEL_SEQUENCES       # reference: base/src/config.h:97
STEP_TELEMETRY_EVERY = 8          # reference: base/src/config.h:170


def parse_request_line(line: str) -> Optional[Tuple[int, int, int, list]]:
    """(id, max_tokens, n_seqs, tokens) or None with a message on standard error."""
    fields = line.split()
    if not fields:
        return None
    try:
        rid = int(fields[0])
    except ValueError:
        print(f"request line dropped, it does not start with an integer id: {line.strip()!r}", file=sys.stderr)
        return None
    try:
        max_tokens = int(fields[1])
        if max_tokens < 1:
            raise ValueError
    except (IndexError, ValueError):
        print(f"request {rid} dropped: max_tokens is missing or below 1", file=sys.stderr)
        return None
    try:
        n_seqs = int(fields[2])
        if not 1 <= n_seqs <= MAX_PARALLEL_SEQUENCES:
            raise ValueError
    except (IndexError, ValueError):
        print(f"request {rid} dropped: n_seqs is missing or not in 1..{MAX_PARALLEL_SEQUENCES}", file=sys.stderr)
        return None
    tokens = []
    for f in fields[3:]:
        try:
            tokens.append(int(f))
        except ValueError:
            break
    if not tokens:
        print(f"request {rid} dropped: no prompt token ids follow its three header fields", file=sys.stderr)
        return None
    return rid, max_tokens, n_seqs, tokens


def serve_tune_rows(max_seqs: int, chunk_size: Optional[int], max_batch_tokens: int) -> list:
    """Row counts a server has the vendor library's algorithms timed for: its decode batches and
    the size of the prompt portions its steps are mostly made of."""
    from ..ops.gemm_bf16 import decode_tune_rows
    rows = decode_tune_rows(max_seqs)
    portion = min(int(chunk_size or max_batch_tokens), int(max_batch_tokens))
    if portion > max_seqs and portion not in rows:
        rows.append(portion)
    return rows


def _reader(inbox: "queue.Queue") -> None:
    for line in sys.stdin:
        req = parse_request_line(line)
        if req is not None:
            inbox.put(req)
    inbox.put(None)


def emit(obj: dict) -> None:
    sys.stdout.write(json.dumps(obj) + "\n")
    sys.stdout.flush()


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="serve", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model_dir", nargs="?", default=os.environ.get("MODEL_DIR"))
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--cache-mode", choices=["paged", "contiguous"], default="paged")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-seqs", type=int, default=64)
    ap.add_argument("--max-seq-len", type=int, default=None)
    ap.add_argument("--cache-tokens", type=int, default=None)
    ap.add_argument("--max-batch-tokens", type=int, default=3072)
    ap.add_argument("--chunk-size", type=int, default=None)
    ap.add_argument("--gemm-tune-rows", default="auto",
                    help="comma list of row counts (tokens per step) for which the vendor GEMM library's "
                         "algorithms are timed at start-up (a few seconds); smaller row counts down to half "
                         "share what is found.  'auto': the powers of two from 32 up to the number of seats, "
                         "that number, and the size of a prompt portion (--chunk-size, else "
                         "--max-batch-tokens); '' for none")
    args = ap.parse_args(argv)
    if not args.model_dir:
        print("no model folder: pass it as the first argument or set MODEL_DIR", file=sys.stderr)
        return 1
    print(f"Model directory: {args.model_dir}", file=sys.stderr)

    env = os.environ
    ignore_eos = env.get("IGNORE_EOS", "")[:1] == "1"
    temperature = max(0.0, float(env.get("TEMPERATURE", "0") or 0))
    seed = int(env.get("SAMPLING_SEED", "0") or 0) & 0xFFFFFFFF
    policy = env.get("ORCA_POLICY", "max")
    if policy not in ("max", "pow2", "oracle"):
        print(f"Unknown ORCA_POLICY '{policy}', expected max|pow2|oracle", file=sys.stderr)
        return 1
    preemption = env.get("PREEMPTION_POLICY", "recompute")
    if preemption != "recompute":
        print(f"PREEMPTION_POLICY '{preemption}' is not supported: this engine preempts by recomputation",
              file=sys.stderr)
        return 1
    penalty = float(env.get("REPETITION_PENALTY", "1.15") or 1.15)
    if temperature > 0:
        print(f"Sampling: temperature {temperature}, seed {seed} (greedy decoding is OFF)", file=sys.stderr)

    from ..engine.engine import Engine, EngineOptions
    from ..engine.runner import Runner, ServeOptions
    engine = Engine(args.model_dir, EngineOptions(
        dtype=args.dtype, cache_mode=args.cache_mode, page_size=args.page_size, max_seqs=args.max_seqs,
        max_seq_len=args.max_seq_len, cache_tokens=args.cache_tokens, max_batch_tokens=args.max_batch_tokens,
        max_logit_rows=args.max_seqs,         # one sampled token per request and step
        gemm_tune_rows=serve_tune_rows(args.max_seqs, args.chunk_size, args.max_batch_tokens)
        if args.gemm_tune_rows == "auto" else [int(r) for r in args.gemm_tune_rows.split(",") if r.strip()]))
    runner = Runner(engine, ServeOptions(
        temperature=temperature, sampling_seed=seed, ignore_eos=ignore_eos, repetition_penalty=penalty,
        max_batch_tokens=args.max_batch_tokens, chunk_size=args.chunk_size, reserve_policy=policy))
    emit({"type": "engine_config", "mechanism": args.cache_mode, "batch_size": args.max_seqs,
          "max_batch_tokens": args.max_batch_tokens, "max_seq_len": engine.max_seq_len,
          "page_size": args.page_size, "temperature": temperature, "sampling_seed": seed,
          "reserve_policy": policy, "preemption_policy": preemption, "repetition_penalty": penalty,
          "dtype": args.dtype, "kv_pool_tokens": engine.cache.num_pages * args.page_size,
          "architecture": engine.spec.architecture})

    inbox: "queue.Queue" = queue.Queue()
    threading.Thread(target=_reader, args=(inbox,), daemon=True).start()
    t_start = time.perf_counter()
    first_token_at: Dict[Tuple[int, int], float] = {}
    submitted_at: Dict[int, float] = {}
    prompt_len: Dict[int, int] = {}
    eof = False
    decode_steps = 0
    while True:
        # take what has arrived; block only when there is nothing to run
        while True:
            try:
                req = inbox.get(block=runner.idle() and not eof, timeout=None)
            except queue.Empty:
                break
            if req is None:
                eof = True
                break
            rid, max_tokens, n_seqs, tokens = req
            runner.submit(tokens, max_tokens, request_id=rid, n_seqs=n_seqs)
            submitted_at[rid] = time.perf_counter()
            prompt_len[rid] = len(tokens)
        if runner.idle():
            if eof:
                break
            continue
        t0 = time.perf_counter()
        events = runner.step()
        step_ms = (time.perf_counter() - t0) * 1e3
        now = time.perf_counter()
        decoded = False
        for ev in events:
            key = (ev.request_id, ev.seq_index)
            if ev.kind == "token":
                emit({"id": ev.request_id, "slot": ev.seat, "seq": ev.seq_index, "tok": ev.token})
                if key not in first_token_at:
                    first_token_at[key] = now
                    n = prompt_len.get(ev.request_id, 0)
                    waited = (now - submitted_at.get(ev.request_id, now)) * 1e3
                    emit({"type": "prefill_stats", "id": ev.request_id, "slot": ev.seat,
                          "speed": n / (waited / 1e3) if waited > 0 else 0.0, "time_ms": waited,
                          "prompt_tokens": n, "resumed_tokens": 0})
                else:
                    decoded = True
            elif ev.kind == "done":
                t_first = first_token_at.pop(key, now)
                decode_ms = (now - t_first) * 1e3
                out = {"id": ev.request_id, "slot": ev.seat, "seq": ev.seq_index, "done": True,
                       "tokens": ev.tokens, "decode_time": decode_ms,
                       "decode_speed": ev.tokens / (decode_ms / 1e3) if decode_ms > 0 else 0.0}
                if ev.reason not in ("eos", "length"):
                    out["error"] = ev.reason
                emit(out)
            elif ev.kind == "rejected":
                emit({"id": ev.request_id, "slot": -1, "seq": ev.seq_index, "done": True, "tokens": 0,
                      "decode_time": 0.0, "decode_speed": 0.0, "error": ev.reason})
            elif ev.kind == "preempted":
                emit({"type": "preempted", "id": ev.request_id, "slot": ev.seat, "seq": ev.seq_index,
                      "generated": ev.generated, "policy": "recompute"})
        if decoded:
            decode_steps += 1
            if decode_steps % STEP_TELEMETRY_EVERY == 0:
                st = engine.cache.stats()
                emit({"type": "step", "t_ms": (now - t_start) * 1e3, "running": st["running"],
                      "waiting": len(runner.scheduler.waiting), "kv_tokens_reserved": st["kv_tokens_reserved"],
                      "kv_tokens_live": st["kv_tokens_live"], "kv_tokens_total": st["kv_tokens_total"],
                      "fragmentation_failures": st["fragmentation_failures"],
                      "preemptions": runner.scheduler.preemptions, "pages_reused": st["pages_reused"],
                      "step_ms": step_ms})
    return 0


if __name__ == "__main__":
    sys.exit(main())
