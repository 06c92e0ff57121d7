"""Sweeps of the serving loop: batch size x cache mode x model shape, one JSON line per run.

    python -m kv_cache_optimization_for_llm_amd.cli.sweep --shapes 1b --batches 1,8,64 \\
        --cache-modes paged,contiguous --prompt-len 512 --new-tokens 256

The reference drives its two servers through staged experiments (``sweep.py:693-712``,
``bench.py:43-78``) to compare the paged cache with the contiguous, reserved one.  Here one
engine has both cache modes, so a run is: build the model shape with random weights on the
device, submit ``batch`` requests of seeded uniform token ids, run the serving loop to the end
and report what the reference's reports are made of - tokens per second and step latency for the
decoding phase, prompt throughput, cache occupancy (reserved against live tokens, the paper's
comparison, ``paged_attention/src/engine.cu:755-768``, ``base/src/engine.cu:513-525``), pages
reused, preemptions, fragmentation failures - plus the fraction of the HBM roofline a decode step
reached.

Workloads: ``uniform`` (every prompt ``--prompt-len`` long) and ``mixed`` (prompt lengths uniform
in ``[--prompt-min, --prompt-len]``, the shape of the reference's trace-driven runs without their
datasets).  ``--layers`` runs fewer layers than the shape has (the line then names both numbers).
With ``--out FILE`` the sweep can be resumed: a run whose line the file already holds is skipped
unless ``--force`` is given (the reference's driver skips finished runs the same way,
``sweep.py:270-288``).
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from typing import Dict, List

HBM_PEAK_GBS = 8000.0
WARM_STEPS = 3


def _llama(hidden, layers, heads, kv_heads, head_dim, inter, tied, factor, max_pos=131072):
    return dict(
        architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=hidden,
        intermediate_size=inter, num_hidden_layers=layers, num_attention_heads=heads,
        num_key_value_heads=kv_heads, head_dim=head_dim, rms_norm_eps=1e-5, rope_theta=500000.0,
        max_position_embeddings=max_pos,
        rope_scaling=dict(rope_type="llama3", factor=factor, low_freq_factor=1.0, high_freq_factor=4.0,
                          original_max_position_embeddings=8192),
        tie_word_embeddings=tied, hidden_act="silu", torch_dtype="bfloat16")


SHAPES: Dict[str, dict] = {
    "1b": _llama(2048, 16, 32, 8, 64, 8192, True, 32.0),
    "3b": _llama(3072, 28, 24, 8, 128, 8192, True, 32.0),
    "8b": _llama(4096, 32, 32, 8, 128, 14336, False, 8.0),
}


def weight_bytes(cfg, elem=2) -> int:
    H, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    q, kv = cfg["num_attention_heads"] * cfg["head_dim"], cfg["num_key_value_heads"] * cfg["head_dim"]
    return (L * ((q + 2 * kv) * H + H * q + 3 * I * H + 2 * H) + H + V * H) * elem


def kv_bytes_per_token(cfg, elem=2) -> int:
    return 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * cfg["num_hidden_layers"] * elem


def run_one(args, shape: str, batch: int, mode: str) -> dict:
    import torch
    from ..engine.engine import Engine, EngineOptions
    from ..engine.runner import Runner, ServeOptions
    from ..ops.gemm_bf16 import decode_tune_rows

    cfg = dict(SHAPES[shape]) if shape in SHAPES else json.load(open(shape))
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = min(args.layers, full_layers)
    longest = args.prompt_len + args.new_tokens + 1
    if shape in SHAPES:
        cfg["max_position_embeddings"] = max(2048, 1 << (longest - 1).bit_length())
    elif longest > cfg["max_position_embeddings"]:
        raise SystemExit(f"{shape}: prompts of {args.prompt_len} plus {args.new_tokens} new tokens do not fit "
                         f"max_position_embeddings {cfg['max_position_embeddings']}")
    seats = min(batch, args.max_seqs) if args.max_seqs else batch
    pool = args.cache_tokens or seats * (longest + 2 * args.page_size) * (2 if mode == "contiguous" else 1)
    engine = Engine(None, EngineOptions(dtype="bfloat16", cache_mode=mode, page_size=args.page_size,
                                        cache_tokens=pool, max_seqs=seats, max_seq_len=longest,
                                        use_graphs=not args.no_graphs,
                                        max_batch_tokens=max(8192, args.max_batch_tokens), max_logit_rows=seats,
                                        gemm_tune_rows=decode_tune_rows(seats) if args.tune_gemm else []),
                    config_dict=cfg, random_seed=args.seed)
    runner = Runner(engine, ServeOptions(ignore_eos=True, max_batch_tokens=args.max_batch_tokens,
                                         chunk_size=args.chunk_size, reserve_policy=args.reserve_policy,
                                         run_ahead=not args.no_run_ahead))
    gen = torch.Generator().manual_seed(args.seed)
    # one short request first, untimed: kernels are loaded and library workspaces made
    runner.submit([int(t) for t in torch.randint(0, engine.vocab_size, (8,), generator=gen)], 3)
    while not runner.idle():
        runner.step()
    lens: List[int] = []
    for _ in range(batch):
        n = args.prompt_len if args.workload == "uniform" else \
            int(torch.randint(args.prompt_min, args.prompt_len + 1, (1,), generator=gen))
        lens.append(n)
        runner.submit([int(t) for t in torch.randint(0, engine.vocab_size, (n,), generator=gen)], args.new_tokens)

    sched = runner.scheduler
    emitted = done = 0
    peak_reserved = peak_live = 0
    decode_steps = decode_tokens = seen_decode_steps = 0
    decode_time = 0.0
    decode_bytes = 0.0
    wbytes, kvbytes = weight_bytes(cfg), kv_bytes_per_token(cfg)
    reasons: Dict[str, int] = {}
    torch.cuda.synchronize()
    t_start = time.perf_counter()
    t_first_decode = None
    last = t_start
    while not runner.idle():
        prefilling = bool(sched.waiting) or any(s.prefilling for s in sched.running)
        # what this step has to read if it is a decode step: every weight once and the keys and
        # values of the requests that are still decoding (early finishers have left)
        step_bytes = wbytes + kvbytes * sum(s.computed + 1 for s in sched.running)
        events = runner.step()
        now = time.perf_counter()
        tokens = sum(1 for e in events if e.kind == "token")
        emitted += tokens
        for e in events:
            if e.kind in ("done", "rejected"):
                done += 1
                reasons[e.reason] = reasons.get(e.reason, 0) + 1
        if not prefilling:
            # a step of decoding only: with the loop running ahead of the device the time between
            # two such calls is one step of the device
            if t_first_decode is None:
                t_first_decode = now
            seen_decode_steps += 1
            if seen_decode_steps > WARM_STEPS:      # the first steps of a batch shape run eagerly, then capture a graph
                decode_steps += 1
                decode_tokens += tokens
                decode_time += now - last
                decode_bytes += step_bytes
        st = engine.cache.stats()
        peak_reserved = max(peak_reserved, st["kv_tokens_reserved"])
        peak_live = max(peak_live, st["kv_tokens_live"])
        last = now
    torch.cuda.synchronize()
    wall = time.perf_counter() - t_start
    st = engine.cache.stats()
    engine.cache.check()
    out = {
        "shape": shape, "layers": cfg["num_hidden_layers"], "layers_full": full_layers, "batch": batch,
        "cache_mode": mode, "reserve_policy": args.reserve_policy if mode == "contiguous" else None,
        "workload": args.workload, "prompt_tokens": sum(lens), "new_tokens_each": args.new_tokens,
        "seats": seats, "cache_tokens": st["kv_tokens_total"],
        "tokens_emitted": emitted, "requests_done": done, "finish_reasons": reasons,
        "wall_s": round(wall, 3),
        "prefill_s": round((t_first_decode or time.perf_counter()) - t_start, 3),
        "prefill_tok_s": round(sum(lens) / max(1e-9, (t_first_decode or time.perf_counter()) - t_start), 1),
        "decode_steps": decode_steps,
        "decode_ms_per_step": round(decode_time / decode_steps * 1e3, 4) if decode_steps else None,
        "decode_tok_s": round(decode_tokens / decode_time, 1) if decode_time > 0 else None,
        "peak_kv_tokens_reserved": peak_reserved, "peak_kv_tokens_live": peak_live,
        "reserved_over_live": round(peak_reserved / peak_live, 3) if peak_live else None,
        "pages_reused": st["pages_reused"], "preemptions": sched.preemptions,
        "fragmentation_failures": st["fragmentation_failures"],
    }
    if decode_steps:
        gbs = decode_bytes / decode_time / 1e9          # bytes of the steps that were timed, rows as they were
        out["decode_hbm_gbs"] = round(gbs, 1)
        out["decode_hbm_frac"] = round(gbs / HBM_PEAK_GBS, 4)
    return out


RUN_KEY = ("shape", "layers_asked", "batch", "cache_mode", "reserve_policy", "workload", "prompt_len",
           "prompt_min", "new_tokens_each", "page_size", "max_seqs", "cache_tokens_asked", "max_batch_tokens",
           "chunk_size", "seed")


def run_key(args, shape: str, batch: int, mode: str) -> dict:
    """What identifies a run: a line with the same key in the output file is that run's result."""
    return {"shape": shape, "layers_asked": args.layers, "batch": batch, "cache_mode": mode,
            "reserve_policy": args.reserve_policy if mode == "contiguous" else None, "workload": args.workload,
            "prompt_len": args.prompt_len, "prompt_min": args.prompt_min if args.workload == "mixed" else None,
            "new_tokens_each": args.new_tokens, "page_size": args.page_size, "max_seqs": args.max_seqs,
            "cache_tokens_asked": args.cache_tokens, "max_batch_tokens": args.max_batch_tokens,
            "chunk_size": args.chunk_size, "seed": args.seed}


def finished_runs(path: str) -> list:
    """Keys of the runs whose lines a file of earlier results holds (a cut-off last line is ignored)."""
    import os
    done = []
    if path and os.path.isfile(path):
        with open(path) as f:
            for line in f:
                try:
                    rec = json.loads(line)
                except json.JSONDecodeError:
                    continue
                if isinstance(rec, dict) and rec.get("requests_done") is not None:
                    done.append({k: rec.get(k) for k in RUN_KEY})
    return done


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--shapes", default="1b",
                    help="comma list of " + ", ".join(SHAPES) + ", or paths of config.json files")
    ap.add_argument("--batches", default="1,8,64")
    ap.add_argument("--cache-modes", default="paged", help="comma list of paged, contiguous")
    ap.add_argument("--reserve-policy", default="max", choices=["max", "pow2", "oracle"],
                    help="contiguous mode: what a request reserves at admission (ORCA_POLICY)")
    ap.add_argument("--workload", default="uniform", choices=["uniform", "mixed"])
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--prompt-min", type=int, default=128, help="mixed workload: shortest prompt")
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the shape has")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-seqs", type=int, default=None, help="seats (default: the batch size)")
    ap.add_argument("--cache-tokens", type=int, default=None, help="pool size in tokens (default: room for all)")
    ap.add_argument("--max-batch-tokens", type=int, default=3072)
    ap.add_argument("--chunk-size", type=int, default=None)
    ap.add_argument("--tune-gemm", action="store_true",
                    help="time the vendor GEMM library's algorithms at start-up for decode batches above 16")
    ap.add_argument("--no-graphs", action="store_true", help="launch every step's kernels one by one")
    ap.add_argument("--no-run-ahead", action="store_true")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--out", default=None, help="also append the lines to this file; a run whose line is "
                                                 "there already is skipped (the sweep can be resumed)")
    ap.add_argument("--force", action="store_true", help="run again what the --out file already holds")
    return ap


def main(argv=None) -> int:
    ap = build_parser()
    args = ap.parse_args(argv)
    import os
    done = [] if args.force else finished_runs(args.out)
    for shape in args.shapes.split(","):
        if shape not in SHAPES and not os.path.isfile(shape):
            ap.error(f"shape {shape!r} is neither one of {', '.join(SHAPES)} nor a config.json file")
    for shape in args.shapes.split(","):
        for mode in args.cache_modes.split(","):
            for batch in (int(b) for b in args.batches.split(",")):
                key = run_key(args, shape, batch, mode)
                if key in done:
                    print(f"[sweep] {shape} batch {batch} {mode}: already in {args.out}, skipped (--force runs it again)",
                          file=sys.stderr, flush=True)
                    continue
                line = json.dumps({**run_one(args, shape, batch, mode), **key})
                print(line, flush=True)
                if args.out:
                    with open(args.out, "a") as f:
                        f.write(line + "\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
