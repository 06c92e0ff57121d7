#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, Llama-3.2-1B shape, random bf16 weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  ``value`` is decoded tokens per second of the default run: a batch of 8
requests whose contexts end at 8,192 tokens, driven by the serving loop; a "step" is one decode
step (scheduling, model forward over the paged cache, greedy sampling, token ids back on the host).  The same line carries the
2,048-token prefill, the decode roofline (bytes the step has to read / time / HBM peak) and the
batch-1 and batch-64 points.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_PEAK_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

# the benchmark configuration: Llama 3.2 1B shape
CONFIG_1B = dict(
    architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=128256, hidden_size=2048,
    intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8,
    head_dim=64, rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=8192,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=True, hidden_act="silu", torch_dtype="bfloat16",
)
CONTEXT = 8192
PAGE = 16
PREFILL_TOKENS = 2048


def weight_bytes(cfg, elem=2):
    H, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    q, kv = cfg["num_attention_heads"] * cfg["head_dim"], cfg["num_key_value_heads"] * cfg["head_dim"]
    per_layer = (q + 2 * kv) * H + H * q + 3 * I * H + 2 * H
    head = V * H if cfg["tie_word_embeddings"] else V * H      # the output matrix is read once either way
    return (L * per_layer + H + head) * elem


def kv_bytes_per_token(cfg, elem=2):
    return 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * cfg["num_hidden_layers"] * elem


def prefill_flops(cfg, T):
    H, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    q, kv = cfg["num_attention_heads"] * cfg["head_dim"], cfg["num_key_value_heads"] * cfg["head_dim"]
    linear = 2 * T * L * ((q + 2 * kv) * H + H * q + 3 * I * H)
    attn = L * 4 * cfg["num_attention_heads"] * cfg["head_dim"] * T * (T + 1) / 2
    return linear + attn + 2 * V * H


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=CONTEXT)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the 16 of the configuration")
    ap.add_argument("--no-gemm-tuning", action="store_true",
                    help="leave the vendor GEMM library its own choice of algorithm (no timing at start-up)")
    ap.add_argument("--skip-points", action="store_true", help="only the default decode run and the prefill")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (this engine runs on a single MI355X)")
        return 2

    import torch
    from kv_cache_optimization_for_llm_amd.engine.batch import StepEntry
    from kv_cache_optimization_for_llm_amd.engine.engine import Engine, EngineOptions
    from kv_cache_optimization_for_llm_amd.engine.runner import Runner, ServeOptions

    cfg = dict(CONFIG_1B)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    max_batch = 64 if not args.skip_points else args.batch
    ctx = args.context
    cfg["max_position_embeddings"] = max(cfg["max_position_embeddings"], ctx)      # a longer --context
    # room for max_batch requests at the context, one more page each for the tokens decoded
    pool = max_batch * (ctx + 2 * PAGE)
    # the vendor library's algorithms are timed once, at start-up, for the row counts whose
    # products go to it here: the prefill's 2,048 tokens and decode batches above 16
    tune_rows = [] if args.no_gemm_tuning else [PREFILL_TOKENS] + [b for b in {args.batch, max_batch} if b > 16]
    engine = Engine(None, EngineOptions(dtype="bfloat16", page_size=PAGE, cache_tokens=pool,
                                        max_seqs=max_batch, max_seq_len=cfg["max_position_embeddings"],
                                        max_batch_tokens=32768, gemm_tune_rows=tune_rows),
                    config_dict=cfg, random_seed=0)
    dev = engine.device
    gen = torch.Generator().manual_seed(0)

    def decode_run(batch, steps, warmup, context):
        """Times ``steps`` decode steps of ``batch`` requests through the serving loop (scheduler,
        step function, sampler; a step is launched while the host still waits for the previous
        step's tokens).  The prompts are prefilled first, in portions; their lengths are set so
        that the longest context ENDS at ``context``.  Returns (seconds, mean context length
        over the timed steps)."""
        budget = 32768
        runner = Runner(engine, ServeOptions(ignore_eos=True, run_ahead=True, max_batch_tokens=budget))
        lead = warmup + steps + 2
        first = context - lead
        first -= (batch * first + budget - 1) // budget + 1      # steps that other requests' prompts take
        if first < 1:
            raise SystemExit(f"context {context} is too short for {steps} + {warmup} steps")
        for _ in range(batch):
            prompt = [int(t) for t in torch.randint(0, engine.vocab_size, (first,), generator=gen)]
            runner.submit(prompt, context - first - 1)
        sched = runner.scheduler
        while sched.waiting or any(s.prefilling for s in sched.running):
            runner.step()
        for _ in range(warmup):
            runner.step()
        torch.cuda.synchronize()
        if len(sched.running) != batch or any(s.prefilling for s in sched.running):
            raise SystemExit(f"bench: {len(sched.running)} of {batch} requests are decoding after the prompts "
                             f"(waiting {len(sched.waiting)}, preemptions {sched.preemptions}): the pool or the "
                             f"token budget does not fit context {context}")
        ctx0 = sum(s.computed for s in sched.running) / batch
        t0 = time.perf_counter()
        for _ in range(steps):
            runner.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(sched.running) == batch and max(s.computed for s in sched.running) <= context
        mean_ctx = ctx0 + steps / 2
        # drop the requests (their remaining budget is not part of the measurement)
        runner._resolve_in_flight()
        for s_ in list(sched.running) + list(sched.closing):
            sched._finish(s_, "length", [])
        return dt, mean_ctx

    dt, mean_ctx = decode_run(args.batch, args.steps, args.warmup, ctx)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = weight_bytes(cfg) + args.batch * mean_ctx * kv_bytes_per_token(cfg)
    achieved = step_bytes / (ms_per_step * 1e-3) / 1e9

    # prefill of 2,048 tokens: one request, one step, logits at the last place
    prompt = [int(t) for t in torch.randint(0, engine.vocab_size, (PREFILL_TOKENS,), generator=gen)]
    pre_ms = []
    for i in range(6):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry(f"p{i}", prompt, [PREFILL_TOKENS - 1])])
        torch.cuda.synchronize()
        pre_ms.append((time.perf_counter() - t0) * 1e3)
        engine.release(f"p{i}")
    p_ms = min(pre_ms[1:])
    flops = prefill_flops(cfg, PREFILL_TOKENS)
    prefill = {"value": round(PREFILL_TOKENS / (p_ms * 1e-3), 1), "tokens": PREFILL_TOKENS,
               "ms": round(p_ms, 3), "frac": round(flops / (p_ms * 1e-3) / (PEAK_TFLOPS["bf16"] * 1e12), 4)}

    points = {}
    if not args.skip_points:
        for b in (1, 64):
            k = max(16, args.steps // 2)
            d, _ = decode_run(b, k, 8, ctx)
            points[f"decode_b{b}"] = round(b * k / d, 1)
        # the serving workload of the comparison: 512-token prompts, 256 generated tokens
        for b in (1, 8, 64):
            d, _ = decode_run(b, 240, 8, 512 + 256)
            points[f"decode_b{b}_p512_g256"] = round(b * 240 / d, 1)

    out = {
        "metric": f"decode tok/s at batch {args.batch} (context {ctx}), Llama-3.2-1B shape", "value": round(value, 1),
        "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic: random weights N(0,0.02), seeded uniform token ids (prompts are prefilled, then decoded)",
        "config": {"model": "llama-3.2-1b-shape", "global_batch": args.batch, "seq_len": ctx,
                   "parallelism": "single-gpu", "layers": cfg["num_hidden_layers"], "layers_full": full_layers,
                   "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
                   "page_size": PAGE, "prefill_tokens": PREFILL_TOKENS, "tied_embeddings": True,
                   "rope": "llama3 factor 32", "sampling": "greedy on device"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": points,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
