#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, Llama-3.2-1B shape, random bf16 weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  ``value`` is decoded tokens per second of the default run: a batch of 8
requests whose contexts end at 8,192 tokens, driven by the serving loop; a "step" is one decode
step (scheduling, model forward over the paged cache, greedy sampling, token ids back on the host).
The same line carries the 2,048-token prefill; the decode roofline (bytes the step has to read /
time / HBM peak, and against what a plain read stream gets from this GPU); ``points``: batch 1 and
batch 64 at the same context and batches 1, 8 and 64 with 512-token prompts and 256 generated
tokens, each with its step time, bytes and fraction of the HBM peak, and the serving loop at the
3B and 8B layer sizes (mixed prompt lengths; paged against contiguous cache occupancy).
``points`` also holds the device time per class of kernel of one decode step and of the prefill
(``kclass_...``; ``--no-kernel-classes`` leaves them out) and, for the serving runs, pages reused,
preemptions and fragmentation failures.
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
    ap.add_argument("--skip-large", action="store_true",
                    help="leave out the serving runs at the 3B and 8B layer sizes (about a minute together)")
    ap.add_argument("--no-kernel-classes", dest="kernel_classes", action="store_false",
                    help="leave out the device time per class of kernel (one decode step and the prefill with events "
                         "around every launch, launched one by one instead of replayed from graphs: a second or two)")
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
    pool = max(max_batch * (ctx + 2 * PAGE), PREFILL_TOKENS + PAGE)      # and room for the prefill's prompt
    # the vendor library's algorithms are timed once, at start-up, for the row counts whose
    # products go to it here: the prefill's 2,048 tokens and decode batches above 16
    tune_rows = [] if args.no_gemm_tuning else [PREFILL_TOKENS] + [b for b in {args.batch, max_batch} if b > 16]
    engine = Engine(None, EngineOptions(dtype="bfloat16", page_size=PAGE, cache_tokens=pool,
                                        max_seqs=max_batch, max_seq_len=cfg["max_position_embeddings"],
                                        max_batch_tokens=32768, max_logit_rows=max(64, args.batch),
                                        gemm_tune_rows=tune_rows),
                    config_dict=cfg, random_seed=0)
    dev = engine.device
    gen = torch.Generator().manual_seed(0)

    def decode_run(batch, steps, warmup, context, decoded_before=0):
        """Times ``steps`` decode steps of ``batch`` requests through the serving loop (scheduler,
        step function, sampler; a step is launched while the host still waits for the previous
        step's tokens).  The prompts are prefilled first, in portions; their lengths are set so
        that the longest context ENDS at ``context``.  ``decoded_before``: the requests have been
        decoding for that many steps when the warm-up steps begin.  Returns (seconds, mean
        context length over the timed steps)."""
        budget = 32768
        runner = Runner(engine, ServeOptions(ignore_eos=True, run_ahead=True, max_batch_tokens=budget))
        warmup += decoded_before
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
        for rid in runner.live_requests():
            runner.cancel(rid)
        assert runner.idle()
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

    def add_point(name, batch, steps, seconds, mean_context):
        """tok/s under the name itself; beside it the step's time, the bytes it has to read (every
        weight once, the cache of the live requests) and the fraction of the HBM peak that is."""
        ms = seconds / steps * 1e3
        gb = (weight_bytes(cfg) + batch * mean_context * kv_bytes_per_token(cfg)) / 1e9
        points[name] = round(batch * steps / seconds, 1)
        points[name + "_ms"] = round(ms, 4)
        points[name + "_gb"] = round(gb, 3)
        points[name + "_frac"] = round(gb / (ms * 1e-3) / HBM_PEAK_GBS, 4)

    if not args.skip_points:
        for b in (1, 64):
            k = max(16, args.steps // 2)
            d, c = decode_run(b, k, 8, ctx)
            add_point(f"decode_b{b}", b, k, d, c)
        # The default run again, with the requests 320 steps into their decoding when the same warm-up
        # and the same timed steps begin.  After a prefill (seconds of matrix products that ask
        # little of the memory) the first third of a second of decode steps runs 6-7 % slower than
        # all that follow: every kernel that streams weights takes 0.5-1 us longer, until the
        # memory has been busy for that long (one run of 8 x 8,192, 40 steps at a time: 1.227 ms
        # seven times, then 1.169, 1.150, 1.149 ..; kernel by kernel in a trace: down and output
        # 8.9 -> 7.9 us, gate/up 14.1 -> 13.1, Q/K/V 7.9 -> 7.4, attention 25.4 -> 24.8).  A server
        # that decodes is past that point; the default run, timed right after its prompts, is not.
        # Every point has such a twin, "..._sustained": about 0.4 s of decode steps first, or, where
        # the context has no room for them, the same run repeated until as much lies behind.
        if ctx >= 400 + args.warmup + args.steps + 64:
            d, c = decode_run(args.batch, args.steps, args.warmup, ctx, decoded_before=320)
            add_point(f"decode_b{args.batch}_sustained", args.batch, args.steps, d, c)
            for b, before in ((1, 400), (64, 96)):
                k = max(16, args.steps // 2)
                d, c = decode_run(b, k, 8, ctx, decoded_before=before)
                add_point(f"decode_b{b}_sustained", b, k, d, c)
        # the serving workload of the comparison: 512-token prompts, 256 generated tokens
        for b in (1, 8, 64):
            d, c = decode_run(b, 240, 8, 512 + 256)
            add_point(f"decode_b{b}_p512_g256", b, 240, d, c)
            spent = d
            while spent < 0.45:                  # the same run again until 0.45 s of decode steps lie behind
                d, c = decode_run(b, 240, 8, 512 + 256)
                spent += d
            d, c = decode_run(b, 240, 8, 512 + 256)
            add_point(f"decode_b{b}_p512_g256_sustained", b, 240, d, c)

    # what a plain read stream gets from this GPU's memory (the published peak is 8 TB/s)
    from kv_cache_optimization_for_llm_amd.ops import kernels as K
    probed_gbs = K.probe_read_bandwidth(dev)

    kernel_ms = None
    if args.kernel_classes:
        graphs, portion_graphs = engine.graphs, engine.portion_graphs
        engine.graphs = engine.portion_graphs = None           # launched one by one, so that events fit between
        kernel_ms = {}
        try:
            # eight requests decoding at the context's end
            ids = [f"k{i}" for i in range(args.batch)]
            base = [int(t) for t in torch.randint(0, engine.vocab_size, (ctx - 8,), generator=gen)]
            for rid in ids:
                for lo in range(0, len(base), 4096):
                    engine.step([StepEntry(rid, base[lo:lo + 4096], [])])
            step = [StepEntry(rid, [5], [0]) for rid in ids]
            engine.step(step)
            with K.KernelClassTimer() as timer:
                engine.step(step)
            kernel_ms[f"decode_b{args.batch}_eager"] = timer.milliseconds()
            for rid in ids:
                engine.release(rid)
            engine.step([StepEntry("kp0", prompt, [PREFILL_TOKENS - 1])])
            engine.release("kp0")
            with K.KernelClassTimer() as timer:
                engine.step([StepEntry("kp1", prompt, [PREFILL_TOKENS - 1])])
            kernel_ms[f"prefill_{PREFILL_TOKENS}_eager"] = timer.milliseconds()
            engine.release("kp1")
        finally:
            engine.graphs, engine.portion_graphs = graphs, portion_graphs

    # The serving loop at the layer sizes of the larger configurations (random weights, seeded
    # uniform token ids): 32 requests with prompts of 128 to 4,096 tokens and 128 new tokens each,
    # portions of 512, at the 3B sizes; 64 concurrent requests of 8,192 + 512 tokens at the 8B
    # sizes, once over the paged cache and once over the contiguous one (what is reserved against
    # what holds a token is the comparison the reference's paper makes).
    if not args.skip_large:
        import gc
        from kv_cache_optimization_for_llm_amd.cli import sweep
        del engine
        gc.collect()
        torch.cuda.empty_cache()
        mixed = sweep.build_parser().parse_args(
            ["--workload", "mixed", "--prompt-len", "4096", "--prompt-min", "128", "--new-tokens", "128",
             "--chunk-size", "512", "--max-batch-tokens", "4096", "--tune-gemm"])
        r = sweep.run_one(mixed, "3b", 32, "paged")
        points.update({"serve_3b_mixed_b32_tok_s": round(r["tokens_emitted"] / r["wall_s"], 1),
                       "serve_3b_mixed_b32_wall_s": r["wall_s"], "serve_3b_mixed_b32_prefill_tok_s": r["prefill_tok_s"],
                       "serve_3b_mixed_b32_decode_tok_s": r["decode_tok_s"],
                       "serve_3b_mixed_b32_decode_frac": r.get("decode_hbm_frac"),
                       "serve_3b_mixed_b32_pages_reused": r["pages_reused"],
                       "serve_3b_mixed_b32_preemptions": r["preemptions"]})
        gc.collect()
        torch.cuda.empty_cache()
        long = sweep.build_parser().parse_args(
            ["--prompt-len", "8192", "--new-tokens", "512", "--max-batch-tokens", "8192", "--chunk-size", "2048",
             "--reserve-policy", "pow2", "--tune-gemm"])
        for mode in ("paged", "contiguous"):
            r = sweep.run_one(long, "8b", 64, mode)
            key = f"serve_8b_b64_ctx8704_{mode}"
            points.update({key + "_decode_tok_s": r["decode_tok_s"], key + "_decode_frac": r.get("decode_hbm_frac"),
                           key + "_prefill_tok_s": r["prefill_tok_s"], key + "_wall_s": r["wall_s"],
                           key + "_kv_tokens_reserved": r["peak_kv_tokens_reserved"],
                           key + "_kv_tokens_live": r["peak_kv_tokens_live"],
                           key + "_reserved_over_live": r["reserved_over_live"],
                           key + "_pages_reused": r["pages_reused"], key + "_preemptions": r["preemptions"],
                           key + "_fragmentation_failures": r["fragmentation_failures"]})
            gc.collect()
            torch.cuda.empty_cache()

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
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "bytes_gb": round(step_bytes / 1e9, 3),
                     "probed_read_stream": round(probed_gbs, 1), "frac_of_probed": round(achieved / probed_gbs, 4)},
        "points": points,
    }
    if kernel_ms is not None:
        out["kernel_ms"] = kernel_ms
        for run, classes in kernel_ms.items():          # and flat, beside the other points
            for cls, ms in classes.items():
                name = "".join(c if c.isalnum() else "_" for c in cls).strip("_")
                while "__" in name:
                    name = name.replace("__", "_")
                points[f"kclass_{run}_{name}_ms"] = ms
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
