"""Single kernels in a loop, for timing and for profilers.

    python -m kv_cache_optimization_for_llm_amd.cli.micro attention --tokens 8192 --kernel lds
    python -m kv_cache_optimization_for_llm_amd.cli.micro attention --batch 8 --context 8192 --splits 32
    python -m kv_cache_optimization_for_llm_amd.cli.micro gemm --rows 8 --shape gate_up
    python -m kv_cache_optimization_for_llm_amd.cli.micro prompt --tokens 8192 --portion 512
    python -m kv_cache_optimization_for_llm_amd.cli.micro stream --megabytes 8.4,67,525

The reference keeps a harness that runs its attention kernels alone over made-up caches
(``micro/harness.cuh``); this is the same idea for the kernels here.  Sizes default to the
Llama-3.2-1B ones.  Every call works on its own copy of the weights or the cache, enough copies
that nothing is served from a cache of the memory system, and one line is printed per case:
microseconds per call, and TFLOP/s or TB/s of what the call has to compute or read.  Calls are
launched one by one from the host: below some 15 us a figure shows the host's launch rate, not
the kernel (inside a HIP graph, as decode steps run, the same kernels take less).
"""
from __future__ import annotations

import argparse
import sys
import time

GEMM_MODES = {"qkv": "plain", "o": "resid", "gate_up": "swiglu", "down": "resid", "lm_head": "f32"}


def gemm_shape(name: str, sizes: str = "1b"):
    """(N, K, mode) of a layer's product at the layer sizes of ``cli.sweep.SHAPES[sizes]``;
    mode: plain | resid | swiglu | f32 (the epilogue the model runs it with)."""
    from .sweep import SHAPES
    cfg = SHAPES[sizes]
    hidden, inter, d = cfg["hidden_size"], cfg["intermediate_size"], cfg["head_dim"]
    q, kv = cfg["num_attention_heads"] * d, cfg["num_key_value_heads"] * d
    n, k = {"qkv": (q + 2 * kv, hidden), "o": (hidden, q), "gate_up": (2 * inter, hidden),
            "down": (hidden, inter), "lm_head": (cfg["vocab_size"], hidden)}[name]
    return n, k, GEMM_MODES[name]


def _time(calls, reps: int) -> float:
    import torch
    for f in calls:
        f()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(reps):
        calls[i % len(calls)]()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps * 1e6


def _time_in_graph(calls, reps: int) -> float:
    """Microseconds per call when the calls run from a HIP graph, one after the other, as the
    kernels of a decode step do (no host launch cost between them)."""
    import torch
    for f in calls:
        f()
    n = max(len(calls), min(reps, 64))
    g = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        for i in range(n):
            calls[i % len(calls)]()
    g.replay()
    torch.cuda.synchronize()
    rounds = max(1, reps // n)
    t0 = time.perf_counter()
    for _ in range(rounds):
        g.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / (rounds * n) * 1e6


def attention(args) -> None:
    import numpy as np
    import torch
    from ..ops import kernels as K

    dev = torch.device("cuda:0")
    nq, nkv, d, page = args.heads, args.kv_heads, args.head_dim, 16
    group = nq // nkv
    scale = d ** -0.5
    if args.tokens:                                # a prompt portion of `tokens` tokens from position `start`
        entries = [(args.start, args.tokens)]
    else:                                          # `batch` decoded tokens at the end of `context`
        entries = [(args.context - 1, 1)] * args.batch
    ctx = max(s + n for s, n in entries)
    blocks = (ctx + page - 1) // page
    copies = max(1, min(8, int(600e6 / (len(entries) * blocks * page * nkv * d * 4)) + 1))
    caches = [(K.keys_to_pages(torch.randn(len(entries) * blocks, nkv, page, d, device=dev).bfloat16()),
               torch.randn(len(entries) * blocks, nkv, d, page, device=dev).bfloat16()) for _ in range(copies)]
    table = torch.arange(len(entries) * blocks, dtype=torch.int32).view(len(entries), blocks).to(dev)
    lens = [n for _, n in entries]
    T = sum(lens)
    qkv = torch.randn(T, nq * d, device=dev).bfloat16()
    out = torch.empty(T, nq * d, dtype=torch.bfloat16, device=dev)
    q_start = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tiles = args.tiles or (2 if args.tokens else 1)
    rows_per_item = {"lds": 128, "wave": 16 * tiles}[args.kernel]
    meta = []
    for e, (start, n) in enumerate(entries):
        for r0 in range(0, n * group, rows_per_item):
            meta.append((q_start[e], n, start, e, r0, 0, 0, 0))
    meta.sort(key=lambda m: -(m[2] + (min(m[4] + rows_per_item, m[1] * group) - 1) // group))
    meta_d = torch.tensor(meta, dtype=torch.int32, device=dev)
    ent = meta_d[:, 3].contiguous()
    row0 = meta_d[:, 4].contiguous()
    seat = torch.arange(len(entries), dtype=torch.int32, device=dev)
    qs = torch.from_numpy(q_start).to(dev)
    sp = torch.tensor([s for s, _ in entries], dtype=torch.int32, device=dev)
    splits, per = 1, 0
    if not args.tokens or args.portion_splits > 1:
        splits = args.portion_splits if args.tokens else args.splits
        per = ((ctx + splits - 1) // splits + 31) // 32 * 32
    if args.kernel == "lds":
        calls = [lambda c=c: K.attention_lds(qkv, nq * d, out, c[0], c[1], table, meta_d, nq, nkv, d, scale, 0, args.pair,
                                             splits, per) for c in caches]
    else:
        pair = bool(args.tokens) and len(meta) * nkv >= 2048 and not args.no_pair
        calls = [lambda c=c: K.attention_mfma(qkv, nq * d, out, c[0], c[1], table, ent, row0, seat, qs, sp, nq, nkv,
                                              d, scale, 0, splits, per, tiles, pair, meta_d) for c in caches]
    us = _time_in_graph(calls, args.reps) if args.graph else _time(calls, args.reps)
    flops = sum(4.0 * nq * d * n * (2 * s + n + 1) / 2 for s, n in entries)
    kv_bytes = sum((s + n) * nkv * d * 4 for s, n in entries)
    what = (f"prompt of {args.tokens}" + (f" from position {args.start}" if args.start else "") +
            (f", {splits} key ranges" if splits > 1 else "")) if args.tokens else f"batch {args.batch} at context {args.context}, {splits} splits"
    print(f"attention {args.kernel:4s} {what}: {us:9.1f} us  {flops / us / 1e6:8.1f} TFLOP/s  "
          f"{kv_bytes / us / 1e6:7.2f} TB/s of keys and values", flush=True)


def gemm(args) -> None:
    import torch
    from ..ops import kernels as K

    dev = torch.device("cuda:0")
    n, k, mode = gemm_shape(args.shape, args.sizes)
    m = args.rows
    copies = min(48, max(4, int(600e6 / (n * k * 2)) + 1))
    x = torch.randn(m, k, device=dev).bfloat16()
    ws = [torch.randn(n, k, device=dev).bfloat16() * 0.02 for _ in range(copies)]
    gemv = args.kernel == "gemv"
    if gemv and not K.gemv_supported(m, n, k):
        raise SystemExit(f"the matrix-vector kernel does not take {m} rows of [{n} x {k}]")
    tiled = ws if gemv else [K.TiledWeight(w, 2 if mode == "swiglu" else 1) for w in ws]
    product = K.gemv if gemv else K.gemm_skinny
    if mode == "resid":
        hidden = torch.zeros(m, n, device=dev).bfloat16()
        scaled = torch.empty_like(hidden)
        ss = torch.empty(m, K.gemv_sumsq_parts(n, k) if gemv else K.gemm_skinny_sumsq_parts(n), device=dev)
        nw = torch.ones(n, device=dev).bfloat16()
        calls = [lambda w=w: product(x, w, None, hidden=hidden, next_weight=nw, scaled_out=scaled, sumsq_out=ss)
                 for w in tiled]
    elif mode == "swiglu":
        out = torch.empty(m, n // 2, device=dev).bfloat16()
        if args.x_tiled:
            xt = K.TiledRows.from_rows(x)
            calls = [lambda w=w: product(xt, w, out, swiglu=True, x_tiled=True) for w in tiled]
        else:
            calls = [lambda w=w: product(x, w, out, swiglu=True) for w in tiled]
    else:
        out = torch.empty(m, n, device=dev, dtype=torch.float32 if mode == "f32" else torch.bfloat16)
        if args.x_tiled:
            xt = K.TiledRows.from_rows(x)
            calls = [lambda w=w: product(xt, w, out, x_tiled=True) for w in tiled]
        else:
            calls = [lambda w=w: product(x, w, out) for w in tiled]
    us = _time_in_graph(calls, args.reps) if args.graph else _time(calls, args.reps)
    name = "matrix-vector kernel" if gemv else "few-rows kernel"
    line = f"gemm {args.shape:8s} rows {m:3d} [{n} x {k}] {name} {us:8.2f} us  {n * k * 2 / us / 1e6:6.2f} TB/s of weights"
    if args.vendor:
        out_v = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
        us_v = _time([lambda w=w: K.gemm_vendor(x, w, out_v) for w in ws], args.reps)
        line += f"   vendor GEMM {us_v:8.2f} us"
    print(line, flush=True)


def prompt(args) -> None:
    """One prompt through the whole engine (Llama-3.2-1B sizes, random weights) in portions of
    ``--portion`` tokens, one portion per step: the time of the fastest of ``--reps`` passes."""
    import torch
    from ..engine.batch import StepEntry
    from ..engine.engine import Engine, EngineOptions
    from .sweep import SHAPES

    cfg = dict(SHAPES[args.sizes])
    cfg["max_position_embeddings"] = max(8192, args.tokens)
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    eng = Engine(None, EngineOptions(dtype="bfloat16", cache_tokens=args.tokens + 64, max_seqs=2,
                                     max_seq_len=cfg["max_position_embeddings"], use_graphs=not args.no_graphs,
                                     max_batch_tokens=max(8192, args.tokens),
                                     gemm_tune_rows=[args.portion] if args.tune_gemm else []),
                 config_dict=cfg, random_seed=0)
    gen = torch.Generator().manual_seed(0)
    tokens = [int(t) for t in torch.randint(0, eng.vocab_size, (args.tokens,), generator=gen)]
    best = float("inf")
    for _ in range(args.reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(0, args.tokens, args.portion):
            part = tokens[i:i + args.portion]
            eng.step([StepEntry("p", part, [len(part) - 1] if i + args.portion >= args.tokens else [])])
        torch.cuda.synchronize()
        best = min(best, time.perf_counter() - t0)
        eng.release("p")
    steps = (args.tokens + args.portion - 1) // args.portion
    from .sweep import weight_bytes
    # matrix products: two flops per weight and token (the head only at the wanted row); attention: causal
    layers, nq, d = cfg["num_hidden_layers"], cfg["num_attention_heads"], cfg["head_dim"]
    head = cfg["vocab_size"] * cfg["hidden_size"]
    flops = 2.0 * (weight_bytes(cfg, 1) - head) * args.tokens + 2.0 * head
    flops += layers * 4.0 * nq * d * args.tokens * (args.tokens + 1) / 2
    print(f"prompt of {args.tokens} in portions of {args.portion} ({steps} steps, {cfg['num_hidden_layers']} layers of the "
          f"{args.sizes} sizes): {best * 1e3:8.2f} ms  {args.tokens / best:9.0f} tok/s  {flops / best / 1e12:6.0f} TFLOP/s", flush=True)


def stream(args) -> None:
    """The floor for kernels that stream weights: a kernel that only reads N bytes once, each call
    on another buffer so that every byte comes from memory, launched one by one and from a graph
    of 200 such kernels (as decode steps run)."""
    import torch
    from ..ops import kernels as K

    dev = torch.device("cuda:0")
    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    print(f"plain read stream over 2 GiB: {K.probe_read_bandwidth(dev):.0f} GB/s")
    # what a compute unit takes in from L2: every workgroup reads the same few hundred kilobytes (the
    # rows of X of a few-rows product), over and over
    for kb in (64, 256, 1024):
        buf = torch.zeros(kb << 10, dtype=torch.uint8, device=dev)
        for wgs in (256, 512, 1024):
            reps = max(4, (64 << 20) // (kb << 10) // 8)
            for _ in range(2):
                K.stream_reread(buf, wgs, reps, sink)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            K.stream_reread(buf, wgs, reps, sink)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            total = wgs * reps * (kb << 10)
            print(f"{wgs} workgroups of 256 each read the same {kb} KB {reps} times: {dt * 1e6:.0f} us = "
                  f"{total / dt / 1e12:.2f} TB/s into the compute units ({total / dt / 1e9 / min(wgs, 256):.0f} GB/s per unit)")
    # two streams into a compute unit at once: 256 workgroups, each with a range of its own from
    # memory (a few-rows product's share of W) and a range all of them read (its rows of X)
    wgs = 256
    own_sets = [torch.zeros(wgs * (256 << 10), dtype=torch.uint8, device=dev) for _ in range(12)]
    for shared_kb in (64, 128, 256):
        shared = torch.zeros(shared_kb << 10, dtype=torch.uint8, device=dev)
        line = []
        for what in ("own", "shared", "both"):
            calls = [(lambda o=o: K.stream_mixed(o if what != "shared" else None,
                                                 shared if what != "own" else None, wgs, sink)) for o in own_sets]
            g = torch.cuda.CUDAGraph()
            for c in calls[:2]:
                c()
            torch.cuda.synchronize()
            with torch.cuda.graph(g):
                for i in range(120):
                    calls[i % len(calls)]()
            g.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(5):
                g.replay()
            torch.cuda.synchronize()
            line.append((time.perf_counter() - t0) / (5 * 120) * 1e6)
        print(f"{wgs} workgroups, each 256 KB of its own from memory and the same {shared_kb} KB from L2: "
              f"own alone {line[0]:.2f} us, shared alone {line[1]:.2f} us, both at once {line[2]:.2f} us")
    for mb in [float(x) for x in args.megabytes.split(",")]:
        n = int(mb * 1e6) // 16 * 16
        copies = max(2, min(200, int(3e9 // n)))
        bufs = [torch.zeros(n, dtype=torch.uint8, device=dev) for _ in range(copies)]
        for wgs in [int(w) for w in args.workgroups.split(",")]:
            eager = _time([(lambda b=b: K.stream_read(b, wgs, sink)) for b in bufs], 200)
            g = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            with torch.cuda.graph(g):
                for i in range(200):
                    K.stream_read(bufs[i % copies], wgs, sink)
            g.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(5):
                g.replay()
            torch.cuda.synchronize()
            in_graph = (time.perf_counter() - t0) / (5 * 200) * 1e6
            print(f"read {mb:g} MB, {wgs} workgroups of 256: {eager:.2f} us launched one by one, "
                  f"{in_graph:.2f} us in a graph = {n / in_graph / 1e6:.2f} TB/s")


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description="one kernel in a loop")
    sub = ap.add_subparsers(dest="what", required=True)
    a = sub.add_parser("attention")
    a.add_argument("--kernel", choices=["wave", "lds"], default="wave",
                   help="one wavefront per work item, or a workgroup sharing key blocks through LDS")
    a.add_argument("--tokens", type=int, default=0, help="a prompt of this many tokens (else decoded tokens)")
    a.add_argument("--start", type=int, default=0, help="with --tokens: the portion's first position (keys before it are in the cache)")
    a.add_argument("--portion-splits", type=int, default=1, help="with --tokens: cut the keys into this many ranges")
    a.add_argument("--batch", type=int, default=8)
    a.add_argument("--context", type=int, default=8192)
    a.add_argument("--splits", type=int, default=32)
    a.add_argument("--heads", type=int, default=32)
    a.add_argument("--kv-heads", type=int, default=8)
    a.add_argument("--head-dim", type=int, default=64)
    a.add_argument("--reps", type=int, default=20)
    a.add_argument("--no-pair", action="store_true", help="wave kernel: never give a wave two items")
    a.add_argument("--tiles", type=int, default=0, help="wave kernel: row tiles of 16 per item (default 2 for a prompt, 1 for decoded tokens)")
    a.add_argument("--pair", action="store_true", help="workgroup kernel: a workgroup takes item i and item n-1-i")
    a.add_argument("--graph", action="store_true", help="time the calls inside a HIP graph (no host launch cost)")
    g = sub.add_parser("gemm")
    g.add_argument("--shape", choices=sorted(GEMM_MODES), default="gate_up")
    g.add_argument("--sizes", choices=["1b", "3b", "8b"], default="1b", help="whose layer sizes (cli.sweep.SHAPES)")
    g.add_argument("--rows", type=int, default=8)
    g.add_argument("--vendor", action="store_true", help="also time the vendor GEMM on the plain weight")
    g.add_argument("--kernel", choices=["few-rows", "gemv"], default="few-rows",
                   help="the matrix-core kernel over the tiled weight, or the matrix-vector kernel (one or two rows)")
    g.add_argument("--graph", action="store_true", help="time the launches inside a captured graph")
    g.add_argument("--x-tiled", action="store_true", help="gated product: the rows of X laid out [K / 8][rows][8]")
    g.add_argument("--reps", type=int, default=48)
    pr = sub.add_parser("prompt")
    pr.add_argument("--tokens", type=int, default=8192)
    pr.add_argument("--portion", type=int, default=512)
    pr.add_argument("--sizes", choices=["1b", "3b", "8b"], default="1b", help="whose layer sizes (cli.sweep.SHAPES)")
    pr.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has")
    pr.add_argument("--reps", type=int, default=4)
    pr.add_argument("--no-graphs", action="store_true")
    pr.add_argument("--tune-gemm", action="store_true", help="time the vendor library's algorithms for the portion's rows first")
    st = sub.add_parser("stream", help="a kernel that only reads: the floor for weight-streaming kernels")
    st.add_argument("--megabytes", default="8.4,12.6,33.5,67,525", help="comma list of sizes to read")
    st.add_argument("--workgroups", default="256,1024,2048")
    args = ap.parse_args(argv)
    if args.what == "prompt":
        prompt(args)
        return 0
    if args.what == "stream":
        stream(args)
        return 0
    if args.what == "attention":
        if args.kernel == "lds" and not args.tokens:
            ap.error("the workgroup kernel is for prompts: give --tokens")
        attention(args)
    else:
        gemm(args)
    return 0


if __name__ == "__main__":
    sys.exit(main())
