"""A small client for the serving process, in the manner of the reference's ``client.py`` and
``bench.py``: it starts the engine as a child process, writes request lines to its standard
input, reads JSON lines back, and reports counts, speeds, an order-sensitive checksum per
sequence (``h = h * 1000003 + tok mod 2^32``, reference ``bench.py:226-237``) and the token-count
invariant (with ``IGNORE_EOS=1`` every sequence emits exactly its budget, ``bench.py:334-338``).

    python -m kv_cache_optimization_for_llm_amd.cli.client MODEL_DIR [N] [--prompts FILE] ...

Prompts are token ids: one prompt per line of ``--prompts FILE`` (ids separated by spaces), or
``N`` seeded random prompts.  No tokenizer is needed.  ``STALL_TIMEOUT_S`` (default 120) ends the
run when the engine says nothing for that long (reference ``base/client.py:30``).
"""
from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys
import threading
import time
from typing import Dict, List, Tuple


def checksum(tokens: List[int]) -> int:
    h = 0
    for t in tokens:
        h = (h * 1000003 + t) & 0xFFFFFFFF
    return h


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="client", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model_dir")
    ap.add_argument("num_prompts", nargs="?", type=int, default=4)
    ap.add_argument("--prompts", help="file with one prompt per line, token ids separated by spaces")
    ap.add_argument("--prompt-len", type=int, default=32)
    ap.add_argument("--max-new-tokens", type=int, default=32)
    ap.add_argument("--num-seqs", type=int, default=1)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--out", help="write the result as JSON to this file")
    argv = list(sys.argv[1:] if argv is None else argv)
    engine_args = []
    if "--" in argv:            # everything after -- goes to the engine
        cut = argv.index("--")
        argv, engine_args = argv[:cut], argv[cut + 1:]
    args = ap.parse_args(argv)
    stall = float(os.environ.get("STALL_TIMEOUT_S", "120"))

    if args.prompts:
        with open(args.prompts) as f:
            prompts = [[int(x) for x in line.split()] for line in f if line.strip()]
        if args.num_prompts > len(prompts):
            print(f"Asked for {args.num_prompts} prompts but {args.prompts} only has {len(prompts)}.", file=sys.stderr)
            return 1
        prompts = prompts[:args.num_prompts]
    else:
        import numpy as np
        with open(os.path.join(args.model_dir, "config.json")) as f:
            vocab = json.load(f)["vocab_size"]
        rng = np.random.default_rng(args.seed)
        prompts = [[int(t) for t in rng.integers(0, vocab, args.prompt_len)] for _ in range(args.num_prompts)]

    extra = engine_args
    env = dict(os.environ)
    env.setdefault("IGNORE_EOS", "1")
    cmd = [sys.executable, "-m", "kv_cache_optimization_for_llm_amd.cli.serve", args.model_dir, *extra]
    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    env["PYTHONPATH"] = root + os.pathsep + env.get("PYTHONPATH", "")
    engine = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=sys.stderr,
                              text=True, bufsize=1, env=env)
    tokens: Dict[Tuple[int, int], List[int]] = {}
    done: Dict[Tuple[int, int], dict] = {}
    other: List[dict] = []
    last_line = [time.time()]

    def reader():
        for line in engine.stdout:
            last_line[0] = time.time()
            try:
                msg = json.loads(line)
            except json.JSONDecodeError:
                continue
            if msg.get("done"):
                done[(msg["id"], msg["seq"])] = msg
            elif "tok" in msg:
                tokens.setdefault((msg["id"], msg["seq"]), []).append(msg["tok"])
            else:
                other.append(msg)

    threading.Thread(target=reader, daemon=True).start()
    t0 = time.time()
    for i, p in enumerate(prompts):
        engine.stdin.write(f"{i} {args.max_new_tokens} {args.num_seqs} {' '.join(map(str, p))}\n")
    engine.stdin.flush()
    engine.stdin.close()
    expected = len(prompts) * args.num_seqs
    status = "ok"
    while len(done) < expected:
        if engine.poll() is not None and len(done) < expected:
            time.sleep(0.2)
            if len(done) < expected:
                status = f"engine exited with {engine.returncode}"
                break
        if time.time() - last_line[0] > stall:
            status = f"stalled: nothing from the engine for {stall:.0f} s"
            engine.kill()
            break
        time.sleep(0.01)
    wall = time.time() - t0
    try:
        engine.wait(timeout=30)
    except subprocess.TimeoutExpired:
        engine.kill()

    total = sum(len(v) for v in tokens.values())
    broken = [k for k, d in done.items() if d["tokens"] != len(tokens.get(k, []))]
    short = [k for k, d in done.items() if env["IGNORE_EOS"] == "1" and "error" not in d
             and d["tokens"] != args.max_new_tokens]
    result = {
        "status": status, "requests": len(prompts), "sequences_done": len(done), "tokens": total,
        "wall_s": round(wall, 3), "tokens_per_s": round(total / wall, 1) if wall > 0 else 0.0,
        "count_mismatches": len(broken), "budget_mismatches": len(short),
        "errors": sorted({d["error"] for d in done.values() if "error" in d}),
        "checksums": {f"{k[0]}.{k[1]}": checksum(v) for k, v in sorted(tokens.items())},
        "preemptions": sum(1 for m in other if m.get("type") == "preempted"),
        "engine_config": next((m for m in other if m.get("type") == "engine_config"), None),
    }
    print(json.dumps(result, indent=2))
    if args.out:
        with open(args.out, "w") as f:
            json.dump(result, f, indent=2)
    return 0 if status == "ok" and not broken and not short else 1


if __name__ == "__main__":
    sys.exit(main())
