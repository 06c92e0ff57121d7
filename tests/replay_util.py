"""Drives bin/trace_run as a user would and gathers its logits per (request, position)."""
import json
import os
import subprocess
import sys
from typing import Dict, List, Tuple

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def run_trace(model_dir: str, dtype: str, steps: List[dict], max_tokens: int, out_dir: str,
              vocab: int, extra_args=()) -> Dict[Tuple[str, int], np.ndarray]:
    """Feeds ``steps`` one at a time (the next only after ``done``) and returns
    {(request, position): logits row}."""
    os.makedirs(out_dir, exist_ok=True)
    cmd = [sys.executable, TRACE_RUN, "--model", model_dir, "--dtype", dtype, "--out", out_dir,
           "--max-tokens", str(max_tokens), *extra_args]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    pos: Dict[str, int] = {}
    rows: Dict[Tuple[str, int], np.ndarray] = {}
    try:
        for st in steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline()
            assert line.strip() == f"done {st['step']}", f"trace_run said {line!r} (exit {proc.poll()})"
            wanted = [(e["id"], pos.get(e["id"], 0) + i) for e in st["entries"] for i in e.get("want", [])]
            for e in st["entries"]:
                pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
            for rid in st.get("end", []):
                pos.pop(rid, None)
            if wanted:
                data = np.fromfile(os.path.join(out_dir, f"{st['step']}.f32"), dtype="<f4")
                data = data.reshape(len(wanted), vocab)
                for key, row in zip(wanted, data):
                    rows[key] = row
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    return rows


def cache_stats(out_dir: str) -> dict:
    """What trace_run's cache manager counted during the replay that wrote ``out_dir``."""
    with open(os.path.join(out_dir, "cache_stats.json")) as f:
        return json.load(f)


def whole(requests: Dict[str, List[int]]) -> List[dict]:
    """Each request alone and whole, one step each, logits everywhere."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
             "end": [rid]} for i, (rid, toks) in enumerate(requests.items())]


def tail_decoded(requests: Dict[str, List[int]], tail: int = 32) -> List[dict]:
    """Most of each request in one step, its last ``tail`` tokens one by one."""
    steps, n = [], 0
    for rid, toks in requests.items():
        cut = max(1, len(toks) - tail)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:cut], "want": list(range(cut))}], "end": []})
        n += 1
        for i in range(cut, len(toks)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}],
                          "end": [rid] if i == len(toks) - 1 else []})
            n += 1
        if cut == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def chunked(requests: Dict[str, List[int]], sizes=(7, 16, 5, 2, 33, 3, 64, 2)) -> List[dict]:
    """Each request alone, in portions of changing size, down to two tokens."""
    steps, n = [], 0
    for rid, toks in requests.items():
        i, k = 0, 0
        while i < len(toks):
            m = min(sizes[k % len(sizes)], len(toks) - i)
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[i:i + m], "want": list(range(m))}],
                          "end": [rid] if i + m == len(toks) else []})
            n, i, k = n + 1, i + m, k + 1
    return steps


def mixed(requests: Dict[str, List[int]], seed: int = 0, max_live: int = 4, prompt_frac: float = 0.6,
          chunk_sizes=(2, 5, 16, 9, 31)) -> List[dict]:
    """Up to ``max_live`` live requests: portions of some prompts beside single decoded tokens of
    others; a request may sit a step out.  Requests start as others end, so pages are reused."""
    rng = np.random.default_rng(seed)
    pending = list(requests.items())
    live: Dict[str, dict] = {}
    steps, n = [], 0
    while pending or live:
        while pending and len(live) < max_live:
            rid, toks = pending.pop(0)
            live[rid] = {"toks": toks, "done": 0, "prompt": max(2, int(len(toks) * prompt_frac))}
        entries, ended = [], []
        for rid, st in list(live.items()):
            if len(live) > 1 and rng.random() < 0.2:
                continue    # sits this step out
            if st["done"] < st["prompt"]:
                m = int(min(chunk_sizes[rng.integers(len(chunk_sizes))], st["prompt"] - st["done"]))
                if st["prompt"] - st["done"] - m == 1:
                    m += 1   # never leave a one-token portion of a prompt
            else:
                m = 1
            toks = st["toks"][st["done"]:st["done"] + m]
            entries.append({"id": rid, "tokens": toks, "want": list(range(len(toks)))})
            st["done"] += len(toks)
            if st["done"] == len(st["toks"]):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": n, "entries": entries, "end": ended})
            n += 1
    return steps


def max_live_tokens(steps: List[dict], unit: int = 64) -> int:
    """Most tokens live requests hold at any time, each count rounded up to ``unit``."""
    held: Dict[str, int] = {}
    peak = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum((v + unit - 1) // unit * unit for v in held.values()))
        for rid in st.get("end", []):
            held.pop(rid, None)
    return peak
