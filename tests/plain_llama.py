"""A plain, slow Llama: whole sequences, no cache, one function per part.

Written from the reference's formulas; every function cites the reference file and lines it
restates.  It shares no code with the package under test: it reads ``config.json`` keys and
safetensors tensors by itself and uses only torch on the CPU.

``act`` is the rounding applied to every op's output: identity for the 32-bit model, a
bfloat16 round trip to mimic the reference's storage of every intermediate in bf16
(``base/src/engine.cuh:40-51``).
"""
from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional, Sequence

import numpy as np
import torch


def identity(x: torch.Tensor) -> torch.Tensor:
    return x


def round_bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype)


# ----------------------------------------------------------------------------- loading
def load_model_dir(model_dir: str, dtype=torch.float32):
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    weights = {k: v.to(dtype) for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, weights


def head_dim_of(cfg) -> int:
    return cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]


# ----------------------------------------------------------------------------- parts
def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """base/src/kernels.cu:10-36: r = sqrt(sum(x^2)/H + eps); y = (x / r) * w."""
    r = torch.sqrt((x * x).sum(dim=-1, keepdim=True) / x.shape[-1] + eps)
    return (x / r) * w


def rope_inv_freq(head_dim: int, theta: float, scaling: Optional[dict]) -> np.ndarray:
    """base/src/kernels.cu:56-88 (float arithmetic throughout, as there)."""
    f = np.float32
    half = head_dim // 2
    inv = np.zeros(half, dtype=f)
    for i in range(half):
        inv[i] = f(1.0) / f(np.power(f(theta), f(f(2.0) * f(i)) / f(head_dim)))
    if not scaling or scaling.get("rope_type", scaling.get("type")) in (None, "default"):
        return inv
    assert scaling.get("rope_type", scaling.get("type")) == "llama3"
    factor, low, high = f(scaling["factor"]), f(scaling["low_freq_factor"]), f(scaling["high_freq_factor"])
    orig = f(scaling["original_max_position_embeddings"])
    low_wl, high_wl = f(orig / low), f(orig / high)
    out = inv.copy()
    for i in range(half):
        wavelen = f(f(2.0) * f(math.pi) / inv[i])
        if wavelen > low_wl:
            out[i] = f(inv[i] / factor)
        elif wavelen >= high_wl:
            smooth = f(f(orig / wavelen - low) / f(high - low))
            out[i] = f(f(f(1.0) - smooth) * f(inv[i] / factor) + f(smooth * inv[i]))
    return out


def rope_cos_sin(positions: Sequence[int], inv_freq: np.ndarray):
    """base/src/kernels.cu:90-106: angle = pos * inv_freq in float; cos and sin of it."""
    pos = np.asarray(positions, dtype=np.float32)[:, None]
    angle = (pos * inv_freq[None, :]).astype(np.float32)
    return np.cos(angle).astype(np.float32), np.sin(angle).astype(np.float32)


def apply_rope(x: torch.Tensor, cos: np.ndarray, sin: np.ndarray) -> torch.Tensor:
    """base/src/kernels.cu:289-319: rotate-half pairing, element j with j + d/2, angle index j:
    out[j] = x[j] c - x[j+d/2] s ; out[j+d/2] = x[j] s + x[j+d/2] c.   x: [T, heads, d]."""
    half = x.shape[-1] // 2
    c = torch.from_numpy(cos).to(x.dtype)[:, None, :]
    s = torch.from_numpy(sin).to(x.dtype)[:, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * c - x2 * s, x1 * s + x2 * c], dim=-1)


def causal_gqa_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                         window: int = 0) -> torch.Tensor:
    """base/src/kernels.cu:156-225 (decode) and :361-466 (prefill): per query head h, kv head
    h // (nq / nkv); score = (q . k) * scale over keys 0..p of the same sequence; softmax;
    weighted sum of V.   q: [T, nq, d]; k, v: [T, nkv, d]  ->  [T, nq, d]."""
    T, nq, d = q.shape
    nkv = k.shape[1]
    group = nq // nkv
    out = torch.zeros_like(q)
    for h in range(nq):
        kh = h // group
        for t in range(T):
            lo = max(0, t - window + 1) if window > 0 else 0
            scores = (k[lo:t + 1, kh, :] @ q[t, h, :]) * scale
            m = scores.max()
            p = torch.exp(scores - m)
            out[t, h, :] = (p[:, None] * v[lo:t + 1, kh, :]).sum(dim=0) / p.sum()
    return out


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """base/src/engine.cu:652-671: y = x W^T for a row-major [out, in] weight, no bias."""
    return x @ w.t()


def swiglu(x: torch.Tensor, w_gate, w_up, w_down, act: Callable = identity) -> torch.Tensor:
    """base/src/engine.cu:780-858 and kernels.cu:45-52: down( g * (1 / (1 + exp(-g))) * u )."""
    g = act(linear(x, w_gate))
    u = act(linear(x, w_up))
    a = act(g * (1.0 / (1.0 + torch.exp(-g))) * u)
    return act(linear(a, w_down))


def attention_block(x, W, prefix, cfg, positions, act: Callable = identity, window: int = 0):
    """base/src/engine.cu:652-762: q,k,v projections -> rope(q), rope(k) -> attention -> o."""
    nq, nkv, d = cfg["num_attention_heads"], cfg.get("num_key_value_heads") or cfg["num_attention_heads"], head_dim_of(cfg)
    T = x.shape[0]
    q = act(linear(x, W[prefix + "q_proj.weight"])).view(T, nq, d)
    k = act(linear(x, W[prefix + "k_proj.weight"])).view(T, nkv, d)
    v = act(linear(x, W[prefix + "v_proj.weight"])).view(T, nkv, d)
    inv = rope_inv_freq(d, cfg.get("rope_theta", 10000.0), cfg.get("rope_scaling"))
    cos, sin = rope_cos_sin(positions, inv)
    q, k = act(apply_rope(q, cos, sin)), act(apply_rope(k, cos, sin))
    o = act(causal_gqa_attention(q, k, v, 1.0 / math.sqrt(d), window)).reshape(T, nq * d)
    return act(linear(o, W[prefix + "o_proj.weight"]))


def hidden_states(cfg, W: Dict[str, torch.Tensor], tokens: Sequence[int], act: Callable = identity,
                  first_position: int = 0) -> torch.Tensor:
    """base/src/engine.cu:637-860: embed; per layer h += attn(norm(h)); h += mlp(norm(h));
    final norm.  Returns the normed hidden state of every token."""
    eps = cfg["rms_norm_eps"]
    T = len(tokens)
    positions = list(range(first_position, first_position + T))
    h = W["model.embed_tokens.weight"][torch.as_tensor(list(tokens), dtype=torch.long)].clone()
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        x = act(rms_norm(h, W[p + "input_layernorm.weight"], eps))
        h = act(h + attention_block(x, W, p + "self_attn.", cfg, positions, act))
        x = act(rms_norm(h, W[p + "post_attention_layernorm.weight"], eps))
        h = act(h + swiglu(x, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"],
                           W[p + "mlp.down_proj.weight"], act))
    return act(rms_norm(h, W["model.norm.weight"], eps))


def logits_all(cfg, W, tokens: Sequence[int], act: Callable = identity) -> torch.Tensor:
    """base/src/engine.cu:872-890: logits = x E^T with the token table (tied), or lm_head."""
    x = hidden_states(cfg, W, tokens, act)
    head = W["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else W["lm_head.weight"]
    return linear(x, head)


# ----------------------------------------------------------------------------- sampling
def counter_uniform(seed: int, key: int, step: int) -> float:
    """base/src/kernels.cu:638-649 and python/sampling_reference.py:26-35."""
    M = (1 << 64) - 1
    z = (((key & 0xFFFFFFFF) << 32) ^ (step & 0xFFFFFFFF)) & M
    z ^= (seed * 0x9E3779B97F4A7C15) & M
    z = (z + 0x9E3779B97F4A7C15) & M
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
    z = z ^ (z >> 31)
    return (z >> 40) * (1.0 / 16777216.0)


def penalised(logits: np.ndarray, emitted: Sequence[int], penalty: float) -> np.ndarray:
    """base/src/kernels.cu:504-513: an already emitted token's logit l becomes l / p if l > 0
    else l * p."""
    out = np.array(logits, dtype=np.float64)
    for t in set(emitted):
        out[t] = out[t] / penalty if out[t] > 0 else out[t] * penalty
    return out


def greedy(logits: np.ndarray) -> int:
    """base/src/kernels.cu:489-496: the maximum; ties go to the lowest token id."""
    return int(np.argmax(logits))


def sample_temperature(logits: np.ndarray, temperature: float, u: float) -> int:
    """python/sampling_reference.py:85-89: flat inverse CDF, first index whose cumulative weight
    exceeds u * total."""
    w = np.exp((np.asarray(logits, dtype=np.float64) - np.max(logits)) / temperature)
    cdf = np.cumsum(w)
    return int(min(np.searchsorted(cdf, u * cdf[-1], side="right"), len(w) - 1))


def generate(cfg, W, prompt: Sequence[int], max_new_tokens: int, *, temperature: float = 0.0,
             seed: int = 0, rng_key: int = 0, repetition_penalty: float = 1.0,
             eos: Sequence[int] = (), act: Callable = identity) -> List[int]:
    """Whole-sequence recomputation for every new token.  The uniform for the token that will
    sit at absolute position p is counter_uniform(seed, rng_key, p).  The penalty applies to
    tokens already emitted, from the second generated token on (base/src/engine.cu:892-907,1260-1268)."""
    seq = list(prompt)
    out: List[int] = []
    for i in range(max_new_tokens):
        l = logits_all(cfg, W, seq, act)[-1].double().numpy()
        if repetition_penalty != 1.0 and i > 0:
            l = penalised(l, out, repetition_penalty)
        if temperature > 0:
            tok = sample_temperature(l, temperature, counter_uniform(seed, rng_key, len(seq)))
        else:
            tok = greedy(l)
        if tok in eos:
            break
        out.append(tok)
        seq.append(tok)
    return out
