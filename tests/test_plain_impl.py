"""Pins the plain implementation by what fixes it beside the reference's text: special cases
that reduce to a library routine, invariants, and the checks the reference's own sampling test
makes (python/sampling_reference.py:92-136)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_llama as plain
from conftest import TINY_A, TINY_B, TINY_C

torch.manual_seed(0)


def test_rms_norm_is_the_library_formula_and_the_weight_multiplies_last():
    x, w = torch.randn(5, 48), torch.rand(48) + 0.5
    want = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), want, atol=1e-6)
    y = plain.rms_norm(x, torch.ones(48), 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(5), atol=1e-5)      # unit RMS
    assert torch.allclose(plain.rms_norm(3.0 * x, w, 0.0), plain.rms_norm(x, w, 0.0), atol=1e-5)
    # a zero weight gives zero: the weight is used as stored, not as 1 + w
    assert plain.rms_norm(x, torch.zeros(48), 1e-5).abs().max() == 0


def test_rope_pairs_j_with_j_plus_half_and_turns_counter_clockwise():
    inv = plain.rope_inv_freq(4, 10000.0, None)
    assert inv[0] == 1.0 and abs(inv[1] - 0.01) < 1e-7
    cos, sin = plain.rope_cos_sin([1], inv)
    x = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]])
    out = plain.apply_rope(x, cos, sin)[0, 0]
    assert torch.allclose(out, torch.tensor([math.cos(1.0), 0.0, math.sin(1.0), 0.0]), atol=1e-6)
    x = torch.tensor([[[0.0, 0.0, 1.0, 0.0]]])
    out = plain.apply_rope(x, cos, sin)[0, 0]
    assert torch.allclose(out, torch.tensor([-math.sin(1.0), 0.0, math.cos(1.0), 0.0]), atol=1e-6)


def test_rope_is_complex_multiplication_and_only_distances_count():
    d = 24
    inv = plain.rope_inv_freq(d, 500000.0, TINY_B["rope_scaling"])
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)
    cos, sin = plain.rope_cos_sin([7], inv)
    out = plain.apply_rope(q, cos, sin)[0, 0]
    z = torch.complex(q[0, 0, :d // 2], q[0, 0, d // 2:]) * torch.polar(
        torch.ones(d // 2, dtype=torch.float64), torch.from_numpy((np.float32(7) * inv).astype(np.float64)))
    assert torch.allclose(out[:d // 2], z.real, atol=1e-6) and torch.allclose(out[d // 2:], z.imag, atol=1e-6)
    c0, s0 = plain.rope_cos_sin([0], inv)
    assert torch.equal(plain.apply_rope(q, c0, s0), q)                      # position 0 is the identity

    def dot(m, n):
        cm, sm = plain.rope_cos_sin([m], inv)
        cn, sn = plain.rope_cos_sin([n], inv)
        return (plain.apply_rope(q, cm, sm) * plain.apply_rope(k, cn, sn)).sum().item()
    assert abs(dot(9, 4) - dot(25, 20)) < 1e-4 and abs(dot(9, 4) - dot(5, 0)) < 1e-4
    assert abs(dot(9, 4) - dot(4, 9)) > 1e-3                               # the sign of the distance matters


def test_llama3_scaling_has_three_bands_and_is_continuous():
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=64)
    base = plain.rope_inv_freq(64, 500000.0, None)
    got = plain.rope_inv_freq(64, 500000.0, sc)
    wl = 2 * math.pi / base
    hi, lo = wl < 16, wl > 64
    mid = ~hi & ~lo
    assert hi.any() and lo.any() and mid.any()
    assert np.array_equal(got[hi], base[hi])                                # short waves: unchanged
    assert np.allclose(got[lo], base[lo] / 8.0, rtol=1e-6)                  # long waves: / factor
    assert ((got[mid] < base[mid]) & (got[mid] > base[mid] / 8.0)).all()    # between the two
    # factor 1 changes nothing
    assert np.allclose(plain.rope_inv_freq(64, 500000.0, dict(sc, factor=1.0)), base, rtol=1e-6)


def theta_for_wavelength(wavelen, head_dim, i):
    """The theta that gives frequency index ``i`` (of ``head_dim / 2``) the wavelength
    ``wavelen``: 2 pi theta^(2i/d) = wavelen."""
    return (wavelen / (2 * math.pi)) ** (head_dim / (2.0 * i))


def test_llama3_mid_band_meets_the_outer_bands_at_both_edges():
    """``rope_inv_freq`` itself is evaluated at frequencies put on and just inside both edges of
    the middle band: at wavelength orig / low_freq_factor it must give inv / factor (where the
    long-wave band begins), at orig / high_freq_factor the unscaled inv, and just inside each
    edge a value next to those.  A swapped pair of factors, a smooth that runs the wrong way or
    an interpolation of wavelengths instead of frequencies fails here."""
    d, i, orig, factor, low, high = 64, 8, 256.0, 8.0, 1.0, 4.0
    sc = dict(rope_type="llama3", factor=factor, low_freq_factor=low, high_freq_factor=high,
              original_max_position_embeddings=int(orig))
    low_wl, high_wl = orig / low, orig / high

    def at(wavelen):
        theta = theta_for_wavelength(wavelen, d, i)
        base = plain.rope_inv_freq(d, theta, None)[i]
        assert abs(2 * math.pi / base - wavelen) < 1e-3 * wavelen      # the frequency sits where it was put
        return plain.rope_inv_freq(d, theta, sc)[i] / base              # what scaling made of it

    assert abs(at(low_wl * 1.01) - 1 / factor) < 1e-6          # beyond the long edge: / factor
    assert abs(at(low_wl * 0.999) - 1 / factor) < 2e-3         # just inside: next to it ...
    assert at(low_wl * 0.999) > 1 / factor                     # ... and already above it
    assert abs(at(high_wl * 1.001) - 1.0) < 2e-3               # just inside the short edge: next to unscaled
    assert at(high_wl * 1.001) < 1.0
    assert at(high_wl * 0.99) == 1.0                           # beyond the short edge: unchanged
    # half-way in frequency (wavelength orig / 2.5: smooth = 0.5) the value is the mean of the two ends
    assert abs(at(orig / 2.5) - 0.5 * (1 / factor + 1.0)) < 1e-4
    # the ratio falls as the wavelength grows, all the way through the band
    ratios = [at(w) for w in np.linspace(high_wl * 1.001, low_wl * 0.999, 9)]
    assert all(a > b for a, b in zip(ratios, ratios[1:]))


@pytest.mark.parametrize("nq, nkv, d", [(4, 2, 16), (6, 1, 24), (3, 3, 8)])
def test_attention_is_the_library_routine(nq, nkv, d):
    T = 19
    q, k, v = torch.randn(T, nq, d), torch.randn(T, nkv, d), torch.randn(T, nkv, d)
    got = plain.causal_gqa_attention(q, k, v, 1 / math.sqrt(d))
    rep = nq // nkv
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.repeat_interleave(rep, 1).transpose(0, 1)[None],
        v.repeat_interleave(rep, 1).transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    assert torch.allclose(got, want, atol=2e-6)
    assert torch.allclose(got[0], v[0].repeat_interleave(rep, 0), atol=1e-6)     # one key: out = V
    zero = plain.causal_gqa_attention(torch.zeros_like(q), k, v, 1.0)
    assert torch.allclose(zero[5, 0], v[:6, 0].mean(0), atol=1e-6)               # q = 0: mean of V
    # consecutive query heads share a kv head
    if nkv > 1 and rep > 1:
        q2 = q.clone()
        q2[:, 1] = q[:, 0]
        assert torch.allclose(plain.causal_gqa_attention(q2, k, v, 1.0)[:, 1],
                              plain.causal_gqa_attention(q2, k, v, 1.0)[:, 0])


def test_window_is_a_band_mask():
    T, d, w = 23, 8, 5
    q, k, v = torch.randn(T, 2, d), torch.randn(T, 2, d), torch.randn(T, 2, d)
    i = torch.arange(T)
    mask = (i[None, :] <= i[:, None]) & (i[None, :] > i[:, None] - w)
    want = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                          v.transpose(0, 1)[None], attn_mask=mask)[0].transpose(0, 1)
    assert torch.allclose(plain.causal_gqa_attention(q, k, v, 1 / math.sqrt(d), window=w), want, atol=2e-6)


def test_swiglu_is_silu_times_up_then_down():
    x = torch.randn(4, 12)
    wg, wu, wd = torch.randn(20, 12), torch.randn(20, 12), torch.randn(12, 20)
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(plain.swiglu(x, wg, wu, wd), want, atol=1e-5)
    assert plain.swiglu(x, wg, torch.zeros(20, 12), wd).abs().max() == 0          # up = 0 -> 0


def random_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    d = plain.head_dim_of(cfg)
    nq, nkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    W = {"model.embed_tokens.weight": torch.randn(V, H, generator=g) * 0.5,
         "model.norm.weight": 1 + 0.1 * torch.randn(H, generator=g)}
    if not cfg.get("tie_word_embeddings"):
        W["lm_head.weight"] = torch.randn(V, H, generator=g) * 0.1
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        W[p + "input_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g)
        W[p + "post_attention_layernorm.weight"] = 1 + 0.1 * torch.randn(H, generator=g)
        for n, shape in (("self_attn.q_proj", (nq * d, H)), ("self_attn.k_proj", (nkv * d, H)),
                         ("self_attn.v_proj", (nkv * d, H)), ("self_attn.o_proj", (H, nq * d)),
                         ("mlp.gate_proj", (I, H)), ("mlp.up_proj", (I, H)), ("mlp.down_proj", (H, I))):
            W[p + n + ".weight"] = torch.randn(*shape, generator=g) * 0.15
    return W


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B, TINY_C])
def test_model_is_causal_and_a_shift_of_all_positions_changes_nothing(cfg):
    W = random_weights(cfg, 1)
    toks = [int(t) for t in torch.randint(0, cfg["vocab_size"], (20,))]
    full = plain.logits_all(cfg, W, toks)
    assert full.shape == (20, cfg["vocab_size"])
    part = plain.logits_all(cfg, W, toks[:11])
    assert torch.allclose(full[:11], part, atol=1e-5)             # later tokens do not reach back
    changed = plain.logits_all(cfg, W, toks[:10] + [(toks[10] + 1) % cfg["vocab_size"]] + toks[11:])
    assert torch.allclose(full[:10], changed[:10], atol=1e-5) and not torch.allclose(full[10:], changed[10:], atol=1e-3)
    a = plain.hidden_states(cfg, W, toks, first_position=0)
    b = plain.hidden_states(cfg, W, toks, first_position=37)
    assert torch.allclose(a, b, atol=2e-4)                        # only distances count
    # tied: the table is the output matrix; untied: lm_head is, and the table is not
    x = plain.hidden_states(cfg, W, toks)
    table = W["model.embed_tokens.weight"]
    if cfg.get("tie_word_embeddings"):
        assert torch.allclose(full, F.linear(x, table), atol=1e-6)
    else:
        assert torch.allclose(full, F.linear(x, W["lm_head.weight"]), atol=1e-6)
        assert not torch.allclose(full, F.linear(x, table), atol=1e-2)


def test_bf16_emulation_rounds_every_output():
    W = random_weights(TINY_A, 2)
    toks = list(range(12))
    a = plain.logits_all(TINY_A, W, toks)
    b = plain.logits_all(TINY_A, W, toks, act=plain.round_bf16)
    assert not torch.equal(a, b) and (a - b).abs().max() < 0.05 * a.abs().max()


# ---- the sampler: the reference's own three checks --------------------------------------
def peaked_logits(vocab=128256, seed=0):
    rng = np.random.default_rng(seed)
    logits = rng.normal(0.0, 2.0, vocab)
    logits[rng.choice(vocab, 20, replace=False)] += 12.0
    return logits


def test_counter_uniform_is_splitmix64_of_the_counter():
    """With seed, key and step all 0 the mixed word is splitmix64's first output for state 0,
    0xE220A8397B1DCDAF (the public test vector of that generator); its top 24 bits make u."""
    assert plain.counter_uniform(0, 0, 0) == 0xE220A8 / 2 ** 24
    # key sits in the upper half of the counter, step in the lower half, and the seed is folded in
    # by a multiplication: each of them alone moves the draw
    assert len({plain.counter_uniform(0, 0, 0), plain.counter_uniform(1, 0, 0),
                plain.counter_uniform(0, 1, 0), plain.counter_uniform(0, 0, 1)}) == 4
    assert plain.counter_uniform(0, 1, 0) != plain.counter_uniform(0, 0, 1)


def test_counter_uniform_is_in_range_and_a_pure_function():
    us = [plain.counter_uniform(1234, 7, i) for i in range(2000)]
    assert all(0.0 <= u < 1.0 for u in us) and abs(np.mean(us) - 0.5) < 0.03
    assert plain.counter_uniform(1234, 7, 5) == us[5]
    assert plain.counter_uniform(1234, 8, 5) != us[5] and plain.counter_uniform(1235, 7, 5) != us[5]
    assert all(round(u * 16777216) == u * 16777216 for u in us[:50])       # 24-bit fractions


def test_empirical_distribution_matches_softmax():
    logits = peaked_logits()
    probs = np.exp(logits - logits.max())
    probs /= probs.sum()
    top = np.argsort(probs)[-8:]
    draws = 40000
    cdf = np.cumsum(np.exp(logits - logits.max()))
    counts = np.zeros(len(logits))
    for i in range(draws):
        counts[np.searchsorted(cdf, plain.counter_uniform(99, 3, i) * cdf[-1], side="right")] += 1
    for t in top:
        assert abs(counts[t] / draws - probs[t]) / probs[t] < 0.05
    # and the function under the same draws picks the same tokens
    for i in range(200):
        u = plain.counter_uniform(99, 3, i)
        assert plain.sample_temperature(logits, 1.0, u) == int(np.searchsorted(cdf, u * cdf[-1], side="right"))


def test_boundary_draws_stay_in_range_and_greedy_takes_the_lowest_id():
    logits = peaked_logits(1000)
    for u in (0.0, 1.0 - 2.0 ** -24):
        assert 0 <= plain.sample_temperature(logits, 0.7, u) < 1000
    l = np.zeros(10)
    l[[3, 7]] = 5.0
    assert plain.greedy(l) == 3
    pen = plain.penalised(np.array([2.0, -2.0, 1.0]), [0, 1], 1.15)
    assert np.allclose(pen, [2.0 / 1.15, -2.0 * 1.15, 1.0])
