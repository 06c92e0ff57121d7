"""Generality of the framework, shown with toy parts that live only in this file.

* a mixer with a fixed-size state of its own (no keys and values) is registered, built from a
  model folder and stepped - whole, in portions, token by token, beside another request, and
  after its seat was used by someone else - without a change to the framework's files;
* one model has different mixers in different layers;
* a mixer whose cache entry is not keys and values of heads - one latent vector and one fp32 number
  per token - declares its arrays by name and shape and gets pages, a block table and a pool of
  its own from the same cache manager, beside an attention layer's;
* the run order is data: a layer is run twice (with a cache of its own each time) and a layer
  reads another call's cache without writing;
* another position encoding (rotation of neighbouring pairs instead of half-apart pairs) and a
  feed-forward with routing (the best of three small experts per token) are registered from here
  and run beside the framework's attention, which then cannot fuse with them and must not try.
"""
import math

import numpy as np
import pytest
import torch

import plain_llama as plain
from kv_cache_optimization_for_llm_amd.config.registry import (BLOCKS, FEED_FORWARDS, MIXERS, POSITION_ENCODINGS,
                                                               register_architecture)
from kv_cache_optimization_for_llm_amd.engine.batch import StepEntry
from kv_cache_optimization_for_llm_amd.engine.engine import Engine, EngineOptions
from kv_cache_optimization_for_llm_amd.models.spec import (LayerCall, LayerSpec, ModelSpec, PartSpec,
                                                           TensorSpec)
from kv_cache_optimization_for_llm_amd.ops import kernels as K
from kv_cache_optimization_for_llm_amd.parts.base import (Block, CacheArray, FeedForward, KVCacheSpec, Mixer,
                                                          MixerContext, PositionEncoding, StateSpec)
from kv_cache_optimization_for_llm_amd.weights.random_init import write_random_model

pytestmark = pytest.mark.gpu
DECAY = 0.75


class ToyDecayMixer(Mixer):
    """s_t = DECAY * s_{t-1} + W_in x_t ;  y_t = W_out s_t.  The state s is all it remembers."""

    def __init__(self, prefix, *, hidden_size, state_size):
        super().__init__(prefix)
        self.h, self.n = hidden_size, state_size

    def tensor_specs(self):
        return {self.prefix + "in.weight": TensorSpec((self.n, self.h)),
                self.prefix + "out.weight": TensorSpec((self.h, self.n))}

    def load(self, tensors):
        self.w_in = tensors[self.prefix + "in.weight"].float()
        self.w_out = tensors[self.prefix + "out.weight"].float()

    def state_spec(self):
        return StateSpec((self.n,), torch.float32)

    def forward(self, x, ctx: MixerContext):
        b = ctx.batch
        u = x.float() @ self.w_in.t()
        y = torch.empty_like(u)
        for e in range(b.num_entries):
            seat, lo, hi = int(b.h_entry_seat[e]), int(b.h_entry_q_start[e]), int(b.h_entry_q_start[e + 1])
            s = ctx.state[seat].clone()
            for t in range(lo, hi):
                s = DECAY * s + u[t]
                y[t] = s
            ctx.state[seat] = s
        return (y @ self.w_out.t()).to(x.dtype)


class ToyBlockwiseDecayMixer(ToyDecayMixer):
    """The same recurrence by a mixer that can only be cut where a block of four positions ends (it
    would update its state block by block): it says so, and records where it was cut."""
    portion_multiple = 4
    cuts = []

    def forward(self, x, ctx: MixerContext):
        b = ctx.batch
        for e in range(b.num_entries):
            n = int(b.h_entry_q_start[e + 1]) - int(b.h_entry_q_start[e])
            if n > 1:
                type(self).cuts.append((int(b.h_entry_start_pos[e]), n))
        return super().forward(x, ctx)


class ToyLatentMixer(Mixer):
    """Attention over one latent vector per token: c_t = W_c x_t, g_t = 1 + tanh(w_g . x_t) (kept in
    32-bit), q_t = W_q x_t; y_t = W_o sum_{s<=t} softmax_s(q_t . c_s / sqrt(w)) g_s c_s.  What it
    keeps per token is not keys and values of heads but two arrays of its own, of different widths
    and types; it reads them back through the block table it is handed."""

    def __init__(self, prefix, *, hidden_size, latent_size):
        super().__init__(prefix)
        self.h, self.w = hidden_size, latent_size

    def tensor_specs(self):
        p = self.prefix
        return {p + "c.weight": TensorSpec((self.w, self.h)), p + "q.weight": TensorSpec((self.w, self.h)),
                p + "g.weight": TensorSpec((1, self.h)), p + "o.weight": TensorSpec((self.h, self.w))}

    def load(self, tensors):
        p = self.prefix
        self.wc, self.wq, self.wg, self.wo = (tensors[p + n + ".weight"].float() for n in "cqgo")

    def kv_cache_spec(self):
        return KVCacheSpec((CacheArray("latent", (self.w,), token_axis=0),
                            CacheArray("gain", (1,), token_axis=0, dtype=torch.float32)))

    def forward(self, x, ctx: MixerContext):
        b, kv = ctx.batch, ctx.kv
        xf = x.float()
        c, q, g = xf @ self.wc.t(), xf @ self.wq.t(), 1 + torch.tanh(xf @ self.wg.t())
        latent, gain = kv.arrays["latent"], kv.arrays["gain"]           # [pages, page, w], [pages, page, 1]
        assert latent.shape[1:] == (kv.page_size, self.w) and gain.dtype == torch.float32
        if kv.writes:
            slots = kv.slot_mapping.long()
            latent.view(-1, self.w)[slots] = c.to(latent.dtype)
            gain.view(-1)[slots] = g[:, 0]
        y = torch.empty_like(c)
        for e in range(b.num_entries):
            seat, lo, hi = int(b.h_entry_seat[e]), int(b.h_entry_q_start[e]), int(b.h_entry_q_start[e + 1])
            start = int(b.h_entry_start_pos[e])
            ctx_len = start + hi - lo
            pages = kv.block_table[seat, :(ctx_len + kv.page_size - 1) // kv.page_size].long()
            cs = latent[pages].reshape(-1, self.w)[:ctx_len].float()      # what the cache holds (rounded to its type)
            gs = gain[pages].reshape(-1)[:ctx_len]
            scores = q[lo:hi] @ cs.t() / math.sqrt(self.w)
            keys = torch.arange(ctx_len, device=x.device)[None, :]
            mine = (start + torch.arange(hi - lo, device=x.device))[:, None]
            prob = torch.softmax(scores.masked_fill(keys > mine, float("-inf")), dim=-1)
            y[lo:hi] = (prob * gs[None, :]) @ cs
        return (y @ self.wo.t()).to(x.dtype)


class ToyNeighbourRotary(PositionEncoding):
    """Rotates the pairs (2j, 2j+1) of every head by position * theta^(-2j/d): the pairing of
    the original rotary paper, not the half-apart pairing the framework's kernels know."""

    def __init__(self, *, head_dim, theta):
        super().__init__("")
        self.inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))

    def apply_and_cache(self, qkv, positions, num_q_heads, num_kv_heads, head_dim, kv):
        T = qkv.shape[0]
        ang = positions.to(torch.float64)[:, None] * self.inv.to(qkv.device)[None, :]
        cos, sin = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]
        heads = num_q_heads + num_kv_heads
        x = qkv[:, :heads * head_dim].float().view(T, heads, head_dim // 2, 2)
        a, b = x[..., 0], x[..., 1]
        rot = torch.stack([a * cos - b * sin, a * sin + b * cos], dim=-1).view(T, heads * head_dim)
        qkv[:, :heads * head_dim] = rot.to(qkv.dtype)
        if kv is not None and kv.writes:        # the framework's kernel only stores K and V here
            K.rope_kv_write(qkv, positions, num_q_heads, num_kv_heads, head_dim, None, None,
                            kv.k_cache, kv.v_cache, kv.slot_mapping, kv.page_size)


class ToyRoutedFFN(FeedForward):
    """y = p * W2_e relu(W1_e x), e = the router's best expert for the token, p its softmax weight."""

    def __init__(self, prefix, *, hidden_size, inner_size, experts):
        super().__init__(prefix)
        self.h, self.i, self.e = hidden_size, inner_size, experts

    def tensor_specs(self):
        p = self.prefix
        return {p + "router.weight": TensorSpec((self.e, self.h)),
                p + "w1": TensorSpec((self.e, self.i, self.h)), p + "w2": TensorSpec((self.e, self.h, self.i))}

    def load(self, tensors):
        p = self.prefix
        self.router, self.w1, self.w2 = (tensors[p + n].float() for n in ("router.weight", "w1", "w2"))

    def forward(self, x, ctx):
        xf = x.float()
        prob = torch.softmax(xf @ self.router.t() * ROUTER_GAIN, dim=-1)
        p, e = prob.max(dim=-1)
        y = torch.zeros_like(xf)
        for k in range(self.e):                      # data-dependent shapes: not for a HIP graph
            rows = (e == k).nonzero().flatten()
            if rows.numel():
                y[rows] = torch.relu(xf[rows] @ self.w1[k].t()) @ self.w2[k].t()
        return (y * p[:, None]).to(x.dtype)


ROUTER_GAIN = 40.0


def toy_config(kind, dtype="float32"):
    return dict(architectures=[kind], vocab_size=97, hidden_size=40, state_size=24, intermediate_size=56,
                num_heads=4, num_kv_heads=2, head_dim=16, eps=1e-5, theta=10000.0, latent_size=12,
                max_position_embeddings=256, torch_dtype=dtype)


def toy_layer(c, i, mixer):
    p = f"blocks.{i}."
    if mixer in ("toy_decay", "toy_blockwise_decay"):
        mx = PartSpec(mixer, dict(prefix=p + "mix.", hidden_size=c["hidden_size"], state_size=c["state_size"]))
    elif mixer == "toy_latent":
        mx = PartSpec("toy_latent", dict(prefix=p + "lat.", hidden_size=c["hidden_size"], latent_size=c["latent_size"]))
    else:
        pos = PartSpec("rotary", dict(head_dim=c["head_dim"], max_positions=c["max_position_embeddings"],
                                      theta=c["theta"]))
        mx = PartSpec("gqa_attention", dict(prefix=p + "attn.", hidden_size=c["hidden_size"],
                                            num_heads=c["num_heads"], num_kv_heads=c["num_kv_heads"],
                                            head_dim=c["head_dim"], scale=1 / math.sqrt(c["head_dim"]),
                                            position=pos))
    norm = lambda n: PartSpec("rmsnorm", dict(prefix=p + n + ".", width=c["hidden_size"], eps=c["eps"]))
    return LayerSpec(block=PartSpec("pre_norm"), mixer=mx,
                     feed_forward=PartSpec("swiglu", dict(prefix=p + "ffn.", hidden_size=c["hidden_size"],
                                                          intermediate_size=c["intermediate_size"])),
                     norms={"mixer": norm("n1"), "feed_forward": norm("n2")}, prefix=p)


def toy_spec(kind, mixers, order):
    def build(c):
        return ModelSpec(architecture=kind, hidden_size=c["hidden_size"], vocab_size=c["vocab_size"],
                         embedding_name="embed.weight",
                         layers=tuple(toy_layer(c, i, m) for i, m in enumerate(mixers)), order=tuple(order),
                         final_norm=PartSpec("rmsnorm", dict(prefix="final.", width=c["hidden_size"], eps=c["eps"])),
                         final_norm_prefix="final.", head_name="head.weight",
                         max_positions=c["max_position_embeddings"])
    return build


def routed_spec(c):
    p = "blocks.0."
    pos = PartSpec("toy_neighbour_rotary", dict(head_dim=c["head_dim"], theta=c["theta"]))
    norm = lambda n: PartSpec("rmsnorm", dict(prefix=p + n + ".", width=c["hidden_size"], eps=c["eps"]))
    layer = LayerSpec(
        block=PartSpec("pre_norm"),
        mixer=PartSpec("gqa_attention", dict(prefix=p + "attn.", hidden_size=c["hidden_size"],
                                             num_heads=c["num_heads"], num_kv_heads=c["num_kv_heads"],
                                             head_dim=c["head_dim"], scale=1 / math.sqrt(c["head_dim"]), position=pos)),
        feed_forward=PartSpec("toy_routed", dict(prefix=p + "moe.", hidden_size=c["hidden_size"],
                                                 inner_size=c["intermediate_size"], experts=3)),
        norms={"mixer": norm("n1"), "feed_forward": norm("n2")}, prefix=p)
    return ModelSpec(architecture="ToyRoutedLM", hidden_size=c["hidden_size"], vocab_size=c["vocab_size"],
                     embedding_name="embed.weight", layers=(layer,), order=(LayerCall(0, 0),),
                     final_norm=PartSpec("rmsnorm", dict(prefix="final.", width=c["hidden_size"], eps=c["eps"])),
                     final_norm_prefix="final.", head_name="head.weight", max_positions=c["max_position_embeddings"])


class ToySandwichBlock(Block):
    """Another arrangement of a layer, with four norms: each branch is normalised before AND after,
    ``h += post(branch(pre(h)))``.  It does not start with a norm that a product could prepare
    (``first_norm`` stays None), so it takes the stream and a plain branch output as they are."""

    graph_safe = True
    NORM_NAMES = ("pre_mixer", "post_mixer", "pre_ffn", "post_ffn")

    def forward(self, hidden, delta, ctx, next_norm=None):
        if delta is not None:
            K.residual_add(hidden, delta)
        a = self.mixer.forward(self.norms["pre_mixer"].forward(hidden), ctx)
        K.residual_add(hidden, self.norms["post_mixer"].forward(a))
        f = self.feed_forward.forward(self.norms["pre_ffn"].forward(hidden), ctx)
        return hidden, self.norms["post_ffn"].forward(f)


SANDWICH = dict(embedding_scale=6.5, logit_scale=3.0, logit_softcap=3.0)


def sandwich_spec(c):
    layers = []
    for i in range(2):
        base = toy_layer(c, i, "gqa_attention")
        p = base.prefix
        norm = lambda n: PartSpec("rmsnorm", dict(prefix=p + n + ".", width=c["hidden_size"], eps=c["eps"]))
        layers.append(LayerSpec(block=PartSpec("toy_sandwich"), mixer=base.mixer, feed_forward=base.feed_forward,
                                norms={n: norm(n) for n in ToySandwichBlock.NORM_NAMES}, prefix=p))
    return ModelSpec(architecture="ToySandwichLM", hidden_size=c["hidden_size"], vocab_size=c["vocab_size"],
                     embedding_name="embed.weight", layers=tuple(layers), order=(LayerCall(0, 0), LayerCall(1, 1)),
                     final_norm=PartSpec("rmsnorm", dict(prefix="final.", width=c["hidden_size"], eps=c["eps"])),
                     final_norm_prefix="final.", head_name="head.weight", max_positions=c["max_position_embeddings"],
                     **SANDWICH)


@pytest.fixture(scope="module", autouse=True)
def registered():
    BLOCKS.register("toy_sandwich", ToySandwichBlock, replace=True)
    register_architecture("ToySandwichLM", dict, sandwich_spec, replace=True)
    MIXERS.register("toy_decay", ToyDecayMixer, replace=True)
    MIXERS.register("toy_latent", ToyLatentMixer, replace=True)
    MIXERS.register("toy_blockwise_decay", ToyBlockwiseDecayMixer, replace=True)
    register_architecture("ToyBlockwiseLM", dict, toy_spec(
        "ToyBlockwiseLM", ["toy_blockwise_decay", "gqa_attention"], [LayerCall(0, 0), LayerCall(1, 1)]), replace=True)
    register_architecture("ToyLatentLM", dict, toy_spec(
        "ToyLatentLM", ["toy_latent", "gqa_attention", "toy_latent"],
        [LayerCall(0, 0), LayerCall(1, 1), LayerCall(2, 2)]), replace=True)
    POSITION_ENCODINGS.register("toy_neighbour_rotary", ToyNeighbourRotary, replace=True)
    FEED_FORWARDS.register("toy_routed", ToyRoutedFFN, replace=True)
    register_architecture("ToyRoutedLM", dict, routed_spec, replace=True)
    register_architecture("ToyStateLM", dict, toy_spec(
        "ToyStateLM", ["toy_decay", "gqa_attention"], [LayerCall(0, 0), LayerCall(1, 1)]), replace=True)
    register_architecture("ToyStateOnlyLM", dict, toy_spec(
        "ToyStateOnlyLM", ["toy_decay", "toy_decay"], [LayerCall(0, 0), LayerCall(1, 1)]), replace=True)
    register_architecture("ToyOrderLM", dict, toy_spec(
        "ToyOrderLM", ["gqa_attention", "gqa_attention"],
        [LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2), LayerCall(1, 1, writes_cache=False)]), replace=True)
    yield
    MIXERS.unregister("toy_decay")
    MIXERS.unregister("toy_latent")
    MIXERS.unregister("toy_blockwise_decay")
    BLOCKS.unregister("toy_sandwich")
    POSITION_ENCODINGS.unregister("toy_neighbour_rotary")
    FEED_FORWARDS.unregister("toy_routed")


# ---- plain references, from the plain implementation's parts ---------------------------
def ref_ffn(c, W, p, h):
    x = plain.rms_norm(h, W[p + "n2.weight"], c["eps"])
    return h + plain.swiglu(x, W[p + "ffn.gate_proj.weight"], W[p + "ffn.up_proj.weight"], W[p + "ffn.down_proj.weight"])


def ref_qkv(c, W, p, x, T):
    inv = plain.rope_inv_freq(c["head_dim"], c["theta"], None)
    cos, sin = plain.rope_cos_sin(range(T), inv)
    q = plain.apply_rope(plain.linear(x, W[p + "attn.q_proj.weight"]).view(T, c["num_heads"], c["head_dim"]), cos, sin)
    k = plain.apply_rope(plain.linear(x, W[p + "attn.k_proj.weight"]).view(T, c["num_kv_heads"], c["head_dim"]), cos, sin)
    v = plain.linear(x, W[p + "attn.v_proj.weight"]).view(T, c["num_kv_heads"], c["head_dim"])
    return q, k, v


def ref_attn_layer(c, W, i, h, kv=None):
    """One attention layer; with ``kv`` it attends to the given keys and values instead of its own."""
    p, T = f"blocks.{i}.", h.shape[0]
    x = plain.rms_norm(h, W[p + "n1.weight"], c["eps"])
    q, k, v = ref_qkv(c, W, p, x, T)
    if kv is not None:
        k, v = kv
    o = plain.causal_gqa_attention(q, k, v, 1 / math.sqrt(c["head_dim"])).reshape(T, -1)
    return ref_ffn(c, W, p, h + plain.linear(o, W[p + "attn.o_proj.weight"])), (k, v)


def ref_state_model(c, W, toks):
    h = W["embed.weight"][torch.tensor(toks)]
    x = plain.rms_norm(h, W["blocks.0.n1.weight"], c["eps"])
    u = x @ W["blocks.0.mix.in.weight"].t()
    s, ys = torch.zeros(c["state_size"]), []
    for t in range(len(toks)):
        s = DECAY * s + u[t]
        ys.append(s)
    h = ref_ffn(c, W, "blocks.0.", h + torch.stack(ys) @ W["blocks.0.mix.out.weight"].t())
    h, _ = ref_attn_layer(c, W, 1, h)
    return plain.rms_norm(h, W["final.weight"], c["eps"]) @ W["head.weight"].t()


def ref_order_model(c, W, toks):
    h = W["embed.weight"][torch.tensor(toks)]
    h, _ = ref_attn_layer(c, W, 0, h)
    h, kv1 = ref_attn_layer(c, W, 1, h)
    h, _ = ref_attn_layer(c, W, 0, h)            # the same weights again, keys and values of its own
    h, _ = ref_attn_layer(c, W, 1, h, kv=kv1)    # reads what the second call cached, writes nothing
    return plain.rms_norm(h, W["final.weight"], c["eps"]) @ W["head.weight"].t()


def load_plain(d):
    from safetensors.torch import load_file
    import os
    return {k: v.float() for k, v in load_file(os.path.join(d, "model.safetensors")).items()}


def err(got, ref):
    return float((got.cpu() - ref).abs().max() / ref.abs().max())


@pytest.mark.parametrize("dtype, tol", [("float32", 3e-5), ("bfloat16", 2e-2)])
def test_toy_mixer_with_state_is_registered_built_and_stepped(dtype, tol, tmp_path, gpu):
    c = toy_config("ToyStateLM", "bfloat16")
    d = write_random_model(str(tmp_path / "toy"), c, seed=5)
    W = load_plain(d)
    eng = Engine(d, EngineOptions(dtype=dtype, max_seqs=2, max_seq_len=128, cache_tokens=256))
    assert eng.graphs is None                         # the toy mixer does not claim to be graph safe
    assert len(eng.cache.groups) == 1 and list(eng.cache.state) == [0]
    rng = np.random.default_rng(0)
    a = [int(t) for t in rng.integers(0, 97, 50)]
    b = [int(t) for t in rng.integers(0, 97, 23)]
    ra, rb = ref_state_model(c, W, a), ref_state_model(c, W, b)
    # whole
    assert err(eng.step([StepEntry("a", a, list(range(50)))]), ra) <= tol
    eng.release("a")
    # portions of a beside single tokens of b; the state of each sits in its own seat
    rows_a, rows_b, ia, ib = [], [], 0, 0
    for n in (7, 2, 16, 1, 1, 5, 18):
        step = [StepEntry("a", a[ia:ia + n], list(range(n)))]
        if ib < len(b):
            step.append(StepEntry("b", [b[ib]], [0]))
        out = eng.step(step).cpu()
        rows_a.append(out[:n])
        if ib < len(b):
            rows_b.append(out[n:])
            ib += 1
        ia += n
    assert ia == 50
    assert err(torch.cat(rows_a), ra) <= tol and err(torch.cat(rows_b), rb[:ib]) <= tol
    # seats are reused: a newcomer must find a zeroed state, not its predecessor's
    eng.release("a")
    eng.release("b")
    assert err(eng.step([StepEntry("c", b, list(range(23)))]), rb) <= tol
    eng.cache.check()


def ref_latent_layer(c, W, i, h, cache_dtype):
    p, w = f"blocks.{i}.", c["latent_size"]
    x = plain.rms_norm(h, W[p + "n1.weight"], c["eps"])
    cs = (x @ W[p + "lat.c.weight"].t()).to(cache_dtype).float()         # the cache stores the latent in its type
    q, g = x @ W[p + "lat.q.weight"].t(), 1 + torch.tanh(x @ W[p + "lat.g.weight"].t())[:, 0]
    T = h.shape[0]
    scores = (q @ cs.t() / math.sqrt(w)).masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), float("-inf"))
    y = (torch.softmax(scores, dim=-1) * g[None, :]) @ cs
    return ref_ffn(c, W, p, h + y @ W[p + "lat.o.weight"].t())


# (bfloat16: three layers of N(0, 1 / sqrt(in)) matrices; rounding every op's output to bfloat16 moves
# the plain two-layer models' logits by 1.0-1.5 % of their scale, so 3 % here; the 32-bit run is the
# one that would show a wrong page or a wrong array)
@pytest.mark.parametrize("dtype, tol", [("float32", 3e-5), ("bfloat16", 3e-2)])
def test_a_mixer_whose_cache_entry_is_one_vector_per_token(dtype, tol, tmp_path, gpu):
    """The cache manager allocates what a mixer's description says - here a latent vector of 12
    elements and one 32-bit number per token, pages ``[page, 12]`` and ``[page, 1]`` - beside an
    attention layer's keys and values, which form a group of their own with its own pool and block
    table; the engine sizes the pool from the same description (no pool size is given).  Whole,
    in portions beside another request's decoded tokens, and on pages that were used before."""
    c = toy_config("ToyLatentLM", "bfloat16")
    d = write_random_model(str(tmp_path / "toy"), c, seed=31, gain=1.0)
    W = load_plain(d)
    page = 8
    eng = Engine(d, EngineOptions(dtype=dtype, max_seqs=2, max_seq_len=96, page_size=page))
    assert eng.graphs is None
    elem = 4 if dtype == "float32" else 2
    groups = {tuple(a.name for a in g.spec.arrays): g for g in eng.cache.groups}
    assert sorted(groups) == [("k", "v"), ("latent", "gain")]
    lat, att = groups[("latent", "gain")], groups[("k", "v")]
    assert lat.slot_ids == [0, 2] and att.slot_ids == [1]
    assert lat.arrays["latent"].shape == (2, lat.num_pages, page, 12) and lat.arrays["gain"].dtype == torch.float32
    assert att.arrays["v"].shape == (1, att.num_pages, 2, 16, page)
    assert att.arrays["k"].shape == (1, att.num_pages, 2, 16 // 8, page, 8)       # a key in chunks of 8 elements
    assert eng.cache.page_bytes() == page * (2 * (12 * elem + 4) + 2 * 2 * 16 * elem)
    assert lat.num_pages == 2 * 96 // page            # every seat at its longest: nothing more is worth having

    def ref(toks):
        h = W["embed.weight"][torch.tensor(toks)]
        h = ref_latent_layer(c, W, 0, h, eng.dtype)
        h, _ = ref_attn_layer(c, W, 1, h)
        h = ref_latent_layer(c, W, 2, h, eng.dtype)
        return plain.rms_norm(h, W["final.weight"], c["eps"]) @ W["head.weight"].t()

    rng = np.random.default_rng(6)
    a = [int(t) for t in rng.integers(0, 97, 61)]
    b = [int(t) for t in rng.integers(0, 97, 30)]
    ra, rb = ref(a), ref(b)
    assert err(eng.step([StepEntry("w", a, list(range(61)))]), ra) <= tol
    eng.release("w")
    reused_before = sum(g.pool.reuses for g in eng.cache.groups)
    rows_a, rows_b, ia, ib = [], [], 0, 0
    for n in (7, 2, 16, 1, 1, 5, 29):
        step = [StepEntry("a", a[ia:ia + n], list(range(n)))]
        if ib < len(b):
            step.append(StepEntry("b", [b[ib]], [0]))
        out = eng.step(step).cpu()
        rows_a.append(out[:n])
        if ib < len(b):
            rows_b.append(out[n:])
            ib += 1
        ia += n
    assert ia == 61 and err(torch.cat(rows_a), ra) <= tol and err(torch.cat(rows_b), rb[:ib]) <= tol
    assert sum(g.pool.reuses for g in eng.cache.groups) > reused_before       # on pages the first request gave back
    eng.cache.check()


def test_a_model_that_keeps_no_keys_at_all(tmp_path, gpu):
    """Two layers of the stateful toy mixer and no attention: the cache manager has no paged group,
    only state slots; the pool is sized from nothing, admission asks no group for pages, and the
    serving loop generates through the same scheduler."""
    from kv_cache_optimization_for_llm_amd.engine.runner import Runner, ServeOptions
    c = toy_config("ToyStateOnlyLM", "bfloat16")
    d = write_random_model(str(tmp_path / "toy"), c, seed=17, gain=1.0)
    W = load_plain(d)

    def ref(toks):
        h = W["embed.weight"][torch.tensor(toks)]
        for i in range(2):
            p = f"blocks.{i}."
            u = plain.rms_norm(h, W[p + "n1.weight"], c["eps"]) @ W[p + "mix.in.weight"].t()
            s, ys = torch.zeros(c["state_size"]), []
            for t in range(len(toks)):
                s = DECAY * s + u[t]
                ys.append(s)
            h = ref_ffn(c, W, p, h + torch.stack(ys) @ W[p + "mix.out.weight"].t())
        return plain.rms_norm(h, W["final.weight"], c["eps"]) @ W["head.weight"].t()

    eng = Engine(d, EngineOptions(dtype="float32", max_seqs=2, max_seq_len=96))       # no pool size given
    assert eng.cache.groups == [] and sorted(eng.cache.state) == [0, 1]
    rng = np.random.default_rng(4)
    toks = [int(t) for t in rng.integers(0, 97, 40)]
    want = ref(toks)
    rows, i = [], 0
    for n in (11, 1, 1, 20, 7):
        rows.append(eng.step([StepEntry("p", toks[i:i + n], list(range(n)))]).cpu())
        i += n
    assert err(torch.cat(rows), want) <= 3e-5
    eng.release("p")
    # generation: three requests through two seats; greedy tokens are the plain model's
    runner = Runner(eng, ServeOptions(ignore_eos=True, max_batch_tokens=32, chunk_size=16))
    prompts = [[int(t) for t in rng.integers(0, 97, n)] for n in (5, 33, 18)]
    ids = [runner.submit(p, 6) for p in prompts]
    out = {i: [] for i in ids}
    for ev in runner.run_until_idle():
        if ev.kind == "token":
            out[ev.request_id].append(ev.token)
    for rid, p in zip(ids, prompts):
        seq = list(p)
        for tok in out[rid]:
            assert tok == int(ref(seq)[-1].argmax())
            seq.append(tok)
        assert len(out[rid]) == 6
    eng.cache.check()
    assert eng.cache.free_seats == 2


def test_the_scheduler_cuts_prompts_where_a_mixer_says_it_can_be_cut(tmp_path, gpu):
    """A model with a mixer that takes portions only up to multiples of four positions, beside an
    attention layer that takes any cut: the serving loop asks the model and cuts prompts there
    (token budget 23, portions of at most 10 tokens: 8 at a time), a prompt's last portion ends
    where the prompt ends, and what is generated is what the same weights generate under the mixer
    that takes any cut."""
    from kv_cache_optimization_for_llm_amd.engine.runner import Runner, ServeOptions
    c = toy_config("ToyBlockwiseLM", "float32")
    d = write_random_model(str(tmp_path / "toy"), c, seed=23, gain=1.0)
    c2 = dict(c, architectures=["ToyStateLM"])
    d2 = write_random_model(str(tmp_path / "toy2"), c2, seed=23, gain=1.0)
    rng = np.random.default_rng(9)
    prompts = [[int(t) for t in rng.integers(0, 97, n)] for n in (3, 30, 17, 41)]
    results = []
    for folder in (d, d2):
        eng = Engine(folder, EngineOptions(dtype="float32", max_seqs=3, max_seq_len=96, cache_tokens=512))
        runner = Runner(eng, ServeOptions(ignore_eos=True, max_batch_tokens=23, chunk_size=10))
        if folder == d:
            assert eng.model.portion_multiple == 4 and runner.scheduler.portion_multiple == 4
            ToyBlockwiseDecayMixer.cuts.clear()
        else:
            assert eng.model.portion_multiple == 1
        ids = [runner.submit(p, 5) for p in prompts]
        out = {i: [] for i in ids}
        for ev in runner.run_until_idle():
            if ev.kind == "token":
                out[ev.request_id].append(ev.token)
        results.append([out[i] for i in ids])
        eng.cache.check()
    assert results[0] == results[1] and all(len(g) == 5 for g in results[0])
    cuts = ToyBlockwiseDecayMixer.cuts
    lengths = {len(p) for p in prompts}
    assert cuts and all(start % 4 == 0 and ((start + n) % 4 == 0 or start + n in lengths) for start, n in cuts), cuts
    assert any((start + n) % 4 == 0 and n == 8 for start, n in cuts)


@pytest.mark.parametrize("dtype, tol", [("float32", 3e-5), ("bfloat16", 2e-2)])
def test_run_order_names_a_layer_twice_and_shares_a_cache(dtype, tol, tmp_path, gpu):
    c = toy_config("ToyOrderLM", "bfloat16")
    d = write_random_model(str(tmp_path / "toy"), c, seed=9)
    W = load_plain(d)
    eng = Engine(d, EngineOptions(dtype=dtype, max_seqs=2, max_seq_len=128, cache_tokens=256))
    assert len(eng.cache.groups) == 1 and eng.cache.groups[0].slot_ids == [0, 1, 2]
    rng = np.random.default_rng(1)
    toks = [int(t) for t in rng.integers(0, 97, 70)]
    ref = ref_order_model(c, W, toks)
    assert err(eng.step([StepEntry("w", toks, list(range(70)))]), ref) <= tol
    rows, i = [], 0
    for n in (9, 1, 1, 30, 2, 27):
        rows.append(eng.step([StepEntry("p", toks[i:i + n], list(range(n)))]).cpu())
        i += n
    assert err(torch.cat(rows), ref) <= tol


def ref_routed_model(c, W, toks):
    """Plain counterpart of ToyRoutedLM; also returns, per token, how decisive the routing was."""
    T, d, p = len(toks), c["head_dim"], "blocks.0."
    h = W["embed.weight"][torch.tensor(toks)]
    x = plain.rms_norm(h, W[p + "n1.weight"], c["eps"])
    inv = 1.0 / (c["theta"] ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
    ang = torch.arange(T, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]

    def rot(t, heads):
        t = t.view(T, heads, d // 2, 2)
        a, b = t[..., 0], t[..., 1]
        return torch.stack([a * cos - b * sin, a * sin + b * cos], dim=-1).view(T, heads, d)
    q = rot(plain.linear(x, W[p + "attn.q_proj.weight"]), c["num_heads"])
    k = rot(plain.linear(x, W[p + "attn.k_proj.weight"]), c["num_kv_heads"])
    v = plain.linear(x, W[p + "attn.v_proj.weight"]).view(T, c["num_kv_heads"], d)
    o = plain.causal_gqa_attention(q, k, v, 1 / math.sqrt(d)).reshape(T, -1)
    h = h + plain.linear(o, W[p + "attn.o_proj.weight"])
    x = plain.rms_norm(h, W[p + "n2.weight"], c["eps"])
    logits = x @ W[p + "moe.router.weight"].t() * ROUTER_GAIN
    prob = torch.softmax(logits, dim=-1)
    pe, e = prob.max(dim=-1)
    y = torch.stack([torch.relu(x[t] @ W[p + "moe.w1"][e[t]].t()) @ W[p + "moe.w2"][e[t]].t() for t in range(T)])
    h = h + y * pe[:, None]
    top2 = logits.topk(2, dim=-1).values
    return plain.rms_norm(h, W["final.weight"], c["eps"]) @ W["head.weight"].t(), top2[:, 0] - top2[:, 1], e


@pytest.mark.parametrize("dtype, tol", [("float32", 3e-5), ("bfloat16", 2e-2)])
def test_another_position_encoding_and_a_routed_feed_forward(dtype, tol, tmp_path, gpu):
    c = toy_config("ToyRoutedLM", "bfloat16")
    d = write_random_model(str(tmp_path / "toy"), c, seed=13)
    W = load_plain(d)
    eng = Engine(d, EngineOptions(dtype=dtype, max_seqs=2, max_seq_len=128, cache_tokens=256))
    assert eng.graphs is None                         # the routed feed-forward is not graph safe
    rng = np.random.default_rng(2)
    toks = [int(t) for t in rng.integers(0, 97, 60)]
    ref, gap, chosen = ref_routed_model(c, W, toks)
    assert len(set(chosen.tolist())) == 3             # every expert is used
    # a token whose two best experts are nearly tied may go either way in bfloat16
    sure = gap > (0.0 if dtype == "float32" else 0.5)
    assert sure.float().mean() > 0.8
    whole = eng.step([StepEntry("w", toks, list(range(60)))]).cpu()
    assert err(whole[sure], ref[sure]) <= tol
    # in portions and token by token (few rows: the attention's products may fuse, its neighbours do not)
    rows, i = [], 0
    for n in (5, 1, 1, 20, 2, 1, 30):
        rows.append(eng.step([StepEntry("p", toks[i:i + n], list(range(n)))]).cpu())
        i += n
    assert err(torch.cat(rows)[sure], ref[sure]) <= tol
    eng.cache.check()


def ref_sandwich_model(c, W, toks):
    T, eps = len(toks), c["eps"]
    h = W["embed.weight"][torch.tensor(toks)] * SANDWICH["embedding_scale"]
    for i in range(2):
        p = f"blocks.{i}."
        x = plain.rms_norm(h, W[p + "pre_mixer.weight"], eps)
        q, k, v = ref_qkv(c, W, p, x, T)
        o = plain.causal_gqa_attention(q, k, v, 1 / math.sqrt(c["head_dim"])).reshape(T, -1)
        h = h + plain.rms_norm(plain.linear(o, W[p + "attn.o_proj.weight"]), W[p + "post_mixer.weight"], eps)
        x = plain.rms_norm(h, W[p + "pre_ffn.weight"], eps)
        f = plain.swiglu(x, W[p + "ffn.gate_proj.weight"], W[p + "ffn.up_proj.weight"], W[p + "ffn.down_proj.weight"])
        h = h + plain.rms_norm(f, W[p + "post_ffn.weight"], eps)
    raw = plain.rms_norm(h, W["final.weight"], eps) @ W["head.weight"].t()
    logits = raw * SANDWICH["logit_scale"]
    return SANDWICH["logit_softcap"] * torch.tanh(logits / SANDWICH["logit_softcap"]), float(raw.abs().max())


@pytest.mark.parametrize("dtype, tol", [("float32", 3e-5), ("bfloat16", 2e-2)])
def test_a_block_with_four_norms_and_constants_on_embedding_and_logits(dtype, tol, tmp_path, gpu):
    """A layer arrangement with norms after its branches too, a multiplier on the embeddings, a
    scale and a soft cap on the logits: a block class and a ModelSpec in this file, nothing changed
    in the framework.  Decoded tokens run from captured graphs (the toy block says it may)."""
    c = toy_config("ToySandwichLM", "bfloat16")
    d = write_random_model(str(tmp_path / "toy"), c, seed=21, gain=1.0)
    W = load_plain(d)
    eng = Engine(d, EngineOptions(dtype=dtype, max_seqs=2, max_seq_len=128, cache_tokens=256))
    assert (eng.graphs is not None) == (dtype == "bfloat16")
    rng = np.random.default_rng(3)
    toks = [int(t) for t in rng.integers(0, 97, 64)]
    ref, raw_scale = ref_sandwich_model(c, W, toks)
    assert ref.abs().max() > 0.8 * SANDWICH["logit_softcap"] and ref.abs().max() <= SANDWICH["logit_softcap"]
    # A rounding error of the head's product is a fraction of ITS scale (raw_scale); the logit scale
    # multiplies it, the cap (slope at most 1) does not shrink it, but the cap does shrink the scale
    # the result is measured by, to logit_softcap.
    tol = tol * max(1.0, SANDWICH["logit_scale"] * raw_scale / SANDWICH["logit_softcap"])
    assert err(eng.step([StepEntry("w", toks, list(range(64)))]), ref) <= tol
    rows, i = [], 0
    for n in (9, 30, 2) + (1,) * 23:
        rows.append(eng.step([StepEntry("p", toks[i:i + n], list(range(n)))]).cpu().clone())
        i += n
    assert i == 64 and err(torch.cat(rows), ref) <= tol
    if eng.graphs is not None:
        assert eng.graphs.replays > 0
    # the arrangement is checked against the names it is given
    with pytest.raises(ValueError) as e:
        ToySandwichBlock(None, None, {"pre_mixer": None})
    assert "post_ffn" in str(e.value)


def test_garbage_of_an_earlier_engine_is_not_collected_inside_a_graph_capture(tmp_path, gpu):
    """An engine that has become unreachable (pinned block tables, events, captured graphs) is
    freed by Python's collector at some later allocation - also one made while the next engine
    captures a decode graph, where freeing such things is forbidden and fails inside a destructor.
    The capture keeps the collector off: with a collector set to run at every few allocations, a
    second engine captures and replays its graphs next to the garbage of a first."""
    import gc
    from conftest import TINY
    cfg = TINY["A"][0]
    write_random_model(str(tmp_path / "m"), cfg, 2)
    prompt = [3, 1, 4, 1, 5, 9, 2, 6]

    def decode_some(engine, name):
        logits = engine.step([StepEntry(name, prompt, [len(prompt) - 1])])
        tok = int(logits[0].argmax())
        out = [tok]
        for _ in range(6):                                    # the same shape again and again: warm-up, capture, replays
            logits = engine.step([StepEntry(name, [tok], [0])])
            tok = int(logits[0].argmax())
            out.append(tok)
        engine.release(name)
        return out

    first = Engine(str(tmp_path / "m"), EngineOptions(dtype="bfloat16", max_seqs=2, max_seq_len=64))
    want = decode_some(first, "a")
    assert first.graphs.captures >= 1
    ring = [first]
    ring.append(ring)                                         # a cycle: only the collector can free it
    del first, ring
    old = gc.get_threshold()
    gc.set_threshold(5, 2, 2)
    try:
        second = Engine(str(tmp_path / "m"), EngineOptions(dtype="bfloat16", max_seqs=2, max_seq_len=64))
        got = decode_some(second, "b")
        assert second.graphs.captures >= 1 and second.graphs.replays >= 1
    finally:
        gc.set_threshold(*old)
    assert got == want
