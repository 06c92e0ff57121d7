"""Seeded random configurations (head sizes from 8 to 256, any number of heads and groups, widths,
intermediate sizes and vocabularies that are no powers of two, several page sizes) replayed in
process the way bin/trace_run drives the engine, against the plain implementation."""
import numpy as np
import pytest

import plain_llama as plain
import replay_util as ru
from kv_cache_optimization_for_llm_amd.engine.batch import StepEntry
from kv_cache_optimization_for_llm_amd.engine.engine import Engine, EngineOptions
from kv_cache_optimization_for_llm_amd.weights.random_init import write_random_model

pytestmark = pytest.mark.gpu
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def random_config(rng):
    d = int(rng.choice([8, 16, 24, 32, 40, 48, 64, 80, 96, 112, 128, 160, 192, 256]))
    nkv = int(rng.integers(1, 5))
    nq = nkv * int(rng.integers(1, 6))
    hidden = int(rng.choice([nq * d, 2 * int(rng.integers(17, 200)), 8 * int(rng.integers(5, 60)),
                             32 * int(rng.integers(2, 24))]))
    inter = int(rng.choice([2 * int(rng.integers(9, 300)), 8 * int(rng.integers(3, 100)),
                            32 * int(rng.integers(2, 40)), int(rng.integers(17, 400))]))
    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=int(rng.integers(37, 3000)),
               hidden_size=hidden, intermediate_size=inter, num_hidden_layers=int(rng.integers(1, 4)),
               num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d,
               rms_norm_eps=float(rng.choice([1e-5, 1e-6, 3e-4])),
               rope_theta=float(rng.choice([10000.0, 500000.0, 1234.5])), max_position_embeddings=1024,
               tie_word_embeddings=bool(rng.integers(2)), hidden_act="silu", torch_dtype="bfloat16")
    if rng.integers(2):
        cfg["rope_scaling"] = dict(rope_type="llama3", factor=float(rng.choice([2.0, 8.0, 32.0])),
                                   low_freq_factor=1.0, high_freq_factor=float(rng.choice([2.0, 4.0])),
                                   original_max_position_embeddings=int(rng.choice([64, 256, 8192])))
    return cfg


def replay(model_dir, dtype, steps, page):
    unit = max(64, page)
    pool = ru.max_live_tokens(steps, unit)
    eng = Engine(model_dir, EngineOptions(dtype=dtype, page_size=page, cache_tokens=pool, max_seqs=8,
                                          max_seq_len=pool))
    pos, rows = {}, {}
    for st in steps:
        logits = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in st["entries"]]).float().cpu().numpy()
        wanted = [(e["id"], pos.get(e["id"], 0) + i) for e in st["entries"] for i in e["want"]]
        for e in st["entries"]:
            pos[e["id"]] = pos.get(e["id"], 0) + len(e["tokens"])
        for rid in st["end"]:
            pos.pop(rid)
            eng.release(rid)
        rows.update(zip(wanted, logits))
    eng.cache.check()
    return rows


def wide_group_config(nq, nkv, d):
    """More than 16 query heads on one kv head: a decoded token is then more than one tile of 16
    query rows for the matrix-core attention kernel."""
    return dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=211, hidden_size=nq * d // 4,
                intermediate_size=320, num_hidden_layers=2, num_attention_heads=nq, num_key_value_heads=nkv,
                head_dim=d, rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=1024,
                tie_word_embeddings=False, hidden_act="silu", torch_dtype="bfloat16")


def wide_config(hidden, inter, nq, nkv, d, tied):
    """Widths that are multiples of 512: one or two decoded tokens take the matrix-vector kernel
    (with its rotation epilogue where half a head is a multiple of the pairs a wavefront works on,
    whatever the attention kernel needs), the other row counts the few-rows kernel or the library."""
    return dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=1003, hidden_size=hidden,
                intermediate_size=inter, num_hidden_layers=2, num_attention_heads=nq, num_key_value_heads=nkv,
                head_dim=d, rms_norm_eps=1e-5, rope_theta=10000.0, max_position_embeddings=1024,
                tie_word_embeddings=tied, hidden_act="silu", torch_dtype="bfloat16")


WIDE = {"512 wide, head 64": (512, 1024, 8, 2, 64, True), "1024 wide, head 24": (1024, 1000, 6, 3, 24, False),
        "1536 wide, head 96": (1536, 512, 4, 1, 96, True)}


@pytest.mark.parametrize("case", list(range(12)) + ["32 heads on 1", "40 heads on 2", "17 heads on 1"] + list(WIDE))
def test_random_configuration_under_two_cuts(case, tmp_path, gpu):
    if case in WIDE:
        rng = np.random.default_rng(sum(WIDE[case][:5]))
        cfg, case = wide_config(*WIDE[case]), WIDE[case][0]
    elif isinstance(case, str):
        nq, nkv, d = {"32 heads on 1": (32, 1, 64), "40 heads on 2": (40, 2, 32), "17 heads on 1": (17, 1, 16)}[case]
        rng = np.random.default_rng(nq * 100 + d)
        cfg, case = wide_group_config(nq, nkv, d), nq
    else:
        rng = np.random.default_rng(4000 + case)
        cfg = random_config(rng)
    page = int(rng.choice([16, 16, 8, 32, 4]))
    lengths = [int(x) for x in rng.integers(1, 200, 5)]
    model_dir = write_random_model(str(tmp_path / "m"), cfg, case)
    pcfg, W = plain.load_model_dir(model_dir)
    reqs = {f"r{i}": [int(t) for t in rng.integers(0, cfg["vocab_size"], n)] for i, n in enumerate(lengths)}
    ref = {rid: plain.logits_all(pcfg, W, t).numpy() for rid, t in reqs.items()}
    for dtype in ("float32", "bfloat16"):
        for what, steps in (("mixed", ru.mixed(reqs, seed=case)), ("tail decoded", ru.tail_decoded(reqs))):
            rows = replay(model_dir, dtype, steps, page)
            for rid, toks in reqs.items():
                scale = float(np.abs(ref[rid]).max())
                for p in range(len(toks)):
                    err = float(np.abs(rows[(rid, p)] - ref[rid][p]).max()) / scale
                    assert err <= TOL[dtype], (f"{cfg} page {page}: {what} [{dtype}] differs by {err:.3g} of the "
                                               f"logits' scale at {(rid, p)}")
