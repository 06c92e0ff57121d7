"""The engine through its Python entry point: generation, long decoding, cache modes, preemption,
HIP-graph replays, and a toy architecture with a stateful mixer registered from this file."""
import json
import os

import numpy as np
import pytest
import torch

import plain_llama as plain
from conftest import TINY
from kv_cache_optimization_for_llm_amd.engine.batch import StepEntry
from kv_cache_optimization_for_llm_amd.engine.engine import CacheExhausted, Engine, EngineOptions
from kv_cache_optimization_for_llm_amd.engine.runner import LLM, ServeOptions

pytestmark = pytest.mark.gpu
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


@pytest.fixture(scope="module")
def model_dirs(sharp_model_dirs):
    """Generation is tested on the weights whose attention rows are not uniform (conftest)."""
    return sharp_model_dirs


def prompts_for(name, lengths, seed=1):
    rng = np.random.default_rng(seed)
    v = TINY[name][0]["vocab_size"]
    return [[int(t) for t in rng.integers(0, v, n)] for n in lengths]


def check_choices(cfg, W, prompt, got, dtype, temperature=0.0, seed=0, key=0, penalty=1.0):
    """Every generated token is what the plain model would pick given the same prefix: exactly
    for float32; for bfloat16 the pick must be within rounding of the plain model's best."""
    ref = plain.logits_all(cfg, W, prompt + got).double().numpy()
    for i, tok in enumerate(got):
        row = ref[len(prompt) - 1 + i]
        if penalty != 1.0 and i > 0:
            row = plain.penalised(row, got[:i], penalty)
        if temperature > 0:
            u = plain.counter_uniform(seed, key, len(prompt) + i)
            want = plain.sample_temperature(row, temperature, u)
            if tok != want:
                w = np.exp((row - row.max()) / temperature)
                cdf = np.cumsum(w) / w.sum()
                lo = cdf[tok - 1] if tok > 0 else 0.0
                slack = 1e-4 if dtype == "float32" else 3e-2
                assert lo - slack <= u <= cdf[tok] + slack, f"token {i}: {tok} is not the draw's token {want}"
        else:
            best = row.max()
            assert row[tok] >= best - TOL[dtype] * np.abs(row).max(), f"token {i}: {tok} is not the best"
            if dtype == "float32":
                assert tok == int(np.argmax(row))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_greedy_generation_through_the_entry_point(name, dtype, model_dirs, gpu):
    cfg, W = plain.load_model_dir(model_dirs[name])
    lengths = {"A": [5, 17, 33], "B": [1, 9, 40, 70], "C": [3, 20, 64], "D": [2, 31, 50]}[name]
    prompts = prompts_for(name, lengths)
    llm = LLM(model_dirs[name], EngineOptions(dtype=dtype, page_size=8 if name == "B" else 16, max_seqs=4,
                                              max_seq_len=128),
              ServeOptions(chunk_size=16 if name == "B" else None, max_batch_tokens=64))
    got, reasons = llm.generate(prompts, max_new_tokens=8, ignore_eos=True, return_reasons=True)
    assert reasons == ["length"] * len(prompts)
    for p, g in zip(prompts, got):
        assert len(g) == 8
        check_choices(cfg, W, p, g, dtype)
    if dtype == "float32":
        assert got == [plain.generate(cfg, W, p, 8) for p in prompts]
    llm.engine.cache.check()
    assert llm.engine.cache.free_seats == 4


@pytest.mark.parametrize("name, batch", [("A", 20), ("C", 40), ("D", 64), ("E", 24), ("F", 40), ("E", 64)])
def test_many_requests_decoding_together(name, batch, model_dirs, gpu, monkeypatch):
    """17 to 64 decoded tokens per step: the shapes of the few-rows products whose waves share X
    through LDS, of the vendor GEMM at few rows and of decode graphs for large batches; at head
    sizes 64 and 128 (E, F) also of the attention kernel that rotates and caches the tokens' keys
    itself.  Every pick must be the plain model's (within bf16 rounding), for every request."""
    from kv_cache_optimization_for_llm_amd.ops import kernels as K
    calls = []
    inside = K.attention_mfma_rope
    monkeypatch.setattr(K, "attention_mfma_rope", lambda *a, **k: (calls.append(1), inside(*a, **k))[1])
    cfg, W = plain.load_model_dir(model_dirs[name])
    rng = np.random.default_rng(7)
    lengths = [int(n) for n in rng.integers(1, 12, batch)]
    prompts = prompts_for(name, lengths, seed=5)
    llm = LLM(model_dirs[name], EngineOptions(dtype="bfloat16", page_size=16, max_seqs=batch, max_seq_len=64),
              ServeOptions(max_batch_tokens=1024))
    got, reasons = llm.generate(prompts, max_new_tokens=10, ignore_eos=True, return_reasons=True)
    assert reasons == ["length"] * batch
    for p, g in zip(prompts, got):
        assert len(g) == 10
        check_choices(cfg, W, p, g, "bfloat16")
    assert llm.engine.graphs.replays > 0
    assert bool(calls) == (name in "EF"), "rotation inside the attention kernel: taken where it should not be, or not where it should"
    llm.engine.cache.check()
    assert llm.engine.cache.free_seats == batch


@pytest.mark.parametrize("lengths", [[520], [700, 530], [1030], [2040]])
def test_one_or_two_requests_decode_without_a_merge_launch(lengths, sharp_model_dirs, tmp_path, gpu, monkeypatch):
    """Model E (512 wide, heads of 64): from 512 keys on the attention kernel leaves the key ranges
    of one or two decoded tokens as partial results - four ranges a workgroup - and the output
    projection's matrix-vector kernel adds them up where it would have read the tokens (up to
    2,048 keys in 16 ranges; one request up to 4,096 keys in 32: the run that starts at 2,040 keys
    crosses into those).  On the weights that spread attention over far keys, every pick against the plain model; eagerly and
    from the decode graph."""
    from kv_cache_optimization_for_llm_amd.ops import kernels as K
    calls = []
    inside = K.gemv_merged
    monkeypatch.setattr(K, "gemv_merged", lambda x, *a, **k: (calls.append(x.parts), inside(x, *a, **k))[1])
    from kv_cache_optimization_for_llm_amd.weights.random_init import write_random_model
    model_dir = sharp_model_dirs["E"]
    if max(lengths) > 2000:                                      # the same model with room for 4,096 positions
        model_dir = write_random_model(str(tmp_path / "e4k"), dict(TINY["E"][0], max_position_embeddings=4096),
                                       TINY["E"][1], gain=1.0)
    cfg, W = plain.load_model_dir(model_dir)
    prompts = prompts_for("E", lengths, seed=11)
    llm = LLM(model_dir, EngineOptions(dtype="bfloat16", page_size=16, max_seqs=2, max_seq_len=2100),
              ServeOptions(max_batch_tokens=2048))
    got = llm.generate(prompts, max_new_tokens=12, ignore_eos=True)
    for p, g in zip(prompts, got):
        assert len(g) == 12
        check_choices(cfg, W, p, g, "bfloat16")
    assert calls and all(2 <= parts <= K.gemv_merge_max_parts(len(lengths)) for parts in calls)
    if lengths == [2040]:
        assert 4 in calls and 8 in calls
    assert llm.engine.graphs.replays > 0
    llm.engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_temperature_sampling_and_penalty_follow_the_plain_sampler(dtype, model_dirs, gpu):
    cfg, W = plain.load_model_dir(model_dirs["B"])
    prompts = prompts_for("B", [1, 9, 40, 70], seed=4)
    llm = LLM(model_dirs["B"], EngineOptions(dtype=dtype, page_size=8, max_seqs=4, max_seq_len=128),
              ServeOptions(chunk_size=16))
    got = llm.generate(prompts, max_new_tokens=10, temperature=0.7, seed=1234, ignore_eos=True)
    for i, (p, g) in enumerate(zip(prompts, got)):
        assert len(g) == 10
        check_choices(cfg, W, p, g, dtype, temperature=0.7, seed=1234, key=i * 8)
    again = llm.generate(prompts, max_new_tokens=10, temperature=0.7, seed=1234, ignore_eos=True)
    other = llm.generate(prompts, max_new_tokens=10, temperature=0.7, seed=99, ignore_eos=True)
    assert again == got and other != got            # a pure function of (seed, request, position)
    pen = llm.generate(prompts[:2], max_new_tokens=10, repetition_penalty=1.15, ignore_eos=True)
    for p, g in zip(prompts, pen):
        check_choices(cfg, W, p, g, dtype, penalty=1.15)


def test_eos_ends_generation_and_is_not_returned(model_dirs, gpu):
    cfg, W = plain.load_model_dir(model_dirs["C"])
    prompt = prompts_for("C", [12])[0]
    free = plain.generate(cfg, W, prompt, 6)
    # make the third generated token the end-of-sequence token
    d = json.load(open(os.path.join(model_dirs["C"], "config.json")))
    import tempfile, shutil
    with tempfile.TemporaryDirectory() as tmp:
        shutil.copy(os.path.join(model_dirs["C"], "model.safetensors"), tmp)
        d["eos_token_id"] = [free[2], 388]
        json.dump(d, open(os.path.join(tmp, "config.json"), "w"))
        llm = LLM(tmp, EngineOptions(dtype="float32", max_seqs=2, max_seq_len=64))
        got, reasons = llm.generate([prompt], max_new_tokens=6, return_reasons=True)
        assert got == [free[:free.index(free[2])]] and reasons == ["eos"]
        got, reasons = llm.generate([prompt], max_new_tokens=6, ignore_eos=True, return_reasons=True)
        assert got == [free] and reasons == ["length"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_ahead_of_the_device_changes_nothing_that_is_emitted(dtype, model_dirs, gpu):
    """The serving loop launches a step before it has seen the previous step's tokens (they stay
    on the device).  Same requests with and without that: same tokens, same reasons - with
    end-of-sequence tokens arriving at different times, more requests than seats, a repetition
    penalty and a temperature."""
    name = "C"
    prompts = prompts_for(name, [12, 3, 40, 25, 7, 18], seed=11)
    d = json.load(open(os.path.join(model_dirs[name], "config.json")))
    import shutil
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        shutil.copy(os.path.join(model_dirs[name], "model.safetensors"), tmp)
        json.dump(d, open(os.path.join(tmp, "config.json"), "w"))
        probe = LLM(tmp, EngineOptions(dtype=dtype, max_seqs=3, max_seq_len=128), ServeOptions(run_ahead=False))
        free = probe.generate(prompts, max_new_tokens=24, ignore_eos=True)
        # end-of-sequence ids that some requests meet early, some late and some never
        d["eos_token_id"] = [free[0][5], free[2][14], free[4][1]]
        json.dump(d, open(os.path.join(tmp, "config.json"), "w"))
        results = {}
        for ahead in (False, True):
            llm = LLM(tmp, EngineOptions(dtype=dtype, max_seqs=3, max_seq_len=128),
                      ServeOptions(run_ahead=ahead, max_batch_tokens=32, chunk_size=16))
            results[ahead] = [
                llm.generate(prompts, max_new_tokens=24, return_reasons=True),
                llm.generate(prompts, max_new_tokens=24, return_reasons=True, temperature=0.9, seed=3,
                             repetition_penalty=1.15),
            ]
            llm.engine.cache.check()
            assert llm.engine.cache.free_seats == 3
        assert results[True] == results[False]
        got, reasons = results[True][0]
        assert "eos" in reasons and "length" in reasons
        eos = set(d["eos_token_id"])
        for g, f, r in zip(got, free, reasons):
            stop = next((i for i, t in enumerate(f) if t in eos), None)
            if dtype == "float32":
                assert g == (f if stop is None else f[:stop]) and r == ("length" if stop is None else "eos")
            assert not eos & set(g)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_workloads_emit_the_same_with_and_without_running_ahead(seed, model_dirs, gpu):
    """Random prompt lengths and output budgets, more requests than seats, so few pages that
    requests are preempted and recomputed, end-of-sequence ids that do occur, a temperature: the
    loop that runs ahead of the device emits, per request, exactly what the synchronous loop does."""
    from kv_cache_optimization_for_llm_amd.engine.runner import Runner
    rng = np.random.default_rng(100 + seed)
    cfg = TINY["A"][0]
    # room for the longest request alone (59 + 39 tokens) and little more: three live ones do not fit
    eng = Engine(model_dirs["A"], EngineOptions(dtype="float32", max_seqs=3, max_seq_len=128, cache_tokens=112))
    requests = [([int(t) for t in rng.integers(0, cfg["vocab_size"], int(rng.integers(1, 60)))],
                 int(rng.integers(3, 40))) for _ in range(9)]
    probe = Runner(eng, ServeOptions(run_ahead=False, ignore_eos=True, temperature=0.8, sampling_seed=seed))
    for p, n in requests:
        probe.submit(p, n)
    seen = [ev.token for ev in probe.run_until_idle() if ev.kind == "token"]
    ids_seen, counts = np.unique(seen, return_counts=True)
    # ids that the requests do sample, but rarely: some requests stop early, most run on
    eos = [int(t) for t in ids_seen[np.argsort(counts, kind="stable")[:3]]]
    results = {}
    for ahead in (False, True):
        runner = Runner(eng, ServeOptions(run_ahead=ahead, temperature=0.8, sampling_seed=seed,
                                          max_batch_tokens=48, chunk_size=16))
        runner.scheduler.eos = frozenset(eos)
        ids = [runner.submit(p, n) for p, n in requests]
        out = {i: [] for i in ids}
        reasons = {}
        for ev in runner.run_until_idle():
            if ev.kind == "token":
                assert ev.request_id not in reasons, "a token after the request was done"
                out[ev.request_id].append(ev.token)
            elif ev.kind in ("done", "rejected"):
                reasons[ev.request_id] = ev.reason
        results[ahead] = (out, reasons, runner.scheduler.preemptions)
        eng.cache.check()
        assert eng.cache.free_seats == 3 and all(g.free_pages() == g.num_pages for g in eng.cache.groups)
    assert results[True][0] == results[False][0] and results[True][1] == results[False][1]
    assert set(results[True][1].values()) <= {"eos", "length"} and len(results[True][1]) == len(requests)
    assert not any(set(eos) & set(toks) for toks in results[True][0].values())
    assert results[False][2] > 0 and results[True][2] > 0                 # pages do run out, for every seed


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(dtype, model_dirs, gpu):
    """300 tokens decoded one by one from a one-token start: crosses many pages and several
    context buckets of the graphs; every position is compared with the plain logits."""
    name = "C"
    cfg, W = plain.load_model_dir(model_dirs[name])
    toks = prompts_for(name, [301], seed=8)[0]
    ref = plain.logits_all(cfg, W, toks).numpy()
    scale = np.abs(ref).max()
    for use_graphs in (True, False):
        eng = Engine(model_dirs[name], EngineOptions(dtype=dtype, max_seqs=2, max_seq_len=320,
                                                     cache_tokens=320, use_graphs=use_graphs))
        worst = 0.0
        for i, t in enumerate(toks):
            row = eng.step([StepEntry("x", [t], [0])]).cpu().numpy()[0]
            worst = max(worst, float(np.abs(row - ref[i]).max() / scale))
        assert worst <= TOL[dtype], f"graphs={use_graphs}: worst error {worst:.3g}"
        if use_graphs and dtype == "bfloat16":
            assert eng.graphs.replays > 250 and eng.graphs.captures >= 2
        eng.release("x")
        eng.cache.check()


def test_graph_replays_equal_eager_steps_with_work_in_between(model_dirs, gpu):
    """Every replay is checked against the same step run eagerly by a second engine; prompt
    portions (eager work) and synchronisations come between the replays."""
    name = "A"
    opts = dict(dtype="bfloat16", max_seqs=4, max_seq_len=256, cache_tokens=1024)
    a = Engine(model_dirs[name], EngineOptions(use_graphs=True, **opts))
    b = Engine(model_dirs[name], EngineOptions(use_graphs=False, **opts))
    rng = np.random.default_rng(0)
    v = TINY[name][0]["vocab_size"]
    for eng in (a, b):
        eng.step([StepEntry(r, [int(t) for t in rng.integers(0, v, n)], []) for r, n in (("p", 20), ("q", 3))])
        rng = np.random.default_rng(0)
    for i in range(40):
        step = [StepEntry("p", [int(rng.integers(v))], [0]), StepEntry("q", [int(rng.integers(v))], [0])]
        la, lb = a.step(step), b.step(step)
        torch.cuda.synchronize()
        # the graph splits the keys for its whole context bucket, the eager step for the context
        # it sees: same arithmetic, another grouping of the sums
        assert (la - lb).abs().max() <= 4e-3 * lb.abs().max(), f"replay {i} differs from the eager step"
        if i % 7 == 3:      # eager work between replays: a prompt portion of a third request
            extra = [StepEntry("r", [int(t) for t in rng.integers(0, v, 5)], [4])]
            assert torch.equal(a.step(extra), b.step(extra))
    assert a.graphs.replays >= 30


def test_portion_graph_replays_equal_eager_steps(gpu, monkeypatch):
    """Steps with prompt portions whose shape comes back run from a graph of that shape: every
    replay is checked against the same step run eagerly by a second engine (whose steps are the
    eager work between the replays), at layer sizes where the vendor library's large-product
    kernels take part; portions alone, portions beside decoded tokens, pages used again.  A
    graph cuts the keys into splits by its context bucket, an eager step by the context it sees:
    here the eager steps are given the bucket too, and then every replay must be bit for bit
    what the eager step gives."""
    import kv_cache_optimization_for_llm_amd.engine.engine as engine_module
    from kv_cache_optimization_for_llm_amd.engine.graphs import context_bucket
    plain_build = engine_module.build_batch

    def build_with_bucket(*args, **kwargs):
        batch = plain_build(*args, **kwargs)
        batch.max_context = context_bucket(batch.max_context)
        return batch
    monkeypatch.setattr(engine_module, "build_batch", build_with_bucket)
    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=1531, hidden_size=2048,
               intermediate_size=8192, num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8,
               head_dim=64, rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=8192,
               tie_word_embeddings=True, hidden_act="silu", torch_dtype="bfloat16")
    opts = dict(dtype="bfloat16", max_seqs=4, max_seq_len=4608, cache_tokens=3 * 4608)
    a = Engine(None, EngineOptions(use_graphs=True, **opts), config_dict=cfg, random_seed=3)
    b = Engine(None, EngineOptions(use_graphs=False, **opts), config_dict=cfg, random_seed=3)
    rng = np.random.default_rng(1)
    toks = lambda n: [int(t) for t in rng.integers(0, 1531, n)]
    n_steps = 0

    def both(step):
        nonlocal n_steps
        la, lb = a.step(step), b.step(step)
        torch.cuda.synchronize()
        assert torch.equal(la, lb), f"step {n_steps} from its graph is not what the eager step gives"
        n_steps += 1

    for round_ in range(2):            # the second round reuses the pages the first gave back
        # three prompts in portions of 512, each alone in its step
        for chunk in range(8):
            for r in ("x", "y", "z"):
                both([StepEntry(r, toks(512), [511] if chunk >= 5 else [])])
        # two of them decode beside portions of a fourth request; then portions of 200 beside three decoding
        for r in ("x",):
            a.release(r), b.release(r)
        for i in range(6):
            both([StepEntry("y", toks(1), [0]), StepEntry("z", toks(1), [0]), StepEntry("w", toks(256), [255])])
        for i in range(5):
            both([StepEntry("y", toks(1), [0]), StepEntry("z", toks(1), [0]), StepEntry("w", toks(1), [0]),
                  StepEntry("x", toks(200), [])])
        for r in ("x", "y", "z", "w"):
            a.release(r), b.release(r)
    a.cache.check(), b.cache.check()
    assert a.portion_graphs.captures >= 4 and a.portion_graphs.replays >= 40, \
        (a.portion_graphs.captures, a.portion_graphs.replays, n_steps)


def test_a_long_prompt_in_portions_takes_the_split_kernels_and_matches_plain(tmp_path, gpu, monkeypatch):
    """A 4,352-token prompt in portions of 1,024, then 256: late portions are few workgroups that
    each walk thousands of keys, so the workgroup attention kernel cuts their keys into ranges
    (and the 256-token portion takes the one-wavefront kernel with two row tiles and key splits);
    with the policy's own thresholds, against the plain model."""
    from kv_cache_optimization_for_llm_amd.ops import kernels as K
    from kv_cache_optimization_for_llm_amd.weights.random_init import write_random_model
    cfg = dict(architectures=["LlamaForCausalLM"], model_type="llama", vocab_size=997, hidden_size=1024,
               intermediate_size=1408, num_hidden_layers=2, num_attention_heads=16, num_key_value_heads=4,
               head_dim=64, rms_norm_eps=1e-5, rope_theta=500000.0, max_position_embeddings=8192,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=2048),
               tie_word_embeddings=True, hidden_act="silu", torch_dtype="bfloat16")
    model_dir = write_random_model(str(tmp_path / "m"), cfg, 77)
    pcfg, W = plain.load_model_dir(model_dir)
    rng = np.random.default_rng(12)
    prompt = [int(t) for t in rng.integers(0, 997, 4352)]
    ref = plain.logits_all(pcfg, W, prompt).numpy()
    seen = {"lds_splits": 0, "wave_splits": 0}
    real_lds, real_mfma = K.attention_lds, K.attention_mfma

    def lds(*a, **kw):
        seen["lds_splits"] += 1 if a[13] > 1 else 0
        return real_lds(*a, **kw)

    def mfma(*a, **kw):
        seen["wave_splits"] += 1 if (a[16] > 1 and a[18] == 2) else 0
        return real_mfma(*a, **kw)
    monkeypatch.setattr(K, "attention_lds", lds)
    monkeypatch.setattr(K, "attention_mfma", mfma)
    eng = Engine(model_dir, EngineOptions(dtype="bfloat16", max_seqs=2, max_seq_len=4608, cache_tokens=4608))
    at, scale = 0, float(np.abs(ref).max())
    for n in (1024, 1024, 1024, 1024, 256):
        want = list(range(0, n, 97)) + [n - 1]
        out = eng.step([StepEntry("p", prompt[at:at + n], want)]).float().cpu().numpy()
        err = float(np.abs(out - ref[[at + i for i in want]]).max()) / scale
        assert err <= TOL["bfloat16"], f"portion at {at}: {err:.3g}"
        at += n
    assert seen["lds_splits"] >= 2 * cfg["num_hidden_layers"] and seen["wave_splits"] >= cfg["num_hidden_layers"], seen
    eng.cache.check()


def test_graphs_kept_are_bounded_and_a_dropped_shape_is_captured_again(model_dirs, gpu):
    """Only so many captured shapes are kept (the least recently used goes first); a shape that
    was dropped and comes back is captured again, and every step still equals the eager step."""
    name = "D"
    opts = dict(dtype="bfloat16", max_seqs=6, max_seq_len=256, cache_tokens=1536)
    a = Engine(model_dirs[name], EngineOptions(use_graphs=True, **opts))
    b = Engine(model_dirs[name], EngineOptions(use_graphs=False, **opts))
    a.graphs.MAX_SHAPES, a.portion_graphs.MAX_SHAPES = 2, 1
    rng = np.random.default_rng(2)
    v = TINY[name][0]["vocab_size"]
    toks = lambda n: [int(t) for t in rng.integers(0, v, n)]
    for eng_step in (lambda st: (a.step(st), b.step(st)),):
        for r in "pqrs":
            eng_step([StepEntry(r, toks(20), [])])
        for i in range(48):
            live = "pqrs"[:1 + (i // 4) % 4]            # batch sizes 1, 2, 3, 4, four steps each, then again
            la, lb = eng_step([StepEntry(r, toks(1), [0]) for r in live])
            torch.cuda.synchronize()
            assert (la - lb).abs().max() <= 4e-3 * lb.abs().max(), f"decode step {i}"
            if i % 3 == 0:                              # two portion shapes, a few steps each, then again
                n = 24 if (i // 6) % 2 == 0 else 40
                for r in ("x", "y"):
                    la, lb = eng_step([StepEntry(r + str(i), toks(n), [n - 1])])
                    torch.cuda.synchronize()
                    assert (la - lb).abs().max() <= 4e-3 * lb.abs().max(), f"portion step {i}"
                    a.release(r + str(i)), b.release(r + str(i))
    assert len(a.graphs.slots) <= 2 and len(a.portion_graphs.slots) <= 1
    assert a.graphs.captures > 4 and a.portion_graphs.captures > 2        # shapes came back after being dropped
    a.cache.check(), b.cache.check()


@pytest.mark.parametrize("run_ahead", [False, True])
def test_serving_with_small_portions_replays_portion_graphs(run_ahead, model_dirs, gpu):
    """A small token budget and portions of 24 tokens: the same step shapes (a portion alone,
    decoded tokens beside a portion) come back again and again and are replayed from graphs, with
    the serving loop one step ahead of the device or not; every token is the plain model's choice."""
    name = "D"
    cfg, W = plain.load_model_dir(model_dirs[name])
    prompts = prompts_for(name, [96, 120, 96, 72, 120, 96, 48, 96], seed=4)
    llm = LLM(model_dirs[name], EngineOptions(dtype="bfloat16", max_seqs=3, max_seq_len=256, cache_tokens=512),
              ServeOptions(chunk_size=24, max_batch_tokens=40, run_ahead=run_ahead))
    got = llm.generate(prompts, max_new_tokens=12, ignore_eos=True)
    for p, g in zip(prompts, got):
        assert len(g) == 12
        check_choices(cfg, W, p, g, "bfloat16")
    pg = llm.engine.portion_graphs
    assert pg.captures >= 2 and pg.replays >= 10, (pg.captures, pg.replays)
    llm.engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_contiguous_mode_gives_the_same_logits(dtype, model_dirs, gpu):
    name = "A"
    cfg, W = plain.load_model_dir(model_dirs[name])
    reqs = {f"r{i}": p for i, p in enumerate(prompts_for(name, [30, 75, 50], seed=2))}
    ref = {r: plain.logits_all(cfg, W, t).numpy() for r, t in reqs.items()}
    eng = Engine(model_dirs[name], EngineOptions(dtype=dtype, cache_mode="contiguous", max_seqs=4,
                                                 max_seq_len=128, cache_tokens=192))
    for r in reqs:
        assert eng.add_request(r, reserve_tokens=len(reqs[r])) is not None or r == "r2"
    assert not eng.has_request("r2")                 # runs of 2 + 8 + 4 pages do not fit 12
    for r in ("r0", "r1"):
        toks = reqs[r]
        rows = [eng.step([StepEntry(r, toks[:20], list(range(20)))]).cpu().numpy()]
        rows += [eng.step([StepEntry(r, [t], [0])]).cpu().numpy() for t in toks[20:]]
        got = np.concatenate(rows)
        assert np.abs(got - ref[r]).max() / np.abs(ref[r]).max() <= TOL[dtype]
    with pytest.raises(CacheExhausted):
        eng.step([StepEntry("r0", [1, 2, 3], [])])   # r0 reserved 30 -> 32 tokens, all used
    eng.release("r0")
    assert eng.add_request("r2", reserve_tokens=50) is not None
    got = eng.step([StepEntry("r2", reqs["r2"], list(range(50)))]).cpu().numpy()
    assert np.abs(got - ref["r2"]).max() / np.abs(ref["r2"]).max() <= TOL[dtype]
    eng.cache.check()
    st = eng.cache.stats()
    assert st["kv_tokens_reserved"] == 128 + 64 and st["kv_tokens_live"] == 75 + 50


@pytest.mark.parametrize("policy", ["max", "pow2", "oracle"])
def test_contiguous_mode_with_a_pool_for_two_makes_the_others_wait(policy, model_dirs, gpu):
    """Five equal requests, a contiguous pool that holds two reservations: through the entry
    point with its default loop (one step ahead of the device), every request gets its full
    budget - the queue head waits while the holders of its room only wait for their last token -
    and the tokens are those of a roomy paged run (``base/src/engine.cu:432-437``: nothing that
    fits is refused)."""
    name = "A"
    prompts = prompts_for(name, [20] * 5, seed=8)
    paged = LLM(model_dirs[name], EngineOptions(dtype="float32", max_seqs=4, max_seq_len=64, cache_tokens=1024))
    want = paged.generate(prompts, max_new_tokens=12, ignore_eos=True)
    tight = LLM(model_dirs[name], EngineOptions(dtype="float32", cache_mode="contiguous", max_seqs=4,
                                                max_seq_len=64, cache_tokens=128),
                ServeOptions(reserve_policy=policy))
    assert tight.serve_options.run_ahead
    got, reasons = tight.generate(prompts, max_new_tokens=12, ignore_eos=True, return_reasons=True)
    assert reasons == ["length"] * 5 and got == want
    st = tight.engine.cache.stats()
    assert st["running"] == 0 and st["kv_tokens_reserved"] == 0
    tight.engine.cache.check()
    # and a request can be ended from outside while others go on
    from kv_cache_optimization_for_llm_amd.engine.runner import Runner
    runner = Runner(paged.engine, ServeOptions(ignore_eos=True))
    ids = [runner.submit(p, 30) for p in prompts[:3]]
    out = {i: [] for i in ids}
    done = {}
    steps = 0
    while not runner.idle():
        evs = runner.step()
        steps += 1
        if steps == 6:
            evs += runner.cancel(ids[1])
        for ev in evs:
            if ev.kind == "token":
                out[ev.request_id].append(ev.token)
            elif ev.kind == "done":
                done[ev.request_id] = (ev.reason, ev.tokens)
    assert done[ids[1]][0] == "cancelled" and done[ids[1]][1] == len(out[ids[1]]) < 30
    assert done[ids[0]] == ("length", 30) and done[ids[2]] == ("length", 30)
    assert runner.live_requests() == []
    paged.engine.cache.check()
    assert paged.engine.cache.free_seats == 4


def test_preempted_requests_finish_with_the_tokens_of_an_unpreempted_run(model_dirs, gpu):
    name = "A"
    prompts = prompts_for(name, [30, 30, 30], seed=6)
    big = LLM(model_dirs[name], EngineOptions(dtype="float32", max_seqs=4, max_seq_len=128, cache_tokens=1024))
    want = big.generate(prompts, max_new_tokens=50, ignore_eos=True)
    assert big.last_runner.scheduler.preemptions == 0
    small = LLM(model_dirs[name], EngineOptions(dtype="float32", max_seqs=4, max_seq_len=128,
                                                cache_tokens=11 * 16))    # 3 x 5 pages do not fit
    got = small.generate(prompts, max_new_tokens=50, ignore_eos=True, temperature=0.0)
    assert small.last_runner.scheduler.preemptions > 0 and got == want
    small.engine.cache.check()
    assert small.engine.cache.stats()["pages_reused"] > 0
    # with temperature too: draws depend on (seed, request, position) only
    want_t = big.generate(prompts, max_new_tokens=50, ignore_eos=True, temperature=0.8, seed=5)
    got_t = small.generate(prompts, max_new_tokens=50, ignore_eos=True, temperature=0.8, seed=5)
    assert got_t == want_t


@pytest.mark.parametrize("name", ["D", "F"])
@pytest.mark.parametrize("split_keys", [False, True])
def test_prompt_portions_through_the_workgroup_attention_kernel(split_keys, name, model_dirs, gpu, monkeypatch):
    """The attention kernel that shares key blocks through LDS is chosen for steps with many long
    rows; with its thresholds lowered it runs on a tiny model (head size 32) and on one with the
    served models' head size of 128, which has thresholds of its own: whole prompts, portions that
    start deep in a request, and portions beside decoded tokens (two launches) all match the plain
    implementation - also with the keys cut into ranges of 64, one workgroup each, and merged."""
    from kv_cache_optimization_for_llm_amd.ops import attention as policy
    from kv_cache_optimization_for_llm_amd.ops import kernels as K
    calls = {"lds": 0, "split": 0}
    real = K.attention_lds

    def counted(*a, **kw):
        calls["lds"] += 1
        calls["split"] += 1 if a[13] > 1 else 0
        return real(*a, **kw)
    monkeypatch.setattr(policy, "_LDS_MIN_GROUPS", 1)
    monkeypatch.setattr(policy, "_LDS_MANY_GROUPS", 1)
    if split_keys:
        monkeypatch.setattr(policy, "_LDS_MIN_KEYS_PER_SPLIT", 64)
        monkeypatch.setattr(policy, "_LDS_MIN_KEYS_PER_SPLIT_WIDE_HEADS", 64)
    monkeypatch.setattr(K, "attention_lds", counted)
    cfg, W = plain.load_model_dir(model_dirs[name])
    eng = Engine(model_dirs[name], EngineOptions(dtype="bfloat16", max_seqs=3, max_seq_len=512))
    pa, pb, pc = prompts_for(name, [300, 140, 77], seed=9)
    ref = {k: plain.logits_all(cfg, W, p) for k, p in (("a", pa), ("b", pb), ("c", pc))}

    def worst(got, want):
        return float((got.float().cpu() - want).abs().max() / want.abs().max())
    out = eng.step([StepEntry("a", pa[:200], list(range(200))), StepEntry("b", pb[:60], list(range(60)))])
    assert worst(out[:200], ref["a"][:200]) <= TOL["bfloat16"] and worst(out[200:], ref["b"][:60]) <= TOL["bfloat16"]
    assert calls["lds"] == cfg["num_hidden_layers"]
    # a's next token beside b's rest and all of c: decoded rows and prompt rows in one step
    out = eng.step([StepEntry("a", pa[200:201], [0]), StepEntry("b", pb[60:], list(range(80))),
                    StepEntry("c", pc, list(range(77)))])
    assert worst(out[:1], ref["a"][200:201]) <= TOL["bfloat16"]
    assert worst(out[1:81], ref["b"][60:]) <= TOL["bfloat16"] and worst(out[81:], ref["c"]) <= TOL["bfloat16"]
    assert calls["lds"] == 2 * cfg["num_hidden_layers"]
    out = eng.step([StepEntry("a", pa[201:], list(range(99)))])          # a portion that starts at 201
    assert worst(out, ref["a"][201:]) <= TOL["bfloat16"]
    assert calls["split"] == (calls["lds"] if split_keys else 0)
    eng.cache.check()


def test_a_tensor_stored_in_32_bit_is_used_in_32_bit(model_dirs, tmp_path, gpu):
    """Norm weights and one projection stored as float32 in a bfloat16 engine stay float32."""
    from safetensors.torch import load_file, save_file
    import shutil
    d = str(tmp_path / "mixed")
    shutil.copytree(model_dirs["A"], d)
    w = load_file(os.path.join(d, "model.safetensors"))
    for k in list(w):
        if "layernorm" in k or k == "model.norm.weight" or k.endswith("layers.0.mlp.down_proj.weight"):
            w[k] = (w[k].float() + 1e-4 * torch.randn(w[k].shape))      # not representable in bf16
    save_file(w, os.path.join(d, "model.safetensors"))
    eng = Engine(d, EngineOptions(dtype="bfloat16", max_seqs=2, max_seq_len=64))
    assert eng.model.final_norm.weight.dtype == torch.float32
    assert eng.model.blocks[0].feed_forward.down.weight.dtype == torch.float32
    assert eng.model.blocks[1].feed_forward.down.weight.dtype == torch.bfloat16
    cfg, W = plain.load_model_dir(d)
    toks = prompts_for("A", [25])[0]
    got = eng.step([StepEntry("x", toks, list(range(25)))]).cpu().numpy()
    ref = plain.logits_all(cfg, W, toks).numpy()
    assert np.abs(got - ref).max() / np.abs(ref).max() <= TOL["bfloat16"]


def test_engine_refuses_what_it_cannot_run(model_dirs, gpu):
    eng = Engine(model_dirs["A"], EngineOptions(dtype="float32", max_seqs=2, max_seq_len=64, cache_tokens=64))
    with pytest.raises(Exception) as e:
        eng.step([StepEntry("x", [1, 2, 999], [0])])
    assert "token id" in str(e.value)
    with pytest.raises(Exception):
        eng.step([StepEntry("x", [1], [0]), StepEntry("x", [2], [0])])
    with pytest.raises(CacheExhausted):
        eng.step([StepEntry("y", list(range(65)), [])])
    eng.release("y")
    eng.step([StepEntry("a", [1, 2], []), StepEntry("b", [3], [])])
    with pytest.raises(CacheExhausted):
        eng.step([StepEntry("c", [3], [])])           # no seat left
    from kv_cache_optimization_for_llm_amd.ops import kernels as K
    with pytest.raises(K.KernelError) as e:
        K.rmsnorm(torch.zeros(2, 8), torch.ones(8), 1e-5, torch.zeros(2, 8))
    assert "GPU only" in str(e.value)


def test_pool_comes_from_free_memory_and_a_step_is_bounded(gpu):
    """No pool size given: the engine takes what the device has left after the weights, less a
    margin and a step's activations, never more than every seat at its longest; and a step that
    brings more tokens than ``max_batch_tokens`` is refused before anything is mapped."""
    from conftest import MID_F
    from kv_cache_optimization_for_llm_amd.engine.engine import EngineError
    cfg = dict(MID_F, max_position_embeddings=131072)
    torch.cuda.empty_cache()               # what earlier tests left in torch's cache is free memory too
    free, _ = torch.cuda.mem_get_info(gpu)
    page_bytes = 2 * 2 * 2 * 128 * 16 * 2                      # layers x (K, V) x kv heads x head size x tokens x bf16
    # as on a device with 3 GiB to spare: the margin takes the rest
    eng = Engine(None, EngineOptions(dtype="bfloat16", max_seqs=64, memory_margin_bytes=free - 3 * 2 ** 30,
                                     max_batch_tokens=256, max_logit_rows=4, use_graphs=False),
                 config_dict=cfg, random_seed=1)
    # the largest step's intermediate results have their memory already (taken once, kept by torch's allocator)
    assert eng.step_arena_bytes == eng.model.step_activation_bytes(256, 4) > 256 * 640 * 2
    assert torch.cuda.memory_reserved(gpu) - torch.cuda.memory_allocated(gpu) >= eng.step_arena_bytes
    pool_bytes = eng.cache.num_pages * page_bytes
    assert eng.max_seq_len == 131072 and eng.cache.num_pages < 64 * 131072 // 16
    assert 2 * 2 ** 30 < pool_bytes <= 3 * 2 ** 30
    stats = eng.cache.stats()
    assert stats["kv_tokens_total"] == eng.cache.num_pages * 16
    # a request longer than one step may bring is cut by its caller; the engine refuses the whole
    logits = eng.step([StepEntry("a", list(range(256)), [255])])
    assert logits.shape == (1, cfg["vocab_size"])
    with pytest.raises(EngineError) as e:
        eng.step([StepEntry("a", list(range(200)), []), StepEntry("b", list(range(57)), [])])
    assert "max_batch_tokens" in str(e.value)
    with pytest.raises(EngineError) as e:
        eng.step([StepEntry("a", list(range(8)), [0, 1, 2, 3, 4])])
    assert "max_logit_rows" in str(e.value)
    assert not eng.has_request("b") and eng.length("a") == 256 and eng.cache.free_seats == 63
    eng.cache.check()
    del eng
    torch.cuda.empty_cache()
    # a small model with few seats: every seat at its longest fits and is what the pool holds
    eng = Engine(None, EngineOptions(dtype="float32", max_seqs=2, max_seq_len=100), config_dict=cfg, random_seed=1)
    assert eng.cache.num_pages == 2 * 7
