"""Trace replay against the plain implementation: every way of cutting the same requests gives
the same logits, in 32-bit and in bfloat16."""
import numpy as np
import pytest
import torch

import plain_llama as plain
import replay_util as ru
from conftest import TINY

pytestmark = pytest.mark.gpu

# Largest |difference| allowed, as a fraction of the largest |logit| of the plain result.
# float32: both sides are fp32 arithmetic in another order.  bfloat16: every op's output is
# rounded to 8 bits of mantissa (relative 2^-9 each), a few dozen roundings deep.
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def make_requests(vocab, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": [int(t) for t in rng.integers(0, vocab, n)] for i, n in enumerate(lengths)}


@pytest.fixture(scope="module")
def plain_rows(model_dirs):
    cache = {}

    def get(name, requests):
        key = (name, tuple((k, tuple(v)) for k, v in requests.items()))
        if key not in cache:
            cfg, W = plain.load_model_dir(model_dirs[name])
            cache[key] = {rid: plain.logits_all(cfg, W, toks).numpy() for rid, toks in requests.items()}
        return cache[key]
    return get


def compare(rows, ref, requests, dtype, what):
    assert len(rows) == sum(len(t) for t in requests.values()), f"{what}: some logits rows are missing"
    worst = (0.0, None)
    for rid, toks in requests.items():
        scale = float(np.abs(ref[rid]).max())
        for p in range(len(toks)):
            err = float(np.abs(rows[(rid, p)] - ref[rid][p]).max()) / scale
            if err > worst[0]:
                worst = (err, (rid, p))
    assert worst[0] <= TOL[dtype], (f"{what} [{dtype}]: logits differ from the plain implementation by "
                                    f"{worst[0]:.3g} of their scale at (request, position) {worst[1]}")


LENGTHS = {"A": [5, 17, 33, 70, 131], "B": [1, 9, 40, 70, 97], "C": [3, 66, 130, 45, 200],
           "D": [2, 35, 90, 64, 150], "E": [4, 130, 300, 65, 517], "F": [2, 257, 48, 330, 129]}


# the page size each configuration is replayed at (B: the 8 its baseline configuration names)
PAGE = {"A": 16, "B": 8, "C": 16, "D": 16, "E": 16, "F": 16}


def same_rows(a, b, dtype, what):
    """float32: every reduction has a fixed order that does not depend on the batch, so two cuts
    give the same bits.  bfloat16: the split counts of attention and of the few-rows products
    depend on the batch, which changes rounding only."""
    assert a.keys() == b.keys()
    if dtype == "float32":
        bad = [k for k in a if not np.array_equal(a[k], b[k])]
        assert not bad, f"{what}: float32 logits are not bit-identical at {bad[:5]} ({len(bad)} rows)"
    else:
        for k in a:
            scale = float(np.abs(a[k]).max())
            assert float(np.abs(a[k] - b[k]).max()) <= 2 * TOL[dtype] * scale, f"{what}: rows differ at {k}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F"])
def test_every_cut_matches_plain(name, dtype, model_dirs, plain_rows, tmp_path, gpu):
    vocab = TINY[name][0]["vocab_size"]
    requests = make_requests(vocab, LENGTHS[name], seed=5)
    ref = plain_rows(name, requests)
    page = ["--page-size", str(PAGE[name])]
    got = {}
    for what, steps in (("whole", ru.whole(requests)), ("tail decoded", ru.tail_decoded(requests)),
                        ("portions", ru.chunked(requests)), ("mixed", ru.mixed(requests, seed=3))):
        budget = ru.max_live_tokens(steps)
        out = str(tmp_path / what.replace(" ", "_"))
        rows = ru.run_trace(model_dirs[name], dtype, steps, budget, out, vocab, page)
        compare(rows, ref, requests, dtype, what)
        got[what] = rows
        if what == "mixed":
            # the pool holds the most that is live at a time, less than all requests together:
            # later requests can only have run on pages that earlier ones gave back
            stats = ru.cache_stats(out)
            assert stats["pages_reused"] > 0 and stats["kv_tokens_total"] < sum(
                (len(t) + 63) // 64 * 64 for t in requests.values()), f"mixed: no page was used again: {stats}"
    # the same mixed trace over the contiguous (buddy) cache: every request reserves one run that
    # holds the longest of them, four runs fill the pool, and runs are handed out again
    longest = max(len(t) for t in requests.values())
    run = PAGE[name]
    while run < longest:
        run *= 2
    out = str(tmp_path / "mixed_contiguous")
    rows = ru.run_trace(model_dirs[name], dtype, ru.mixed(requests, seed=3), 4 * run, out, vocab,
                        page + ["--cache-mode", "contiguous", "--reserve-tokens", str(run)])
    compare(rows, ref, requests, dtype, "mixed, contiguous")
    got["mixed, contiguous"] = rows
    assert ru.cache_stats(out)["kv_tokens_total"] == 4 * run
    # and the cuts agree with each other, not only with the plain implementation
    for what in ("tail decoded", "portions", "mixed", "mixed, contiguous"):
        same_rows(got["whole"], got[what], dtype, f"whole against {what}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "F"])
def test_mixed_cuts_match_plain_on_weights_that_spread_attention(name, dtype, sharp_model_dirs, tmp_path, gpu):
    """The same drives on matrices N(0, 1 / sqrt(in)): scores spread over several units, so one
    page of wrong keys moves the logits by tens of percent of their scale (with the N(0, 0.02)
    matrices above: 2-4 %, about the bfloat16 tolerance there).  The bfloat16 tolerance here is
    measured, not chosen: twice what rounding every op's output to bfloat16 does to the plain
    implementation's own logits for these requests."""
    vocab = TINY[name][0]["vocab_size"]
    requests = make_requests(vocab, LENGTHS[name], seed=9)
    cfg, W = plain.load_model_dir(sharp_model_dirs[name])
    ref = {rid: plain.logits_all(cfg, W, toks).numpy() for rid, toks in requests.items()}
    tol = TOL["float32"]
    if dtype == "bfloat16":
        rounded = {rid: plain.logits_all(cfg, W, toks, act=plain.round_bf16).numpy() for rid, toks in requests.items()}
        noise = max(float(np.abs(rounded[r] - ref[r]).max()) / float(np.abs(ref[r]).max()) for r in requests)
        tol = 2 * noise
        assert 0.005 < tol < 0.05, f"rounding noise {noise:.3g} of the logits' scale is not what this test was sized for"
    page = ["--page-size", str(PAGE[name])]
    steps = ru.mixed(requests, seed=4)
    longest = max(len(t) for t in requests.values())
    run = PAGE[name]
    while run < longest:
        run *= 2
    got = {}
    for what, extra, budget in (("mixed", [], ru.max_live_tokens(steps)),
                                ("mixed, contiguous", ["--cache-mode", "contiguous", "--reserve-tokens", str(run)], 4 * run)):
        out = str(tmp_path / what.replace(", ", "_"))
        rows = ru.run_trace(sharp_model_dirs[name], dtype, steps, budget, out, vocab, page + extra)
        assert len(rows) == sum(len(t) for t in requests.values())
        worst = max((float(np.abs(rows[(rid, p)] - ref[rid][p]).max()) / float(np.abs(ref[rid]).max()), rid, p)
                    for rid, toks in requests.items() for p in range(len(toks)))
        assert worst[0] <= tol, (f"{what} [{dtype}]: logits differ from the plain implementation by {worst[0]:.3g} "
                                 f"of their scale (allowed {tol:.3g}) at request {worst[1]}, position {worst[2]}")
        got[what] = rows
    assert ru.cache_stats(str(tmp_path / "mixed"))["pages_reused"] > 0
    if dtype == "float32":
        same_rows(got["mixed"], got["mixed, contiguous"], dtype, "paged against contiguous")
