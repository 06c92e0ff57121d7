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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F"])
def test_every_cut_matches_plain(name, dtype, model_dirs, plain_rows, tmp_path, gpu):
    vocab = TINY[name][0]["vocab_size"]
    requests = make_requests(vocab, LENGTHS[name], seed=5)
    ref = plain_rows(name, requests)
    for what, steps in (("whole", ru.whole(requests)), ("tail decoded", ru.tail_decoded(requests)),
                        ("portions", ru.chunked(requests)), ("mixed", ru.mixed(requests, seed=3))):
        budget = ru.max_live_tokens(steps)
        rows = ru.run_trace(model_dirs[name], dtype, steps, budget, str(tmp_path / what.replace(" ", "_")), vocab)
        compare(rows, ref, requests, dtype, what)
