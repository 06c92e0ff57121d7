"""The matrix-vector product of one or two tokens (csrc/gemv.hip) against a plain fp64 product and
against the epilogues done one after the other, at sizes other than the engine's: every K instance
class (rows in flight 8, 4, 2, 1), row counts that end inside a wavefront's unit of rows."""
import pytest
import torch

from kv_cache_optimization_for_llm_amd.ops import kernels as K

pytestmark = pytest.mark.gpu


def rnd(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


SHAPES = [(37, 512), (1001, 1024), (130, 1536), (2050, 2048), (77, 2560), (64, 3584), (515, 4096), (91, 5120),
          (33, 8192)]


def test_supported_shapes():
    assert K.gemv_supported(1, 5, 512) and K.gemv_supported(2, 128256, 2048) and K.gemv_supported(1, 8, 7168)
    assert not K.gemv_supported(3, 64, 512)            # more than two tokens
    assert not K.gemv_supported(1, 64, 768)            # K is no multiple of 512
    assert not K.gemv_supported(1, 64, 4608)           # between instances
    assert not K.gemv_supported(1, 64, 8704)           # beyond the largest
    assert K.gemv_qkv_rope_supported(1, 2048, 64) and K.gemv_qkv_rope_supported(2, 512, 16)
    assert not K.gemv_qkv_rope_supported(1, 512, 6)    # half a head is no multiple of the 4 pairs in flight


@pytest.mark.parametrize("m", [1, 2])
@pytest.mark.parametrize("n, k", SHAPES)
def test_product_bf16_and_fp32_outputs_and_row_scale(m, n, k, gpu):
    x, w = rnd(m, k), rnd(n, k, scale=0.05, seed=1)
    want = x.double() @ w.double().t()
    # x given as the first rows of a wider buffer: the row stride is its own argument
    wide = torch.zeros((m, k + 64), dtype=torch.bfloat16, device=gpu)
    wide[:, :k] = x.to(gpu)
    for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 6e-3)):
        out = torch.full((m, n), float("nan"), dtype=dt, device=gpu)
        K.gemv(x.to(gpu), w.to(gpu), out)
        err = (out.double().cpu() - want).abs().max() / want.abs().max()
        assert err <= tol, f"{dt}: {err:.3g}"
        out2 = torch.full((m, n), float("nan"), dtype=dt, device=gpu)
        K.gemv(wide[:, :k], w.to(gpu), out2)
        assert torch.equal(out, out2)
    # the input's unfinished norm: per-token scale from partial sums of squares
    parts, width, eps = 7, 300, 3e-6
    sumsq = torch.rand(m, parts, generator=torch.Generator().manual_seed(5)) * 50 + 1
    out = torch.empty((m, n), dtype=torch.float32, device=gpu)
    K.gemv(x.to(gpu), w.to(gpu), out, sumsq=sumsq.to(gpu), norm_width=width, eps=eps)
    scaled = want * torch.rsqrt(sumsq.double().sum(-1, keepdim=True) / width + eps)
    assert (out.double().cpu() - scaled).abs().max() <= 1e-5 * scaled.abs().max()
    # a token's result does not depend on the token beside it (bitwise)
    if m == 2:
        one = torch.empty((1, n), dtype=torch.float32, device=gpu)
        two = torch.empty((2, n), dtype=torch.float32, device=gpu)
        K.gemv(x.to(gpu), w.to(gpu), two)
        K.gemv(x[1:].contiguous().to(gpu), w.to(gpu), one)
        assert torch.equal(one[0], two[1])


@pytest.mark.parametrize("m", [1, 2])
@pytest.mark.parametrize("inter, k", [(333, 512), (250, 1024), (8192, 2048), (57, 2560), (100, 6144), (31, 8192)])
def test_gated_product(m, inter, k, gpu):
    x, w = rnd(m, k), rnd(2 * inter, k, scale=0.1, seed=2)
    g = x.double() @ w[:inter].double().t()
    u = x.double() @ w[inter:].double().t()
    want = g * (1 / (1 + torch.exp(-g))) * u
    out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=gpu)
    K.gemv(x.to(gpu), w.to(gpu), out, swiglu=True)
    err = (out.double().cpu() - want).abs().max() / want.abs().max()
    assert err <= 6e-3, f"{err:.3g}"
    # the same values as the few-rows kernel leaves, up to the order of its sums
    few = torch.empty_like(out)
    K.gemm_skinny(x.to(gpu), K.TiledWeight(w.to(gpu), halves=2), few, swiglu=True)
    assert (few.float() - out.float()).abs().max() <= 8e-3 * want.abs().max()


def rms(h, w, eps):
    return h * torch.rsqrt((h * h).mean(-1, keepdim=True) + eps) * w


@pytest.mark.parametrize("m", [1, 2])
@pytest.mark.parametrize("n, k", [(2048, 2048), (515, 512), (96, 1536), (389, 3072), (512, 8192), (61, 5120)])
def test_product_adds_into_the_stream_and_prepares_the_next_norm(m, n, k, gpu):
    x, w = rnd(m, k), rnd(n, k, scale=0.05, seed=1)
    h0 = rnd(m, n, seed=2)
    w_next = (1 + 0.1 * torch.randn(n, generator=torch.Generator().manual_seed(3)))
    eps = 2e-6
    parts = K.gemv_sumsq_parts(n, k)
    assert 1 <= parts <= n
    for wn in (w_next.to(torch.bfloat16), w_next.float(), None):
        hidden = h0.clone().to(gpu)
        scaled = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=gpu)
        sumsq = torch.full((m, parts), float("nan"), device=gpu)
        K.gemv(x.to(gpu), w.to(gpu), None, hidden=hidden, next_weight=None if wn is None else wn.to(gpu),
               scaled_out=scaled, sumsq_out=sumsq)
        want_h = (h0.float() + (x.double() @ w.double().t()).float()).to(torch.bfloat16)
        diff = (hidden.cpu().float() - want_h.float()).abs().max() / want_h.float().abs().max()
        assert diff <= 8e-3                                            # one bf16 ulp where a sum sits on a tie
        hf = hidden.cpu().float()
        assert torch.allclose(sumsq.cpu().sum(-1), (hf * hf).sum(-1), rtol=1e-5)
        wf = torch.ones(n) if wn is None else wn.float()
        assert torch.equal(scaled.cpu(), (hf * wf).to(torch.bfloat16))
        # finishing the norm alone, and inside a following product
        fin = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
        K.normed_rows_finish(scaled, sumsq, n, eps, fin)
        want_norm = rms(hf, wf, eps)
        assert (fin.cpu().float() - want_norm).abs().max() <= 1.2e-2 * want_norm.abs().max()
        if K.gemv_supported(m, 80, n):
            w2 = rnd(80, n, scale=0.05, seed=4)
            out = torch.empty((m, 80), dtype=torch.float32, device=gpu)
            K.gemv(scaled, w2.to(gpu), out, sumsq=sumsq, norm_width=n, eps=eps)
            want = want_norm.double() @ w2.double().t()
            assert (out.cpu().double() - want).abs().max() <= 6e-3 * want.abs().max()


@pytest.mark.parametrize("m", [1, 2])
@pytest.mark.parametrize("nq, nkv, d, page, k", [(4, 2, 32, 16, 512), (6, 1, 96, 8, 1536), (3, 3, 64, 4, 2048),
                                                 (32, 8, 64, 16, 2048), (5, 5, 16, 16, 1024), (2, 1, 128, 32, 4096),
                                                 (7, 1, 48, 16, 8192), (3, 1, 8, 16, 512)])
@pytest.mark.parametrize("rotate, normed", [(True, False), (True, True), (False, False)])
def test_qkv_product_rotates_and_writes_the_cache(m, nq, nkv, d, page, k, rotate, normed, gpu):
    """The fused projection equals product -> round -> rotate-half rotation -> cache write done
    one after the other in fp32 (the cache is checked slot by slot, untouched slots stay zero)."""
    import plain_llama as plain
    n = (nq + 2 * nkv) * d
    x, w = rnd(m, k), rnd(n, k, scale=0.05, seed=1)
    pos = [(37 * i + 211) % 300 for i in range(m)]
    pages = 4
    slots = torch.randperm(pages * page, generator=torch.Generator().manual_seed(m + d))[:m].to(torch.int32)
    inv = plain.rope_inv_freq(d, 20000.0, dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0,
                                               high_freq_factor=2.0, original_max_position_embeddings=64))
    cos, sin = plain.rope_cos_sin(range(300), inv)
    y = x.double() @ w.double().t()
    extra = {}
    if normed:
        parts = 5
        sumsq = torch.rand(m, parts, generator=torch.Generator().manual_seed(9)) * 40 + 1
        eps, width = 3e-6, 100
        y = y * torch.rsqrt(sumsq.double().sum(-1, keepdim=True) / width + eps)
        extra = dict(sumsq=sumsq.to(gpu), norm_width=width, eps=eps)
    y = y.float().to(torch.bfloat16).float()                            # what a separate product leaves
    q_want = y[:, :nq * d].view(m, nq, d).clone()
    k_want = y[:, nq * d:(nq + nkv) * d].view(m, nkv, d).clone()
    v_want = y[:, (nq + nkv) * d:].view(m, nkv, d)
    if rotate:
        c, s = plain.rope_cos_sin(pos, inv)
        q_want = plain.apply_rope(q_want, c, s)
        k_want = plain.apply_rope(k_want, c, s)
    tables = (torch.from_numpy(cos).to(gpu), torch.from_numpy(sin).to(gpu)) if rotate else (None, None)
    positions = torch.tensor(pos, dtype=torch.int32, device=gpu)
    assert K.gemv_qkv_rope_supported(m, k, d)
    for some_unwritten in (False, True):
        sl = slots.clone()
        if some_unwritten:
            sl[m - 1] = -1                          # a token whose keys are not kept
        k_cache = K.keys_to_pages(torch.zeros(pages, nkv, page, d, dtype=torch.bfloat16, device=gpu))
        v_cache = torch.zeros(pages, nkv, d, page, dtype=torch.bfloat16, device=gpu)
        q = torch.full((m, nq * d), float("nan"), dtype=torch.bfloat16, device=gpu)
        K.gemv_qkv_rope(x.to(gpu), w.to(gpu), q, nq, nkv, d, positions, *tables, k_cache, v_cache, sl.to(gpu), page,
                        **extra)
        scale = y.abs().max()
        assert (q.float().cpu().view(m, nq, d) - q_want).abs().max() <= 1e-2 * scale
        kc, vc = K.pages_to_keys(k_cache).float().cpu(), v_cache.float().cpu()
        for t in range(m):
            s_ = int(sl[t])
            if s_ < 0:
                continue
            assert (kc[s_ // page, :, s_ % page, :] - k_want[t]).abs().max() <= 1e-2 * scale, f"k of row {t}"
            assert (vc[s_ // page, :, :, s_ % page] - v_want[t]).abs().max() <= 1e-2 * scale, f"v of row {t}"
        written = {int(s_) for s_ in sl if s_ >= 0}
        for s_ in range(pages * page):
            if s_ not in written:
                assert kc[s_ // page, :, s_ % page, :].abs().max() == 0 and vc[s_ // page, :, :, s_ % page].abs().max() == 0
    # without a cache only Q is produced
    q2 = torch.empty_like(q)
    K.gemv_qkv_rope(x.to(gpu), w.to(gpu), q2, nq, nkv, d, positions, *tables, None, None, None, 0, **extra)
    assert torch.equal(q2, q)
    # the few-rows kernel leaves the same queries up to the order of its sums
    if K.gemm_skinny_qkv_rope_supported(m, k, d):
        q3 = torch.empty_like(q)
        K.gemm_skinny_qkv_rope(x.to(gpu), K.TiledWeight(w.to(gpu)), q3, nq, nkv, d, positions, *tables, None, None,
                               None, 0, **extra)
        assert (q3.float() - q.float()).abs().max() <= 1.6e-2 * scale


def test_refusals(gpu):
    x, w = rnd(1, 768).to(gpu), rnd(16, 768).to(gpu)
    with pytest.raises(K.KernelError):
        K.gemv(x, w, torch.empty((1, 16), dtype=torch.bfloat16, device=gpu))          # K has no instance
    x, w = rnd(3, 512).to(gpu), rnd(16, 512).to(gpu)
    with pytest.raises(K.KernelError):
        K.gemv(x, w, torch.empty((3, 16), dtype=torch.bfloat16, device=gpu))          # three tokens
    with pytest.raises(K.KernelError):
        K.gemv(x[:1], w, torch.empty((1, 17), dtype=torch.bfloat16, device=gpu))      # output of another width
    with pytest.raises(K.KernelError):
        K.gemv(x[:1], w.t().contiguous().t(), torch.empty((1, 16), dtype=torch.bfloat16, device=gpu))   # not row-major
    with pytest.raises(K.KernelError):
        K.gemv_qkv_rope(x[:1], rnd(4 * 6, 512).to(gpu), torch.empty((1, 12), dtype=torch.bfloat16, device=gpu), 2, 1, 6,
                        torch.zeros(1, dtype=torch.int32, device=gpu), None, None, None, None, None, 0)


@pytest.mark.parametrize("m", [1, 2])
@pytest.mark.parametrize("n, k, d, parts", [(2048, 2048, 64, 3), (515, 512, 64, 2), (96, 1536, 96, 4), (389, 3072, 128, 4),
                                            (130, 4096, 128, 3), (77, 2560, 16, 2), (64, 3584, 8, 4), (40, 1024, 32, 3),
                                            (2048, 2048, 64, 8), (61, 512, 32, 5), (200, 4096, 64, 7)])
def test_product_over_an_attention_output_still_in_partial_results(m, n, k, d, parts, gpu):
    """The residual-epilogue product whose input is what an attention kernel left per key range
    (running maximum in the base-2 domain, sum of exponentials, unnormalised output) against the
    ranges added up here and the ordinary product over that sum; one range of one head without a
    key (maximum -inf, everything else zero), which must weigh nothing."""
    if parts > K.gemv_merge_max_parts(m):
        assert m == 2 and not K.gemv_merged_supported(m, n, k, d, parts)       # more than four only for one token
        return
    heads = k // d
    g = torch.Generator().manual_seed(n + k + parts + m)
    part_o = torch.randn(m * heads, parts, d, generator=g)
    ml = torch.stack([torch.randn(m * heads, parts, generator=g) * 3, torch.rand(m * heads, parts, generator=g) * 5 + 0.5], -1)
    part_o[1, parts - 1] = 0.0
    ml[1, parts - 1, 0], ml[1, parts - 1, 1] = float("-inf"), 0.0
    wgt = torch.exp2(ml[..., 0] - ml[..., 0].max(-1, keepdim=True).values)           # [rows, parts]
    merged = (part_o * wgt[..., None]).sum(1) / (ml[..., 1] * wgt).sum(-1, keepdim=True)
    x = merged.reshape(m, k).to(torch.bfloat16)
    w = rnd(n, k, scale=0.05, seed=1)
    h0 = rnd(m, n, seed=2)
    w_next = (1 + 0.1 * torch.randn(n, generator=torch.Generator().manual_seed(3))).to(torch.bfloat16)
    p_out = K.gemv_sumsq_parts(n, k)
    assert K.gemv_merged_supported(m, n, k, d, parts)
    hidden_a, hidden_b = h0.clone().to(gpu), h0.clone().to(gpu)
    scaled_a, scaled_b = (torch.empty((m, n), dtype=torch.bfloat16, device=gpu) for _ in range(2))
    ss_a, ss_b = (torch.empty((m, p_out), device=gpu) for _ in range(2))
    K.gemv_merged(K.AttentionPartials(part_o.to(gpu), ml.to(gpu), m, heads), w.to(gpu), hidden_a, w_next.to(gpu), scaled_a, ss_a)
    K.gemv(x.to(gpu), w.to(gpu), None, hidden=hidden_b, next_weight=w_next.to(gpu), scaled_out=scaled_b, sumsq_out=ss_b)
    want = (h0.float() + (x.double() @ w.double().t()).float())
    scale = want.abs().max()
    assert (hidden_a.cpu().float() - want).abs().max() <= 8e-3 * scale
    # against the ordinary product: the same but for inputs that the two ways of adding up round differently
    assert (hidden_a.float() - hidden_b.float()).abs().max() <= 8e-3 * scale
    hf = hidden_a.cpu().float()
    assert torch.allclose(ss_a.cpu().sum(-1), (hf * hf).sum(-1), rtol=1e-5)
    assert torch.equal(scaled_a.cpu(), (hf * w_next.float()).to(torch.bfloat16))


def test_what_the_merging_product_takes():
    assert K.gemv_merge_max_parts(1) >= K.gemv_merge_max_parts(2) >= 4
    assert K.gemv_merged_supported(1, 2048, 2048, 64, 2) and K.gemv_merged_supported(2, 4096, 4096, 128, 4)
    assert not K.gemv_merged_supported(1, 2048, 2048, 64, 1)         # nothing to add up
    assert not K.gemv_merged_supported(1, 2048, 2048, 64, K.gemv_merge_max_parts(1) + 1)
    assert not K.gemv_merged_supported(2, 2048, 2048, 64, K.gemv_merge_max_parts(2) + 1)
    assert not K.gemv_merged_supported(1, 2048, 5120, 64, 2)         # K beyond 4,096
    assert not K.gemv_merged_supported(1, 2048, 2048, 12, 2)         # heads of no multiple of 8
    assert not K.gemv_merged_supported(1, 2048, 2048, 80, 2)         # heads that do not divide K
    assert not K.gemv_merged_supported(3, 2048, 2048, 64, 2)
