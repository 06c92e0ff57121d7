"""The few-rows matrix-core product against a plain fp32 product, at sizes other than the engine's."""
import pytest
import torch

from kv_cache_optimization_for_llm_amd.ops import kernels as K

pytestmark = pytest.mark.gpu


def rnd(*shape, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


@pytest.mark.parametrize("m", [1, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("n, k", [(16, 32), (100, 96), (389, 128), (2048, 2048), (3072, 1024), (48, 8192)])
def test_skinny_product_bf16_and_fp32_outputs(m, n, k, gpu):
    assert K.gemm_skinny_supported(m, n, k)
    x, w = rnd(m, k), rnd(n, k, scale=0.05, seed=1)
    want = x.double() @ w.double().t()
    for dt, tol in ((torch.float32, 1e-5), (torch.bfloat16, 6e-3)):
        out = torch.full((m, n), float("nan"), dtype=dt, device=gpu)
        K.gemm_skinny(x.to(gpu), K.TiledWeight(w.to(gpu)), out)
        err = (out.double().cpu() - want).abs().max() / want.abs().max()
        assert err <= tol, f"{dt}: {err:.3g}"
    # a token's result does not depend on the batch it is in (bitwise)
    one = torch.empty((1, n), dtype=torch.float32, device=gpu)
    full = torch.empty((m, n), dtype=torch.float32, device=gpu)
    K.gemm_skinny(x.to(gpu), K.TiledWeight(w.to(gpu)), full)
    K.gemm_skinny(x[m - 1:].contiguous().to(gpu), K.TiledWeight(w.to(gpu)), one)
    assert torch.equal(one[0], full[m - 1])


@pytest.mark.parametrize("m", [1, 5, 16, 40, 64])
@pytest.mark.parametrize("inter, k", [(16, 64), (250, 96), (8192, 2048), (56, 160)])
def test_skinny_product_with_swiglu_epilogue(m, inter, k, gpu):
    x, w = rnd(m, k), rnd(2 * inter, k, scale=0.2, seed=2)
    g = x.double() @ w[:inter].double().t()
    u = x.double() @ w[inter:].double().t()
    want = g * (1 / (1 + torch.exp(-g))) * u
    out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=gpu)
    K.gemm_skinny(x.to(gpu), K.TiledWeight(w.to(gpu), halves=2), out, swiglu=True)
    err = (out.double().cpu() - want).abs().max() / want.abs().max()
    assert err <= 6e-3, f"{err:.3g}"


def test_skinny_product_refuses_what_it_cannot_do(gpu):
    assert not K.gemm_skinny_supported(65, 16, 32) and not K.gemm_skinny_supported(4, 16, 40)
    x, w = rnd(4, 40).to(gpu), rnd(16, 40).to(gpu)
    with pytest.raises(K.KernelError):
        K.TiledWeight(w)                                   # K is not a multiple of 32
    with pytest.raises(K.KernelError):
        K.gemm_skinny(x, w, torch.empty((4, 16), dtype=torch.bfloat16, device=gpu))
    tw = K.TiledWeight(rnd(50, 64).to(gpu))                # 50 rows are padded to 64
    assert tw.data.shape == (4, 2, 16, 32) and tw.data[3, :, 2:].abs().max() == 0


def rms(h, w, eps):
    return h * torch.rsqrt((h * h).mean(-1, keepdim=True) + eps) * w


@pytest.mark.parametrize("m", [1, 8, 33, 64])
@pytest.mark.parametrize("n, k", [(2048, 2048), (96, 160), (389, 64)])
def test_product_adds_into_the_stream_and_prepares_the_next_norm(m, n, k, gpu):
    """EPI_RESID: hidden += x W^T (rounded), scaled = round(hidden * w_next), partial sums of
    hidden^2; a following product that takes (scaled, sumsq) equals norm-then-product."""
    x, w = rnd(m, k), rnd(n, k, scale=0.05, seed=1)
    h0 = rnd(m, n, seed=2)
    w_next = (1 + 0.1 * torch.randn(n, generator=torch.Generator().manual_seed(3)))
    eps = 2e-6
    for wn in (w_next.to(torch.bfloat16), w_next.float()):            # norm weight stored in bf16 or fp32
        hidden = h0.clone().to(gpu)
        scaled = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
        parts = K.gemm_skinny_sumsq_parts(n)
        assert parts == (n + 15) // 16
        sumsq = torch.full((m, parts), float("nan"), device=gpu)
        K.gemm_skinny(x.to(gpu), K.TiledWeight(w.to(gpu)), None, hidden=hidden, next_weight=wn.to(gpu), scaled_out=scaled,
                      sumsq_out=sumsq)
        want_h = (h0.float() + (x.double() @ w.double().t()).float()).to(torch.bfloat16)
        diff = (hidden.cpu().float() - want_h.float()).abs().max() / want_h.float().abs().max()
        assert diff <= 8e-3                                            # one bf16 ulp where a sum sits on a tie
        hf = hidden.cpu().float()
        assert torch.allclose(sumsq.cpu().sum(-1), (hf * hf).sum(-1), rtol=1e-5)
        assert torch.equal(scaled.cpu(), (hf * wn.float()).to(torch.bfloat16))
        # finishing the norm alone
        fin = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
        K.normed_rows_finish(scaled, sumsq, n, eps, fin)
        want_norm = rms(hf, wn.float(), eps)
        assert (fin.cpu().float() - want_norm).abs().max() <= 1.2e-2 * want_norm.abs().max()
        rows = torch.tensor([m - 1, 0, m - 1], dtype=torch.int32, device=gpu)
        fin3 = torch.empty((3, n), dtype=torch.bfloat16, device=gpu)
        K.normed_rows_finish(scaled, sumsq, n, eps, fin3, rows)
        assert torch.equal(fin3.cpu(), fin.cpu()[rows.cpu().long()])
        # a following product finishes the norm in its epilogue (needs its K = n to be a multiple of 32)
        if n % 32 == 0:
            w2 = rnd(80, n, scale=0.05, seed=4)
            out = torch.empty((m, 80), dtype=torch.float32, device=gpu)
            K.gemm_skinny(scaled, K.TiledWeight(w2.to(gpu)), out, sumsq=sumsq, norm_width=n, eps=eps)
            want = want_norm.double() @ w2.double().t()
            assert (out.cpu().double() - want).abs().max() <= 6e-3 * want.abs().max()
            act = torch.empty((m, 40), dtype=torch.bfloat16, device=gpu)
            K.gemm_skinny(scaled, K.TiledWeight(w2.to(gpu), halves=2), act, swiglu=True, sumsq=sumsq, norm_width=n, eps=eps)
            g, u = want[:, :40], want[:, 40:]
            want_act = g * (1 / (1 + torch.exp(-g))) * u
            assert (act.cpu().double() - want_act).abs().max() <= 1e-2 * want_act.abs().max()


def test_wide_matrices_give_a_wave_several_tiles(gpu):
    """N >= 32768 and >= 65536 switch to 2 and 4 n-tiles per wave (the vocabulary-sized product)."""
    for n in (32768 + 48, 65536 + 16, 128256):
        x, w = rnd(5, 64), rnd(n, 64, scale=0.1, seed=n)
        out = torch.full((5, n), float("nan"), dtype=torch.float32, device=gpu)
        K.gemm_skinny(x.to(gpu), K.TiledWeight(w.to(gpu)), out)
        want = x.double() @ w.double().t()
        assert (out.cpu().double() - want).abs().max() <= 1e-5 * want.abs().max()
