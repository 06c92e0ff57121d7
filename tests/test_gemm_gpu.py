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
        K.gemm_skinny(x.to(gpu), w.to(gpu), out)
        err = (out.double().cpu() - want).abs().max() / want.abs().max()
        assert err <= tol, f"{dt}: {err:.3g}"
    # a token's result does not depend on the batch it is in (bitwise)
    one = torch.empty((1, n), dtype=torch.float32, device=gpu)
    full = torch.empty((m, n), dtype=torch.float32, device=gpu)
    K.gemm_skinny(x.to(gpu), w.to(gpu), full)
    K.gemm_skinny(x[m - 1:].contiguous().to(gpu), w.to(gpu), one)
    assert torch.equal(one[0], full[m - 1])


@pytest.mark.parametrize("m", [1, 5, 16, 40, 64])
@pytest.mark.parametrize("inter, k", [(16, 64), (250, 96), (8192, 2048), (56, 160)])
def test_skinny_product_with_swiglu_epilogue(m, inter, k, gpu):
    x, w = rnd(m, k), rnd(2 * inter, k, scale=0.2, seed=2)
    g = x.double() @ w[:inter].double().t()
    u = x.double() @ w[inter:].double().t()
    want = g * (1 / (1 + torch.exp(-g))) * u
    out = torch.full((m, inter), float("nan"), dtype=torch.bfloat16, device=gpu)
    K.gemm_skinny(x.to(gpu), w.to(gpu), out, swiglu=True)
    err = (out.double().cpu() - want).abs().max() / want.abs().max()
    assert err <= 6e-3, f"{err:.3g}"


def test_skinny_product_refuses_what_it_cannot_do(gpu):
    assert not K.gemm_skinny_supported(65, 16, 32) and not K.gemm_skinny_supported(4, 16, 40)
    x, w = rnd(4, 40).to(gpu), rnd(16, 40).to(gpu)
    with pytest.raises(K.KernelError):
        K.gemm_skinny(x, w, torch.empty((4, 16), dtype=torch.bfloat16, device=gpu))
