"""vrl_gemm_nt: out = y @ x.T on the matrix cores (the d hidden / d W products of the LM-head backward), against the fp64
product of the same 16-bit operands: every element within one rounding to the output type plus the fp32 accumulation
error of a contraction of that length."""

import pytest
import torch

from verl_amd import gemm

pytestmark = pytest.mark.gpu


def _check(out, x, y, base=None, ulps=1.0):
    ref = y.double() @ x.double().t()
    if base is not None:
        ref = ref + base.double()
    eps = 2.0 ** -8 if out.dtype == torch.bfloat16 else 2.0 ** -11
    K = x.shape[1]
    # one rounding to the output type, plus fp32 accumulation over K products of magnitude <= |x||y|
    acc = (y.double().abs() @ x.double().abs().t()) * (K ** 0.5) * 2.0 ** -23
    bound = ulps * eps * ref.abs() + acc + 1e-30
    err = (out.double() - ref).abs()
    worst = (err / bound).max().item()
    assert worst <= 1.0, worst


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("NX,NY,K", [(256, 256, 128), (512, 256, 192), (260, 300, 256), (768, 1024, 4096), (3584, 512, 1024)])
def test_product_against_fp64(dev, dtype, NX, NY, K):
    g = torch.Generator(device=dev).manual_seed(NX + NY + K)
    x = (torch.randn(NX, K, generator=g, device=dev) * 0.5).to(dtype)
    y = (torch.randn(NY, K, generator=g, device=dev) * 0.5).to(dtype)
    for parts in (None, 1, 2, 3):
        if parts is not None and K // 64 // parts < 2:
            continue
        out = gemm.gemm_nt(x, y, k_parts=parts)
        _check(out, x, y)
        base = (torch.randn(NY, NX, generator=g, device=dev)).to(dtype)
        acc = base.clone()
        gemm.gemm_nt(x, y, out=acc, accumulate=True, k_parts=parts)
        _check(acc, x, y, base=base)


def test_strided_operands_and_output(dev):
    g = torch.Generator(device=dev).manual_seed(3)
    xb = (torch.randn(512, 640 + 64, generator=g, device=dev) * 0.5).bfloat16()
    yb = (torch.randn(384, 640 + 8, generator=g, device=dev) * 0.5).bfloat16()
    x, y = xb[:, :640], yb[:, :640]
    outb = torch.full((384, 512 + 4), 7.0, dtype=torch.bfloat16, device=dev)
    out = outb[:, :512]
    gemm.gemm_nt(x, y, out=out)
    _check(out, x, y)
    assert torch.all(outb[:, 512:] == 7.0)          # the padding of the output rows is left alone


def test_ranges_of_the_contraction_do_not_change_the_result_much(dev):
    g = torch.Generator(device=dev).manual_seed(5)
    x = (torch.randn(512, 8192, generator=g, device=dev) * 0.2).bfloat16()
    y = (torch.randn(256, 8192, generator=g, device=dev) * 0.2).bfloat16()
    a = gemm.gemm_nt(x, y, k_parts=1)
    b = gemm.gemm_nt(x, y, k_parts=8)
    c = gemm.gemm_nt(x, y, k_parts=8)
    assert torch.equal(b, c)                          # fixed summation order: reproducible
    assert (a.float() - b.float()).abs().max().item() <= 2.0 ** -7 * a.float().abs().max().item()


def test_backward_shapes_of_the_lm_head(dev):
    """d hidden = G @ W and d W += G.T @ H at a chunk of 1024 tokens, hidden 3584, vocabulary 152064 / 151936."""
    for V in (152064, 151936):
        g = torch.Generator(device=dev).manual_seed(V)
        T, D = 1024, 3584
        G = (torch.randn(T, V, generator=g, device=dev) * 0.01).bfloat16()
        W = (torch.randn(V, D, generator=g, device=dev) * 0.02).bfloat16()
        H = (torch.randn(T, D, generator=g, device=dev) * 0.5).bfloat16()
        dH = gemm.gemm_nt(W.t().contiguous(), G)                     # (T, D)
        ref = (G.float() @ W.float())
        assert (dH.float() - ref).abs().max().item() <= 2.0 ** -7 * ref.abs().max().item()
        dW = torch.zeros(V, D, dtype=torch.bfloat16, device=dev)
        gemm.gemm_nt(H.t().contiguous(), G.t().contiguous(), out=dW, accumulate=True)   # (V, D)
        ref = (G.float().t() @ H.float())
        assert (dW.float() - ref).abs().max().item() <= 2.0 ** -7 * ref.abs().max().item()


def test_argument_errors(dev):
    x = torch.zeros(256, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        gemm.gemm_nt(x[:128], x)                       # fewer than 256 rows
    with pytest.raises(ValueError):
        gemm.gemm_nt(x[:, :64], x[:, :64])             # contraction shorter than 128
    with pytest.raises(ValueError):
        gemm.gemm_nt(x, x.half())
    with pytest.raises(ValueError):
        gemm.gemm_nt(x, x, out=torch.zeros(256, 128, dtype=torch.bfloat16, device=dev))
    with pytest.raises(ValueError):
        gemm.gemm_nt(x, x, accumulate=True)
    with pytest.raises(RuntimeError):
        gemm.gemm_nt(x.cpu(), x.cpu())
