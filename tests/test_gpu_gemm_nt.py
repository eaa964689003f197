"""vrl_gemm / vrl_gemm_nt: out = y @ x.T on the matrix cores (the d hidden / d W products of the LM-head backward), against
the fp64 product of the same 16-bit operands: every element within one rounding to the output type plus the fp32
accumulation error of a contraction of that length. Operands stored contraction-major (x_t / y_t) must give the very
bits of the row-major product: the same elements meet in the same matrix instructions in the same order."""

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
@pytest.mark.parametrize("NX,NY,K", [(256, 256, 128), (512, 256, 192), (260, 300, 256), (768, 1024, 4096), (3584, 512, 1024),
                                     # more than 8 patches of work items with smaller ones at both edges: whole patches go
                                     # to the XCDs, the last few are dealt item by item
                                     (3584, 3008, 384), (2304, 2816, 192)])
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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("NX,NY,K", [(256, 256, 128), (512, 256, 192), (264, 304, 256), (768, 1024, 4096), (3584, 512, 1024),
                                     (1000, 520, 320)])
def test_contraction_major_operands_give_the_same_bits(dev, dtype, NX, NY, K):
    g = torch.Generator(device=dev).manual_seed(NX * 3 + NY + K)
    x = (torch.randn(NX, K, generator=g, device=dev) * 0.5).to(dtype)
    y = (torch.randn(NY, K, generator=g, device=dev) * 0.5).to(dtype)
    xt, yt = x.t().contiguous(), y.t().contiguous()          # (K, NX), (K, NY)
    base = torch.randn(NY, NX, generator=g, device=dev).to(dtype)
    for parts in (None, 2):
        if parts is not None and K // 64 // parts < 2:
            continue
        want = gemm.gemm_nt(x, y, k_parts=parts)
        _check(want, x, y)
        want_acc = base.clone()
        gemm.gemm_nt(x, y, out=want_acc, accumulate=True, k_parts=parts)
        for x_t, y_t in ((True, False), (False, True), (True, True)):
            got = gemm.gemm(xt if x_t else x, yt if y_t else y, x_t, y_t, k_parts=parts)
            assert torch.equal(got, want), (x_t, y_t, parts)
            acc = base.clone()
            gemm.gemm(xt if x_t else x, yt if y_t else y, x_t, y_t, out=acc, accumulate=True, k_parts=parts)
            assert torch.equal(acc, want_acc), (x_t, y_t, parts)


def test_contraction_major_operands_with_row_strides(dev):
    """Views into wider buffers: a contraction-major operand's row stride is the distance between consecutive
    contraction indices."""
    g = torch.Generator(device=dev).manual_seed(11)
    NX, NY, K = 520, 776, 448
    xb = (torch.randn(K, NX + 24, generator=g, device=dev) * 0.5).bfloat16()
    yb = (torch.randn(K, NY + 8, generator=g, device=dev) * 0.5).bfloat16()
    xt, yt = xb[:, 8:8 + NX], yb[:, :NY]
    want = gemm.gemm_nt(xt.t().contiguous(), yt.t().contiguous())
    got = gemm.gemm(xt, yt, True, True)
    assert torch.equal(got, want)
    _check(got, xt.t().contiguous(), yt.t().contiguous())


def test_random_shapes_strides_and_layouts(dev):
    """Seeded random shapes (edge tiles on both sides, odd tile counts, contraction ranges), operands as views into wider
    buffers, every layout pair, stored and accumulated: bit-equal to the row-major product of contiguous copies, which is
    itself checked against fp64."""
    import random

    rng = random.Random(20240607)
    g = torch.Generator(device=dev).manual_seed(17)
    for case in range(12):
        NX = rng.randrange(256, 1100, 8)
        NY = rng.randrange(256, 1100, 8)
        K = rng.randrange(128, 1100, 64)
        dtype = (torch.bfloat16, torch.float16)[case % 2]
        parts = rng.choice([None, 1, 2]) if K >= 256 else None
        x = (torch.randn(NX, K, generator=g, device=dev) * 0.5).to(dtype)
        y = (torch.randn(NY, K, generator=g, device=dev) * 0.5).to(dtype)
        base = torch.randn(NY, NX, generator=g, device=dev).to(dtype)
        want = gemm.gemm_nt(x, y, k_parts=parts)
        _check(want, x, y)
        want_acc = base.clone()
        gemm.gemm_nt(x, y, out=want_acc, accumulate=True, k_parts=parts)

        def widened(t, pad):                      # the same values as a view into a buffer with a longer row
            buf = torch.full((t.shape[0], t.shape[1] + pad), 3.0, dtype=t.dtype, device=dev)
            buf[:, :t.shape[1]] = t
            return buf[:, :t.shape[1]]

        px, py = 8 * rng.randrange(0, 4), 8 * rng.randrange(0, 4)
        for x_t, y_t in ((False, False), (True, False), (False, True), (True, True)):
            xo = widened(x.t().contiguous() if x_t else x, px)
            yo = widened(y.t().contiguous() if y_t else y, py)
            got = gemm.gemm(xo, yo, x_t, y_t, k_parts=parts)
            assert torch.equal(got, want), (case, NX, NY, K, x_t, y_t, parts)
            acc = base.clone()
            gemm.gemm(xo, yo, x_t, y_t, out=acc, accumulate=True, k_parts=parts)
            assert torch.equal(acc, want_acc), (case, NX, NY, K, x_t, y_t, parts)


def test_backward_products_of_the_lm_head_read_in_place(dev):
    """d hidden = G @ W and d W (+)= G.T @ H from G (tokens, vocab), W (vocab, hidden) and H (tokens, hidden) as they
    lie, against the same products through transposed copies (bit-equal) and against fp32 (tolerance)."""
    V, T, D = 151936, 1024, 3584
    g = torch.Generator(device=dev).manual_seed(V)
    G = (torch.randn(T, V, generator=g, device=dev) * 0.01).bfloat16()
    W = (torch.randn(V, D, generator=g, device=dev) * 0.02).bfloat16()
    H = (torch.randn(T, D, generator=g, device=dev) * 0.5).bfloat16()
    dH = gemm.gemm(W, G, x_t=True)                                        # (T, D)
    assert torch.equal(dH, gemm.gemm_nt(W.t().contiguous(), G))
    ref = G.float() @ W.float()
    assert (dH.float() - ref).abs().max().item() <= 2.0 ** -7 * ref.abs().max().item()
    dW = torch.empty(V, D, dtype=torch.bfloat16, device=dev)
    gemm.gemm(H, G, x_t=True, y_t=True, out=dW)                           # (V, D), stored
    gemm.gemm(H, G, x_t=True, y_t=True, out=dW, accumulate=True)          # and added once more
    want = torch.zeros(V, D, dtype=torch.bfloat16, device=dev)
    Ht, Gt = H.t().contiguous(), G.t().contiguous()
    gemm.gemm_nt(Ht, Gt, out=want)
    gemm.gemm_nt(Ht, Gt, out=want, accumulate=True)
    assert torch.equal(dW, want)
    ref = 2.0 * (G.float().t() @ H.float())
    assert (dW.float() - ref).abs().max().item() <= 2.0 ** -6 * ref.abs().max().item()


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
    wide = torch.zeros(256, 264, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        gemm.gemm(wide[:, :260], wide[:, :256], x_t=True)    # a contraction-major operand needs whole groups of 8 rows
    with pytest.raises(ValueError):
        gemm.gemm(wide[:, :256], wide[:, :192], x_t=True)    # contraction lengths differ (256 rows against 192 columns)
