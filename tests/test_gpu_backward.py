"""Backward of the row op (vrl_rowscore_backward through torch.autograd) against torch's autograd of the
oracle's composition on the same inputs.

fp32 logits: absolute 2e-6 (gradient entries are bounded by |g_logprob| + |g_entropy| * (|log p| + H) / T).
bf16 logits: the reference gradient is the fp32 autograd result rounded to bf16; the kernel computes in fp32 and
rounds once, so the two agree to one bf16 ulp (2^-8 relative) plus the fp32 difference.
"""

import pytest
import torch

from verl_amd import torch_functional as vf
from oracle import scoring

pytestmark = pytest.mark.gpu


def _reference_grad(x, lab, temp, w_lp, w_h):
    xr = x.detach().float().requires_grad_(True)
    lp, h = scoring.score_reference(xr, lab, temp)
    loss = 0.0
    if w_lp is not None:
        loss = loss + (lp * w_lp).sum()
    if w_h is not None:
        loss = loss + (h * w_h).sum()
    loss.backward()
    return xr.grad


def _ours(x, lab, temp, w_lp, w_h):
    xo = x.detach().clone().requires_grad_(True)
    lp, h = vf.fused_logprob_entropy(xo, lab, temp)
    loss = 0.0
    if w_lp is not None:
        loss = loss + (lp * w_lp).sum()
    if w_h is not None:
        loss = loss + (h * w_h).sum()
    loss.backward()
    assert xo.grad.dtype == x.dtype and xo.grad.shape == x.shape
    return xo.grad


def _compare(got, ref, dtype, scale=4.0):
    """``scale`` bounds the incoming gradients (|w| of a standard normal stays below 4 here). The exponent
    x*c - lse*log2(e) is formed in fp32 at magnitude ~25, so p carries ~1e-6 relative error: 4e-6 * scale absolute."""
    got, ref = got.float(), ref.float()
    floor = 4e-6 * scale
    if dtype == torch.float32:
        assert (got - ref).abs().max().item() <= floor
    else:
        # one ulp of the 16-bit result (2^-8 relative for bf16, 2^-11 for fp16; fp16 also has subnormals below 6e-5)
        rel = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
        assert ((got - ref).abs() <= ref.abs() * rel + floor + (6e-8 if dtype == torch.float16 else 0.0)).all(), \
            (got - ref).abs().max().item()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,V", [(5, 1), (9, 7), (33, 1000), (17, 4099), (6, 32000), (4, 151936)])
@pytest.mark.parametrize("which", ["both", "logprob", "entropy"])
def test_gradient_matches_torch_autograd(dev, dtype, n, V, which):
    g = torch.Generator(device=dev).manual_seed(n * 100 + V)
    x = (torch.randn(n, V, generator=g, device=dev) * 3).to(dtype)
    lab = torch.randint(0, V, (n,), generator=g, device=dev)
    temp = torch.rand(n, generator=g, device=dev) + 0.5
    w_lp = torch.randn(n, generator=g, device=dev) if which in ("both", "logprob") else None
    w_h = torch.randn(n, generator=g, device=dev) if which in ("both", "entropy") else None
    for t in (None, temp):
        _compare(_ours(x, lab, t, w_lp, w_h), _reference_grad(x, lab, t, w_lp, w_h), dtype)


def test_leading_dims_strided_rows_and_separate_functions(dev):
    g = torch.Generator(device=dev).manual_seed(8)
    base = torch.randn(3, 4, 1030, generator=g, device=dev)
    lab = torch.randint(0, 1021, (3, 4), generator=g, device=dev)
    w1 = torch.randn(3, 4, generator=g, device=dev)
    w2 = torch.randn(3, 4, generator=g, device=dev)
    # a strided, misaligned view: rows start 3 elements into each 1030-element row
    leaf = base.clone().requires_grad_(True)
    view = leaf[..., 3:1024]
    lp = vf.logprobs_from_logits(view, lab, inplace_backward=False)
    h = vf.entropy_from_logits(view)
    ((lp * w1).sum() + (h * w2).sum()).backward()
    ref_leaf = base.clone().requires_grad_(True)
    rlp = scoring.logprobs_from_logits(ref_leaf[..., 3:1024], lab)
    rh = scoring.entropy_from_logits(ref_leaf[..., 3:1024])
    ((rlp * w1).sum() + (rh * w2).sum()).backward()
    assert (leaf.grad - ref_leaf.grad).abs().max().item() <= 1.6e-5
    assert leaf.grad[..., :3].abs().max().item() == 0


def test_inplace_backward_writes_over_the_logits(dev):
    g = torch.Generator(device=dev).manual_seed(9)
    leaf = (torch.randn(64, 5000, generator=g, device=dev)).requires_grad_(True)
    lab = torch.randint(0, 5000, (64,), generator=g, device=dev)
    w = torch.randn(64, generator=g, device=dev)
    z = leaf * 1.0                      # a non-leaf tensor, like `logits / temperature` in the engine
    ptr = z.data_ptr()
    lp = vf.logprobs_from_logits(z, lab)            # inplace_backward=True by default, as in the reference
    (lp * w).sum().backward()
    ref = _reference_grad(leaf, lab, None, w, None)
    assert (leaf.grad - ref).abs().max().item() <= 1.6e-5
    assert z.data_ptr() == ptr and (z.detach() - ref).abs().max().item() <= 1.6e-5   # z now holds its own gradient
    # a leaf is never overwritten
    leaf2 = leaf.detach().clone().requires_grad_(True)
    keep = leaf2.detach().clone()
    (vf.logprobs_from_logits(leaf2, lab) * w).sum().backward()
    assert torch.equal(leaf2.detach(), keep) and (leaf2.grad - ref).abs().max().item() <= 1.6e-5


def test_minus_inf_logits_and_unused_outputs(dev):
    x = torch.randn(4, 300, device=dev)
    x[0, :50] = float("-inf")
    lab = torch.tensor([100, 1, 2, 3], device=dev)
    xo = x.clone().requires_grad_(True)
    lp, h = vf.fused_logprob_entropy(xo, lab)
    lp.sum().backward()                      # entropy unused: its gradient is absent, not zero-filled
    ref = _reference_grad(x, lab, None, torch.ones(4, device=dev), None)
    assert torch.isfinite(xo.grad).all() and (xo.grad - ref).abs().max().item() <= 4e-6
    assert xo.grad[0, :50].abs().max().item() == 0
    # no grad requested: plain forward, no graph
    with torch.no_grad():
        lp2, _ = vf.fused_logprob_entropy(xo, lab)
    assert not lp2.requires_grad and torch.equal(lp2, lp.detach())


def test_full_vocab_bf16_c3_shape_slice(dev):
    """256 rows of the c3 shape (V = 151936 bf16), both gradients, temperature 0.7."""
    g = torch.Generator(device=dev).manual_seed(12)
    n, V = 256, 151936
    x = (torch.randn(n, V, generator=g, device=dev) * 3).bfloat16()
    lab = torch.randint(0, V, (n,), generator=g, device=dev)
    temp = torch.full((n,), 0.7, device=dev)
    w1 = torch.randn(n, generator=g, device=dev)
    w2 = torch.randn(n, generator=g, device=dev)
    _compare(_ours(x, lab, temp, w1, w2), _reference_grad(x, lab, temp, w1, w2).bfloat16(), torch.bfloat16)


@pytest.mark.parametrize("use_reentrant", [False, True])
def test_entropy_under_activation_checkpointing(dev, use_reentrant):
    """The engines may wrap the entropy function in torch.utils.checkpoint (entropy_checkpointing,
    fsdp/transformer_impl.py:1371-1374 in the reference): the forward then runs twice, the gradient is the same."""
    from torch.utils.checkpoint import checkpoint

    g = torch.Generator(device=dev).manual_seed(21)
    x = (torch.randn(40, 5003, generator=g, device=dev) * 2).requires_grad_(True)
    w = torch.randn(40, generator=g, device=dev)
    (vf.entropy_from_logits(x * 1.0) * w).sum().backward()
    plain = x.grad.clone()
    x.grad = None
    h = checkpoint(vf.entropy_from_logits, x * 1.0, use_reentrant=use_reentrant)
    (h * w).sum().backward()
    assert torch.equal(x.grad, plain)


def test_fp32_peaked_rows_at_low_temperature_stay_as_close_to_fp64_as_torch(dev):
    """|z| ~ 100 (logits up to 35 at temperature 0.36): the exponent must not pick up roundings of size ulp(|z|) that
    torch's own fp32 autograd does not have. Compared with the fp64 gradient of the same composition."""
    g = torch.Generator(device=dev).manual_seed(31)
    n, V = 6, 58902
    x = torch.randn(n, V, generator=g, device=dev) * 8.0
    x[torch.arange(n), torch.randint(0, V, (n,), generator=g, device=dev)] = 35.0
    lab = torch.randint(0, V, (n,), generator=g, device=dev)
    temp = torch.tensor([0.36, 0.5, 0.7, 1.0, 1.8, 0.36], device=dev)
    g1 = torch.randn(n, generator=g, device=dev)
    g2 = torch.randn(n, generator=g, device=dev) * 0.3

    def grad(xx, fn, cast):
        xx = xx.requires_grad_(True)
        lp, h = fn(xx)
        ((lp * g1.to(cast)).sum() + (h * g2.to(cast)).sum()).backward()
        return xx.grad

    g64 = grad(x.double(), lambda t: scoring.score_reference(t, lab, temp.double()), torch.float64)
    g32 = grad(x.clone(), lambda t: scoring.score_reference(t, lab, temp), torch.float32)
    ours = grad(x.clone(), lambda t: vf.fused_logprob_entropy(t, lab, temp), torch.float32)
    e_torch = (g32.double() - g64).abs().max().item()
    e_ours = (ours.double() - g64).abs().max().item()
    assert e_ours <= 2.0 * e_torch + 2e-6, (e_ours, e_torch)


@pytest.mark.parametrize("dtype,n,V", [(torch.bfloat16, 1100, 32760), (torch.float32, 1100, 16388),
                                       (torch.float16, 600, 65544),
                                       # rows of 513 vectors, one more than a wavefront's trip: nearly every trip holds two rows
                                       (torch.bfloat16, 8300, 4104), (torch.float32, 8300, 2052)])
def test_rows_back_to_back_take_the_walk_without_rows_with_the_same_bits(dev, dtype, n, V):
    """Contiguous rows of 64 MiB or more are differentiated by workgroups that walk them as one array
    (rowscore_backward_flat_kernel), every other input by one workgroup per row: same arithmetic per element, so the same
    bits. Rows here are no multiple of a wavefront's 512-vector trip, so trips straddle rows; labels sit on the first and
    last element of rows and on both sides of vector borders; also in place."""
    from verl_amd import _lib

    lib = _lib.load()
    code = {torch.float32: _lib.VRL_F32, torch.bfloat16: _lib.VRL_BF16, torch.float16: _lib.VRL_F16}[dtype]
    g = torch.Generator(device=dev).manual_seed(n + V)
    x = (torch.randn(n, V, generator=g, device=dev) * 3).to(dtype)
    assert x.numel() * x.element_size() >= (1 << 26)
    lab = torch.randint(0, V, (n,), generator=g, device=dev)
    per_vec = 16 // x.element_size()
    lab[:8] = torch.tensor([0, V - 1, per_vec - 1, per_vec, V - per_vec, V - per_vec - 1, 1, V // 2], device=dev)
    temp = torch.rand(n, generator=g, device=dev) + 0.5
    lse = torch.logsumexp(x.float() / temp[:, None], -1)
    ent = torch.rand(n, generator=g, device=dev) * 4
    gl = torch.randn(n, generator=g, device=dev)
    gh = torch.randn(n, generator=g, device=dev)
    wide = torch.zeros(n, V + 2 * per_vec, dtype=dtype, device=dev)        # the same rows with a pitch: one workgroup per row
    wide[:, :V] = x
    out_flat = torch.empty_like(x)
    out_rows = torch.zeros_like(wide)
    stream = _lib.stream_ptr(dev)
    with torch.cuda.device(dev):
        for src, dst in ((x, out_flat), (wide, out_rows)):
            st = lib.vrl_rowscore_backward(src.data_ptr(), code, n, V, src.stride(0), lab.data_ptr(), temp.data_ptr(),
                                           lse.data_ptr(), ent.data_ptr(), gl.data_ptr(), gh.data_ptr(), dst.data_ptr(),
                                           dst.stride(0), stream)
            assert st == _lib.VRL_OK
        bits = torch.int16 if x.element_size() == 2 else torch.int32
        assert torch.equal(out_flat.view(bits), out_rows[:, :V].contiguous().view(bits))
        assert not bool(out_rows[:, V:].any())
        # the label term landed where it belongs: the gradient of the log-prob alone sums to g / T * (1 - 1) = 0 per row
        st = lib.vrl_rowscore_backward(x.data_ptr(), code, n, V, V, lab.data_ptr(), temp.data_ptr(), lse.data_ptr(), None,
                                       gl.data_ptr(), None, out_flat.data_ptr(), V, stream)
        assert st == _lib.VRL_OK
        sums = out_flat.double().sum(-1)
        tol = 2e-2 if dtype != torch.float32 else 1e-4
        assert bool((sums.abs() <= tol * (gl.abs().double() / temp.double() + 1)).all()), sums.abs().max().item()
        # in place
        y = x.clone()
        st = lib.vrl_rowscore_backward(y.data_ptr(), code, n, V, V, lab.data_ptr(), temp.data_ptr(), lse.data_ptr(),
                                       ent.data_ptr(), gl.data_ptr(), gh.data_ptr(), y.data_ptr(), V, stream)
        assert st == _lib.VRL_OK
        assert torch.equal(y.view(bits), out_rows[:, :V].contiguous().view(bits))
