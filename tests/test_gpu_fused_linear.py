"""LM head + scoring in token chunks (verl_amd.fused_linear) against torch on the same inputs.

Tolerances are the reference's own for this comparison (tests/utils/test_linear_cross_entropy.py:211-224,
261-269): forward atol = rtol = 1e-4 against the fp32 torch composition, gradients atol 1e-2 / rtol 1e-4,
with inputs drawn like there (uniform(-0.5, 0.5), temperature 1.5).
"""

import pytest
import torch

from verl_amd.fused_linear import linear_cross_entropy, FusedLinearForPPO, fused_linear_for_ppo
from oracle import fused_linear as ofl

pytestmark = pytest.mark.gpu


def _torch_reference(hidden, weight, labels, temperature):
    """The reference's composition in fp32 (run_torch_entropy of its test, tests/utils/test_linear_cross_entropy.py:97-118),
    as oracle/fused_linear.py states it; differentiable with respect to hidden and weight."""
    lp, ent, _ = ofl.forward(hidden, weight, labels, temperature, dtype=torch.float32)
    return lp, ent


@pytest.mark.parametrize("T,D,V,chunk", [(300, 256, 32256, 128), (257, 128, 10007, 512), (64, 64, 151936, 17)])
def test_fp32_forward_and_backward_match_torch(dev, T, D, V, chunk):
    g = torch.Generator(device=dev).manual_seed(T + V)
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).requires_grad_()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    g_ent = torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=g)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    temperature = 1.5

    ref_lp, ref_ent = _torch_reference(hidden, weight, labels, temperature)
    d_ref_h, d_ref_w = torch.autograd.grad((ref_ent, ref_lp), (hidden, weight), (g_ent, g_lp))

    from verl_amd import gemm

    before = gemm.counters["gemm"]
    lp, ent = fused_linear_for_ppo(hidden, weight, labels, temperature, chunk_size=chunk, keep_logits=False)
    assert lp.dtype == torch.float32 and lp.shape == (T,) and ent.shape == (T,)
    torch.testing.assert_close(ref_lp, lp, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(ref_ent, ent, atol=1e-4, rtol=1e-4)
    d_h, d_w = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
    torch.testing.assert_close(d_ref_h, d_h, atol=1e-2, rtol=1e-4)
    torch.testing.assert_close(d_ref_w, d_w, atol=1e-2, rtol=1e-4)
    # much closer than the reference asks for
    assert (d_ref_h - d_h).abs().max().item() <= 2e-4 and (d_ref_w - d_w).abs().max().item() <= 2e-4
    # an fp32 model is served by the library GEMM + the row kernels on purpose: none of the 16-bit matrix-core products ran
    assert gemm.counters["gemm"] == before


def test_bf16_module_3d_inputs(dev):
    """bf16 like the engine runs it; 3-D hidden states as the reference's module accepts them."""
    g = torch.Generator(device=dev).manual_seed(5)
    B, S, D, V = 2, 150, 256, 32256
    hidden = torch.empty(B, S, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    labels = torch.randint(0, V, (B, S), generator=g, device=dev)
    # the default forward keeps the logits in fp32: it sits on the all-fp32 reference
    d_lp, d_ent = FusedLinearForPPO(chunk_size=64, keep_logits=False)(hidden, weight, labels, temperature=1.5)
    f_lp, f_ent = _torch_reference(hidden.detach().view(-1, D), weight.detach(), labels.view(-1), 1.5)
    assert (d_lp.view(-1) - f_lp).abs().max().item() <= 1e-4 and (d_ent.view(-1) - f_ent).abs().max().item() <= 1e-4
    mod = FusedLinearForPPO(chunk_size=64, keep_logits=False, kernels="library")
    lp, ent = mod(hidden, weight, labels, temperature=1.5)
    assert lp.shape == (B, S) and ent.shape == (B, S)
    # the kernels' share, exactly: fp32 math on the bf16 logits the library GEMM produced
    logits = torch.matmul(hidden.detach().view(-1, D), weight.detach().t()).float() / 1.5
    ref_lp = torch.log_softmax(logits, -1).gather(-1, labels.view(-1, 1)).squeeze(-1)
    ref_ent = torch.logsumexp(logits, -1) - (torch.softmax(logits, -1) * logits).sum(-1)
    assert (lp.view(-1) - ref_lp).abs().max().item() <= 2e-3 and (ent.view(-1) - ref_ent).abs().max().item() <= 2e-3
    # against the all-fp32 reference the difference is the bf16 rounding of the logits (|logit| ~ 2.3 here)
    f_lp, f_ent = _torch_reference(hidden.detach().view(-1, D), weight.detach(), labels.view(-1), 1.5)
    assert (lp.view(-1) - f_lp).abs().max().item() <= 5e-2
    g_lp = torch.empty(B, S, device=dev).uniform_(-1, 1, generator=g)
    g_ent = torch.empty(B, S, device=dev).uniform_(-0.5, 0.5, generator=g)
    d_h, d_w = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
    hf = hidden.detach().float().requires_grad_()
    wf = weight.detach().float().requires_grad_()
    r_lp, r_ent = _torch_reference(hf.view(-1, D), wf, labels.view(-1), 1.5)
    d_rh, d_rw = torch.autograd.grad((r_ent, r_lp), (hf, wf), (g_ent.view(-1), g_lp.view(-1)))
    assert d_h.dtype == torch.bfloat16 and d_h.shape == hidden.shape and d_w.shape == weight.shape
    torch.testing.assert_close(d_rh, d_h.float(), atol=2e-2, rtol=4e-2)   # the reference's bf16-kernel tolerance (:271-276)
    torch.testing.assert_close(d_rw, d_w.float(), atol=2e-2, rtol=4e-2)


def test_bf16_long_batch_uses_transposed_operands(dev):
    """From 2048 tokens on the backward multiplies by a transposed copy of the weight (and always by a transposed
    copy of the hidden chunk for 16-bit operands): same gradients as the products on the operands as stored."""
    g = torch.Generator(device=dev).manual_seed(11)
    T, D, V = 2304, 192, 20011
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    g_ent = torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=g)
    lp, ent = fused_linear_for_ppo(hidden, weight, labels, 0.9, chunk_size=1000, keep_logits=False)
    d_h, d_w = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
    lp1, ent1 = fused_linear_for_ppo(hidden, weight, labels, 0.9)          # default chunk: one chunk here
    # the library may sum a product of another height in another order: a bf16 logit can move by one rounding step
    torch.testing.assert_close(lp, lp1, atol=2e-2, rtol=0)
    torch.testing.assert_close(ent, ent1, atol=2e-2, rtol=0)
    hf = hidden.detach().float().requires_grad_()
    wf = weight.detach().float().requires_grad_()
    r_lp, r_ent = _torch_reference(hf, wf, labels, 0.9)
    d_rh, d_rw = torch.autograd.grad((r_ent, r_lp), (hf, wf), (g_ent, g_lp))
    torch.testing.assert_close(d_rh, d_h.float(), atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(d_rw, d_w.float(), atol=2e-2, rtol=4e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_keep_logits_same_results_one_backward(dev, dtype):
    g = torch.Generator(device=dev).manual_seed(12)
    T, D, V = 2100, 128, 10007
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).to(dtype).requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).to(dtype).requires_grad_()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    g_ent = torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=g)
    lp0, ent0 = fused_linear_for_ppo(hidden, weight, labels, 1.3, chunk_size=512, keep_logits=False)
    dh0, dw0 = torch.autograd.grad((ent0, lp0), (hidden, weight), (g_ent, g_lp))
    lp1, ent1 = fused_linear_for_ppo(hidden, weight, labels, 1.3, chunk_size=512, keep_logits=True)
    assert torch.equal(lp0, lp1) and torch.equal(ent0, ent1)
    dh1, dw1 = torch.autograd.grad((ent1, lp1), (hidden, weight), (g_ent, g_lp), retain_graph=True)
    # same per-token gradient over the logits; the products differ in summation order (and, for d W, in not being
    # rounded to the operand type once per chunk)
    tol = dict(atol=2e-2, rtol=4e-2) if dtype == torch.bfloat16 else dict(atol=2e-5, rtol=1e-4)
    torch.testing.assert_close(dh0.float(), dh1.float(), **tol)
    torch.testing.assert_close(dw0.float(), dw1.float(), **tol)
    with pytest.raises(RuntimeError, match="overwritten by the first backward"):
        torch.autograd.grad((ent1, lp1), (hidden, weight), (g_ent, g_lp))
    # without gradients nothing is kept
    with torch.no_grad():
        lp2, _ = fused_linear_for_ppo(hidden, weight, labels, 1.3, chunk_size=512, keep_logits=True)
    assert torch.equal(lp2, lp0)
    mod = FusedLinearForPPO(chunk_size=512, keep_logits=True)
    lp3, ent3 = mod(hidden, weight, labels, 1.3)
    assert torch.equal(lp3, lp0)


def test_linear_cross_entropy_call_and_reductions(dev):
    """The call of the reference's Triton-backed function (verl/utils/kernel/linear_cross_entropy.py:38-119): 3-D
    hidden states, flattened fp32 outputs, reduction on the log-probs only; checked the way the reference checks its
    kernel against torch (tests/utils/test_linear_cross_entropy.py:211-224)."""
    g = torch.Generator(device=dev).manual_seed(9)
    B, S, D, V = 2, 70, 128, 4099
    hidden = torch.empty(B, S, D, device=dev).uniform_(-0.5, 0.5, generator=g).requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).requires_grad_()
    labels = torch.randint(0, V, (B, S), generator=g, device=dev)
    ref_lp, ref_ent = _torch_reference(hidden.detach().view(-1, D), weight.detach(), labels.view(-1), 1.5)
    lp, ent = linear_cross_entropy(hidden, weight, labels, 1.5, "none")
    assert lp.shape == (B * S,) and ent.shape == (B * S,) and lp.dtype == torch.float32
    torch.testing.assert_close(lp, ref_lp, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(ent, ref_ent, atol=1e-4, rtol=1e-4)
    for red, want in (("sum", ref_lp.sum()), ("mean", ref_lp.mean()), ("MEAN", ref_lp.mean())):
        lp_r, ent_r = linear_cross_entropy(hidden, weight, labels, 1.5, red)
        assert lp_r.shape == () and ent_r.shape == (B * S,)
        torch.testing.assert_close(lp_r, want, atol=1e-3, rtol=1e-4)
    lp_m, ent_m = linear_cross_entropy(hidden, weight, labels, 1.5, "mean")
    (lp_m + ent_m.sum()).backward()
    hf = hidden.detach().clone().requires_grad_()
    wf = weight.detach().clone().requires_grad_()
    r_lp, r_ent = _torch_reference(hf.view(-1, D), wf, labels.view(-1), 1.5)
    (r_lp.mean() + r_ent.sum()).backward()
    torch.testing.assert_close(hidden.grad, hf.grad, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(weight.grad, wf.grad, atol=1e-4, rtol=1e-4)
    with pytest.raises(ValueError, match="Invalid reduction"):
        linear_cross_entropy(hidden, weight, labels, 1.5, "max")
    with pytest.raises(TypeError):
        linear_cross_entropy(hidden, weight, labels, 1)
    with pytest.raises(NotImplementedError):
        linear_cross_entropy(hidden, weight, labels, 1.5, "none", dist_process_group=object())


def test_input_checks(dev):
    h = torch.randn(4, 8, device=dev)
    w = torch.randn(16, 8, device=dev)
    ids = torch.zeros(4, dtype=torch.long, device=dev)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        fused_linear_for_ppo(h.cpu(), w.cpu(), ids.cpu())
    with pytest.raises(TypeError):
        fused_linear_for_ppo(h, w.bfloat16(), ids)
    with pytest.raises(ValueError):
        fused_linear_for_ppo(h, w, ids[:3])
    with pytest.raises(ValueError):
        fused_linear_for_ppo(h, w, ids, chunk_size=0, keep_logits=False)
    with pytest.raises(IndexError):
        fused_linear_for_ppo(h, w, torch.full((4,), 16, device=dev))
    # the kernels read the ids through a raw device pointer: ids that live on the host are moved, never dereferenced
    got = fused_linear_for_ppo(h, w, ids.cpu())
    want = fused_linear_for_ppo(h, w, ids)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    with pytest.raises(TypeError):
        fused_linear_for_ppo(h, w, ids.float())
    with pytest.raises(TypeError):
        fused_linear_for_ppo(h, w, ids.bool())
    lp, ent = fused_linear_for_ppo(h[:0], w, ids[:0])
    assert lp.shape == (0,) and ent.shape == (0,)
