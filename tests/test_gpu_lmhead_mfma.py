"""vrl_lmhead_score (LM head + scoring in one matrix-core kernel, no logits in memory) against torch.

The kernel keeps the logits in fp32, so the reference is the all-fp32 composition on the same bf16/fp16 operands
(products of 16-bit values are exact in fp32; only the summation order differs): 2e-5 absolute at these sizes.
Against the library-GEMM path (which rounds the logits to the operand type) the difference is that rounding."""

import pytest
import torch

from verl_amd import _lib
from verl_amd.fused_linear import fused_linear_for_ppo, lm_head_score_mfma
from oracle import fused_linear as ofl

pytestmark = pytest.mark.gpu


def _reference(h, w, ids, temp):
    """fp64 value of the reference's forward on these operands (oracle/fused_linear.py, pinned on the CPU by
    tests/test_oracle_fused_linear.py)."""
    lp, ent, _ = ofl.forward(h, w, ids, temp, dtype=torch.float64)
    return lp, ent


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,V,K,splits", [(256, 256, 64, 1), (256, 512, 128, 2), (512, 1024, 256, 3), (300, 700, 192, 2),
                                          (1000, 300, 64, 1), (257, 18992, 512, None), (2048, 4099, 320, None),
                                          (1024, 32000, 1024, 8)])
def test_matches_fp64_composition(dev, dtype, T, V, K, splits):
    g = torch.Generator(device=dev).manual_seed(T + V + K)
    h = (torch.randn(T, K, generator=g, device=dev) * 0.5).to(dtype)
    w = (torch.randn(V, K, generator=g, device=dev) * 0.2).to(dtype)
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    temp = torch.rand(T, generator=g, device=dev) + 0.5
    for t in (1.0, 0.7, temp):
        lp, ent = lm_head_score_mfma(h, w, ids, t, n_splits=splits)
        r_lp, r_ent = _reference(h, w, ids, None if t == 1.0 else t) if not isinstance(t, torch.Tensor) else _reference(h, w, ids, t)
        assert lp.dtype == torch.float32 and lp.shape == (T,)
        assert (lp.double() - r_lp).abs().max().item() <= 2e-5
        assert (ent.double() - r_ent).abs().max().item() <= 2e-5


def test_xcd_aware_workgroup_order_covers_every_token_block_and_split(dev):
    """32 token blocks x 8 splits takes the XCD-aware (token block, split) mapping of the workgroups (it needs the
    block count to divide by 8 and the split count by 4): every token of every block must come out right, which a
    wrong mapping (a block or split served twice, another never) would not."""
    T, V, K, splits = 8192, 8192, 256, 8
    g = torch.Generator(device=dev).manual_seed(99)
    h = (torch.randn(T, K, generator=g, device=dev) * 0.5).bfloat16()
    w = (torch.randn(V, K, generator=g, device=dev) * 0.2).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    temp = torch.rand(T, generator=g, device=dev) + 0.5
    lp, ent = lm_head_score_mfma(h, w, ids, temp, n_splits=splits)
    r_lp, r_ent = _reference(h, w, ids, temp)
    assert (lp.double() - r_lp).abs().max().item() <= 2e-5
    assert (ent.double() - r_ent).abs().max().item() <= 2e-5


def test_benchmark_shape_against_the_chunked_fp64_composition(dev):
    """8192 tokens x 3584 -> 152064 bf16 (the shape bench.py --lm-head times; 594 vocabulary tiles over 8 splits,
    the last split shorter, XCD-aware order): all tokens against the fp64 composition, formed 256 tokens at a time."""
    T, K, V = 8192, 3584, 152064
    g = torch.Generator(device=dev).manual_seed(4000)
    h = torch.empty(T, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    w = (torch.empty(V, K, device=dev).uniform_(-0.5, 0.5, generator=g) * 0.05).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    lp, ent = lm_head_score_mfma(h, w, ids, 1.5)
    w64 = w.double()
    worst_lp = worst_ent = 0.0
    for lo in range(0, T, 256):
        r_lp, r_ent = _reference(h[lo:lo + 256], w64, ids[lo:lo + 256], 1.5)
        worst_lp = max(worst_lp, (lp[lo:lo + 256].double() - r_lp).abs().max().item())
        worst_ent = max(worst_ent, (ent[lo:lo + 256].double() - r_ent).abs().max().item())
    print(f"[lmhead 8192x3584->152064] max abs err vs fp64: log-prob {worst_lp:.2e}, entropy {worst_ent:.2e}", flush=True)
    assert worst_lp <= 2e-5 and worst_ent <= 2e-5


def _dlogits_reference(h, w, ids, temp, g_lp, g_h):
    """fp64 gradient of sum(g_lp * logprob + g_h * entropy) with respect to the logits (closed form of
    verl/utils/experimental/torch_functional.py:66-78 as oracle/fused_linear.py states it), with the logsumexp and
    entropy the backward kernel is handed."""
    z = ofl.logits_of(h, w, temp, dtype=torch.float64)
    lp, ent, lse = ofl.forward(h, w, ids, temp, dtype=torch.float64)
    d = ofl.dlogits(z, ids, None if g_lp is None else g_lp.double(), None if g_h is None else g_h.double(), temp)
    return d, lse, ent


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,V,K,splits", [(256, 256, 64, 1), (300, 704, 192, 2), (512, 1024, 256, 3), (1000, 304, 64, 1),
                                          (257, 18992, 512, None), (2048, 4104, 320, None)])
def test_dlogits_matches_fp64_autograd(dev, dtype, T, V, K, splits):
    """vrl_lmhead_dlogits (logits formed again on the matrix cores, gradient written from registers) against the fp64
    gradient: the result is the fp32 formula rounded once to the operand type (half an ulp of it, 2^-9 relative for
    bf16, 2^-12 for fp16) plus the fp32 arithmetic's own 1e-6. Edge tiles in both directions, every combination of
    incoming gradients, per-token temperatures."""
    lib = _lib.load()
    g = torch.Generator(device=dev).manual_seed(T * 3 + V + K)
    h = (torch.randn(T, K, generator=g, device=dev) * 0.5).to(dtype)
    w = (torch.randn(V, K, generator=g, device=dev) * 0.2).to(dtype)
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    temp = torch.rand(T, generator=g, device=dev) + 0.5
    g_lp = torch.randn(T, generator=g, device=dev)
    g_h = torch.randn(T, generator=g, device=dev) * 0.3
    code = _lib.VRL_BF16 if dtype == torch.bfloat16 else _lib.VRL_F16
    n_splits = lib.vrl_lmhead_plan(T, V) if splits is None else splits
    pitch = V + 8     # rows of the output need not be dense
    for gl, gh, tt in ((g_lp, g_h, temp), (g_lp, None, None), (None, g_h, temp)):
        want, lse, ent = _dlogits_reference(h, w, ids, tt, gl, gh)
        lse32, ent32 = lse.float().contiguous(), ent.float().contiguous()
        out = torch.full((T, pitch), float("nan"), dtype=dtype, device=dev)
        with torch.cuda.device(dev):
            st = lib.vrl_lmhead_dlogits(h.data_ptr(), w.data_ptr(), code, T, V, K, K, K, ids.data_ptr(),
                                        None if tt is None else tt.data_ptr(), lse32.data_ptr(), ent32.data_ptr(),
                                        None if gl is None else gl.data_ptr(), None if gh is None else gh.data_ptr(),
                                        n_splits, out.data_ptr(), pitch, _lib.stream_ptr(dev))
        assert st == _lib.VRL_OK, lib.vrl_strerror(st)
        got = out[:, :V].double()
        assert torch.isfinite(got).all()                       # every element of the (T, V) block was written
        assert torch.isnan(out[:, V:].float()).all()           # and nothing beyond it
        rel = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        err = (got - want).abs()
        assert bool((err <= rel * want.abs() + 2e-6).all()), err.max().item()


@pytest.mark.parametrize("kernels", ["auto", "mfma"])
def test_backward_products_come_from_the_matrix_core_kernel(dev, kernels):
    """Unless told "library", the backward forms d hidden and d W with vrl_gemm, reading the weight, the hidden states and
    the gradient buffer in place: same tolerances against torch autograd as the other paths, and the launches are
    counted (two per chunk; with kept logits one d hidden and one d W product over all tokens)."""
    from verl_amd import gemm

    g = torch.Generator(device=dev).manual_seed(78)
    T, D, V = 2304, 512, 32256
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    g_ent = torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=g)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    logits = torch.matmul(hidden.float(), weight.float().t()) / 1.5
    ref_ent = torch.logsumexp(logits, -1) - (torch.softmax(logits, -1) * logits).sum(-1)
    ref_lp = -torch.nn.functional.cross_entropy(logits, labels, reduction="none")
    d_ref_h, d_ref_w = torch.autograd.grad((ref_ent, ref_lp), (hidden, weight), (g_ent, g_lp))
    for chunk, keep, launches in ((1024, False, 6), (4096, False, 2), (4096, True, 2)):
        before = gemm.counters["gemm"]
        lp, ent = fused_linear_for_ppo(hidden, weight, labels, 1.5, chunk_size=chunk, keep_logits=keep, kernels=kernels)
        d_h, d_w = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
        assert gemm.counters["gemm"] == before + launches
        torch.testing.assert_close(d_ref_h.float(), d_h.float(), atol=1e-2, rtol=1e-2)
        torch.testing.assert_close(d_ref_w.float(), d_w.float(), atol=1e-2, rtol=1e-2)
    before = gemm.counters["gemm"]
    lp, ent = fused_linear_for_ppo(hidden, weight, labels, 1.5, kernels="library")
    torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
    assert gemm.counters["gemm"] == before


def test_benchmark_shape_backward_against_fp64(dev):
    """8192 tokens x 3584 -> 152064 bf16, chunks of 4096 (what bench.py --lm-head times): d hidden and d W of the
    recomputing path (vrl_lmhead_dlogits + vrl_gemm, two chunks, the second accumulated) and of the default at this size
    (logits kept by the forward kernel, vrl_rowscore_backward in place, one product each) against the closed-form gradient in fp64,
    formed 1024 tokens at a time; the all-library path is measured against the same reference beside it. Bar: 2^-7 +
    2^-10 of the largest reference element: a row of either gradient is dominated by its label term, whose factor from
    the gradient buffer is rounded to bf16 once (up to 2^-8 relative) before the product is rounded to bf16 again (2^-8);
    both paths round that factor alike, so their errors agree to three digits (6.5e-3 and 6.2e-3)."""
    T, K, V = 8192, 3584, 152064
    temp = 1.5
    g = torch.Generator(device=dev).manual_seed(4001)
    h = torch.empty(T, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    w = (torch.empty(V, K, device=dev).uniform_(-0.5, 0.5, generator=g) * 0.05).bfloat16().requires_grad_()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    g_ent = torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=g)
    got = {}
    for name, kernels, keep in (("auto", "auto", False), ("library", "library", False), ("auto, logits kept", "auto", None)):
        lp, ent = fused_linear_for_ppo(h, w, ids, temp, chunk_size=4096, keep_logits=keep, kernels=kernels)
        got[name] = torch.autograd.grad((lp, ent), (h, w), (g_lp, g_ent))
        del lp, ent
    w64 = w.detach().double()
    ref_dw = torch.zeros(V, K, dtype=torch.float64, device=dev)
    ref_dh = torch.empty(T, K, dtype=torch.float64, device=dev)
    for lo in range(0, T, 1024):
        h64 = h.detach()[lo:lo + 1024].double()
        z = (h64 @ w64.t()) / temp
        logp = torch.log_softmax(z, -1)
        p = logp.exp()
        ent64 = -(p * logp).sum(-1)
        G = -(g_ent[lo:lo + 1024].double()[:, None]) * p * (logp + ent64[:, None]) - g_lp[lo:lo + 1024].double()[:, None] * p
        G[torch.arange(G.shape[0], device=dev), ids[lo:lo + 1024]] += g_lp[lo:lo + 1024].double()
        G /= temp
        ref_dh[lo:lo + 1024] = G @ w64
        ref_dw += G.t() @ h64
        del z, logp, p, G
    for kernels, (dh, dw) in got.items():
        e_h = (dh.double() - ref_dh).abs().max().item() / ref_dh.abs().max().item()
        e_w = (dw.double() - ref_dw).abs().max().item() / ref_dw.abs().max().item()
        print(f"[lmhead backward 8192x3584->152064, kernels={kernels}] max err / max |ref|: d hidden {e_h:.2e}, d W {e_w:.2e}",
              flush=True)
        assert e_h <= 2.0 ** -7 + 2.0 ** -10 and e_w <= 2.0 ** -7 + 2.0 ** -10, (kernels, e_h, e_w)


def test_fused_linear_with_the_matrix_core_kernels(dev):
    """fused_linear_for_ppo(kernels="mfma"): forward from vrl_lmhead_score, backward through vrl_lmhead_dlogits and the
    two products, against torch autograd on the fp32 composition at the reference's tolerances
    (tests/utils/test_linear_cross_entropy.py:261-276) and against the library-GEMM path."""
    g = torch.Generator(device=dev).manual_seed(77)
    T, D, V = 1200, 256, 32256
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    g_ent = torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=g)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    logits = torch.matmul(hidden.float(), weight.float().t()) / 1.5
    ref_ent = torch.logsumexp(logits, -1) - (torch.softmax(logits, -1) * logits).sum(-1)
    ref_lp = -torch.nn.functional.cross_entropy(logits, labels, reduction="none")
    d_ref_h, d_ref_w = torch.autograd.grad((ref_ent, ref_lp), (hidden, weight), (g_ent, g_lp))
    for chunk in (512, 4096):
        lp, ent = fused_linear_for_ppo(hidden, weight, labels, 1.5, chunk_size=chunk, keep_logits=False, kernels="mfma")
        torch.testing.assert_close(ref_lp, lp, atol=1e-4, rtol=1e-4)     # the same single kernel with gradients: fp32 logits
        torch.testing.assert_close(ref_ent, ent, atol=1e-4, rtol=1e-4)
        d_h, d_w = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
        assert d_h.dtype == torch.bfloat16 and d_w.dtype == torch.bfloat16
        torch.testing.assert_close(d_ref_h.float(), d_h.float(), atol=1e-2, rtol=1e-2)
        torch.testing.assert_close(d_ref_w.float(), d_w.float(), atol=1e-2, rtol=1e-2)
        lp2, ent2 = fused_linear_for_ppo(hidden, weight, labels, 1.5, chunk_size=chunk, keep_logits=False, kernels="library")
        d_h2, d_w2 = torch.autograd.grad((ent2, lp2), (hidden, weight), (g_ent, g_lp))
        assert (d_h.float() - d_h2.float()).abs().max().item() <= 2e-2 * max(d_h2.float().abs().max().item(), 1e-3)
        assert (d_w.float() - d_w2.float()).abs().max().item() <= 2e-2 * max(d_w2.float().abs().max().item(), 1e-3)
    # without gradients the same switch takes the single forward kernel: fp32 logits, no buffer
    with torch.no_grad():
        lp, ent = fused_linear_for_ppo(hidden, weight, labels, 1.5, kernels="mfma")
    torch.testing.assert_close(ref_lp, lp, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(ref_ent, ent, atol=1e-4, rtol=1e-4)
    with pytest.raises(ValueError):
        fused_linear_for_ppo(hidden, weight, labels, 1.5, kernels="cublas")


def test_fused_linear_fp16_model(dev):
    """The same default path on an fp16 model (v_mfma_f32_16x16x32_f16): forward at the fp32 tolerance, gradients at the
    reference's tolerances, two chunks with a padded tail."""
    g = torch.Generator(device=dev).manual_seed(79)
    T, D, V = 600, 256, 4096
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).half().requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).half().requires_grad_()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    g_ent = torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=g)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    logits = torch.matmul(hidden.float(), weight.float().t()) / 0.7
    ref_ent = torch.logsumexp(logits, -1) - (torch.softmax(logits, -1) * logits).sum(-1)
    ref_lp = -torch.nn.functional.cross_entropy(logits, labels, reduction="none")
    d_ref_h, d_ref_w = torch.autograd.grad((ref_ent, ref_lp), (hidden, weight), (g_ent, g_lp))
    from verl_amd import gemm
    before = gemm.counters["gemm"]
    lp, ent = fused_linear_for_ppo(hidden, weight, labels, 0.7, chunk_size=256, keep_logits=False)
    torch.testing.assert_close(ref_lp, lp, atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(ref_ent, ent, atol=1e-4, rtol=1e-4)
    d_h, d_w = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
    assert gemm.counters["gemm"] == before + 4          # chunks [0, 256) and [256, 600), two products each
    assert d_h.dtype == torch.float16 and d_w.dtype == torch.float16
    torch.testing.assert_close(d_ref_h.float(), d_h.float(), atol=2e-3, rtol=1e-2)
    torch.testing.assert_close(d_ref_w.float(), d_w.float(), atol=2e-3, rtol=1e-2)


def test_close_to_the_library_path_and_3d_inputs(dev):
    g = torch.Generator(device=dev).manual_seed(4)
    B, S, K, V = 2, 260, 256, 5008
    h = torch.empty(B, S, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    w = torch.empty(V, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    ids = torch.randint(0, V, (B, S), generator=g, device=dev)
    lp, ent = lm_head_score_mfma(h, w, ids, 1.5)
    with torch.no_grad():
        lp2, ent2 = fused_linear_for_ppo(h, w, ids, 1.5, kernels="library")
        lp3, ent3 = fused_linear_for_ppo(h, w, ids, 1.5)
    assert lp.shape == (B, S)
    # the library path rounds |logit| ~ 3 to bf16 (2^-8 relative) before the softmax
    assert (lp - lp2).abs().max().item() <= 3e-2 and (ent - ent2).abs().max().item() <= 3e-2
    # the default forward IS this kernel
    assert torch.equal(lp3, lp) and torch.equal(ent3, ent)


def test_default_forward_is_the_same_with_and_without_gradients_and_for_any_token_count(dev):
    """A trainer compares old log-probs (no gradients, its own micro-batching) with new ones (gradients, other
    micro-batches) of the same weights: the default forward must give the same bits for a token whatever the call
    looks like. Fewer than 256 tokens are padded to one block."""
    g = torch.Generator(device=dev).manual_seed(14)
    T, K, V = 700, 128, 3000
    h = torch.empty(T, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    w = torch.empty(V, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    with torch.no_grad():
        lp_all, ent_all = fused_linear_for_ppo(h, w, ids, 0.8)
    hg, wg = h.clone().requires_grad_(), w.clone().requires_grad_()
    lp_g, ent_g = fused_linear_for_ppo(hg, wg, ids, 0.8, chunk_size=256, keep_logits=False)
    assert torch.equal(lp_g.detach(), lp_all) and torch.equal(ent_g.detach(), ent_all)
    for lo, hi in ((0, 100), (100, 356), (356, 700), (699, 700)):
        with torch.no_grad():
            lp_p, ent_p = fused_linear_for_ppo(h[lo:hi], w, ids[lo:hi], 0.8)
        assert torch.equal(lp_p, lp_all[lo:hi]) and torch.equal(ent_p, ent_all[lo:hi]), (lo, hi)
        lp_q, ent_q = fused_linear_for_ppo(hg[lo:hi], wg, ids[lo:hi], 0.8)
        assert torch.equal(lp_q.detach(), lp_all[lo:hi]), (lo, hi)
    # gradients through the padded call
    lp_q, ent_q = fused_linear_for_ppo(hg[:100], wg, ids[:100], 0.8)
    d_h, d_w = torch.autograd.grad((lp_q.sum() + 0.1 * ent_q.sum(),), (hg, wg))
    hf, wf = h.float().requires_grad_(), w.float().requires_grad_()
    z = (hf[:100] @ wf.t()) / 0.8
    ref = torch.log_softmax(z, -1).gather(-1, ids[:100, None]).sum() + 0.1 * (torch.logsumexp(z, -1) - (torch.softmax(z, -1) * z).sum(-1)).sum()
    r_h, r_w = torch.autograd.grad(ref, (hf, wf))
    torch.testing.assert_close(r_h, d_h.float(), atol=2e-2, rtol=4e-2)
    torch.testing.assert_close(r_w, d_w.float(), atol=2e-2, rtol=4e-2)
    assert not d_h[100:].any()


def test_token_results_do_not_depend_on_the_call(dev):
    """The forward kernel hands a token's softmax state over at fixed places of the vocabulary (every three tiles, per
    wavefront quarter) and the finishing kernel merges the states in a fixed order: the same token gives the same bits
    in calls of any size and for any number of splits (which only deals the work to workgroups), with and without
    gradients. A trainer's old and new log-probs of unchanged weights are therefore bit-identical whatever its
    micro-batch sizes."""
    g = torch.Generator(device=dev).manual_seed(15)
    K, V = 64, 16384 + 264                               # 66 vocabulary tiles, the last one partial
    T = 16640
    h = torch.empty(T, K, device=dev).uniform_(-1.0, 1.0, generator=g).bfloat16()
    w = torch.empty(V, K, device=dev).uniform_(-1.0, 1.0, generator=g).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    lib = _lib.load()
    plans = {n: lib.vrl_lmhead_plan(n, V) for n in (256, 2048, 8192, 8448, T)}
    assert len(set(plans.values())) >= 3, plans          # the sizes below are dealt differently
    with torch.no_grad():
        lp_all, ent_all = fused_linear_for_ppo(h, w, ids, 0.9)
        for lo, hi in ((0, 8192), (8192, T), (0, 256), (0, 2048), (300, 2348), (8000, T), (5, 6), (1000, 1300)):
            lp_p, ent_p = fused_linear_for_ppo(h[lo:hi], w, ids[lo:hi], 0.9)
            assert torch.equal(lp_p, lp_all[lo:hi]) and torch.equal(ent_p, ent_all[lo:hi]), (lo, hi)
        for splits in (1, 2, 7, 22, 64):
            lp_p, ent_p = fused_linear_for_ppo(h[:2048], w, ids[:2048], 0.9, forward_splits=splits)
            assert torch.equal(lp_p, lp_all[:2048]) and torch.equal(ent_p, ent_all[:2048]), splits
        # 65 token blocks: (block, split) pairs past the last whole round of 256 workgroups are dealt in 8 equal runs, and
        # the last group of 8 splits is narrower
        for splits in (5, 13, 22):
            lp_p, ent_p = fused_linear_for_ppo(h, w, ids, 0.9, forward_splits=splits)
            assert torch.equal(lp_p, lp_all) and torch.equal(ent_p, ent_all), splits
    hg = h[:300].clone().requires_grad_()
    lp_g, _ = fused_linear_for_ppo(hg, w, ids[:300], 0.9)                            # and with gradients
    assert torch.equal(lp_g.detach(), lp_all[:300])
    lp_g, _ = fused_linear_for_ppo(hg, w, ids[:300], 0.9, keep_logits=True)
    assert torch.equal(lp_g.detach(), lp_all[:300])
    with pytest.raises(ValueError):
        fused_linear_for_ppo(h[:256], w, ids[:256], 0.9, forward_splits=65)


def test_the_plan_fills_whole_rounds_of_workgroups(dev):
    """vrl_lmhead_plan: one workgroup per CU runs at a time, so the splits are chosen to make (rounds of workgroups) x
    (tiles of the longest share) smallest; every split gets tiles, in whole runs of three."""
    lib = _lib.load()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    for T, V in ((8192, 152064), (10240, 152064), (12288, 152064), (256, 152064), (2304, 152064), (4096, 32000),
                 (100000, 128256), (20000, 1000)):
        s = lib.vrl_lmhead_plan(T, V)
        tblocks, runs = -(-T // 256), -(-(-(-V // 256)) // 3)
        assert 1 <= s <= min(64, runs)
        share = -(-runs // s)
        assert -(-runs // share) == s                         # no split without tiles

        def cost(k):
            return -(-tblocks * k // cus) * (2 * -(-runs // k) * 3 + 1)

        assert cost(s) == min(cost(k) for k in range(1, min(64, runs) + 1)), (T, V, s)
    assert lib.vrl_lmhead_plan(8192, 152064) == 8 if cus == 256 else True
    assert lib.vrl_lmhead_partials(8192, 152064) == 198 * 12 * 8192 and lib.vrl_lmhead_partials(0, 5) == 0


def test_matrix_core_entry_points_replay_from_a_graph(dev):
    """vrl_lmhead_score, vrl_lmhead_dlogits and vrl_gemm (d hidden stored, d W accumulated) only enqueue kernels: captured
    once into a graph and replayed three times with new inputs in the same buffers, every replay equals the eager
    result bit for bit."""
    lib = _lib.load()
    T, K, V = 512, 256, 1024
    BF = _lib.VRL_BF16
    gd = torch.Generator(device=dev).manual_seed(21)
    h = torch.empty(T, K, dtype=torch.bfloat16, device=dev)
    w = torch.empty(V, K, dtype=torch.bfloat16, device=dev)
    ids = torch.empty(T, dtype=torch.int64, device=dev)
    g_lp = torch.empty(T, device=dev)
    g_ent = torch.empty(T, device=dev)
    splits = lib.vrl_lmhead_plan(T, V)
    partials = torch.empty(int(lib.vrl_lmhead_partials(T, V)), device=dev)
    lp = torch.empty(T, device=dev); ent = torch.empty(T, device=dev); lse = torch.empty(T, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    G = torch.empty(T, V, dtype=torch.bfloat16, device=dev)
    d_h = torch.empty(T, K, dtype=torch.bfloat16, device=dev)
    d_w = torch.empty(V, K, dtype=torch.bfloat16, device=dev)
    d_w0 = torch.empty(V, K, dtype=torch.bfloat16, device=dev)

    def fill():
        h.copy_(torch.empty(T, K, device=dev).uniform_(-0.5, 0.5, generator=gd))
        w.copy_(torch.empty(V, K, device=dev).uniform_(-0.5, 0.5, generator=gd))
        ids.copy_(torch.randint(0, V, (T,), generator=gd, device=dev))
        g_lp.copy_(torch.empty(T, device=dev).uniform_(-1, 1, generator=gd))
        g_ent.copy_(torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=gd))
        d_w0.copy_(torch.empty(V, K, device=dev).uniform_(-1, 1, generator=gd))

    def call(stream):
        assert lib.vrl_lmhead_score(h.data_ptr(), w.data_ptr(), BF, T, V, K, K, K, ids.data_ptr(), None, splits,
                                    partials.data_ptr(), lp.data_ptr(), ent.data_ptr(), lse.data_ptr(), flag.data_ptr(),
                                    None, 0, 0, stream) == 0
        assert lib.vrl_lmhead_dlogits(h.data_ptr(), w.data_ptr(), BF, T, V, K, K, K, ids.data_ptr(), None, lse.data_ptr(),
                                      ent.data_ptr(), g_lp.data_ptr(), g_ent.data_ptr(), lib.vrl_lmhead_plan(T, V),
                                      G.data_ptr(), V, stream) == 0
        # d hidden = G . W (W contraction-major), d W = d W0 + G^T . H (both contraction-major, accumulated)
        assert lib.vrl_gemm(w.data_ptr(), G.data_ptr(), BF, K, T, V, K, V, 1, 0, d_h.data_ptr(), K, 0, 1, None, stream) == 0
        d_w.copy_(d_w0)
        assert lib.vrl_gemm(h.data_ptr(), G.data_ptr(), BF, K, V, T, K, V, 1, 1, d_w.data_ptr(), K, 1, 1, None, stream) == 0

    outs = (lp, ent, lse, G, d_h, d_w)
    fill()
    call(torch.cuda.current_stream(dev).cuda_stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream(dev).cuda_stream)
    for _ in range(3):
        fill()
        call(torch.cuda.current_stream(dev).cuda_stream)
        torch.cuda.synchronize()
        eager = [t.clone() for t in outs]
        for t in outs:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(eager, outs):
            assert torch.equal(a, b)
        assert torch.isfinite(d_w.float()).all() and int(flag.item()) == 0


def test_special_values_and_errors(dev):
    g = torch.Generator(device=dev).manual_seed(6)
    T, V, K = 256, 512, 64
    h = (torch.randn(T, K, generator=g, device=dev) * 0.5).bfloat16()
    w = (torch.randn(V, K, generator=g, device=dev) * 0.2).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    bad = ids.clone()
    bad[7] = V
    with pytest.raises(IndexError):
        lm_head_score_mfma(h, w, bad)
    short = lm_head_score_mfma(h[:100], w, ids[:100])               # fewer than 256 tokens: padded to one block
    full = lm_head_score_mfma(h, w, ids)
    assert torch.equal(short[0], full[0][:100]) and torch.equal(short[1], full[1][:100])
    with pytest.raises(ValueError):
        lm_head_score_mfma(h, w[:200], ids.clamp(max=199))         # fewer than 256 vocabulary entries
    with pytest.raises(ValueError):
        lm_head_score_mfma(h[:, :32], w[:, :32], ids)              # hidden size not a multiple of 64
    with pytest.raises(TypeError):
        lm_head_score_mfma(h.float(), w.float(), ids)
    with pytest.raises(NotImplementedError):
        lm_head_score_mfma(h.clone().requires_grad_(), w, ids)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        lm_head_score_mfma(h.cpu(), w.cpu(), ids.cpu())
    # a token whose hidden state is zero: uniform distribution, log-prob -log V, entropy log V
    h0 = h.clone()
    h0[3] = 0
    lp, ent = lm_head_score_mfma(h0, w, ids)
    import math
    assert abs(lp[3].item() + math.log(V)) <= 1e-6 and abs(ent[3].item() - math.log(V)) <= 1e-6
    assert lib_plan_is_sane()


def lib_plan_is_sane():
    lib = _lib.load()
    return (lib.vrl_lmhead_plan(8192, 152064) == 8 and lib.vrl_lmhead_plan(256, 256) == 1
            and 1 <= lib.vrl_lmhead_plan(100000, 151936) <= 64 and lib.vrl_lmhead_plan(256, 151936) == 50)   # 198 runs in shares of 4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,V,K", [(256, 256, 64), (300, 704, 192), (1000, 304, 64), (2048, 4104, 320), (257, 18992, 512)])
def test_forward_also_writes_the_logits_when_asked(dev, dtype, T, V, K):
    """vrl_lmhead_score with logits_out: the scores are bit for bit those of the call without it, and the stored logits are
    the fp64 products rounded once to the operand type (half an ulp: up to 2^-8 relative for bf16, 2^-11 for fp16, plus the
    fp32 sum's own error), every element of the (T, V) block and nothing beyond it. Edge tiles in both directions."""
    lib = _lib.load()
    g = torch.Generator(device=dev).manual_seed(T + 2 * V + K)
    h = (torch.randn(T, K, generator=g, device=dev) * 0.5).to(dtype)
    w = (torch.randn(V, K, generator=g, device=dev) * 0.2).to(dtype)
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    temp = torch.rand(T, generator=g, device=dev) + 0.5
    code = _lib.VRL_BF16 if dtype == torch.bfloat16 else _lib.VRL_F16
    splits = lib.vrl_lmhead_plan(T, V)
    part = torch.empty(int(lib.vrl_lmhead_partials(T, V)), device=dev)
    pitch = V + 16
    outs = []
    for keep in (False, True):
        lp, ent, lse = (torch.empty(T, device=dev) for _ in range(3))
        flag = torch.zeros(1, dtype=torch.int32, device=dev)
        logits = torch.full((T, pitch), float("nan"), dtype=dtype, device=dev)
        with torch.cuda.device(dev):
            st = lib.vrl_lmhead_score(h.data_ptr(), w.data_ptr(), code, T, V, K, K, K, ids.data_ptr(), temp.data_ptr(), splits,
                                      part.data_ptr(), lp.data_ptr(), ent.data_ptr(), lse.data_ptr(), flag.data_ptr(),
                                      logits.data_ptr() if keep else None, pitch if keep else 0, T if keep else 0,
                                      _lib.stream_ptr(dev))
        assert st == _lib.VRL_OK, lib.vrl_strerror(st)
        outs.append((lp, ent, lse, logits))
    for a, b in zip(outs[0][:3], outs[1][:3]):
        assert torch.equal(a, b)
    logits = outs[1][3]
    z = ofl.logits_of(h, w, None, dtype=torch.float64)
    assert torch.isnan(logits[:, V:].float()).all()
    got = logits[:, :V].double()
    assert torch.isfinite(got).all()
    rel = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    assert bool(((got - z).abs() <= rel * z.abs() + 2e-6).all()), (got - z).abs().max().item()


@pytest.mark.parametrize("T,V,D", [(2304, 32256, 512), (300, 4104, 256), (100, 1000, 320), (4100, 8200, 256)])
def test_kept_logits_backward_runs_on_the_package_kernels(dev, T, V, D):
    """keep_logits=True on a 16-bit model: the forward kernel writes the logits, vrl_rowscore_backward turns them into
    their gradient in place, vrl_gemm forms d hidden and d W once each (counted; no library product except the partial
    last step of a vocabulary that is not a multiple of 64). Token counts that are not a multiple of 64 or below one
    256-token block are padded with zero rows. Against fp32 autograd of the reference composition at its own tolerances,
    and against the recomputing default path."""
    from verl_amd import gemm

    g = torch.Generator(device=dev).manual_seed(T + V)
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    g_ent = torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=g)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    r_lp, r_ent, _ = ofl.forward(hidden, weight, labels, 1.5, dtype=torch.float32)
    d_ref_h, d_ref_w = torch.autograd.grad((r_ent, r_lp), (hidden, weight), (g_ent, g_lp))
    lp0, ent0 = fused_linear_for_ppo(hidden, weight, labels, 1.5, keep_logits=False)
    dh0, dw0 = torch.autograd.grad((ent0, lp0), (hidden, weight), (g_ent, g_lp))
    before = gemm.counters["gemm"]
    lp, ent = fused_linear_for_ppo(hidden, weight, labels, 1.5, keep_logits=True)
    assert torch.equal(lp, lp0) and torch.equal(ent, ent0)          # the scores do not depend on keeping the logits
    assert (lp - r_lp).abs().max().item() <= 1e-4 and (ent - r_ent).abs().max().item() <= 1e-4
    d_h, d_w = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp), retain_graph=True)
    assert gemm.counters["gemm"] == before + 2
    torch.testing.assert_close(d_ref_h.float(), d_h.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(d_ref_w.float(), d_w.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(dh0.float(), d_h.float(), atol=1e-2, rtol=2e-2)
    torch.testing.assert_close(dw0.float(), d_w.float(), atol=1e-2, rtol=2e-2)
    with pytest.raises(RuntimeError, match="overwritten by the first backward"):
        torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
    # one gradient only, and a single incoming gradient
    lp, ent = fused_linear_for_ppo(hidden, weight.detach(), labels, 1.5, keep_logits=True)
    (only_h,) = torch.autograd.grad(lp, hidden, g_lp)
    lp_r, _, _ = ofl.forward(hidden, weight.detach(), labels, 1.5, dtype=torch.float32)
    (ref_h,) = torch.autograd.grad(lp_r, hidden, g_lp)
    torch.testing.assert_close(ref_h.float(), only_h.float(), atol=1e-2, rtol=1e-2)


def test_logits_are_kept_by_default_when_they_fit_the_budget(dev, monkeypatch):
    """keep_logits=None: kept when tokens x vocab x element size fits DEFAULT_KEEP_LOGITS_BYTES (a kept graph can be
    differentiated once), recomputed chunk by chunk otherwise (any number of times); the scores are the same bits."""
    from verl_amd import fused_linear as fl

    g = torch.Generator(device=dev).manual_seed(31)
    T, D, V = 512, 256, 4096
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    lp, _ = fused_linear_for_ppo(hidden, weight, labels)
    torch.autograd.grad(lp, hidden, g_lp, retain_graph=True)
    with pytest.raises(RuntimeError, match="overwritten by the first backward"):
        torch.autograd.grad(lp, hidden, g_lp)
    monkeypatch.setattr(fl, "DEFAULT_KEEP_LOGITS_BYTES", 256 * V * 2 - 1)      # not even one 256-token block
    lp2, _ = fused_linear_for_ppo(hidden, weight, labels)
    a = torch.autograd.grad(lp2, hidden, g_lp, retain_graph=True)[0]
    b = torch.autograd.grad(lp2, hidden, g_lp)[0]
    assert torch.equal(a, b) and torch.equal(lp, lp2)


@pytest.mark.parametrize("T,V,D,budget_rows", [(1100, 4104, 256, 600), (2304, 8192, 512, 2303), (1300, 1000, 320, 600),
                                               (1536, 1024, 256, 1100)])
def test_a_budget_below_all_logits_keeps_the_leading_blocks(dev, monkeypatch, T, V, D, budget_rows):
    """keep_logits=None with a budget that holds only some of the logits: the forward kernel writes the logits of the
    leading tokens, as many whole 256-token blocks as fit and leave whole chunks (vrl_lmhead_score's logits_rows), the
    backward turns those into their gradient
    in place and forms the rest again chunk by chunk, adding its share of d W. Same scores as both other paths, gradients
    within the tolerances those two agree to."""
    from verl_amd import fused_linear as fl
    from verl_amd import gemm

    g = torch.Generator(device=dev).manual_seed(T + V)
    hidden = torch.empty(T, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    weight = torch.empty(V, D, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16().requires_grad_()
    labels = torch.randint(0, V, (T,), generator=g, device=dev)
    g_ent = torch.empty(T, device=dev).uniform_(-0.5, 0.5, generator=g)
    g_lp = torch.empty(T, device=dev).uniform_(-1, 1, generator=g)
    r_lp, r_ent, _ = ofl.forward(hidden, weight, labels, 1.5, dtype=torch.float32)
    d_ref_h, d_ref_w = torch.autograd.grad((r_ent, r_lp), (hidden, weight), (g_ent, g_lp))
    lp0, ent0 = fused_linear_for_ppo(hidden, weight, labels, 1.5, keep_logits=False, chunk_size=512)
    dh0, dw0 = torch.autograd.grad((ent0, lp0), (hidden, weight), (g_ent, g_lp))
    monkeypatch.setattr(fl, "DEFAULT_KEEP_LOGITS_BYTES", budget_rows * V * 2)
    again = -(-(T - budget_rows) // 512) * 512          # what is formed again is whole chunks (of 512 tokens here)
    kept_rows = max(T - again, 0) // 256 * 256
    seen = {}
    real = fl._own_forward

    def spy(*a, **k):
        out = real(*a, **k)
        seen["kept"] = None if out[3] is None else tuple(out[3].shape)
        return out

    monkeypatch.setattr(fl, "_own_forward", spy)
    lp, ent = fused_linear_for_ppo(hidden, weight, labels, 1.5, chunk_size=512)
    assert seen["kept"] == (kept_rows, V)
    assert torch.equal(lp, lp0) and torch.equal(ent, ent0)
    before = gemm.counters["gemm"]
    d_h, d_w = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp), retain_graph=True)
    assert gemm.counters["gemm"] > before + 2            # the kept part's two products and the chunks' after them
    torch.testing.assert_close(d_ref_h.float(), d_h.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(d_ref_w.float(), d_w.float(), atol=1e-2, rtol=1e-2)
    torch.testing.assert_close(dh0.float(), d_h.float(), atol=1e-2, rtol=2e-2)
    torch.testing.assert_close(dw0.float(), d_w.float(), atol=1e-2, rtol=2e-2)
    with pytest.raises(RuntimeError, match="overwritten by the first backward"):
        torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))


def test_only_the_first_logits_rows_are_written(dev):
    """vrl_lmhead_score with logits_rows below the token count: those rows hold what the full call writes, the rest of the
    buffer is untouched, the scores are the same bits."""
    lib = _lib.load()
    g = torch.Generator(device=dev).manual_seed(9)
    T, V, K, rows = 1000, 1032, 128, 512
    h = torch.empty(T, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    w = torch.empty(V, K, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
    ids = torch.randint(0, V, (T,), generator=g, device=dev)
    splits = 2
    part = torch.empty(int(lib.vrl_lmhead_partials(T, V)), device=dev)
    outs = []
    for n_rows in (T, rows, 1):
        lp, ent, lse = (torch.empty(T, device=dev) for _ in range(3))
        flag = torch.zeros(1, dtype=torch.int32, device=dev)
        logits = torch.full((T, V), float("nan"), dtype=torch.bfloat16, device=dev)
        with torch.cuda.device(dev):
            st = lib.vrl_lmhead_score(h.data_ptr(), w.data_ptr(), _lib.VRL_BF16, T, V, K, K, K, ids.data_ptr(), None, splits,
                                      part.data_ptr(), lp.data_ptr(), ent.data_ptr(), lse.data_ptr(), flag.data_ptr(),
                                      logits.data_ptr(), V, n_rows, _lib.stream_ptr(dev))
        assert st == _lib.VRL_OK, lib.vrl_strerror(st)
        outs.append((lp, ent, lse, logits))
    full = outs[0][3]
    assert torch.isfinite(full.float()).all()
    for (lp, ent, lse, logits), n_rows in zip(outs[1:], (rows, 1)):
        assert torch.equal(lp, outs[0][0]) and torch.equal(ent, outs[0][1]) and torch.equal(lse, outs[0][2])
        assert torch.equal(logits[:n_rows], full[:n_rows])
        assert torch.isnan(logits[n_rows:].float()).all()
