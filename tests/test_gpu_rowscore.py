"""Parity of the HIP row kernel (through the C ABI) with the CPU oracle.

Tolerances (absolute): 1e-5 for fp32 logits, 2e-3 for bf16 logits against the
reference formula on logits.float(). The fp64 C oracle is compared as well, with
a tighter bound, to show the error is the kernel's accumulation and not the
oracle's own fp32 rounding.
"""

import math

import numpy as np
import pytest
import torch

import verl_amd
from verl_amd import synthetic
from verl_amd import torch_functional as vf
from oracle import c_oracle, scoring

pytestmark = pytest.mark.gpu

from _parity import assert_scores_match


def _check(logits, labels, temperature=None, tol=None, tol64=None):
    lp, h = vf.fused_logprob_entropy(logits, labels, temperature)
    assert lp.dtype == torch.float32 and h.dtype == torch.float32
    assert lp.shape == labels.shape and h.shape == labels.shape
    return assert_scores_match(lp, h, logits, labels, temperature, tol=tol, tol64=tol64)


def test_c1_full_size(dev):
    w = synthetic.WORKLOADS["c1"]
    d = synthetic.make_padded(w, dev, seed=1000)
    rep = _check(d["logits"], d["labels"])
    # at this size torch's own fp32 result is close enough to the exact value for the plain 1e-5 bar
    assert rep["log-prob_vs_torch_gpu"] <= 1e-5 and rep["entropy_vs_torch_gpu"] <= 1e-5
    assert rep["log-prob_vs_torch_cpu"] <= 1e-5 and rep["entropy_vs_torch_cpu"] <= 1e-5


@pytest.mark.parametrize("name,B,T", [("c2", 4, 96), ("c3", 3, 100), ("c5", 5, 60)])
def test_bf16_workloads_scaled_rows_full_vocab(dev, name, B, T):
    w = synthetic.WORKLOADS[name].scaled(B=B, T=T)
    d = synthetic.make_padded(w, dev, seed=2000)
    _check(d["logits"], d["labels"])


def test_c4_fp32_temperature_scaled_rows_full_vocab(dev):
    w = synthetic.WORKLOADS["c4"].scaled(B=2, T=128)
    d = synthetic.make_padded(w, dev, seed=4000)
    _check(d["logits"], d["labels"], d["temperature"])


def test_per_token_temperature_and_clamp(dev):
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn(64, 4099, generator=g, device=dev) * 2
    lab = torch.randint(0, 4099, (64,), generator=g, device=dev)
    temp = torch.rand(64, generator=g, device=dev) * 1.5 + 0.3
    _check(x, lab, temp)
    _check(x.bfloat16(), lab, temp)
    # a temperature below the clamp behaves like 1e-8: the row is one-hot on its arg-max
    tiny = torch.full((64,), 1e-12, device=dev)
    lp, h = vf.fused_logprob_entropy(x, x.argmax(-1), tiny)
    assert lp.abs().max().item() <= 1e-5 and h.abs().max().item() <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("V", [1, 2, 7, 8, 9, 63, 64, 65, 257, 1023, 1024, 1025, 4096, 8191, 32000, 50257])
def test_vocab_sizes_and_ragged_tails(dev, dtype, V):
    g = torch.Generator(device=dev).manual_seed(V)
    x = (torch.randn(37, V, generator=g, device=dev) * 3).to(dtype)
    lab = torch.randint(0, V, (37,), generator=g, device=dev)
    _check(x, lab)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_misaligned_and_strided_rows(dev, dtype):
    g = torch.Generator(device=dev).manual_seed(11)
    base = (torch.randn(33, 3001, generator=g, device=dev) * 2).to(dtype)
    for lo, hi in [(1, 3001), (3, 2990), (0, 2999), (5, 1290)]:
        view = base[:, lo:hi]  # row stride 3001 elements, start not 16-byte aligned
        assert not view.is_contiguous()
        lab = torch.randint(0, hi - lo, (33,), generator=g, device=dev)
        _check(view, lab)


def test_leading_shapes_and_separate_entry_points(dev):
    g = torch.Generator(device=dev).manual_seed(3)
    x = torch.randn(3, 5, 777, generator=g, device=dev)
    lab = torch.randint(0, 777, (3, 5), generator=g, device=dev)
    lp, h = vf.fused_logprob_entropy(x, lab)
    assert lp.shape == (3, 5) and h.shape == (3, 5)
    for fn in (vf.logprobs_from_logits, vf.logprobs_from_logits_v2, vf.logprobs_from_logits_naive):
        assert torch.equal(fn(x, lab), lp)
    assert torch.equal(vf.logprobs_from_logits(x, lab, inplace_backward=False), lp)
    assert torch.equal(vf.entropy_from_logits(x), h)
    assert torch.equal(vf.entropy_from_logits_with_chunking(x.reshape(15, 777), chunk_size=4), h.reshape(15))
    ref = scoring.logprobs_from_logits(x.cpu(), lab.cpu())
    assert (lp.cpu() - ref).abs().max() <= 1e-5
    ref_h = scoring.entropy_from_logits_with_chunking(x.cpu().reshape(15, 777), chunk_size=4)
    assert (h.cpu().reshape(15) - ref_h).abs().max() <= 1e-5
    # 1-D logits: a single distribution
    lp1, h1 = vf.fused_logprob_entropy(x[0, 0], lab[0, 0])
    assert lp1.shape == () and torch.equal(lp1, lp[0, 0]) and torch.equal(h1, h[0, 0])


def test_empty_batch(dev):
    x = torch.empty(0, 100, device=dev)
    lab = torch.empty(0, dtype=torch.int64, device=dev)
    lp, h = vf.fused_logprob_entropy(x, lab)
    assert lp.shape == (0,) and h.shape == (0,)


def test_closed_forms_on_device(dev):
    # uniform row: logp = -log V, H = log V
    for V, dtype in [(151936, torch.bfloat16), (32000, torch.float32), (5, torch.float32)]:
        x = torch.full((4, V), 1.25, device=dev, dtype=dtype)
        lab = torch.tensor([0, 1, V // 2, V - 1], device=dev)
        lp, h = vf.fused_logprob_entropy(x, lab)
        assert (lp + math.log(V)).abs().max().item() <= 2e-6
        assert (h - math.log(V)).abs().max().item() <= 2e-6
    # the reference's peaked row (tests/utils/test_linear_cross_entropy.py:352-395): one logit a, rest b
    a, b = 3.0, -15.0
    for V in (152064, 149 * 1024):
        x = torch.full((2, V), b, device=dev, dtype=torch.bfloat16)
        x[:, 0] = a
        lab = torch.tensor([0, 7], device=dev)
        lp, h = vf.fused_logprob_entropy(x, lab)
        lse = math.log(math.exp(a) + (V - 1) * math.exp(b))
        ent = lse - (a * math.exp(a) + (V - 1) * b * math.exp(b)) / math.exp(lse)
        assert abs(lp[0].item() - (a - lse)) <= 2e-6
        assert abs(lp[1].item() - (b - lse)) <= 4e-6
        assert (h - ent).abs().max().item() <= 2e-6
    # one-hot without NaN
    x = torch.zeros(1, 1000, device=dev)
    x[0, 17] = 1e4
    lp, h = vf.fused_logprob_entropy(x, torch.tensor([17], device=dev))
    assert abs(lp.item()) <= 1e-6 and abs(h.item()) <= 1e-6


def test_extreme_magnitudes_fp32(dev):
    # the reference's extreme rows (tests/utils/test_torch_functional.py:142-150), widened
    x = torch.tensor([[1000.0, 1001.0, 999.0], [-1000.0, -999.0, -998.0]], device=dev)
    lab = torch.tensor([1, 0], device=dev)
    # at |x| = 1000 one fp32 ulp of the inputs' shift is 6e-5; compare against fp64 truth loosely
    lp, h = vf.fused_logprob_entropy(x, lab)
    c_lp, c_h = c_oracle.rowscore(x.cpu(), lab.cpu())
    assert np.abs(lp.cpu().double().numpy() - c_lp).max() <= 1e-4
    assert np.abs(h.cpu().double().numpy() - c_h).max() <= 1e-4
    g = torch.Generator(device=dev).manual_seed(9)
    big = torch.randn(16, 5000, generator=g, device=dev) * 40 + 300
    # log-probs are ~ -150 here: one fp32 ulp of the OUTPUT is 1.5e-5
    _check(big, torch.randint(0, 5000, (16,), generator=g, device=dev), tol=2e-5, tol64=2e-5)


def test_special_values_match_torch(dev):
    inf = float("inf")
    V = 300
    g = torch.Generator(device=dev).manual_seed(21)
    x = torch.randn(8, V, generator=g, device=dev)
    x[0, 5] = -inf                   # masked-out token (top-k style)
    x[1, :] = -inf                   # nothing allowed
    x[2, 9] = inf
    x[3, 100] = float("nan")
    x[4, :200] = -inf                # leading -inf block: every lane's first elements are -inf
    x[5, 11] = -inf
    lab = torch.tensor([5, 0, 9, 3, 250, 12], device=dev)
    lab = torch.cat([lab, torch.tensor([0, 1], device=dev)])
    lp, h = vf.fused_logprob_entropy(x, lab)
    ref_lp, ref_h = scoring.score_fp32(x.cpu(), lab.cpu())
    got_lp, got_h = lp.cpu(), h.cpu()
    # same NaN / inf pattern as torch, same finite values
    assert torch.equal(torch.isnan(got_lp), torch.isnan(ref_lp)), (got_lp, ref_lp)
    assert torch.equal(torch.isnan(got_h), torch.isnan(ref_h)), (got_h, ref_h)
    assert torch.equal(torch.isinf(got_lp), torch.isinf(ref_lp))
    fin = torch.isfinite(ref_lp)
    assert (got_lp[fin] - ref_lp[fin]).abs().max() <= 1e-5
    finh = torch.isfinite(ref_h)
    assert (got_h[finh] - ref_h[finh]).abs().max() <= 1e-5
    assert got_lp[0].item() == -inf and torch.isnan(got_h[0])      # -inf label: logp -inf, entropy NaN (0 * -inf)
    assert torch.isfinite(got_lp[4]) and torch.isfinite(got_lp[5])


def test_label_out_of_range_raises(dev):
    x = torch.randn(4, 50, device=dev)
    for bad in (50, -1, 10**12):
        lab = torch.tensor([0, 1, bad, 3], device=dev)
        with pytest.raises(IndexError):
            vf.logprobs_from_logits(x, lab)
    lp, _ = vf.fused_logprob_entropy(x, torch.tensor([0, 1, 50, 3], device=dev), check_labels=False)
    assert torch.isnan(lp[2]) and torch.isfinite(lp[[0, 1, 3]]).all()


def test_label_check_modes(dev):
    """Reading the error flag back costs one host synchronisation per call ("sync", the default of direct calls).
    "off" never looks and the bad row is NaN; "deferred" looks later, without waiting for the GPU inside a call."""
    from verl_amd import errors

    x = torch.randn(4, 50, device=dev)
    lab = torch.tensor([0, 1, 50, 3], device=dev)
    with errors.using("off"):
        lp = vf.logprobs_from_logits(x, lab)
        assert torch.isnan(lp[2]) and torch.isfinite(lp[[0, 1, 3]]).all()
        with pytest.raises(IndexError):
            vf.fused_logprob_entropy(x, lab, check_labels=True)      # an explicit request still checks
    with errors.using("deferred"):
        lp = vf.logprobs_from_logits(x, lab)                         # returns at once, the row is NaN
        assert errors.pending() == 1
        with pytest.raises(IndexError):
            errors.check_errors()
        assert errors.pending() == 0
        lp = vf.logprobs_from_logits(x, lab)
        torch.cuda.synchronize()
        with pytest.raises(IndexError):                              # the next call notices what the last one left
            vf.entropy_from_logits(x)
        vf.entropy_from_logits(x)
        errors.check_errors()
    lp, _ = vf.fused_logprob_entropy(x, lab, check_labels="deferred")
    with pytest.raises(IndexError):
        errors.check_errors()
    with pytest.raises(ValueError):
        vf.fused_logprob_entropy(x, lab, check_labels="later")


def test_rejects_cpu_and_unsupported_inputs(dev):
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        vf.logprobs_from_logits(torch.randn(2, 10), torch.zeros(2, dtype=torch.long))
    x = torch.randn(2, 10, device=dev, requires_grad=True)
    assert vf.entropy_from_logits(x).requires_grad          # differentiable when the logits need it
    with torch.no_grad():
        assert not vf.entropy_from_logits(x).requires_grad
    from verl_amd import spec_rl
    with pytest.raises(NotImplementedError):                 # the verify step is forward-only
        spec_rl.fused_score_verify(x, torch.zeros(2, dtype=torch.long, device=dev), torch.zeros(2, device=dev), seed=0,
                                   cu_seqlens=torch.tensor([0, 2], device=dev))
    with pytest.raises(TypeError):
        vf.entropy_from_logits(torch.randn(2, 10, device=dev).double())


def test_fp16_logits_full_vocab(dev):
    g = torch.Generator(device=dev).manual_seed(16)
    x = (torch.randn(64, 151936, generator=g, device=dev) * 3).half()
    lab = torch.randint(0, 151936, (64,), generator=g, device=dev)
    temp = torch.full((64,), 0.7, device=dev)
    _check(x, lab)
    _check(x, lab, temp)
    _check(x[:, 5:150001], lab.clamp(max=149995))


def test_rows_are_independent_and_deterministic(dev):
    g = torch.Generator(device=dev).manual_seed(77)
    x = (torch.randn(512, 151936, generator=g, device=dev) * 3).bfloat16()
    lab = torch.randint(0, 151936, (512,), generator=g, device=dev)
    lp, h = vf.fused_logprob_entropy(x, lab)
    lp2, h2 = vf.fused_logprob_entropy(x, lab)
    assert torch.equal(lp, lp2) and torch.equal(h, h2)
    perm = torch.randperm(512, generator=g, device=dev)
    lp3, h3 = vf.fused_logprob_entropy(x[perm].contiguous(), lab[perm])
    assert torch.equal(lp3, lp[perm]) and torch.equal(h3, h[perm])
    assert torch.all(lp <= 0) and torch.all(h >= 0) and torch.all(h <= math.log(151936) + 1e-5)


def test_full_size_c2_against_torch_fp32_on_device(dev):
    """Whole 64x1024x152064 bf16 workload: the kernel against torch's own fp32 ops on the GPU, chunked."""
    w = synthetic.WORKLOADS["c2"]
    d = synthetic.make_padded(w, dev, seed=2001)
    logits, labels = d["logits"].view(-1, w.V), d["labels"].view(-1)
    lp, h = vf.fused_logprob_entropy(logits, labels)
    worst_lp = worst_h = 0.0
    for lo in range(0, logits.shape[0], 2048):
        z = logits[lo : lo + 2048].float()
        lse = torch.logsumexp(z, -1)
        ref_lp = z.gather(-1, labels[lo : lo + 2048, None]).squeeze(-1) - lse
        ref_h = lse - (torch.softmax(z, -1) * z).sum(-1)
        worst_lp = max(worst_lp, (lp[lo : lo + 2048] - ref_lp).abs().max().item())
        worst_h = max(worst_h, (h[lo : lo + 2048] - ref_h).abs().max().item())
    assert worst_lp <= 2e-3 and worst_h <= 2e-3, (worst_lp, worst_h)
    # and far inside it in practice (torch's own fp32 entropy is ~1e-5 from the exact value at this V)
    assert worst_lp <= 1e-5 and worst_h <= 1e-4, (worst_lp, worst_h)
    assert torch.all(lp <= 0)
    # N(0,3) logits: logsumexp ~ log V + 4.5 = 16.4; 70 % of labels are boosted by 8: mean ~ 0.7*(-8.4) + 0.3*(-16.4)
    assert -12.0 < lp.mean().item() < -9.5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_response_slice_of_longer_logits_is_scored_without_a_copy(dev, dtype, monkeypatch):
    """logits[:, -R-1:-1] of a (B, S, V) tensor (verl/utils/torch_functional.py:615 feeds exactly that): same numbers
    as the contiguous copy, with gradients landing in the right rows of the full tensor."""
    g = torch.Generator(device=dev).manual_seed(17)
    B, S, R, V = 3, 40, 13, 3001
    full = (torch.randn(B, S, V, generator=g, device=dev) * 2).to(dtype)
    lab = torch.randint(0, V, (B, R), generator=g, device=dev)
    temp = torch.rand(B, R, generator=g, device=dev) + 0.5
    view = full[:, -R - 1:-1]
    assert not view.is_contiguous() and vf._is_batch_of_row_slices(view)
    copies = []
    real_contiguous = torch.Tensor.contiguous
    monkeypatch.setattr(torch.Tensor, "contiguous", lambda t, *a, **k: (copies.append(t.numel()), real_contiguous(t, *a, **k))[1])
    lp, h, q = vf.fused_logprob_entropy(view, lab, temp, want_sum_pi_sq=True)
    assert max(copies, default=0) < V          # nothing of the logits' size was copied
    monkeypatch.undo()
    ref = vf.fused_logprob_entropy(view.contiguous(), lab, temp, want_sum_pi_sq=True)
    # A row's summation tree depends on where its 16-byte vectors start and on how many workgroups share it, and
    # both differ between the slice and its copy: same numbers to fp32 rounding, not bit for bit.
    assert lp.shape == (B, R) and (lp - ref[0]).abs().max().item() <= 4e-6 and (h - ref[1]).abs().max().item() <= 4e-6
    assert ((q - ref[2]).abs() <= 4e-6 * ref[2].abs() + 1e-12).all()
    from _parity import assert_scores_match
    assert_scores_match(lp.reshape(-1), h.reshape(-1), view.reshape(-1, V), lab.reshape(-1), temp.reshape(-1), cpu_torch=False)
    assert (vf.entropy_from_logits(view) - vf.entropy_from_logits(view.contiguous())).abs().max().item() <= 4e-6
    assert (vf.logprobs_from_logits(view, lab) - vf.logprobs_from_logits(view.contiguous(), lab)).abs().max().item() <= 4e-6
    # gradient through the slice
    leaf = full.clone().requires_grad_(True)
    w = torch.randn(B, R, generator=g, device=dev)
    (vf.logprobs_from_logits(leaf[:, -R - 1:-1], lab) * w).sum().backward()
    leaf2 = full.clone().requires_grad_(True)
    (vf.logprobs_from_logits(leaf2[:, -R - 1:-1].contiguous(), lab) * w).sum().backward()
    tol = 1e-6 if dtype == torch.float32 else 2.0 ** -7
    assert (leaf.grad.float() - leaf2.grad.float()).abs().max().item() <= tol and bool((leaf.grad[:, :S - R - 1] == 0).all())
    with pytest.raises(ValueError):
        vf.logprobs_from_logits(view, lab[:, :-1])
    with pytest.raises(IndexError):
        bad = lab.clone()
        bad[1, 2] = V
        vf.logprobs_from_logits(view, bad)
