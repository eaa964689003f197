"""oracle/fused_linear.py (the restatement of verl/utils/experimental/torch_functional.py:27-81 that the LM-head GPU
tests check against) pinned on the CPU: closed forms, invariants and fp64 autograd, chosen so that a transposed
operand, a dropped term or a wrong sign fails one of them."""

import math

import pytest
import torch

from oracle import fused_linear as ofl
from oracle import scoring


def _case(T, D, V, seed):
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(T, D, generator=g, dtype=torch.float64) * 0.7
    w = torch.randn(V, D, generator=g, dtype=torch.float64) * 0.5
    ids = torch.randint(0, V, (T,), generator=g)
    g_lp = torch.randn(T, generator=g, dtype=torch.float64)
    g_h = torch.randn(T, generator=g, dtype=torch.float64)
    temp = torch.rand(T, generator=g, dtype=torch.float64) + 0.5
    return h, w, ids, g_lp, g_h, temp


def test_one_hot_hidden_states_make_the_logits_a_column_of_the_weight():
    V, D = 37, 5
    g = torch.Generator().manual_seed(1)
    w = torch.randn(V, D, generator=g)
    ids = torch.tensor([3, 0, 36, 11, 20])
    h = torch.eye(D)                                  # token k selects column k of the weight
    lp, ent, lse = ofl.forward(h, w, ids, 0.8)
    for k in range(D):
        col = (w[:, k].double() / 0.8).float().view(1, V)     # the scoring oracle on that column, fp64 inside
        ref_lp, ref_h = scoring.score_fp64(col, ids[k:k + 1])
        assert abs(lp[k].item() - ref_lp.item()) <= 1e-6 and abs(ent[k].item() - ref_h.item()) <= 1e-6
    # a weight used transposed (D, V) cannot even be multiplied; a wrong contraction axis on a square weight is caught too
    ws = torch.randn(D, D, generator=g)
    lp2, _, _ = ofl.forward(h, ws, torch.arange(D))
    assert torch.allclose(lp2, torch.log_softmax(ws.double().t(), -1).diagonal())       # logits[k] = ws[:, k]
    assert not torch.allclose(lp2, torch.log_softmax(ws.double(), -1).diagonal())


def test_zero_hidden_states_give_the_uniform_distribution():
    V = 1000
    w = torch.randn(V, 16)
    lp, ent, lse = ofl.forward(torch.zeros(4, 16), w, torch.tensor([0, 5, 999, 17]), 1.3)
    assert torch.allclose(lp, torch.full((4,), -math.log(V), dtype=torch.float64), atol=1e-12)
    assert torch.allclose(ent, torch.full((4,), math.log(V), dtype=torch.float64), atol=1e-12)
    d = ofl.dlogits(torch.zeros(4, V, dtype=torch.float64), torch.tensor([0, 5, 999, 17]), None, torch.ones(4, dtype=torch.float64))
    assert d.abs().max().item() <= 1e-15              # the entropy is stationary at the uniform distribution


def test_temperature_divides_the_logits():
    # two vocabulary entries with logits (a, 0): log-prob of entry 0 is -log(1 + exp(-a / T))
    a, T = 1.7, 0.6
    h = torch.tensor([[1.0]], dtype=torch.float64)
    w = torch.tensor([[a], [0.0]], dtype=torch.float64)
    lp, ent, _ = ofl.forward(h, w, torch.tensor([0]), T)
    p = 1.0 / (1.0 + math.exp(-a / T))
    assert abs(lp.item() + math.log1p(math.exp(-a / T))) <= 1e-12
    assert abs(ent.item() + p * math.log(p) + (1 - p) * math.log(1 - p)) <= 1e-12
    per_token = ofl.forward(h, w, torch.tensor([0]), torch.tensor([T], dtype=torch.float64))[0]
    assert abs(per_token.item() - lp.item()) <= 1e-15
    clamped = ofl.forward(h, w, torch.tensor([0]), torch.tensor([0.0]))[0]      # clamped at 1e-8, not a division by zero
    assert torch.isfinite(clamped).all()


@pytest.mark.parametrize("which", ["logprob", "entropy", "both"])
def test_dlogits_invariants_and_autograd(which):
    h, w, ids, g_lp, g_h, temp = _case(6, 4, 19, seed=3)
    gl = None if which == "entropy" else g_lp
    gh = None if which == "logprob" else g_h
    for t in (None, 1.5, temp):
        z = ofl.logits_of(h, w, t)
        d = ofl.dlogits(z, ids, gl, gh, t)
        # softmax gradients live in the plane orthogonal to the all-ones vector
        assert d.sum(-1).abs().max().item() <= 1e-12
        # fp64 autograd with respect to the unscaled logits
        z0 = (h @ w.t()).requires_grad_(True)
        zt = ofl._scaled(z0, t)
        lse = torch.logsumexp(zt, -1)
        lp = zt.gather(-1, ids[:, None]).squeeze(-1) - lse
        ent = lse - (torch.softmax(zt, -1) * zt).sum(-1)
        loss = (0 if gl is None else (lp * gl).sum()) + (0 if gh is None else (ent * gh).sum())
        (ref,) = torch.autograd.grad(loss, z0)
        assert (d - ref).abs().max().item() <= 1e-12
    # sign: raising the label's logit raises its log-prob
    d = ofl.dlogits(ofl.logits_of(h, w), ids, torch.ones(6, dtype=torch.float64), None)
    assert (d.gather(-1, ids[:, None]) > 0).all()


@pytest.mark.parametrize("which", ["logprob", "entropy", "both"])
def test_backward_matches_autograd_through_forward(which):
    h, w, ids, g_lp, g_h, temp = _case(7, 5, 23, seed=4)        # T, D, V all different: a transposed product cannot fit
    gl = None if which == "entropy" else g_lp
    gh = None if which == "logprob" else g_h
    for t in (None, 0.7, temp):
        dh, dw = ofl.backward(h, w, ids, gl, gh, t)
        rh, rw = ofl.autograd_backward(h, w, ids, gl, gh, t)
        assert dh.shape == h.shape and dw.shape == w.shape
        assert (dh - rh).abs().max().item() <= 1e-12 and (dw - rw).abs().max().item() <= 1e-12


def test_fp32_and_fp64_agree_to_fp32_rounding_and_chunks_add_up():
    h, w, ids, g_lp, g_h, _ = _case(40, 8, 300, seed=5)
    lp64, ent64, _ = ofl.forward(h, w, ids, 1.5)
    lp32, ent32, _ = ofl.forward(h.float(), w.float(), ids, 1.5, dtype=torch.float32)
    assert (lp32.double() - lp64).abs().max().item() <= 1e-5 and (ent32.double() - ent64).abs().max().item() <= 1e-5
    # the reference walks the tokens in chunks and accumulates d W (verl/utils/experimental/torch_functional.py:165-199)
    dh, dw = ofl.backward(h, w, ids, g_lp, g_h, 1.5)
    dw_sum = torch.zeros_like(dw)
    for lo in range(0, 40, 16):
        s = slice(lo, lo + 16)
        dh_c, dw_c = ofl.backward(h[s], w, ids[s], g_lp[s], g_h[s], 1.5)
        assert (dh_c - dh[s]).abs().max().item() <= 1e-13
        dw_sum += dw_c
    assert (dw_sum - dw).abs().max().item() <= 1e-12
