"""Pins the scoring oracle (oracle/scoring.py, oracle/vrl_oracle.c) without any GPU.

Every check is chosen so a plausible slip (dropped term, wrong sign, wrong axis, label off by
one, temperature multiplied instead of divided, natural log vs log2) fails at least one of them.
"""

import math

import numpy as np
import pytest
import scipy.special
import scipy.stats
import torch
from hypothesis import given, settings, strategies as st

from oracle import c_oracle, scoring

LOGPROB_FNS = [scoring.logprobs_from_logits, scoring.logprobs_from_logits_v2, scoring.logprobs_from_logits_naive]


# ---- closed forms -----------------------------------------------------------

@pytest.mark.parametrize("fn", LOGPROB_FNS)
@pytest.mark.parametrize("V", [1, 2, 7, 1000, 32000])
def test_uniform_row_logprob_is_minus_log_v(fn, V):
    x = torch.full((3, V), 0.37)
    lab = torch.tensor([0, V // 2, V - 1])
    assert torch.allclose(fn(x, lab), torch.full((3,), -math.log(V)), atol=2e-6)
    assert torch.allclose(scoring.entropy_from_logits(x), torch.full((3,), math.log(V)), atol=2e-6)


@pytest.mark.parametrize("V", [152064, 149 * 1024])
def test_reference_peaked_row_closed_form(V):
    """The reference's regression construction (tests/utils/test_linear_cross_entropy.py:352-395):
    one logit at +3, all others at -15, label on the peak."""
    a, b = 3.0, -15.0
    x = torch.full((2, V), b)
    x[:, 0] = a
    lab = torch.tensor([0, 5])
    lse = math.log(math.exp(a) + (V - 1) * math.exp(b))
    ent = lse - (a * math.exp(a) + (V - 1) * b * math.exp(b)) / math.exp(lse)
    for fn in LOGPROB_FNS:
        # fp64 torch: exact to rounding. fp32 torch on the CPU adds 152063 terms of e^-18 to an
        # accumulator near 1 and loses ~6 % of them (1.4e-4 absolute): the reference's own test of this
        # construction allows 1e-3 (test_linear_cross_entropy.py:393-394), and so does this one.
        lp = fn(x.double(), lab)
        assert abs(lp[0].item() - (a - lse)) < 1e-11 and abs(lp[1].item() - (b - lse)) < 1e-11
        lp = fn(x, lab)
        assert abs(lp[0].item() - (a - lse)) < 1e-3 and abs(lp[1].item() - (b - lse)) < 1e-3
    assert torch.allclose(scoring.entropy_from_logits(x.double()), torch.full((2,), ent, dtype=torch.float64), atol=1e-10)
    assert torch.allclose(scoring.entropy_from_logits(x), torch.full((2,), ent), atol=1e-3)
    c_lp, c_h = c_oracle.rowscore(x, lab)
    assert abs(c_lp[0] - (a - lse)) < 1e-10 and abs(c_lp[1] - (b - lse)) < 1e-10
    assert np.allclose(c_h, ent, atol=1e-10)
    # bf16 inputs hold these two values exactly, so the same closed form applies
    c_lp16, c_h16 = c_oracle.rowscore(x.bfloat16(), lab)
    assert np.array_equal(c_lp16, c_lp) and np.array_equal(c_h16, c_h)


def test_one_hot_row_has_zero_entropy_and_no_nan():
    x = torch.zeros(1, 500)
    x[0, 17] = 1e4
    assert scoring.entropy_from_logits(x).item() == 0.0
    assert scoring.logprobs_from_logits(x, torch.tensor([17])).item() == 0.0
    c_lp, c_h = c_oracle.rowscore(x, torch.tensor([17]))
    assert c_lp[0] == 0.0 and c_h[0] == 0.0


# ---- invariants / brute force -------------------------------------------------

def test_probabilities_of_all_labels_sum_to_one():
    torch.manual_seed(0)
    V = 37
    x = torch.randn(5, V) * 4
    for fn in LOGPROB_FNS:
        total = torch.zeros(5)
        for v in range(V):
            total += torch.exp(fn(x, torch.full((5,), v)))
        assert torch.allclose(total, torch.ones(5), atol=1e-5)
    total = np.zeros(5)
    for v in range(V):
        total += np.exp(c_oracle.rowscore(x, torch.full((5,), v))[0])
    assert np.allclose(total, 1.0, atol=1e-12)


def test_label_picks_the_right_column_and_row():
    # distinct, strictly increasing logits: logp must be increasing in the label, and row-specific
    x = torch.stack([torch.arange(10.0), torch.arange(10.0) * 2])
    for fn in LOGPROB_FNS:
        lp = torch.stack([fn(x, torch.tensor([v, v])) for v in range(10)])
        assert torch.all(lp[1:] > lp[:-1])
        assert not torch.allclose(lp[:, 0], lp[:, 1])
        # difference of two labels' log-probs is the difference of their logits
        assert torch.allclose(lp[7] - lp[2], x[:, 7] - x[:, 2], atol=1e-5)


def test_shift_and_permutation_invariance():
    torch.manual_seed(1)
    x = torch.randn(6, 301) * 3
    lab = torch.randint(0, 301, (6,))
    perm = torch.randperm(301)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(301)
    for fn in LOGPROB_FNS:
        assert torch.allclose(fn(x + 11.5, lab), fn(x, lab), atol=2e-5)
        assert torch.allclose(fn(x[:, perm], inv[lab]), fn(x, lab), atol=2e-6)
    h = scoring.entropy_from_logits(x)
    assert torch.allclose(scoring.entropy_from_logits(x + 11.5), h, atol=3e-5)
    assert torch.allclose(scoring.entropy_from_logits(x[:, perm]), h, atol=2e-6)
    assert torch.all(h >= 0) and torch.all(h <= math.log(301) + 1e-6)


def test_against_scipy_fp64():
    rng = np.random.default_rng(2)
    x = rng.normal(0, 3, size=(16, 2048))
    lab = rng.integers(0, 2048, size=16)
    ref_lp = scipy.special.log_softmax(x, axis=-1)[np.arange(16), lab]
    ref_h = scipy.stats.entropy(scipy.special.softmax(x, axis=-1), axis=-1)
    xt, lt = torch.from_numpy(x), torch.from_numpy(lab)
    for fn in LOGPROB_FNS:
        assert np.allclose(fn(xt, lt).numpy(), ref_lp, atol=1e-12)
        assert np.allclose(fn(xt.float(), lt).numpy(), ref_lp, atol=1e-5)
    assert np.allclose(scoring.entropy_from_logits(xt).numpy(), ref_h, atol=1e-12)
    lp64, h64 = scoring.score_fp64(xt.float(), lt)
    c_lp, c_h = c_oracle.rowscore(xt.float(), lt)
    ref32 = scipy.special.log_softmax(x.astype(np.float32).astype(np.float64), axis=-1)[np.arange(16), lab]
    assert np.allclose(lp64.numpy(), ref32, atol=1e-12) and np.allclose(c_lp, ref32, atol=1e-12)
    assert np.allclose(h64.numpy(), c_h, atol=1e-12)


def test_v2_branches_and_dtypes():
    torch.manual_seed(3)
    x = torch.randn(4, 6, 129) * 2
    lab = torch.randint(0, 129, (4, 6))
    a, b = scoring.logprobs_from_logits_v2(x, lab), scoring.logprobs_from_logits_naive(x, lab)
    assert a.shape == (4, 6) and a.dtype == torch.float32 and torch.allclose(a, b, atol=2e-6)
    # the non-fp32 branch keeps the input dtype (verl/utils/torch_functional.py:199-206)
    xb = x.bfloat16()
    c = scoring.logprobs_from_logits_v2(xb, lab)
    assert c.dtype == torch.bfloat16 and c.shape == (4, 6)
    assert torch.equal(c, torch.log_softmax(xb, -1).gather(-1, lab.unsqueeze(-1)).squeeze(-1))
    assert scoring.entropy_from_logits(xb).dtype == torch.bfloat16
    # the upcast target used for bf16 parity equals the fp32 functions on the upcast values
    lp32, h32 = scoring.score_fp32(xb, lab)
    assert lp32.dtype == torch.float32 and torch.equal(lp32, scoring.logprobs_from_logits(xb.float(), lab))


def test_chunked_entropy_equals_unchunked():
    torch.manual_seed(4)
    x = torch.randn(300, 777)
    full = scoring.entropy_from_logits(x)
    for chunk in (1, 7, 128, 300, 4096):
        assert torch.allclose(scoring.entropy_from_logits_with_chunking(x, chunk), full, atol=1e-6)
    out = scoring.entropy_from_logits_with_chunking(x.bfloat16(), 64)
    assert out.dtype == torch.float32 and torch.allclose(out, scoring.entropy_from_logits(x.bfloat16().float()), atol=1e-6)


def test_entropy_is_monotone_in_temperature():
    torch.manual_seed(5)
    x = torch.randn(8, 500) * 3
    lab = torch.zeros(8, dtype=torch.long)
    prev = None
    for T in (0.25, 0.5, 1.0, 2.0, 4.0):
        _, h = scoring.score_reference(x, lab, torch.full((8,), T))
        if prev is not None:
            assert torch.all(h > prev)
        prev = h


def test_temperature_is_elementwise_ieee_division_with_clamp():
    torch.manual_seed(6)
    x = torch.randn(5, 64) * 10
    t = torch.tensor([0.7, 1.0, 1.3, 0.0, -2.0])
    got = scoring.apply_temperature(x, t).numpy()
    tn = np.maximum(t.numpy(), np.float32(1e-8)).astype(np.float32)
    assert np.array_equal(got, (x.numpy() / tn[:, None]).astype(np.float32))
    # bf16: the temperature is cast to bf16 and the quotient is a bf16
    gb = scoring.apply_temperature(x.bfloat16(), t)
    assert gb.dtype == torch.bfloat16
    assert torch.equal(gb[0], x.bfloat16()[0] / torch.tensor(0.7).bfloat16())
    # the C oracle divides the same way
    lab = torch.randint(0, 64, (3,))
    c_lp, c_h = c_oracle.rowscore(x[:3], lab, t[:3])
    lp64, h64 = scoring.score_fp64(x[:3], lab, t[:3])
    assert np.allclose(c_lp, lp64.numpy(), atol=1e-12) and np.allclose(c_h, h64.numpy(), atol=1e-12)


@pytest.mark.parametrize("shape", [(8, 17), (3, 5, 32), (1, 1024)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_sum_pi_squared_reference_parametrisation(shape, dtype):
    """Same cases as the reference's tests/utils/test_torch_functional.py:126-140."""
    torch.manual_seed(0)
    logits = torch.randn(*shape, dtype=dtype) * 5.0
    actual = scoring.calculate_sum_pi_squared_from_logits(logits)
    expected = torch.softmax(logits, dim=-1).pow(2).sum(dim=-1)
    assert actual.shape == expected.shape
    torch.testing.assert_close(actual, expected, atol=1e-5, rtol=1e-5)
    assert torch.all(actual > 0) and torch.all(actual <= 1.0 + 1e-5)


def test_sum_pi_squared_reference_extreme_values():
    """tests/utils/test_torch_functional.py:142-150."""
    logits = torch.tensor([[1000.0, 1001.0, 999.0], [-1000.0, -999.0, -998.0]], dtype=torch.float64)
    actual = scoring.calculate_sum_pi_squared_from_logits(logits)
    expected = torch.softmax(logits, dim=-1).pow(2).sum(dim=-1)
    assert torch.isfinite(actual).all()
    torch.testing.assert_close(actual, expected, atol=1e-10, rtol=1e-10)


# ---- special values -----------------------------------------------------------

def test_infinities_and_nan_follow_torch_and_c_oracle_agrees():
    inf, nan = float("inf"), float("nan")
    x = torch.tensor([
        [0.0, -inf, 1.0, 2.0],     # a masked-out entry: logp fine, entropy NaN (0 * -inf)
        [-inf, -inf, -inf, -inf],  # nothing allowed: all NaN
        [0.0, inf, 1.0, 2.0],      # +inf
        [0.0, nan, 1.0, 2.0],
    ])
    lab = torch.tensor([0, 1, 0, 0])
    lp, h = scoring.score_fp32(x, lab)
    assert math.isclose(lp[0].item(), -math.log(1 + math.e + math.e**2), rel_tol=1e-6) and math.isnan(h[0].item())
    assert math.isnan(lp[1].item()) and math.isnan(h[1].item())
    assert lp[2].item() == -inf and math.isnan(h[2].item())
    assert math.isnan(lp[3].item()) and math.isnan(h[3].item())
    assert scoring.logprobs_from_logits(x[:1], torch.tensor([1])).item() == -inf
    c_lp, c_h = c_oracle.rowscore(x, lab)
    assert np.array_equal(np.isnan(c_lp), torch.isnan(lp).numpy()) and np.array_equal(np.isnan(c_h), torch.isnan(h).numpy())
    assert c_lp[2] == -inf and abs(c_lp[0] - lp[0].item()) < 1e-6


# ---- layout helpers -------------------------------------------------------------

def test_response_slice_reference_fixture():
    """tests/models/test_fsdp_no_padding_on_gpu.py:170-205: sequences of 5 and 3 tokens (prompts 3 and 2,
    responses 2 and 1), V = 32, seed 0: expected rows are full[2:4] and pad(full[6:7])."""
    torch.manual_seed(0)
    logits = torch.randn(2, 5, 32)
    flat = torch.cat([logits[0, :5], logits[1, :3]], dim=0)
    ids = torch.tensor([11, 12, 13, 14, 15, 21, 22, 23])
    labels = scoring.roll_labels(ids)
    assert labels.tolist() == [12, 13, 14, 15, 21, 22, 23, 11]
    full = scoring.logprobs_from_logits(flat, labels % 32)
    got = scoring.response_slice(full, prompt_lens=[3, 2], response_lens=[2, 1], max_response_len=2)
    expected = torch.stack([full[2:4], torch.nn.functional.pad(full[6:7], (0, 1))])
    assert got.shape == (2, 2) and torch.equal(got, expected)
    # the slice holds the log-probs OF the response tokens: position 2 predicts token 14, 3 predicts 15, 6 predicts 23
    assert labels[2:4].tolist() == [14, 15] and labels[6].item() == 23
    with pytest.raises(AssertionError):
        scoring.response_slice(full, prompt_lens=[0, 2], response_lens=[5, 1])
    with pytest.raises(AssertionError):
        scoring.response_slice(full, prompt_lens=[3, 2], response_lens=[2, 2])


def test_response_from_nested_is_the_padded_slice_without_its_padding():
    """verl/workers/utils/padding.py:194-210 takes the same window per sequence as no_padding_2_padding (:135-138)
    and joins the pieces instead of padding them: on the reference's fixture the pieces are full[2:4] and full[6:7]."""
    full = torch.arange(8, dtype=torch.float32) * 1.5
    vals, offs = scoring.response_from_nested(full, [0, 5, 8], [2, 1])
    assert torch.equal(vals, torch.cat([full[2:4], full[6:7]])) and offs.tolist() == [0, 2, 3]
    g = torch.Generator().manual_seed(8)
    prompt = torch.randint(1, 9, (20,), generator=g)
    resp = torch.randint(0, 30, (20,), generator=g)
    cu = [0] + torch.cumsum(prompt + resp, 0).tolist()
    x = torch.randn(cu[-1], generator=g)
    vals, offs = scoring.response_from_nested(x, cu, resp.tolist())
    padded = scoring.response_slice(x, prompt.tolist(), resp.tolist())
    for b in range(20):
        r = int(resp[b])
        assert torch.equal(vals[offs[b]:offs[b + 1]], padded[b, :r]) and int(offs[b + 1] - offs[b]) == r
    with pytest.raises(ValueError):
        scoring.response_from_nested(x, cu, resp.tolist()[:-1])     # strict zip, like the reference's


def test_roll_is_global_not_per_shard():
    """tests/models/test_fused_kernels_ulysses_sp_on_cpu.py:69-90: roll then slice differs from slice then roll
    exactly at shard boundaries."""
    torch.manual_seed(0)
    ids = torch.randint(0, 10000, (1, 32))
    good = list(torch.chunk(scoring.roll_labels(ids), 4, dim=-1))
    bad = [torch.roll(s, -1, -1) for s in torch.chunk(ids, 4, dim=-1)]
    for g, b in zip(good, bad):
        assert torch.equal(g[..., :-1], b[..., :-1]) and not torch.equal(g[..., -1], b[..., -1])


# ---- torch restatement vs the independent C restatement ---------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V", [1, 5, 1000, 32000])
def test_c_oracle_agrees_with_torch_oracle(dtype, V):
    torch.manual_seed(V)
    x = (torch.randn(9, V) * 3).to(dtype)
    lab = torch.randint(0, V, (9,))
    t = torch.rand(9) + 0.5
    for temp in (None, t):
        lp, h = scoring.score_fp32(x, lab, temp)
        c_lp, c_h = c_oracle.rowscore(x, lab, temp)
        assert np.abs(lp.double().numpy() - c_lp).max() < 5e-6
        # torch's fp32 CPU softmax is good to ~1e-5 relative per element; at V = 32000 that moves the
        # entropy by up to ~6e-5 (a formula slip would move it by >= 1e-2)
        assert np.abs(h.double().numpy() - c_h).max() < 2e-4
        lp64, h64 = scoring.score_fp64(x, lab, temp)
        assert np.abs(lp64.numpy() - c_lp).max() < 1e-11 and np.abs(h64.numpy() - c_h).max() < 1e-10


@settings(max_examples=60, deadline=None)
@given(st.integers(1, 200), st.integers(1, 6), st.floats(0.1, 20.0), st.integers(0, 2**31 - 1))
def test_property_bounds(V, n, scale, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, V, generator=g) * scale
    lab = torch.randint(0, V, (n,), generator=g)
    lp, h = scoring.score_reference(x, lab)
    assert torch.all(lp <= 1e-6) and torch.all(h >= -1e-5) and torch.all(h <= math.log(V) + 1e-5)
    c_lp, c_h = c_oracle.rowscore(x, lab)
    assert np.all(c_lp <= 0) and np.all(c_h >= -1e-12) and np.all(c_h <= math.log(V) + 1e-12)
    # entropy = -sum p log p written out the long way
    p = torch.softmax(x.double(), -1)
    direct = -(p * torch.log(p.clamp_min(1e-300))).sum(-1)
    assert np.allclose(c_h, direct.numpy(), atol=1e-9)


def test_expand_as_nested_values_is_one_value_per_token_of_its_sequence():
    """Pinned without the formula: written out by hand for a small batch, by a per-token loop for a random one, and
    through what it is for (the per-token temperature gives the same scores as scoring each sequence on its own with
    its scalar temperature)."""
    t = torch.tensor([0.5, 2.0, 1.25])
    got = scoring.expand_as_nested_values(t, [0, 2, 2, 5])            # the middle sequence is empty
    assert got.tolist() == [0.5, 0.5, 1.25, 1.25, 1.25]
    g = torch.Generator().manual_seed(3)
    lens = torch.randint(0, 9, (17,), generator=g)
    cu = torch.zeros(18, dtype=torch.int64)
    cu[1:] = torch.cumsum(lens, 0)
    vals = torch.rand(17, generator=g)
    got = scoring.expand_as_nested_values(vals, cu)
    assert got.shape == (int(cu[-1]),)
    for tok in range(int(cu[-1])):
        b = max(i for i in range(17) if int(cu[i]) <= tok and tok < int(cu[i + 1]))
        assert got[tok] == vals[b]
    x = torch.randn(int(cu[-1]), 50, generator=g)
    lab = torch.randint(0, 50, (int(cu[-1]),), generator=g)
    lp_all, h_all = scoring.score_fp64(x, lab, got.double())
    for b in range(17):
        lo, hi = int(cu[b]), int(cu[b + 1])
        if hi > lo:
            lp_b, h_b = scoring.score_fp64(x[lo:hi], lab[lo:hi], torch.full((hi - lo,), float(vals[b]), dtype=torch.float64))
            assert torch.equal(lp_b, lp_all[lo:hi]) and torch.equal(h_b, h_all[lo:hi])
    with pytest.raises(AssertionError):
        scoring.expand_as_nested_values(vals[:-1], cu)
