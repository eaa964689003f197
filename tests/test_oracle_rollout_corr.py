"""Pins oracle/rollout_corr.py with the exact-value cases the reference's own tests hold
(tests/trainer/ppo/test_rollout_corr.py) and with closed forms."""

import math

import pytest
import torch

from oracle import rollout_corr as rc

OPTIONS = [("token_k1", "0.5_1.5"), ("token_k2", 2.0), ("token_k3", 2.0), ("seq_sum_k1", "0.6_1.4"),
           ("seq_sum_k2", 2.5), ("seq_sum_k3", 2.5), ("seq_mean_k1", "0.5_1.5"), ("seq_mean_k2", 2.0),
           ("seq_mean_k3", 2.0), ("seq_max_k2", 2.0), ("seq_max_k3", 2.0)]


def test_reference_mask_mode_case():
    """test_rollout_corr.py:312-366: old -2.0; rollout -1.0 (ratio e^-1 = 0.37, outside [0.5, 2]) and -2.5 (1.65, inside)."""
    old = torch.full((2, 5), -2.0)
    roll = torch.tensor([[-1.0] * 5, [-2.5] * 5])
    mask = torch.ones(2, 5)
    w, new_mask, m = rc.correction_and_rejection_mask(old, roll, mask, rollout_is="token", rollout_is_threshold=2.0,
                                                      rollout_rs="token_k1", rollout_rs_threshold="0.5_2.0")
    assert torch.all(w[0] > 0)
    assert torch.allclose(w[0, 0], torch.tensor(0.368), atol=0.01) and torch.allclose(w[1, 0], torch.tensor(1.649), atol=0.01)
    assert math.isclose(w[0, 0].item(), math.exp(-1.0), rel_tol=1e-6) and math.isclose(w[1, 0].item(), math.exp(0.5), rel_tol=1e-6)
    assert torch.all(new_mask[0] == 0) and torch.all(new_mask[1] == 1)
    assert abs(m["rollout_corr/rollout_rs_masked_fraction"] - 0.5) < 0.01
    assert m["rollout_corr/rollout_rs_seq_masked_fraction"] == 0.5


def test_reference_icepop_case():
    """test_rollout_corr.py:369-394: raw weights 0.4, 0.8, 6.0 with bounds 0.5_5.0."""
    raw = torch.tensor([[0.4, 0.8, 6.0]])
    old = torch.zeros_like(raw)
    roll = -torch.log(raw)
    mask = torch.ones_like(raw)
    w, new_mask, m = rc.correction_and_rejection_mask(old, roll, mask, rollout_is="token", rollout_is_threshold="0.5_5.0")
    torch.testing.assert_close(w, torch.tensor([[0.0, 0.8, 0.0]]), atol=1e-6, rtol=1e-6)
    assert torch.equal(new_mask, mask)
    assert m["rollout_corr/rollout_is_oob_ratio"] == pytest.approx(2.0 / 3.0, abs=1e-6)
    assert m["rollout_corr/rollout_is_std"] == pytest.approx(0.3771236, abs=1e-6)
    assert m["rollout_corr/rollout_is_eff_sample_size"] == pytest.approx(1.0 / 3.0, abs=1e-6)


def test_reference_seq_fraction_high_uses_raw_weights():
    """test_rollout_corr.py:416-442."""
    raw = torch.tensor([[1.0, 6.0], [0.9, 1.1]])
    m = rc.is_metrics(raw.clamp(max=2.0), raw, torch.log(raw), torch.ones_like(raw), "token", 2.0)
    assert m["rollout_is_seq_fraction_high"] == pytest.approx(0.5)


def test_threshold_parsing_errors():
    """test_rollout_corr.py:397-413 rejects a bool; the parsers' other error branches."""
    with pytest.raises(TypeError):
        rc.parse_is_threshold(True)
    assert rc.parse_is_threshold(2) == (2.0, None) and rc.parse_is_threshold("0.5_5.0") == (5.0, 0.5)
    assert rc.parse_is_threshold(" 3.5 ") == (3.5, None)
    for bad in ("", "a_b", "0_2", "3_2", -1.0):
        with pytest.raises(ValueError):
            rc.parse_is_threshold(bad)
    assert rc.normalize_rs_options(" token_k1, seq_max_k3 ,token_k1") == ["token_k1", "seq_max_k3"]
    with pytest.raises(ValueError):
        rc.normalize_rs_options("token_k4")
    th = rc.parse_rs_thresholds(["token_k1", "seq_max_k3"], "0.4_1.8,3.0")
    assert th == {"token_k1": {"lower": 0.4, "upper": 1.8}, "seq_max_k3": {"lower": None, "upper": 3.0}}
    assert rc.parse_rs_thresholds(["token_k1"], 2.0)["token_k1"] == {"lower": 0.5, "upper": 2.0}   # lower defaults to 1/upper
    assert rc.parse_rs_thresholds(["token_k2", "token_k3"], 2.0)["token_k3"]["upper"] == 2.0      # one value shared
    for opts, spec in ((["token_k2"], "1_2"), (["token_k1"], "2_1"), (["token_k1", "token_k2"], "1,2,3"), (["token_k2"], -1.0)):
        with pytest.raises(ValueError):
            rc.parse_rs_thresholds(opts, spec)


@pytest.mark.parametrize("option,threshold", OPTIONS)
def test_each_option_runs_and_masks_consistently(option, threshold):
    """test_rollout_corr.py:127-166 (every option produces its metrics), plus what the option must do."""
    torch.manual_seed(3)
    old = torch.randn(3, 7)
    roll = old + torch.randn(3, 7) * 0.15
    mask = torch.ones(3, 7)
    _, new_mask, m = rc.correction_and_rejection_mask(old, roll, mask, rollout_rs=option, rollout_rs_threshold=threshold)
    assert f"rollout_corr/rollout_rs_{option}_mean" in m and new_mask.shape == mask.shape
    if not option.startswith("token"):
        assert all(row.min() == row.max() for row in new_mask)    # a sequence is kept or dropped as a whole
    frac = m[f"rollout_corr/rollout_rs_{option}_masked_fraction"]
    assert frac == pytest.approx(1.0 - new_mask.mean().item(), abs=1e-6)
    # a huge mismatch on one token is always caught
    roll2 = roll.clone()
    roll2[1, 3] -= 9.0
    _, bad_mask, _ = rc.correction_and_rejection_mask(old, roll2, mask, rollout_rs=option, rollout_rs_threshold=threshold)
    assert bad_mask[1, 3] == 0


def test_identical_policies_closed_form():
    old = -torch.rand(4, 9) * 3
    mask = (torch.arange(9).unsqueeze(0) < torch.tensor([9, 4, 1, 0]).unsqueeze(1)).float()
    for mode in ("token", "sequence"):
        w, new_mask, m = rc.correction_and_rejection_mask(old, old.clone(), mask, rollout_is=mode, rollout_is_threshold=2.0,
                                                          rollout_rs="token_k1,seq_sum_k2,seq_max_k3", rollout_rs_threshold="0.5_2.0,1.0,1.0")
        assert torch.equal(w, mask) and torch.equal(new_mask, mask)
        for k in ("kl", "k3_kl", "chi2_token", "chi2_seq", "log_ppl_diff", "rollout_rs_masked_fraction"):
            assert abs(m[f"rollout_corr/{k}"]) < 1e-6, k
        assert m["rollout_corr/rollout_is_mean"] == pytest.approx(1.0, abs=1e-6)
        assert m["rollout_corr/rollout_is_eff_sample_size"] == pytest.approx(1.0, abs=1e-5)
        assert m["rollout_corr/ppl_ratio"] == pytest.approx(1.0, abs=1e-6)


def test_sequence_weights_and_batch_normalisation():
    torch.manual_seed(5)
    old = torch.randn(4, 10)
    roll = old + torch.randn(4, 10) * 0.1
    mask = torch.ones(4, 10)
    mask[2, 6:] = 0
    w, _, m = rc.correction_and_rejection_mask(old, roll, mask, rollout_is="sequence", rollout_is_threshold=5.0)
    for b in range(4):
        valid = w[b][mask[b].bool()]
        assert torch.allclose(valid, valid[0]) and torch.all(w[b][~mask[b].bool()] == 0)
        expected = min(math.exp(((old - roll) * mask)[b].sum().item()), 5.0)
        assert valid[0].item() == pytest.approx(expected, rel=1e-5)
    wn, mn = rc.correction_weights(old - roll, mask, "token", 2.0, rollout_is_batch_normalize=True)
    assert rc.masked_mean(wn, mask).item() == pytest.approx(1.0, abs=1e-5) and "rollout_is_batch_norm_factor" in mn
    # TIS caps the weights; clamp bound respected for huge ratios (safety bound e^20)
    big = torch.full((1, 3), 50.0)
    wb, _ = rc.correction_weights(big, torch.ones(1, 3), "token", 2.0)
    assert torch.all(wb == 2.0)


def test_offpolicy_metrics_hand_values():
    old = torch.tensor([[-1.0, -2.0, -3.0], [-0.5, -0.5, 0.0]])
    roll = torch.tensor([[-1.5, -2.0, -2.0], [-1.0, -0.5, 0.0]])
    mask = torch.tensor([[1.0, 1.0, 1.0], [1.0, 1.0, 0.0]])
    m = rc.offpolicy_metrics(old, roll, mask)
    lr = [0.5, 0.0, -1.0, 0.5, 0.0]
    assert m["kl"] == pytest.approx(-sum(lr) / 5, abs=1e-6)
    assert m["k3_kl"] == pytest.approx(sum(math.exp(x) - x - 1 for x in lr) / 5, abs=1e-6)
    assert m["training_ppl"] == pytest.approx((math.exp(2.0) + math.exp(0.5)) / 2, rel=1e-6)
    assert m["rollout_log_ppl"] == pytest.approx((5.5 / 3 + 0.75) / 2, rel=1e-6)
    assert m["chi2_token"] == pytest.approx(sum(math.exp(2 * x) for x in lr) / 5 - 1, rel=1e-6)
    assert m["chi2_seq"] == pytest.approx((math.exp(2 * -0.5) + math.exp(2 * 0.5)) / 2 - 1, rel=1e-6)
    assert m["log_ppl_diff_max"] == pytest.approx(max((-5.5 + 6.0) / 3, (-1.5 + 1.0) / 2), abs=1e-6)
    only = rc.offpolicy_metrics(old, None, mask)
    assert set(only) == {"training_ppl", "training_log_ppl"}
    with pytest.raises(ValueError):
        rc.correction_and_rejection_mask(old, roll, torch.zeros_like(mask))
