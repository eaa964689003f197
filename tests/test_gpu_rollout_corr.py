"""Rollout correction on the GPU (one HIP kernel + host-side metric assembly) against the oracle's torch
restatement of verl's rollout_corr_helper, run on the same device tensors, and against the exact cases the
reference's tests hold."""

import math

import pytest
import torch

from verl_amd import rollout_corr as vrc
from oracle import rollout_corr as orc

pytestmark = pytest.mark.gpu

OPTIONS = [("token_k1", "0.5_1.5"), ("token_k2", 2.0), ("token_k3", 2.0), ("seq_sum_k1", "0.6_1.4"),
           ("seq_sum_k2", 2.5), ("seq_sum_k3", 2.5), ("seq_mean_k1", "0.5_1.5"), ("seq_mean_k2", 2.0),
           ("seq_mean_k3", 2.0), ("seq_max_k2", 2.0), ("seq_max_k3", 2.0)]


def _data(dev, B, T, seed, noise=0.3, lengths=None):
    g = torch.Generator(device=dev).manual_seed(seed)
    old = -torch.rand(B, T, generator=g, device=dev) * 4
    roll = old + torch.randn(B, T, generator=g, device=dev) * noise
    if lengths is None:
        lengths = torch.randint(0, T + 1, (B,), generator=torch.Generator().manual_seed(seed))
        lengths[0] = T
    mask = (torch.arange(T, device=dev).unsqueeze(0) < lengths.to(dev).unsqueeze(1)).float()
    return old, roll, mask


def _close_metrics(got, ref, rel=2e-5, abs_=2e-6):
    assert set(got) == set(ref), (sorted(set(got) ^ set(ref)))
    for k, v in ref.items():
        assert got[k] == pytest.approx(v, rel=rel, abs=abs_), (k, got[k], v)


@pytest.mark.parametrize("option,threshold", OPTIONS)
def test_each_rejection_option(dev, option, threshold):
    old, roll, mask = _data(dev, 37, 130, seed=100 + [o for o, _ in OPTIONS].index(option))
    lr = old - roll
    new_mask, m = vrc.compute_rollout_rejection_mask(lr, mask, option, threshold)
    ref_mask, ref_m = orc.rejection_mask(lr, mask, option, threshold)
    assert new_mask.dtype == mask.dtype and torch.equal(new_mask, ref_mask)
    _close_metrics(m, ref_m)


def test_chained_options_and_mixed_thresholds(dev):
    old, roll, mask = _data(dev, 64, 300, seed=7, noise=0.25)
    lr = old - roll
    for rs, th in (("token_k1,seq_max_k3", "0.4_1.8,3.0"), ("token_k2,token_k3,seq_mean_k1,seq_sum_k2", "0.3,0.3,0.8_1.25,4.0"),
                   ("seq_mean_k2,seq_max_k2", 0.2), (",".join(o for o, _ in OPTIONS), ",".join(str(t) for _, t in OPTIONS))):
        new_mask, m = vrc.compute_rollout_rejection_mask(lr, mask.bool(), rs, th)
        ref_mask, ref_m = orc.rejection_mask(lr, mask, rs, th)
        assert new_mask.dtype == torch.bool and torch.equal(new_mask.float(), ref_mask)
        _close_metrics(m, ref_m)


@pytest.mark.parametrize("level", ["token", "sequence"])
@pytest.mark.parametrize("threshold", [2.0, "0.5_5.0", 1.05, "0.9_1.1"])
@pytest.mark.parametrize("normalize", [False, True])
def test_importance_weights(dev, level, threshold, normalize):
    old, roll, mask = _data(dev, 33, 200, seed=11, noise=0.05 if level == "sequence" else 0.4)
    lr = old - roll
    w, m = vrc.compute_rollout_correction_weights(lr, mask, level, threshold, normalize)
    ref_w, ref_m = orc.correction_weights(lr, mask, level, threshold, normalize)
    assert w.shape == ref_w.shape and w.dtype == torch.float32
    # sequence weights exponentiate a sum whose order of summation differs: relative 1e-5
    torch.testing.assert_close(w, ref_w, rtol=2e-5, atol=1e-7)
    _close_metrics(m, ref_m, rel=5e-5, abs_=5e-6)


def test_combined_call_matches_and_uses_reference_pins(dev):
    old, roll, mask = _data(dev, 48, 256, seed=13)
    for kw in (dict(rollout_is="token", rollout_is_threshold=2.0, rollout_rs="token_k1", rollout_rs_threshold="0.5_2.0"),
               dict(rollout_is="sequence", rollout_is_threshold="0.2_5.0", rollout_is_batch_normalize=True,
                    rollout_rs="seq_mean_k3,token_k2", rollout_rs_threshold="0.05,1.0"),
               dict(rollout_is=None, rollout_rs=None),
               dict(rollout_is="token", rollout_is_threshold=3.0)):
        w, new_mask, m = vrc.compute_rollout_correction_and_rejection_mask(old, roll, mask, **kw)
        rw, rmask, rm = orc.correction_and_rejection_mask(old, roll, mask, **kw)
        assert (w is None) == (rw is None)
        if w is not None:
            torch.testing.assert_close(w, rw, rtol=2e-5, atol=1e-7)
        assert torch.equal(new_mask, rmask)
        _close_metrics(m, rm, rel=5e-5, abs_=5e-6)

    # tests/trainer/ppo/test_rollout_corr.py:312-366 (mask mode)
    o = torch.full((2, 5), -2.0, device=dev)
    r = torch.tensor([[-1.0] * 5, [-2.5] * 5], device=dev)
    ones = torch.ones(2, 5, device=dev)
    w, nm, m = vrc.compute_rollout_correction_and_rejection_mask(o, r, ones, rollout_is="token", rollout_is_threshold=2.0,
                                                                 rollout_rs="token_k1", rollout_rs_threshold="0.5_2.0")
    assert torch.all(w[0] > 0)
    assert torch.allclose(w[0, 0], torch.tensor(0.368, device=dev), atol=0.01) and torch.allclose(w[1, 0], torch.tensor(1.649, device=dev), atol=0.01)
    assert torch.all(nm[0] == 0) and torch.all(nm[1] == 1)
    assert abs(m["rollout_corr/rollout_rs_masked_fraction"] - 0.5) < 0.01
    # :369-394 (IcePop exact values)
    raw = torch.tensor([[0.4, 0.8, 6.0]], device=dev)
    w, nm, m = vrc.compute_rollout_correction_and_rejection_mask(torch.zeros_like(raw), -torch.log(raw), torch.ones_like(raw),
                                                                 rollout_is="token", rollout_is_threshold="0.5_5.0")
    torch.testing.assert_close(w, torch.tensor([[0.0, 0.8, 0.0]], device=dev), atol=1e-6, rtol=1e-6)
    assert torch.equal(nm, torch.ones_like(raw))
    assert m["rollout_corr/rollout_is_oob_ratio"] == pytest.approx(2.0 / 3.0, abs=1e-6)
    assert m["rollout_corr/rollout_is_std"] == pytest.approx(0.3771236, abs=1e-6)
    assert m["rollout_corr/rollout_is_eff_sample_size"] == pytest.approx(1.0 / 3.0, abs=1e-6)
    # :416-442 (sequence fraction from raw weights): lr = log(raw), threshold 2
    raw = torch.tensor([[1.0, 6.0], [0.9, 1.1]], device=dev)
    _, m = vrc.compute_rollout_correction_weights(torch.log(raw), torch.ones_like(raw), "token", 2.0)
    assert m["rollout_is_seq_fraction_high"] == pytest.approx(0.5)


def test_offpolicy_metrics_and_errors(dev):
    old, roll, mask = _data(dev, 20, 90, seed=17)
    _close_metrics(vrc.compute_offpolicy_metrics(old, roll, mask), orc.offpolicy_metrics(old, roll, mask))
    _close_metrics(vrc.compute_offpolicy_metrics(old, None, mask), orc.offpolicy_metrics(old, None, mask))
    with pytest.raises(ValueError, match="at least one valid token"):
        vrc.compute_rollout_correction_and_rejection_mask(old, roll, torch.zeros_like(mask))
    with pytest.raises(ValueError):
        vrc.compute_rollout_correction_and_rejection_mask(old, roll[:, :5], mask)
    with pytest.raises(ValueError):
        vrc.compute_rollout_correction_and_rejection_mask(old, roll, mask, rollout_rs="token_k1")     # no threshold
    with pytest.raises(ValueError):
        vrc.compute_rollout_rejection_mask(old - roll, mask, "token_k9", 1.0)
    with pytest.raises(TypeError):
        vrc.compute_rollout_correction_weights(old - roll, mask, "token", True)                       # :397-413
    with pytest.raises(ValueError):
        vrc.compute_rollout_correction_weights(old - roll, mask, "geometric", 2.0)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        vrc.compute_offpolicy_metrics(old.cpu(), roll.cpu(), mask.cpu())
    empty = torch.empty(0, 5, device=dev)
    assert vrc.compute_rollout_rejection_mask(empty, empty, "token_k1", "0.5_2.0")[1] == {}


def test_large_batch_and_extreme_ratios(dev):
    """GRPO-sized (B, T), a few wildly off tokens (safety clamp at +-20), masks with an all-padding row."""
    B, T = 1024, 2048
    old, roll, mask = _data(dev, B, T, seed=19, noise=0.2)
    roll[5, 7] -= 60.0
    roll[9, 100] += 60.0
    mask[3] = 0
    w, nm, m = vrc.compute_rollout_correction_and_rejection_mask(old, roll, mask, rollout_is="token", rollout_is_threshold=2.0,
                                                                 rollout_rs="token_k1,seq_mean_k2", rollout_rs_threshold="0.5_2.0,0.05")
    rw, rmask, rm = orc.correction_and_rejection_mask(old, roll, mask, rollout_is="token", rollout_is_threshold=2.0,
                                                      rollout_rs="token_k1,seq_mean_k2", rollout_rs_threshold="0.5_2.0,0.05")
    torch.testing.assert_close(w, rw, rtol=2e-5, atol=1e-7)
    # sequence means are summed in another order: a sequence whose mean sits within 1e-6 of the bound may flip
    differing = (nm != rmask).any(dim=1)
    assert int(differing.sum()) <= 1
    _close_metrics(m, rm, rel=2e-3 if differing.any() else 1e-4, abs_=1e-5)
    assert math.isfinite(m["rollout_corr/chi2_seq"])
