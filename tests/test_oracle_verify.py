"""Pins the verify oracle: scalar loops (Python), vectorised torch, and C loops against each other, against
hand-computed rows, and against properties the rule fixes."""

import math

import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from oracle import c_oracle, verify as ov

IMPLS = [ov.verify_loops, ov.verify, c_oracle.spec_verify]
KEYS = ("accept", "first_reject", "prefix_len", "near_count")


def _eq(a, b, keys=KEYS):
    for k in keys:
        assert np.array_equal(np.asarray(a[k]), np.asarray(b[k])), k


def _rand(B, T, seed, drift=0.3, mask_p=0.8):
    g = torch.Generator().manual_seed(seed)
    ln = -torch.rand(B, T, generator=g) * 5
    lo = ln + torch.randn(B, T, generator=g) * drift
    lu = torch.log(torch.rand(B, T, generator=g))
    mk = torch.rand(B, T, generator=g) < mask_p
    ids = torch.randint(0, 1000, (B, T), generator=g)
    return ln, lo, lu, mk, ids


@pytest.mark.parametrize("impl", IMPLS)
def test_hand_computed_rows(impl):
    """Constant d = -1 (new -2, old -1) against per-token thresholds, in the style of the reference's exact-input
    mask test (tests/trainer/ppo/test_rollout_corr.py:312-366: old -2.0 vs rollout -1.0 / -2.5)."""
    ln = torch.full((3, 6), -2.0)
    lo = torch.full((3, 6), -1.0)
    lu = torch.tensor([[-2.0] * 6, [-2.0, -2.0, -0.5, -2.0, -0.5, -2.0], [-1.0] * 6])
    mk = torch.tensor([[1, 1, 1, 1, 0, 0], [1, 1, 1, 1, 1, 1], [1, 1, 1, 0, 0, 0]])
    ids = torch.arange(18).view(3, 6) + 100
    r = impl(ln, lo, lu, mk, 0.0, near_eps=1e-6, draft_ids=ids, pad_id=-1)
    assert np.asarray(r["accept"]).tolist() == [[1, 1, 1, 1, 0, 0], [1, 1, 0, 1, 0, 1], [1, 1, 1, 0, 0, 0]]
    assert np.asarray(r["first_reject"]).tolist() == [4, 2, 3]
    assert np.asarray(r["prefix_len"]).tolist() == [4, 2, 3]
    assert np.asarray(r["near_count"]).tolist() == [0, 0, 3]
    assert np.asarray(r["out_ids"]).tolist() == [[100, 101, 102, 103, -1, -1], [106, 107, -1, -1, -1, -1], [112, 113, 114, -1, -1, -1]]
    assert np.asarray(r["out_mask"]).tolist() == [[1, 1, 1, 1, 0, 0], [1, 1, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0]]
    # offset +1 (lenience e, literal): thresholds rise by one; row 0 sits exactly on it and still accepts (>=)
    r = impl(ln, lo, lu, mk, 1.0)
    assert np.asarray(r["first_reject"]).tolist() == [4, 2, 0]
    r = impl(ln, lo, lu, mk, -1.0)
    assert np.asarray(r["first_reject"]).tolist() == [4, 6, 3]


@pytest.mark.parametrize("impl", IMPLS)
def test_special_values(impl):
    nan, inf = float("nan"), float("inf")
    ln = torch.tensor([[-1.0, nan, -1.0, -1.0], [-1.0, -1.0, -inf, -1.0], [-1.0, -1.0, -1.0, -1.0]])
    lo = torch.full((3, 4), -1.0)
    lu = torch.tensor([[-1.0, -1.0, -1.0, -1.0], [-inf, -inf, -inf, -1.0], [-1.0, nan, -inf, -1.0]])
    r = impl(ln, lo, lu, None, 0.0)
    assert np.asarray(r["accept"]).tolist() == [[1, 0, 1, 1], [1, 1, 1, 1], [1, 0, 1, 1]]
    assert np.asarray(r["first_reject"]).tolist() == [1, 4, 1]


@pytest.mark.parametrize("B,T,seed", [(1, 1, 0), (4, 17, 1), (6, 64, 2), (3, 130, 3), (9, 65, 4)])
@pytest.mark.parametrize("off", [0.0, 0.5, -0.5])
def test_three_implementations_agree_padded(B, T, seed, off):
    ln, lo, lu, mk, ids = _rand(B, T, seed)
    a = ov.verify_loops(ln, lo, lu, mk, off, draft_ids=ids, pad_id=7)
    for impl in (ov.verify, c_oracle.spec_verify):
        _eq(a, impl(ln, lo, lu, mk, off, draft_ids=ids, pad_id=7), KEYS + ("out_ids", "out_mask"))
    b = ov.verify_loops(ln, lo, lu, None, off)
    for impl in (ov.verify, c_oracle.spec_verify):
        _eq(b, impl(ln, lo, lu, None, off))


def test_three_implementations_agree_packed():
    lengths = [0, 1, 63, 64, 65, 0, 200, 17]
    cu = np.concatenate([[0], np.cumsum(lengths)])
    N = int(cu[-1])
    ln, lo, lu, mk, ids = (t.reshape(-1) for t in _rand(1, N, 11))
    for m in (None, mk):
        a = ov.verify_loops(ln, lo, lu, m, 0.25, cu_seqlens=cu, draft_ids=ids, pad_id=1)
        for impl in (ov.verify, c_oracle.spec_verify):
            _eq(a, impl(ln, lo, lu, m, 0.25, cu_seqlens=cu, draft_ids=ids, pad_id=1), KEYS + ("out_ids", "out_mask"))
        assert np.asarray(a["first_reject"])[0] == 0 and np.asarray(a["first_reject"])[5] == 0
        assert np.all(np.asarray(a["first_reject"]) <= np.asarray(lengths))


@pytest.mark.parametrize("impl", IMPLS)
def test_rule_properties(impl):
    ln, lo, lu, mk, ids = _rand(7, 90, 21)
    L = mk.sum(1).numpy()
    last_valid = np.array([(np.nonzero(r)[0].max() + 1) if r.any() else 0 for r in mk.numpy()])
    # d >= 0 and offset <= 0: log u <= 0 so everything valid is accepted, first_reject is the end
    r = impl(lo + 0.1, lo, lu, mk, -0.2)
    assert np.array_equal(np.asarray(r["accept"]).astype(bool), mk.numpy())
    assert np.array_equal(np.asarray(r["first_reject"]), last_valid)
    assert np.array_equal(np.asarray(r["prefix_len"]), L)
    # masked tokens never reject, never accept
    r = impl(ln - 100.0, lo, lu, torch.zeros_like(mk), 0.0)
    assert np.asarray(r["accept"]).sum() == 0 and np.all(np.asarray(r["first_reject"]) == 0)
    # accept is monotone in the offset; prefix never exceeds the number of valid tokens
    prev = None
    for off in (-1.0, -0.3, 0.0, 0.3, 1.0):
        r = impl(ln, lo, lu, mk, off)
        acc = np.asarray(r["accept"]).astype(bool)
        if prev is not None:
            assert np.all(acc <= prev)
        prev = acc
        assert np.all(np.asarray(r["prefix_len"]) <= L)
        # every valid token before first_reject is accepted; the one at first_reject (if any) is valid and rejected
        for b in range(7):
            f = int(np.asarray(r["first_reject"])[b])
            assert np.all(acc[b, :f] == mk.numpy()[b, :f])
            if f < last_valid[b]:
                assert mk[b, f] and not acc[b, f]
    # u = 0 (log u = -inf) accepts anything finite
    r = impl(ln - 50.0, lo, torch.full_like(lu, -math.inf), mk, 3.0)
    assert np.array_equal(np.asarray(r["accept"]).astype(bool), mk.numpy())
    # verifying the truncated draft again changes nothing (right-padded masks: with holes a trailing run of
    # masked positions just before the cut would be dropped by the second pass)
    rp = torch.arange(90).unsqueeze(0) < torch.tensor([0, 1, 30, 64, 65, 89, 90]).unsqueeze(1)
    r = impl(ln, lo, lu, rp, 0.0, draft_ids=ids, pad_id=0)
    r2 = impl(ln, lo, lu, torch.as_tensor(np.asarray(r["out_mask"])), 0.0, draft_ids=torch.as_tensor(np.asarray(r["out_ids"])), pad_id=0)
    assert np.array_equal(np.asarray(r2["first_reject"]), np.asarray(r["first_reject"]))
    assert np.array_equal(np.asarray(r2["out_ids"]), np.asarray(r["out_ids"]))
    assert np.array_equal(np.asarray(r2["out_mask"]), np.asarray(r["out_mask"]))


def test_near_count_band():
    ln = torch.tensor([[0.0, 0.0, 0.0, 0.0]])
    lo = torch.zeros(1, 4)
    lu = torch.tensor([[0.0, -5e-7, 5e-7, -2e-6]])
    for impl in IMPLS:
        r = impl(ln, lo, lu, None, 0.0, near_eps=1e-6)
        assert np.asarray(r["near_count"]).tolist() == [3]
        assert np.asarray(r["accept"]).tolist() == [[1, 1, 0, 1]]


@settings(max_examples=80, deadline=None)
@given(st.integers(1, 5), st.integers(1, 70), st.integers(0, 2**31 - 1), st.floats(-1.0, 1.0), st.floats(0.0, 1.0))
def test_property_implementations_agree(B, T, seed, off, mask_p):
    ln, lo, lu, mk, ids = _rand(B, T, seed, mask_p=mask_p)
    a = ov.verify_loops(ln, lo, lu, mk, off, draft_ids=ids)
    _eq(a, ov.verify(ln, lo, lu, mk, off, draft_ids=ids), KEYS + ("out_ids", "out_mask"))
    _eq(a, c_oracle.spec_verify(ln, lo, lu, mk, off, draft_ids=ids), KEYS + ("out_ids", "out_mask"))
