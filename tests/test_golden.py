"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py).

Without a GPU: every oracle implementation reproduces them (so the fixtures and the oracle cannot drift apart
unnoticed). On the GPU: the HIP path reproduces them through the C ABI."""

import os

import numpy as np
import pytest
import torch

from oracle import c_oracle, scoring, verify as ov

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _scores():
    z = np.load(os.path.join(G, "scores_12x2053.npz"))
    x32 = torch.from_numpy(z["logits_f32"])
    x16 = torch.from_numpy(z["logits_bf16_bits"].astype(np.int16)).view(torch.bfloat16)
    return z, x32, x16, torch.from_numpy(z["labels"]), torch.from_numpy(z["temperature"])


def test_score_fixture_is_reproduced_by_the_oracles():
    z, x32, x16, lab, temp = _scores()
    assert torch.equal(x16, x32.bfloat16())
    for tag, x in (("f32", x32), ("bf16", x16)):
        for ttag, t in (("", None), ("_T", temp)):
            c_lp, c_h = c_oracle.rowscore(x, lab, t)
            assert np.array_equal(c_lp, z[f"logprob_{tag}{ttag}"]) and np.array_equal(c_h, z[f"entropy_{tag}{ttag}"])
            lp, h = scoring.score_fp32(x, lab, t)
            assert np.abs(lp.double().numpy() - z[f"logprob_{tag}{ttag}"]).max() < 5e-6
            assert np.abs(h.double().numpy() - z[f"entropy_{tag}{ttag}"]).max() < 2e-5
            lp64, h64 = scoring.score_fp64(x, lab, t)
            assert np.abs(lp64.numpy() - z[f"logprob_{tag}{ttag}"]).max() < 1e-11


def test_verify_fixture_is_reproduced_by_the_oracles():
    z = np.load(os.path.join(G, "verify_6x150.npz"))
    for mtag in ("", "_holes"):
        for otag, off in (("_m05", -0.5), ("_0", 0.0), ("_p05", 0.5)):
            for impl in (ov.verify, c_oracle.spec_verify):
                r = impl(z["logp_new"], z["logp_old"], z["log_u"], z["mask" + mtag], off, draft_ids=z["draft_ids"], pad_id=-1)
                for k in ("accept", "first_reject", "prefix_len", "near_count", "out_ids", "out_mask"):
                    assert np.array_equal(np.asarray(r[k]), z[f"{k}{mtag}{otag}"]), (k, mtag, otag, impl.__name__)


@pytest.mark.gpu
def test_hip_scores_reproduce_fixture(dev):
    from verl_amd import torch_functional as vf

    z, x32, x16, lab, temp = _scores()
    for tag, x, tol in (("f32", x32, 1e-5), ("bf16", x16, 2e-3)):
        for ttag, t in (("", None), ("_T", temp)):
            lp, h = vf.fused_logprob_entropy(x.to(dev), lab.to(dev), None if t is None else t.to(dev))
            e_lp = np.abs(lp.cpu().double().numpy() - z[f"logprob_{tag}{ttag}"]).max()
            e_h = np.abs(h.cpu().double().numpy() - z[f"entropy_{tag}{ttag}"]).max()
            assert e_lp <= tol and e_h <= tol, (tag, ttag, e_lp, e_h)
            assert e_lp <= 4e-6 and e_h <= 4e-6, (tag, ttag, e_lp, e_h)   # fp64 expected values: the kernel's own error


@pytest.mark.gpu
def test_hip_peaked_rows_reproduce_closed_form(dev):
    from verl_amd import torch_functional as vf

    rows = np.load(os.path.join(G, "peaked_rows.npz"))["rows"]
    for V, a, b, lp_peak, lp_rest, ent in rows:
        V = int(V)
        for dtype in (torch.bfloat16, torch.float32):
            x = torch.full((2, V), b, device=dev, dtype=dtype)
            x[:, 0] = a
            lp, h = vf.fused_logprob_entropy(x, torch.tensor([0, V - 1], device=dev))
            assert abs(lp[0].item() - lp_peak) <= 2e-6 and abs(lp[1].item() - lp_rest) <= 4e-6
            assert (h.cpu().double() - ent).abs().max().item() <= 2e-6


@pytest.mark.gpu
def test_hip_verify_reproduces_fixture(dev):
    from verl_amd import spec_rl as sv

    z = np.load(os.path.join(G, "verify_6x150.npz"))
    t = lambda k: torch.from_numpy(z[k]).to(dev)
    for mtag in ("", "_holes"):
        for otag, off in (("_m05", -0.5), ("_0", 0.0), ("_p05", 0.5)):
            r = sv.spec_verify(t("logp_new"), t("logp_old"), t("mask" + mtag), log_u=t("log_u"), thresh_offset=off,
                               draft_ids=t("draft_ids"), pad_id=-1)
            assert np.array_equal(r.accept.cpu().numpy().astype(np.uint8), z[f"accept{mtag}{otag}"])
            assert np.array_equal(r.first_reject.cpu().numpy(), z[f"first_reject{mtag}{otag}"])
            assert np.array_equal(r.prefix_len.cpu().numpy(), z[f"prefix_len{mtag}{otag}"])
            assert np.array_equal(r.near_count.cpu().numpy(), z[f"near_count{mtag}{otag}"])
            assert np.array_equal(r.out_ids.cpu().numpy(), z[f"out_ids{mtag}{otag}"])
            assert np.array_equal(r.out_mask.cpu().numpy().astype(np.uint8), z[f"out_mask{mtag}{otag}"])
