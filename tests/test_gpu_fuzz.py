"""Seeded random shapes, strides, alignments, dtypes, temperatures and special values: the HIP row kernel (forward,
both launch paths) against the fp64 C oracle and torch's NaN/inf pattern. 300 small cases, a few seconds."""

import numpy as np
import pytest
import torch

from verl_amd import torch_functional as vf
from oracle import c_oracle, scoring

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _case(rng, dev):
    dtype = DTYPES[rng.integers(0, 3)]
    n = int(rng.integers(1, 24))
    V = int(rng.choice([rng.integers(1, 70), rng.integers(70, 3000), rng.integers(3000, 70000)]))
    pad_l, pad_r = int(rng.integers(0, 9)), int(rng.integers(0, 9))
    sigma = float(rng.choice([0.1, 1.0, 3.0, 8.0]))
    shift = float(rng.choice([0.0, 0.0, -30.0, 50.0]))
    g = torch.Generator(device=dev).manual_seed(int(rng.integers(0, 2**31)))
    base = (torch.randn(n, pad_l + V + pad_r, generator=g, device=dev) * sigma + shift).to(dtype)
    x = base[:, pad_l:pad_l + V]
    lab = torch.randint(0, V, (n,), generator=g, device=dev)
    temp = None
    if rng.random() < 0.5:
        temp = torch.rand(n, generator=g, device=dev) * 1.7 + 0.3
    special = rng.random() < 0.25
    if special and V > 3:
        r = int(rng.integers(0, n))
        cols = torch.randint(0, V, (max(1, V // 10),), generator=g, device=dev)
        x[r, cols] = float("-inf")
        lab[r] = int(((x[r] > float("-inf")).nonzero()[0]).item()) if bool((x[r] > float("-inf")).any()) else 0
    splits = int(rng.choice([1, 1, 2, 3, 7]))
    return x, lab, temp, splits, special


def test_random_cases_against_fp64_oracle(dev):
    rng = np.random.default_rng(20240607)
    worst = 0.0
    for i in range(300):
        x, lab, temp, splits, special = _case(rng, dev)
        lp, h, q = vf.fused_logprob_entropy(x, lab, temp, n_splits=splits, want_sum_pi_sq=True)
        c_lp, c_h = c_oracle.rowscore(x.cpu().contiguous(), lab.cpu(), None if temp is None else temp.cpu())
        got_lp, got_h = lp.cpu().double().numpy(), h.cpu().double().numpy()
        assert np.array_equal(np.isnan(got_lp), np.isnan(c_lp)), i
        assert np.array_equal(np.isnan(got_h), np.isnan(c_h)), i
        fin = np.isfinite(c_lp)
        # fp32 outputs: one ulp of the result plus the accumulation error. For 16-bit logits with a temperature
        # the oracle (like the reference) rounds every quotient x/T to fp32 before reducing, the kernel does not
        # (it folds 1/T into the exponent's multiplier); that rounding is half an fp32 ulp of the largest |x/T|.
        slack = 0.0
        if temp is not None and x.dtype != torch.float32:
            xf = x.float()
            zmax = float((xf[torch.isfinite(xf)].abs().max() / temp.min()).item())
            slack = 2.4e-7 * zmax
        tol_lp = 4e-6 + 2.4e-7 * np.abs(c_lp[fin]) + slack
        assert np.all(np.abs(got_lp[fin] - c_lp[fin]) <= tol_lp), (i, np.abs(got_lp[fin] - c_lp[fin]).max())
        finh = np.isfinite(c_h)
        assert np.all(np.abs(got_h[finh] - c_h[finh]) <= 4e-6 + 2.4e-7 * np.abs(c_h[finh]) + slack), (i, np.abs(got_h[finh] - c_h[finh]).max())
        worst = max(worst, float(np.abs(got_lp[fin] - c_lp[fin]).max(initial=0.0)), float(np.abs(got_h[finh] - c_h[finh]).max(initial=0.0)))
        if not special:
            z = x.float() if temp is None else scoring.apply_temperature(x.float(), temp)
            ref_q = torch.softmax(z.double(), -1).pow(2).sum(-1)
            assert ((q.double() - ref_q).abs() <= 1e-5 * ref_q + 1e-12).all(), i
            assert bool((lp <= 1e-6).all()) and bool((h >= -1e-5).all())
    print(f"worst absolute error over 300 cases: {worst:.2e}")


def test_random_cases_backward_against_torch_autograd(dev):
    """Gradients of (log-prob, entropy) for the same random cases against torch's autograd of the fp32 composition:
    absolute 4e-6 x the gradient scale for fp32 logits, plus one rounding step of the output type for 16-bit logits."""
    rng = np.random.default_rng(777)
    worst = 0.0
    for i in range(400):
        x, lab, temp, splits, special = _case(rng, dev)
        if special:
            continue
        g = torch.Generator(device=dev).manual_seed(i)
        g1 = torch.randn(x.shape[0], generator=g, device=dev)
        g2 = torch.randn(x.shape[0], generator=g, device=dev) * 0.3
        xr = x.detach().float().requires_grad_(True)
        lpr, hr = scoring.score_reference(xr, lab, temp)
        ((lpr * g1).sum() + (hr * g2).sum()).backward()
        xo = x.detach().clone().requires_grad_(True)
        lp, h = vf.fused_logprob_entropy(xo, lab, temp, n_splits=splits)
        ((lp * g1).sum() + (h * g2).sum()).backward()
        scale = float((g1.abs() + g2.abs() * 30).max()) / (1.0 if temp is None else float(temp.min()))
        rel = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[x.dtype]
        err = (xo.grad.float() - xr.grad).abs()
        tol = xr.grad.abs() * rel + 4e-6 * scale + (6e-8 if x.dtype == torch.float16 else 1e-7)
        assert bool((err <= tol).all()), (i, x.dtype, tuple(x.shape), float((err - tol).max()))
        worst = max(worst, float(err.max()))
    print(f"worst absolute gradient difference: {worst:.2e}")


def test_random_verify_cases_all_forms_against_the_c_oracle(dev):
    """Seeded random batches through the three forms of vrl_spec_verify (one workgroup per sequence with 128-bit or with
    element-wise accesses, two flat passes): packed and padded layouts, empty and one-token sequences, sequences that
    end on tile borders, masks with holes or none, NaN / inf log-probs, ties on the threshold, early and late
    rejections. Bit for bit against the C loops."""
    from verl_amd import spec_rl as sv
    from verl_amd import synthetic

    import os

    rng = np.random.default_rng(int(os.environ.get("VRL_FUZZ_SEED", "20240607")))
    for case in range(int(os.environ.get("VRL_FUZZ_CASES", "120"))):
        g = torch.Generator(device=dev).manual_seed(int(rng.integers(0, 2**31)))
        packed = rng.random() < 0.6
        if packed:
            B = int(rng.integers(1, 40))
            kinds = rng.integers(0, 5, size=B)
            lengths = [int({0: 0, 1: 1, 2: rng.integers(2, 70), 3: rng.integers(70, 3000), 4: 1024 * rng.integers(1, 4)}[k])
                       for k in kinds]
            cu = synthetic.pack_by_lengths(torch.tensor(lengths))
            shape = (int(cu[-1]),)
        else:
            B, T = int(rng.integers(1, 12)), int(rng.choice([1, 7, 64, 100, 1024, 1500, 3000]))
            cu, shape = None, (B, T)
        n = int(np.prod(shape))
        if n == 0:
            continue
        ln = -torch.rand(shape, generator=g, device=dev) * 5
        drift = float(rng.choice([0.003, 0.05, 0.5]))
        lo = ln + torch.randn(shape, generator=g, device=dev) * drift
        lu = torch.log(torch.rand(shape, generator=g, device=dev) * float(rng.choice([1.0, 0.1])))
        flat = (ln.view(-1), lo.view(-1), lu.view(-1))
        for _ in range(int(rng.integers(0, 4))):        # special values and exact ties
            i = int(rng.integers(0, n))
            which = int(rng.integers(0, 4))
            if which == 0:
                flat[0][i] = float("nan")
            elif which == 1:
                flat[2][i] = float("-inf")
            elif which == 2:
                flat[1][i] = float("inf")
            else:
                flat[1][i] = flat[0][i] - flat[2][i]      # d == tau up to rounding
        mask = None
        if rng.random() < 0.7:
            mask = torch.rand(shape, generator=g, device=dev) < float(rng.choice([0.5, 0.9, 0.99]))
        ids = torch.randint(0, 1000, shape, generator=g, device=dev)
        off = float(rng.choice([0.0, 0.5, -0.5]))
        cud = None if cu is None else cu.to(dev)
        ref = c_oracle.spec_verify(ln, lo, lu, mask, off, cu_seqlens=cu, draft_ids=ids, pad_id=-3)
        for form in (False, True):
            res = sv.spec_verify(ln, lo, mask, log_u=lu, thresh_offset=off, cu_seqlens=cud, draft_ids=ids, pad_id=-3,
                                 two_pass=form)
            what = f"case {case} two_pass={form} packed={packed} shape={shape}"
            assert np.array_equal(res.accept.cpu().numpy().astype(np.uint8), ref["accept"]), what
            for k in ("first_reject", "prefix_len", "near_count"):
                assert np.array_equal(getattr(res, k).cpu().numpy(), ref[k]), (what, k)
            assert np.array_equal(res.out_ids.cpu().numpy(), ref["out_ids"]), what
            assert np.array_equal(res.out_mask.cpu().numpy().astype(np.uint8), ref["out_mask"]), what
    print(f"{case + 1} random verify batches")


def test_random_response_slices_against_the_oracle(dev):
    """Seeded random packed batches through vrl_response_slice / vrl_response_pack: every element size the copy units
    1, 2, 4, 8 and 16 bytes come from, trailing dimensions of odd and even sizes, values that are views off the 16-byte
    grid, empty responses, responses as long as their sequence allows, a padded length below, at and above the longest
    response. Bit for bit against the reference's loop (verl/workers/utils/padding.py:133-138, :194-210)."""
    import os

    from verl_amd import layout

    dtypes = [torch.uint8, torch.int16, torch.bfloat16, torch.float16, torch.float32, torch.int32, torch.int64,
              torch.float64]
    rng = np.random.default_rng(int(os.environ.get("VRL_FUZZ_SEED", "20240607")) + 1)
    for case in range(int(os.environ.get("VRL_FUZZ_CASES", "150"))):
        g = torch.Generator().manual_seed(int(rng.integers(0, 2**31)))
        dtype = dtypes[int(rng.integers(0, len(dtypes)))]
        trailing = [(), (1,), (3,), (4,), (7,), (8,), (5, 3), (64,), (130,)][int(rng.integers(0, 9))]
        B = int(rng.integers(1, 20))
        prompt = torch.randint(1, 30, (B,), generator=g)
        kind = rng.integers(0, 4, size=B)
        resp = torch.tensor([int({0: 0, 1: 1, 2: rng.integers(0, 40), 3: rng.integers(40, 700)}[k]) for k in kind])
        cu = torch.zeros(B + 1, dtype=torch.int64)
        cu[1:] = torch.cumsum(prompt + resp, 0)
        N = int(cu[-1])
        inner = int(np.prod(trailing)) if trailing else 1
        lead = int(rng.integers(0, 5))            # elements the view starts behind its buffer's beginning
        flat = torch.randint(0, 251, (lead + N * inner,), generator=g).to(dtype)
        vals = flat[lead:].view((N,) + trailing)
        longest = int(resp.max())
        T = max(0, longest + int(rng.integers(-2, 4)))
        flat_d = flat.to(dev)
        vals_d = flat_d[lead:].view((N,) + trailing)
        if T >= longest:
            got = layout.response_slice(vals_d, cu.to(dev), resp.to(dev), T)
            ref = scoring.response_slice(vals, prompt.tolist(), resp.tolist(), T)
            assert got.dtype == dtype and torch.equal(got.cpu(), ref), (case, dtype, trailing, lead)
        elif T > 0:                                # a response does not fit the block: reported (a block without
            with pytest.raises(ValueError):        # columns is not looked at)
                layout.response_slice(vals_d, cu.to(dev), resp.to(dev), T)
        total = int(resp.sum()) if rng.random() < 0.5 else None
        packed, packed_cu = layout.response_from_packed(vals_d, cu.to(dev), resp.to(dev), total_response_tokens=total)
        ref_p, ref_cu = scoring.response_from_nested(vals, cu.tolist(), resp.tolist())
        assert packed.dtype == dtype and torch.equal(packed.cpu(), ref_p) and torch.equal(packed_cu.cpu(), ref_cu), case
    print(f"{case + 1} random packed batches sliced and packed")
