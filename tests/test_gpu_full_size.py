"""Whole workloads at the sizes the benchmark configurations name, streamed through the fused entry point in
8192-token packed micro-batches (how verl feeds them after padding removal), one reusable logits buffer.

c3: 128 prompts x 8 samples x up to 2048 response tokens, vocab 151936 bf16, lengths U[256, 2048], drift N(0, 0.2),
    lenience e^0.5.
c5: 512 sequences with log-uniform lengths in [32, 16384], Student-t drift, lenience e^0.5.
c4: 16 x 8192, vocab 128256 fp32, temperature 0.7 in-kernel (67 GB resident, one call).

Per micro-batch: log-probs and entropy against torch's fp32 ops on the device (2e-3 for bf16; for fp32 1e-5 on the
log-prob and 5e-5 on the entropy, torch's own fp32 entropy being ~1e-5 from the exact value at this vocabulary),
and the verify outputs bit-exact against the C oracle fed the kernel's log-probs. Size-independent checks over
the whole workload: every sequence verified exactly once, prefix <= length, accepted tokens = sum of the mask.
"""

import numpy as np
import pytest
import torch

from verl_amd import spec_rl as sv
from verl_amd import synthetic
from oracle import c_oracle

pytestmark = pytest.mark.gpu


def _torch_scores(logits, labels, temp=None, chunk=2048):
    lp = torch.empty(logits.shape[0], device=logits.device)
    h = torch.empty_like(lp)
    for lo in range(0, logits.shape[0], chunk):
        z = logits[lo:lo + chunk].float()
        if temp is not None:
            z = z / temp[lo:lo + chunk].clamp(min=1e-8).unsqueeze(-1)
        lse = torch.logsumexp(z, -1)
        lp[lo:lo + chunk] = z.gather(-1, labels[lo:lo + chunk, None]).squeeze(-1) - lse
        h[lo:lo + chunk] = lse - (torch.softmax(z, -1) * z).sum(-1)
    return lp, h


def _micro_batches(lengths, budget):
    """Whole sequences packed greedily up to ``budget`` tokens; a sequence longer than the budget is cut into
    budget-sized pieces (each verified as its own sequence)."""
    batches, cur, tot = [], [], 0
    for L in lengths:
        L = int(L)
        while L > 0:
            take = min(L, budget)
            if tot + take > budget:
                batches.append(cur)
                cur, tot = [], 0
            cur.append(take)
            tot += take
            L -= take
    if cur:
        batches.append(cur)
    return batches


@pytest.mark.parametrize("name", ["c3", "c5"])
def test_whole_workload_in_packed_micro_batches(dev, name):
    w = synthetic.WORKLOADS[name]
    lengths = synthetic.draw_lengths(w, seed=31).tolist()
    batches = _micro_batches(lengths, w.micro_batch_tokens)
    assert sum(sum(b) for b in batches) == sum(lengths)
    off = sv.thresh_offset_from_lenience(w.lenience)
    gd = torch.Generator(device=dev).manual_seed(32)
    worst_lp = worst_h = 0.0
    n_seq = n_tok = n_acc = 0
    prefix_total = 0
    buf = torch.empty((w.micro_batch_tokens, w.V), dtype=w.dtype, device=dev)
    for bi, lens in enumerate(batches):
        n = sum(lens)
        cu = synthetic.pack_by_lengths(torch.tensor(lens))
        logits = buf[:n]
        for lo in range(0, n, 2048):       # refill the reusable buffer
            logits[lo:lo + 2048] = (torch.randn((min(2048, n - lo), w.V), generator=gd, device=dev) * w.sigma).to(w.dtype)
        labels = torch.randint(0, w.V, (n,), generator=gd, device=dev)
        log_u = torch.log(torch.rand(n, generator=gd, device=dev))
        ref_lp, ref_h = _torch_scores(logits, labels)
        old = synthetic.drift_old_logprobs(ref_lp, w, seed=1000 + bi)
        lp, h, res = sv.fused_score_verify(logits, labels, old, None, log_u=log_u, thresh_offset=off, cu_seqlens=cu.to(dev))
        worst_lp = max(worst_lp, (lp - ref_lp).abs().max().item())
        worst_h = max(worst_h, (h - ref_h).abs().max().item())
        ref = c_oracle.spec_verify(lp, old, log_u, None, off, cu_seqlens=cu)
        assert np.array_equal(res.accept.cpu().numpy().astype(np.uint8), ref["accept"]), bi
        assert np.array_equal(res.first_reject.cpu().numpy(), ref["first_reject"]), bi
        assert np.array_equal(res.prefix_len.cpu().numpy(), ref["prefix_len"]), bi
        assert (res.prefix_len.cpu() <= torch.tensor(lens)).all()
        n_seq += len(lens)
        n_tok += n
        n_acc += int(res.accept.sum())
        prefix_total += int(res.prefix_len.sum())
    assert worst_lp <= 2e-3 and worst_h <= 2e-3, (worst_lp, worst_h)
    assert n_tok == sum(lengths) and n_seq >= len(lengths)
    assert 0 < prefix_total <= n_acc <= n_tok
    print(f"{name}: {len(batches)} micro-batches, {n_tok} tokens, {n_seq} sequences; worst |dlogp| {worst_lp:.2e}, "
          f"|dH| {worst_h:.2e}; accepted {n_acc / n_tok:.3f}, reusable prefix {prefix_total / n_tok:.3f}")


def test_c4_whole_workload_resident(dev):
    w = synthetic.WORKLOADS["c4"]
    d = synthetic.make_padded(w, dev, seed=41)
    logits, labels, temp = d["logits"].view(-1, w.V), d["labels"].view(-1), d["temperature"].view(-1)
    ref_lp, ref_h = _torch_scores(logits, labels, temp)
    old = synthetic.drift_old_logprobs(ref_lp.view(w.B, w.T), w, seed=41)
    lp, h, res = sv.fused_score_verify(d["logits"], d["labels"], old, d["mask"], temperature=d["temperature"],
                                       log_u=d["log_u"], lenience=w.lenience)
    assert (lp.view(-1) - ref_lp).abs().max().item() <= 1e-5
    assert (h.view(-1) - ref_h).abs().max().item() <= 5e-5
    ref = c_oracle.spec_verify(lp, old, d["log_u"], d["mask"], res.thresh_offset)
    assert np.array_equal(res.accept.cpu().numpy().astype(np.uint8), ref["accept"])
    assert np.array_equal(res.first_reject.cpu().numpy(), ref["first_reject"])
    assert np.array_equal(res.near_count.cpu().numpy(), ref["near_count"])


@pytest.mark.parametrize("dtype,V", [(torch.float32, (1 << 29) + 100003), (torch.bfloat16, (1 << 30) + 100003)])
def test_one_row_longer_than_two_gibibytes(dev, dtype, V):
    """Offsets inside a row beyond 2^31 bytes (64-bit indexing in the kernels), forward and backward, against the
    closed form for a row of zeros with three raised entries, two of them past the 2 GiB mark."""
    import math
    from verl_amd import torch_functional as vf

    x = torch.zeros(2, V, dtype=dtype, device=dev)
    hot = {V - 1: 5.0, V - 70001: 3.0, 7: 4.0}
    for k, v in hot.items():
        x[:, k] = v
    assert (V - 70001) * x.element_size() > 2**31
    S = (V - 3) + sum(math.exp(v) for v in hot.values())
    lse = math.log(S)
    H = lse - sum(v * math.exp(v) for v in hot.values()) / S
    lab = torch.tensor([V - 1, V - 70001], device=dev)
    for splits in (None, 1):
        lp, h = vf.fused_logprob_entropy(x, lab, n_splits=splits)
        assert abs(lp[0].item() - (5.0 - lse)) <= 4e-6 and abs(lp[1].item() - (3.0 - lse)) <= 4e-6
        # half a billion fp32 additions per sum, result ~20 (one fp32 step there is 1.9e-6): a few steps
        assert abs(h[0].item() - H) <= 1e-5 and abs(h[1].item() - H) <= 1e-5
    # backward, in place over the row: d lp[r] / d x = onehot(label) - p
    xg = x[:1].clone().requires_grad_(True)
    vf.logprobs_from_logits((xg * 1.0), lab[:1], inplace_backward=True).sum().backward()
    g = xg.grad[0]
    # p = exp(x - lse) with lse ~ 20 rounded to fp32: a relative 4e-6 on every probability; one rounding step of the
    # output type for bf16
    tol = 4e-6 if dtype == torch.float32 else 2.0 ** -8
    assert abs(g[V - 1].item() - (1.0 - math.exp(5.0) / S)) <= tol
    assert abs(g[V - 70001].item() + math.exp(3.0) / S) <= tol * math.exp(3.0) / S + 1e-12
    assert abs(g[7].item() + math.exp(4.0) / S) <= tol * math.exp(4.0) / S + 1e-12
    assert abs(g[V // 2].item() + 1.0 / S) <= tol / S + 1e-15
    assert abs(g.double().sum().item()) <= 1e-3   # the gradient of a log-prob sums to zero over the row


@pytest.mark.parametrize("two_pass", [False, True])
def test_very_long_sequences_verify(dev, two_pass):
    """Two padded sequences of five million tokens: positions beyond any 16-bit or LDS-sized assumption; first
    rejections placed by hand near the end and in the middle, the rest accepts by construction (d = 0.5 >= log u).
    In the two-pass form a tile near the end learns from thousands of tiles back that no rejection is pending."""
    T = 5_000_011
    ln = torch.zeros(2, T, device=dev)
    lo = torch.full((2, T), -0.5, device=dev)
    g = torch.Generator(device=dev).manual_seed(1)
    log_u = torch.log(torch.rand(2, T, generator=g, device=dev))          # <= 0 < 0.5
    mask = torch.ones(2, T, dtype=torch.uint8, device=dev)
    mask[1, T - 1000:] = 0
    lo[0, T - 3] = 10.0                                                    # d = -10: rejected whatever u is (log u > -10 here)
    lo[1, 2_345_678] = 10.0
    log_u[0, T - 3] = -1.0
    log_u[1, 2_345_678] = -1.0
    ids = torch.arange(2 * T, device=dev).view(2, T)
    res = sv.spec_verify(ln, lo, mask, log_u=log_u, thresh_offset=0.0, draft_ids=ids, pad_id=-1, two_pass=two_pass)
    assert res.first_reject.tolist() == [T - 3, 2_345_678] and res.prefix_len.tolist() == [T - 3, 2_345_678]
    assert int(res.accept[0].sum()) == T - 1 and int(res.accept[1].sum()) == T - 1000 - 1
    assert bool((res.out_ids[0, :T - 3] == ids[0, :T - 3]).all()) and bool((res.out_ids[0, T - 3:] == -1).all())
    assert int(res.out_mask[1].sum()) == 2_345_678


def test_transpose_beyond_four_gibibytes(dev):
    """70000 x 16384 fp32 = 4.6 GB: byte offsets past 2^32 on both sides. Transposing twice gives the array back,
    and sampled entries sit where the definition puts them."""
    from verl_amd import layout

    rows, cols = 70000, 16384
    x = torch.arange(rows * cols, device=dev, dtype=torch.int32).view(rows, cols)   # every entry names its own place
    y = layout.transpose_2d(x)
    assert y.shape == (cols, rows)
    r = torch.tensor([0, 1, 127, 128, 65535, 65536, 69999], device=dev)
    c = torch.tensor([0, 5, 64, 8191, 16383], device=dev)
    assert torch.equal(y[c][:, r], x[r][:, c].t())
    assert int(y[cols - 1, rows - 1]) == int(x[rows - 1, cols - 1])
    del x
    back = layout.transpose_2d(y)
    expect_first = torch.arange(cols, device=dev, dtype=torch.int32)
    assert torch.equal(back[0], expect_first) and torch.equal(back[rows - 1], expect_first + (rows - 1) * cols)
    # a checksum over everything: sum of all entries mod 2^61 equals the closed form of sum(0 .. n-1) in wrapped int32
    assert int(back.view(-1)[::4097].to(torch.int64).sum()) == int(torch.arange(0, rows * cols, 4097, dtype=torch.int64).to(torch.int32).to(torch.int64).sum())
