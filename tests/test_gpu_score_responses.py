"""vrl_score_responses: one launch from packed logits to the padded (B, T) response blocks — the label roll
(verl/workers/engine/fsdp/transformer_impl.py:1177), temperature, entropy and log-probs (:1357-1399) and
no_padding_2_padding (verl/workers/utils/padding.py:97-141) in the row kernel itself.

Checked against the reference-held fixture, against the oracle's restatement of the same sequence of steps, and bit for
bit against this library's separate entry points (vrl_rowscore followed by vrl_response_slice)."""

import numpy as np
import pytest
import torch

import verl_amd
from verl_amd import _lib, errors, layout
from verl_amd import torch_functional as vf
from oracle import scoring
from _parity import assert_scores_match

pytestmark = pytest.mark.gpu


def _batch(dev, seed, B, V, dtype, max_prompt=40, max_resp=90, scale=2.5):
    g = torch.Generator().manual_seed(seed)
    prompt = torch.randint(1, max_prompt, (B,), generator=g)
    resp = torch.randint(0, max_resp, (B,), generator=g)
    cu = torch.zeros(B + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(prompt + resp, 0)
    n = int(cu[-1])
    gd = torch.Generator(device=dev).manual_seed(seed + 1)
    ids = torch.randint(0, V, (n,), generator=gd, device=dev)
    logits = (torch.randn(n, V, generator=gd, device=dev) * scale).to(dtype)
    return prompt, resp, cu, ids, logits


def test_reference_fixture_through_the_single_launch(dev):
    """tests/models/test_fsdp_no_padding_on_gpu.py:180-201 in the reference: seed 0, vocab 32, sequences of 5 and 3
    tokens with 2 and 1 response tokens -> rows [2:4] and [6:7] of the packed log-probs, zero-padded to (2, 2)."""
    torch.manual_seed(0)
    logits = torch.randn(2, 5, 32)
    flat = torch.cat([logits[0, :5], logits[1, :3]], dim=0).to(dev)
    ids = torch.tensor([11, 12, 13, 14, 15, 21, 22, 23], device=dev)
    cu = torch.tensor([0, 5, 8], device=dev)
    resp = torch.tensor([2, 1], device=dev)
    r_lp, r_h = verl_amd.score_responses(flat, cu, resp, 2, input_ids=ids)
    full = scoring.logprobs_from_logits(flat.cpu(), scoring.roll_labels(ids.cpu()))
    full_h = scoring.entropy_from_logits(flat.cpu())
    expected = torch.stack([full[2:4], torch.nn.functional.pad(full[6:7], (0, 1))])
    expected_h = torch.stack([full_h[2:4], torch.nn.functional.pad(full_h[6:7], (0, 1))])
    assert r_lp.shape == (2, 2) and (r_lp.cpu() - expected).abs().max().item() <= 1e-5
    assert (r_h.cpu() - expected_h).abs().max().item() <= 1e-5
    assert r_lp[1, 1].item() == 0.0 and r_h[1, 1].item() == 0.0
    # ready-made labels instead of the ids give the same block
    r2, _ = verl_amd.score_responses(flat, cu, resp, 2, labels=layout.roll_labels(ids))
    assert torch.equal(r2, r_lp)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-3)])
@pytest.mark.parametrize("with_temperature", [False, True])
def test_random_packed_batches_against_oracle_and_separate_entry_points(dev, dtype, tol, with_temperature):
    B, V = 23, 4099
    prompt, resp, cu, ids, logits = _batch(dev, 77, B, V, dtype)
    n = logits.shape[0]
    temp = None
    if with_temperature:
        per_seq = 0.5 + torch.rand(B, generator=torch.Generator().manual_seed(3))
        temp = torch.repeat_interleave(per_seq, prompt + resp).to(dev)
    for T in (int(resp.max()), int(resp.max()) + 37):
        r_lp, r_h, t_lp, t_h = verl_amd.score_responses(logits, cu.to(dev), resp.to(dev), T, input_ids=ids,
                                                        temperature=temp, per_token=True)
        # bit for bit what the separate launches give
        lp, h = vf.fused_logprob_entropy(logits, layout.roll_labels(ids), temp)
        assert torch.equal(t_lp, lp) and torch.equal(t_h, h)
        assert torch.equal(r_lp, layout.response_slice(lp, cu.to(dev), resp.to(dev), T))
        assert torch.equal(r_h, layout.response_slice(h, cu.to(dev), resp.to(dev), T))
        # without the per-token vectors only the response rows are scored: same blocks
        s_lp, s_h = verl_amd.score_responses(logits, cu.to(dev), resp.to(dev), T, input_ids=ids, temperature=temp)
        assert torch.equal(s_lp, r_lp) and torch.equal(s_h, r_h)
        only_h = verl_amd.score_responses(logits, cu.to(dev), resp.to(dev), T, temperature=temp, want_logprob=False)
        assert only_h[0] is None and torch.equal(only_h[1], r_h)
        only_lp = verl_amd.score_responses(logits, cu.to(dev), resp.to(dev), T, input_ids=ids, temperature=temp,
                                           want_entropy=False)
        assert only_lp[1] is None and torch.equal(only_lp[0], r_lp)
        # the oracle's restatement of the reference's steps: per token with the shared parity rule (the fp64 value
        # within 4e-6; torch's fp32 composition within the bar widened by torch's own distance from the fp64 value) ...
        assert_scores_match(t_lp, t_h, logits, layout.roll_labels(ids), temp)
        # ... and the slicing exactly, on the fp64 values
        ref_lp, ref_h = scoring.score_fp64(logits.cpu(), scoring.roll_labels(ids.cpu()), None if temp is None else temp.cpu())
        want_lp = scoring.response_slice(ref_lp.float(), prompt.tolist(), resp.tolist(), T)
        want_h = scoring.response_slice(ref_h.float(), prompt.tolist(), resp.tolist(), T)
        assert (r_lp.cpu() - want_lp).abs().max().item() <= 4e-6
        assert (r_h.cpu() - want_h).abs().max().item() <= 4e-6
        assert torch.equal(r_lp.cpu() == 0, want_lp == 0)


def test_one_temperature_per_sequence_is_expanded_like_the_engine_does(dev):
    """The engine holds one temperature per sample and repeats it over the sample's tokens before dividing
    (verl/workers/engine/fsdp/transformer_impl.py:1149-1162, expand_as_nested): passing the (B,) tensor gives the
    same bits as passing the expanded (total_nnz,) one."""
    g = torch.Generator().manual_seed(31)
    B, V = 9, 3001
    prompt = torch.randint(1, 20, (B,), generator=g)
    resp = torch.randint(0, 30, (B,), generator=g)
    cu = torch.zeros(B + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(prompt + resp, 0)
    n = int(cu[-1])
    x = (torch.randn(n, V, generator=g) * 2).bfloat16().to(dev)
    ids = torch.randint(0, V, (n,), generator=g).to(dev)
    t_seq = (torch.rand(B, generator=g) + 0.5).to(dev)
    t_tok = scoring.expand_as_nested_values(t_seq.cpu(), cu).to(dev)
    T = int(resp.max())
    a = vf.score_responses(x, cu.to(dev), resp.to(dev), T, input_ids=ids, temperature=t_seq)
    b = vf.score_responses(x, cu.to(dev), resp.to(dev), T, input_ids=ids, temperature=t_tok)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert not torch.equal(a[0], vf.score_responses(x, cu.to(dev), resp.to(dev), T, input_ids=ids)[0])


def test_prompt_rows_do_not_matter_without_per_token_outputs(dev):
    """Only rows inside a response window are scored when no per-token vector is asked for: whatever the prompt rows
    hold (here NaN), the blocks are the same."""
    B, V = 9, 3001
    prompt, resp, cu, ids, logits = _batch(dev, 5, B, V, torch.bfloat16)
    T = int(resp.max())
    want = verl_amd.score_responses(logits, cu.to(dev), resp.to(dev), T, input_ids=ids)
    poisoned = logits.clone()
    for b in range(B):
        end, r = int(cu[b + 1]), int(resp[b])
        poisoned[int(cu[b]):end - r - 1] = float("nan")
        poisoned[end - 1] = float("nan")
    got = verl_amd.score_responses(poisoned, cu.to(dev), resp.to(dev), T, input_ids=ids)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_device_side_checks(dev):
    B, V = 6, 1000
    prompt, resp, cu, ids, logits = _batch(dev, 9, B, V, torch.float32)
    resp = torch.clamp(resp, min=1)
    cu = torch.zeros(B + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(prompt + resp, 0)
    n = int(cu[-1])
    gd = torch.Generator(device=dev).manual_seed(10)
    ids = torch.randint(0, V, (n,), generator=gd, device=dev)
    logits = torch.randn(n, V, generator=gd, device=dev)
    T = int(resp.max())
    cud, rd = cu.to(dev), resp.to(dev)
    good = verl_amd.score_responses(logits, cud, rd, T, input_ids=ids)
    # a sequence whose "response" swallows its prompt: ValueError, and its row is zero when nobody looks
    bad_r = resp.clone()
    bad_r[2] = prompt[2] + resp[2]
    with pytest.raises(ValueError, match="prompt token"):
        verl_amd.score_responses(logits, cud, bad_r.to(dev), int(bad_r.max()), input_ids=ids)
    out = verl_amd.score_responses(logits, cud, bad_r.to(dev), int(bad_r.max()), input_ids=ids, check=False)
    assert torch.all(out[0][2] == 0) and torch.equal(out[0][3, :T], good[0][3])
    # a response longer than the block
    with pytest.raises(ValueError, match="response length"):
        verl_amd.score_responses(logits, cud, rd, T - 1, input_ids=ids)
    # offsets that do not partition the rows
    for bad in ([0] + (cu[1:-1]).tolist() + [n + 5], [1] + cu[1:].tolist(), cu.flip(0).tolist()):
        with pytest.raises(ValueError, match="partition"):
            verl_amd.score_responses(logits, torch.tensor(bad, device=dev), rd, T, input_ids=ids)
    # a label outside the vocabulary lands in the block as NaN and raises IndexError
    bad_ids = ids.clone()
    first_resp_row = int(cu[1]) - int(resp[0]) - 1
    bad_ids[first_resp_row + 1] = V
    with pytest.raises(IndexError):
        verl_amd.score_responses(logits, cud, rd, T, input_ids=bad_ids)
    with errors.using("deferred"):
        out = verl_amd.score_responses(logits, cud, rd, T, input_ids=bad_ids)
        with pytest.raises(IndexError):
            errors.check_errors()
    assert torch.isnan(out[0][0, 0]) and torch.equal(out[0][1:], good[0][1:])
    # argument errors found on the host
    with pytest.raises(ValueError):
        verl_amd.score_responses(logits, cud, rd, T)                                   # no labels for the log-probs
    with pytest.raises(ValueError):
        verl_amd.score_responses(logits, cud, rd, T, input_ids=ids, labels=ids)
    with pytest.raises(ValueError):
        verl_amd.score_responses(logits, cud[:-1], rd, T, input_ids=ids)
    with pytest.raises(ValueError):
        verl_amd.score_responses(logits.view(1, n, V), cud, rd, T, input_ids=ids)
    empty = verl_amd.score_responses(logits[:0], cud[:1], rd[:0], 4, input_ids=ids[:0])
    assert empty[0].shape == (0, 4)


def _separate_steps(logits, labels, temp, cu, resp, T):
    """The same blocks from this library's row op (its own, separately tested, backward) and torch slicing."""
    lp, h = vf.fused_logprob_entropy(logits, labels, temp)
    rows_lp, rows_h = [], []
    for b in range(resp.numel()):
        end, r = int(cu[b + 1]), int(resp[b])
        rows_lp.append(torch.nn.functional.pad(lp[end - r - 1:end - 1], (0, T - r)))
        rows_h.append(torch.nn.functional.pad(h[end - r - 1:end - 1], (0, T - r)))
    return torch.stack(rows_lp), torch.stack(rows_h)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("which", ["both", "logprob", "entropy"])
def test_gradient_equals_the_separate_steps_bit_for_bit(dev, dtype, which):
    """d(blocks)/d(logits) from vrl_score_responses_backward equals what autograd builds from the row op's backward and
    torch's slicing and padding; prompt rows and each sequence's last row get exact zeros."""
    B, V = 11, 4099
    prompt, resp, cu, ids, logits = _batch(dev, 123, B, V, dtype)
    n = logits.shape[0]
    T = int(resp.max()) + 3
    per_seq = 0.5 + torch.rand(B, generator=torch.Generator().manual_seed(4))
    temp = torch.repeat_interleave(per_seq, prompt + resp).to(dev)
    gd = torch.Generator(device=dev).manual_seed(5)
    w_lp = torch.randn(B, T, generator=gd, device=dev)
    w_h = torch.randn(B, T, generator=gd, device=dev)
    labels = layout.roll_labels(ids)

    def loss(r_lp, r_h):
        out = 0.0
        if which in ("both", "logprob"):
            out = out + (r_lp * w_lp).sum()
        if which in ("both", "entropy"):
            out = out + (r_h * w_h).sum()
        return out

    a = logits.clone().requires_grad_(True)
    got = verl_amd.score_responses(a, cu.to(dev), resp.to(dev), T, input_ids=ids, temperature=temp,
                                   want_logprob=which != "entropy", want_entropy=which != "logprob")
    before = dict(vf.counters)
    loss(*got).backward()
    assert vf.counters["backward_passes"] == before["backward_passes"] + 1
    b = logits.clone().requires_grad_(True)
    want = _separate_steps(b, labels, temp, cu, resp, T)
    if which != "entropy":
        assert torch.equal(got[0], want[0])
    if which != "logprob":
        assert torch.equal(got[1], want[1])
    loss(*want).backward()
    assert torch.equal(a.grad, b.grad)
    for s in range(B):
        begin, end, r = int(cu[s]), int(cu[s + 1]), int(resp[s])
        assert not a.grad[begin:end - r - 1].any() and not a.grad[end - 1].any()
    # ready labels instead of ids, and the gradient written over the logits' own storage
    c = logits.clone().requires_grad_(True)
    c2 = c * 1.0
    got2 = verl_amd.score_responses(c2, cu.to(dev), resp.to(dev), T, labels=labels if which != "entropy" else None,
                                    temperature=temp, want_logprob=which != "entropy", want_entropy=which != "logprob",
                                    inplace_backward=True)
    loss(*got2).backward()
    assert torch.equal(c.grad, a.grad)
    assert torch.equal(c2.detach(), a.grad)                  # c2's storage now holds the gradient


def test_gradient_against_fp64_autograd(dev):
    """The gradient itself against torch's fp64 autograd of the reference's sequence of steps (roll, divide, log-softmax
    gather, entropy, slice, pad), fp32 logits: |diff| <= 2e-6 * max|grad|."""
    B, V = 5, 1237
    prompt, resp, cu, ids, logits = _batch(dev, 9, B, V, torch.float32, max_prompt=9, max_resp=20)
    T = int(resp.max())
    gd = torch.Generator(device=dev).manual_seed(6)
    w_lp = torch.randn(B, T, generator=gd, device=dev)
    w_h = torch.randn(B, T, generator=gd, device=dev)
    a = logits.clone().requires_grad_(True)
    r_lp, r_h = verl_amd.score_responses(a, cu.to(dev), resp.to(dev), T, input_ids=ids, temperature=0.7)
    ((r_lp * w_lp).sum() + (r_h * w_h).sum()).backward()
    x = logits.double().cpu().requires_grad_(True)
    z = x / 0.7
    logp = torch.log_softmax(z, -1)
    lp = logp.gather(-1, torch.roll(ids.cpu(), -1)[:, None])[:, 0]
    h = -(logp.exp() * logp).sum(-1)
    total = 0.0
    for s in range(B):
        end, r = int(cu[s + 1]), int(resp[s])
        total = total + (lp[end - r - 1:end - 1] * w_lp[s, :r].double().cpu()).sum()
        total = total + (h[end - r - 1:end - 1] * w_h[s, :r].double().cpu()).sum()
    total.backward()
    assert (a.grad.double().cpu() - x.grad).abs().max().item() <= 2e-6 * x.grad.abs().max().item()


def test_bad_offsets_leave_the_guard_regions_alone(dev):
    from _guards import BAD_OFFSETS, Arena

    lib = _lib.load()
    N, V, B, T = 100, 512, 3, 16
    g = torch.Generator().manual_seed(8)
    for case, offsets in sorted(BAD_OFFSETS.items()):
        ar = Arena(dev)
        logits = ar.make(N * V, torch.bfloat16, (torch.randn(N * V, generator=g) * 2).bfloat16())
        ids = ar.make(N, torch.int64, torch.randint(0, V, (N,), generator=g))
        cu = ar.make(B + 1, torch.int64, torch.tensor(offsets, dtype=torch.int64))
        rl = ar.make(B, torch.int64, torch.tensor([4, 7, 9], dtype=torch.int64))
        t_lp = ar.make(N, torch.float32)
        t_h = ar.make(N, torch.float32)
        r_lp = ar.make(B * T, torch.float32)
        r_h = ar.make(B * T, torch.float32)
        r_lse = ar.make(B * T, torch.float32)
        g_lp = ar.make(B * T, torch.float32, torch.randn(B * T, generator=g))
        g_h = ar.make(B * T, torch.float32, torch.randn(B * T, generator=g))
        dlogits = ar.make(N * V, torch.bfloat16)
        flag = ar.make(1, torch.int32, torch.zeros(1, dtype=torch.int32))
        print(f"[score_responses] cu_seqlens={offsets} over {N} rows", flush=True)
        for per_token in (True, False):
            flag.zero_()
            with torch.cuda.device(dev):
                st = lib.vrl_score_responses(logits.data_ptr(), _lib.VRL_BF16, N, V, V, None, ids.data_ptr(), None,
                                             cu.data_ptr(), rl.data_ptr(), B, T, t_lp.data_ptr() if per_token else None,
                                             t_h.data_ptr() if per_token else None, r_lp.data_ptr(), r_h.data_ptr(),
                                             r_lse.data_ptr(), flag.data_ptr(), _lib.stream_ptr(dev))
            assert st == _lib.VRL_OK
            torch.cuda.synchronize(dev)
            assert int(flag.item()) & _lib.VRL_FLAG_SEQ_RANGE, case
            assert ar.guards_intact(), case
            assert torch.isfinite(r_lp).all() and torch.isfinite(r_h).all(), case   # every block element was written
        # the backward over the same offsets: every row of the gradient is written, nothing else is
        with torch.cuda.device(dev):
            st = lib.vrl_score_responses_backward(logits.data_ptr(), _lib.VRL_BF16, N, V, V, None, ids.data_ptr(), None,
                                                  cu.data_ptr(), rl.data_ptr(), B, T, r_lse.data_ptr(), r_h.data_ptr(),
                                                  g_lp.data_ptr(), g_h.data_ptr(), dlogits.data_ptr(), V,
                                                  _lib.stream_ptr(dev))
        assert st == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert ar.guards_intact(), case
        assert torch.isfinite(dlogits.float()).all(), case


def test_c3_micro_batch_full_size(dev):
    """One 8192-token packed micro-batch at vocabulary 151936 bf16 (the GRPO workload's shape): the single launch
    equals the separate launches bit for bit."""
    V, n = 151936, 8192
    lens = [2048, 1700, 1500, 1200, 1000, 744]
    assert sum(lens) == n
    resp = torch.tensor([1500, 1000, 1499, 600, 999, 700])
    cu = torch.zeros(len(lens) + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(torch.tensor(lens), 0)
    gd = torch.Generator(device=dev).manual_seed(33)
    logits = torch.empty(n, V, dtype=torch.bfloat16, device=dev)
    for i in range(0, n, 1024):
        logits[i:i + 1024] = (torch.randn(1024, V, generator=gd, device=dev) * 3).bfloat16()
    ids = torch.randint(0, V, (n,), generator=gd, device=dev)
    T = 2048
    r_lp, r_h = verl_amd.score_responses(logits, cu.to(dev), resp.to(dev), T, input_ids=ids, temperature=0.9)
    lp, h = vf.fused_logprob_entropy(logits, layout.roll_labels(ids), 0.9)
    assert torch.equal(r_lp, layout.response_slice(lp, cu.to(dev), resp.to(dev), T))
    assert torch.equal(r_h, layout.response_slice(h, cu.to(dev), resp.to(dev), T))
    rows = torch.arange(0, n, 997)
    ref_lp, ref_h = scoring.score_fp32(logits[rows.to(dev)].cpu(), layout.roll_labels(ids)[rows.to(dev)].cpu(),
                                       torch.full((rows.numel(),), 0.9))
    assert (lp[rows.to(dev)].cpu() - ref_lp).abs().max().item() <= 2e-3
    assert (h[rows.to(dev)].cpu() - ref_h).abs().max().item() <= 2e-3


@pytest.mark.parametrize("dtype,V", [(torch.bfloat16, 32760), (torch.float32, 16388)])
def test_gradient_of_back_to_back_rows_takes_the_walk_without_rows_with_the_same_bits(dev, dtype, V):
    """64 MiB or more of contiguous logits from at most 64 sequences: the gradient is written by workgroups that walk
    the rows as one array (score_responses_backward_flat_kernel) instead of one workgroup per row. Same bits as the
    per-row kernel (run here on the same rows with a pitch), zeros for every row outside a response window, and with
    inconsistent offsets nothing outside the gradient's own array is touched."""
    from _guards import Arena

    lib = _lib.load()
    code = _lib.VRL_BF16 if dtype == torch.bfloat16 else _lib.VRL_F32
    per_vec = 16 // torch.empty((), dtype=dtype).element_size()
    lens = torch.tensor([300, 1, 250, 2, 348, 199])          # a one-token sequence and one with a one-token response among them
    resp = torch.tensor([120, 0, 249, 1, 100, 0])
    B, T = len(lens), 260
    cu = torch.zeros(B + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(lens, 0)
    N = int(cu[-1])
    g = torch.Generator(device=dev).manual_seed(V)
    x = (torch.randn(N, V, generator=g, device=dev) * 2.5).to(dtype)
    assert x.numel() * x.element_size() >= (1 << 26)
    ids = torch.randint(0, V, (N,), generator=g, device=dev)
    temp = torch.rand(N, generator=g, device=dev) + 0.5
    r_lp, r_h, r_lse = (torch.empty(B, T, device=dev) for _ in range(3))
    g_lp = torch.randn(B, T, generator=g, device=dev)
    g_h = torch.randn(B, T, generator=g, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    cu_d, rl_d = cu.to(dev), resp.to(dev)
    wide = torch.zeros(N, V + 2 * per_vec, dtype=dtype, device=dev)
    wide[:, :V] = x
    out_flat = torch.full_like(x, float("nan"))
    out_rows = torch.full_like(wide, float("nan"))
    stream = _lib.stream_ptr(dev)
    with torch.cuda.device(dev):
        st = lib.vrl_score_responses(x.data_ptr(), code, N, V, V, None, ids.data_ptr(), temp.data_ptr(), cu_d.data_ptr(),
                                     rl_d.data_ptr(), B, T, None, None, r_lp.data_ptr(), r_h.data_ptr(), r_lse.data_ptr(),
                                     flag.data_ptr(), stream)
        assert st == _lib.VRL_OK
        for src, dst in ((x, out_flat), (wide, out_rows)):
            st = lib.vrl_score_responses_backward(src.data_ptr(), code, N, V, src.stride(0), None, ids.data_ptr(),
                                                  temp.data_ptr(), cu_d.data_ptr(), rl_d.data_ptr(), B, T, r_lse.data_ptr(),
                                                  r_h.data_ptr(), g_lp.data_ptr(), g_h.data_ptr(), dst.data_ptr(),
                                                  dst.stride(0), stream)
            assert st == _lib.VRL_OK
    torch.cuda.synchronize(dev)
    assert int(flag.item()) == 0
    bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
    assert torch.equal(out_flat.view(bits), out_rows[:, :V].contiguous().view(bits))
    in_window = torch.zeros(N, dtype=torch.bool)
    for b in range(B):
        end, r = int(cu[b + 1]), int(resp[b])
        in_window[end - r - 1:end - 1] = True
    assert not bool(out_flat[~in_window.to(dev)].any()) and bool(out_flat[in_window.to(dev)].any(-1).all())
    # inconsistent offsets: the gradient array between guard regions
    for offsets in ([0, 300, 301, 551, 553, 5000, N], [5, 301, 551, 553, 900, 1000, N], [0, 800, 400, 551, 553, 900, N],
                    [-50, 301, 551, 553, 900, 1000, N], [0, 301, 2 ** 40, 551, 900, 1000, N]):
        ar = Arena(dev)
        grad = ar.make(N * V, dtype)
        bad = torch.tensor(offsets, dtype=torch.int64, device=dev)
        with torch.cuda.device(dev):
            st = lib.vrl_score_responses_backward(x.data_ptr(), code, N, V, V, None, ids.data_ptr(), temp.data_ptr(),
                                                  bad.data_ptr(), rl_d.data_ptr(), B, T, r_lse.data_ptr(), r_h.data_ptr(),
                                                  g_lp.data_ptr(), g_h.data_ptr(), grad.data_ptr(), V, stream)
        assert st == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert ar.guards_intact(), offsets
        assert torch.isfinite(grad.float()).all(), offsets        # every element of the gradient was written
        del ar, grad
