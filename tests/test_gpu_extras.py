"""Split path (few rows), sum of squared probabilities, and the response slice, on the GPU."""

import numpy as np
import pytest
import torch

from verl_amd import errors, layout
from verl_amd import torch_functional as vf
from verl_amd import _lib
from oracle import c_oracle, scoring
from _parity import assert_scores_match

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,V", [(1, 151936), (7, 152064), (64, 128256), (300, 32000), (3, 4096), (5, 1000)])
def test_split_path_matches_oracle_and_single_pass(dev, dtype, n, V):
    g = torch.Generator(device=dev).manual_seed(n * 7 + V)
    x = (torch.randn(n, V, generator=g, device=dev) * 3).to(dtype)
    lab = torch.randint(0, V, (n,), generator=g, device=dev)
    temp = torch.rand(n, generator=g, device=dev) + 0.5
    plan = _lib.load().vrl_rowscore_split_plan(0 if dtype == torch.float32 else 1, n, V)
    for t in (None, temp):
        one = vf.fused_logprob_entropy(x, lab, t, n_splits=1, want_sum_pi_sq=True)
        for splits in sorted({plan, 2, 3, 16, 64}):
            got = vf.fused_logprob_entropy(x, lab, t, n_splits=splits, want_sum_pi_sq=True)
            assert_scores_match(got[0], got[1], x, lab, t, cpu_torch=False)
            # a different summation tree, same numbers to fp32 rounding
            assert (got[0] - one[0]).abs().max().item() <= 4e-6
            assert (got[1] - one[1]).abs().max().item() <= 4e-6
            assert ((got[2] - one[2]).abs() <= 4e-6 * one[2].abs() + 1e-12).all()
    auto = vf.fused_logprob_entropy(x, lab)       # what the wrapper picks by itself
    assert_scores_match(auto[0], auto[1], x, lab, None, cpu_torch=False)


def test_split_special_values_and_ragged(dev):
    inf = float("inf")
    V = 40000
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn(6, V, generator=g, device=dev)
    x[0, :30000] = -inf          # whole leading slices are -inf
    x[1, :] = -inf
    x[2, 39999] = inf
    x[3, 5] = float("nan")
    lab = torch.tensor([35000, 0, 1, 2, 3, 39999], device=dev)
    base = x[:, 3:39990]          # misaligned, strided rows
    lab2 = torch.tensor([31000, 0, 1, 2, 3, 39986], device=dev)
    for xx, ll in ((x, lab), (base, lab2)):
        ref_lp, ref_h = scoring.score_fp32(xx, ll)
        for splits in (1, 4, 9):
            lp, h = vf.fused_logprob_entropy(xx, ll, n_splits=splits)
            assert torch.equal(torch.isnan(lp), torch.isnan(ref_lp)) and torch.equal(torch.isnan(h), torch.isnan(ref_h))
            assert torch.equal(torch.isinf(lp), torch.isinf(ref_lp))
            fin = torch.isfinite(ref_lp)
            assert (lp[fin] - ref_lp[fin]).abs().max() <= 1e-5
            finh = torch.isfinite(ref_h)
            assert (h[finh] - ref_h[finh]).abs().max() <= 1e-5
    with pytest.raises(IndexError):
        vf.fused_logprob_entropy(x, torch.full((6,), V, device=dev), n_splits=4)


@pytest.mark.parametrize("shape", [(8, 17), (3, 5, 32), (1, 1024)])
def test_sum_pi_squared_reference_parametrisation(dev, shape):
    """Same cases as the reference's tests/utils/test_torch_functional.py:126-140, fp32 on the GPU."""
    torch.manual_seed(0)
    logits = (torch.randn(*shape) * 5.0).to(dev)
    actual = vf.calculate_sum_pi_squared_from_logits(logits)
    expected = torch.softmax(logits.double(), dim=-1).pow(2).sum(dim=-1)
    assert actual.shape == expected.shape and actual.dtype == torch.float32
    torch.testing.assert_close(actual.double(), expected, atol=1e-6, rtol=1e-5)
    assert torch.all(actual > 0) and torch.all(actual <= 1.0 + 1e-6)
    ref = scoring.calculate_sum_pi_squared_from_logits(logits.cpu())
    torch.testing.assert_close(actual.cpu(), ref, atol=1e-5, rtol=1e-5)


def test_sum_pi_squared_extremes_and_full_vocab(dev):
    # tests/utils/test_torch_functional.py:142-150 (fp64 there; fp32 inputs hold these values exactly)
    logits = torch.tensor([[1000.0, 1001.0, 999.0], [-1000.0, -999.0, -998.0]], device=dev)
    actual = vf.calculate_sum_pi_squared_from_logits(logits)
    expected = torch.softmax(logits.double(), dim=-1).pow(2).sum(dim=-1)
    assert torch.isfinite(actual).all()
    # |x| = 1000 leaves 2^-14 = 6e-5 of input resolution in fp32 after the log2(e) scaling
    torch.testing.assert_close(actual.double(), expected, atol=2e-4, rtol=2e-4)
    g = torch.Generator(device=dev).manual_seed(3)
    for dtype in (torch.bfloat16, torch.float32):
        x = (torch.randn(33, 151936, generator=g, device=dev) * 3).to(dtype)
        lab = torch.randint(0, 151936, (33,), generator=g, device=dev)
        temp = torch.full((33,), 0.7, device=dev)
        lp, h, q = vf.fused_logprob_entropy(x, lab, temp, want_sum_pi_sq=True)
        z = (x.float() / temp.unsqueeze(-1)).double()
        expected = torch.softmax(z, -1).pow(2).sum(-1)
        assert ((q.double() - expected).abs() <= 2e-6 * expected + 1e-12).all()
        lp2, h2 = vf.fused_logprob_entropy(x, lab, temp)
        assert torch.equal(lp, lp2) and torch.equal(h, h2)     # asking for the third output changes nothing else
        uniform = vf.calculate_sum_pi_squared_from_logits(torch.zeros(2, 1000, device=dev, dtype=dtype))
        assert (uniform - 1e-3).abs().max().item() <= 1e-9


def test_response_slice_reference_fixture(dev):
    """tests/models/test_fsdp_no_padding_on_gpu.py:170-205: sequences of 5 and 3 tokens, responses 2 and 1."""
    torch.manual_seed(0)
    logits = torch.randn(2, 5, 32)
    flat = torch.cat([logits[0, :5], logits[1, :3]], dim=0).to(dev)
    ids = torch.tensor([11, 12, 13, 14, 15, 21, 22, 23], device=dev)
    labels = layout.roll_labels(ids)
    assert labels.tolist() == [12, 13, 14, 15, 21, 22, 23, 11]
    full = vf.logprobs_from_logits(flat, labels % 32)
    cu = torch.tensor([0, 5, 8], device=dev)
    got = layout.response_slice(full, cu, torch.tensor([2, 1], device=dev), max_response_len=2)
    expected = torch.stack([full[2:4], torch.nn.functional.pad(full[6:7], (0, 1))])
    assert got.shape == (2, 2) and torch.equal(got, expected)
    ref = scoring.response_slice(full.cpu(), [3, 2], [2, 1], 2)
    assert torch.equal(got.cpu(), ref)
    # max_response_len defaults to the longest response
    assert torch.equal(layout.response_slice(full, cu, torch.tensor([2, 1], device=dev)), expected)


def test_response_slice_random_and_errors(dev):
    g = torch.Generator().manual_seed(4)
    B = 37
    prompt = torch.randint(1, 50, (B,), generator=g)
    resp = torch.randint(0, 300, (B,), generator=g)
    cu = torch.zeros(B + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(prompt + resp, 0)
    vals = torch.randn(int(cu[-1]), generator=g)
    for T in (int(resp.max()), 512):
        got = layout.response_slice(vals.to(dev), cu.to(dev), resp.to(dev), T)
        assert torch.equal(got.cpu(), scoring.response_slice(vals, prompt.tolist(), resp.tolist(), T))
    with pytest.raises(ValueError):   # a sequence without a prompt token
        layout.response_slice(vals.to(dev), cu.to(dev), (prompt + resp).to(dev), 512)
    with pytest.raises(ValueError):   # response longer than the output
        layout.response_slice(vals.to(dev), cu.to(dev), resp.to(dev), int(resp.max()) - 1)
    out = layout.response_slice(vals.to(dev), cu.to(dev), resp.to(dev), int(resp.max()) - 1, check=False)
    assert torch.all(out[resp.argmax()] == 0)
    assert layout.response_slice(vals[:0].to(dev), cu[:1].to(dev), resp[:0].to(dev), 4).shape == (0, 4)


def test_response_from_packed_matches_oracle_and_flags_bad_sequences(dev):
    g = torch.Generator().manual_seed(14)
    B = 53
    prompt = torch.randint(1, 40, (B,), generator=g)
    resp = torch.randint(0, 700, (B,), generator=g)
    resp[7] = 0
    cu = torch.zeros(B + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(prompt + resp, 0)
    vals = torch.randn(int(cu[-1]), generator=g)
    got, got_cu = layout.response_from_packed(vals.to(dev), cu.to(dev), resp.to(dev))
    ref, ref_cu = scoring.response_from_nested(vals, cu.tolist(), resp.tolist())
    assert torch.equal(got.cpu(), ref) and torch.equal(got_cu.cpu(), ref_cu)
    # the reference fixture's windows: full[2:4] and full[6:7]
    full = torch.arange(8, dtype=torch.float32, device=dev)
    v, o = layout.response_from_packed(full, torch.tensor([0, 5, 8], device=dev), torch.tensor([2, 1], device=dev))
    assert v.tolist() == [2.0, 3.0, 6.0] and o.tolist() == [0, 2, 3]
    with pytest.raises(ValueError):   # a sequence without a prompt token
        layout.response_from_packed(vals.to(dev), cu.to(dev), (prompt + resp).to(dev))
    bad = resp.clone()
    bad[3] = -2
    with pytest.raises(ValueError):
        layout.response_from_packed(vals.to(dev), cu.to(dev), bad.to(dev))
    out, out_cu = layout.response_from_packed(vals[:0].to(dev), cu[:1].to(dev), resp[:0].to(dev))
    assert out.shape == (0,) and out_cu.tolist() == [0]
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        layout.response_from_packed(vals, cu, resp)


def _packed_batch(B, seed, max_resp=300):
    g = torch.Generator().manual_seed(seed)
    prompt = torch.randint(1, 50, (B,), generator=g)
    resp = torch.randint(0, max_resp, (B,), generator=g)
    cu = torch.zeros(B + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(prompt + resp, 0)
    return g, prompt, resp, cu


@pytest.mark.parametrize("dtype,trailing", [
    (torch.bfloat16, ()), (torch.float16, ()), (torch.float32, (8,)), (torch.bfloat16, (8,)), (torch.bfloat16, (3,)),
    (torch.float32, (5, 3)), (torch.int64, ()), (torch.int64, (2,)), (torch.uint8, ()), (torch.uint8, (7,)),
    (torch.float64, (3,)), (torch.bool, ()), (torch.bfloat16, (4096,)),
])
def test_response_slice_and_pack_keep_dtype_and_trailing_dimensions(dev, dtype, trailing):
    """no_padding_2_padding takes (total_nnz, *) of any dtype and pads the sequence axis only
    (verl/workers/utils/padding.py:100-101, :133-138); rows are copied bit for bit."""
    B = 9 if trailing == (4096,) else 29
    g, prompt, resp, cu = _packed_batch(B, seed=40 + len(trailing), max_resp=60 if trailing == (4096,) else 300)
    N = int(cu[-1])
    shape = (N,) + trailing
    if dtype.is_floating_point:
        vals = (torch.randn(shape, generator=g) * 3).to(dtype)
    elif dtype == torch.bool:
        vals = torch.rand(shape, generator=g) < 0.5
    else:
        vals = torch.randint(0, 250, shape, generator=g).to(dtype)
    T = int(resp.max()) + 3
    got = layout.response_slice(vals.to(dev), cu.to(dev), resp.to(dev), T)
    ref = scoring.response_slice(vals, prompt.tolist(), resp.tolist(), T)
    assert got.dtype == dtype and got.shape == (B, T) + trailing
    assert torch.equal(got.cpu(), ref)
    packed, packed_cu = layout.response_from_packed(vals.to(dev), cu.to(dev), resp.to(dev),
                                                   total_response_tokens=int(resp.sum()))
    ref_p, ref_cu = scoring.response_from_nested(vals, cu.tolist(), resp.tolist())
    assert packed.dtype == dtype and torch.equal(packed.cpu(), ref_p) and torch.equal(packed_cu.cpu(), ref_cu)


def test_response_slice_of_views_and_of_the_reference_fixture_with_a_trailing_dimension(dev):
    # the reference's fixture (tests/models/test_fsdp_no_padding_on_gpu.py:180-201) with K = 4 values per token
    full = torch.arange(8 * 4, dtype=torch.float32, device=dev).view(8, 4)
    cu = torch.tensor([0, 5, 8], device=dev)
    got = layout.response_slice(full.bfloat16(), cu, torch.tensor([2, 1], device=dev), max_response_len=2)
    want = torch.stack([full[2:4], torch.cat([full[6:7], torch.zeros(1, 4, device=dev)])]).bfloat16()
    assert got.dtype == torch.bfloat16 and torch.equal(got, want)
    # a strided view (every other column of a wider tensor) and a view that starts off the 16-byte grid
    wide = torch.randn(8, 10, device=dev)
    for view in (wide[:, ::2], wide[:, 1:4], wide.bfloat16()[:, 3:]):
        got = layout.response_slice(view, cu, torch.tensor([2, 1], device=dev), 3)
        ref = scoring.response_slice(view.cpu(), [3, 2], [2, 1], 3)
        assert torch.equal(got.cpu(), ref)
    # a wrong total is caught on the device
    with pytest.raises(ValueError):
        layout.response_from_packed(full, cu, torch.tensor([2, 1], device=dev), total_response_tokens=5)
    with pytest.raises(ValueError):
        layout.response_from_packed(full, cu, torch.tensor([2, 1], device=dev), total_response_tokens=2)


def test_response_slice_with_known_lengths_does_not_synchronise(dev):
    g, prompt, resp, cu = _packed_batch(11, seed=50)
    vals = torch.randn(int(cu[-1]), 4, generator=g).to(dev)
    cu_d, resp_d = cu.to(dev), resp.to(dev)
    T, total = int(resp.max()), int(resp.sum())
    layout.response_slice(vals, cu_d, resp_d, T, check="deferred")                      # first calls: library, pinned buffers
    layout.response_from_packed(vals, cu_d, resp_d, check="deferred", total_response_tokens=total)
    torch.cuda.synchronize(dev)
    torch.cuda.set_sync_debug_mode("error")
    try:
        a = layout.response_slice(vals, cu_d, resp_d, T, check="deferred")
        b, _ = layout.response_from_packed(vals, cu_d, resp_d, check="deferred", total_response_tokens=total)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    errors.check_errors()
    assert torch.equal(a.cpu(), scoring.response_slice(vals.cpu(), prompt.tolist(), resp.tolist(), T))
    assert torch.equal(b.cpu(), scoring.response_from_nested(vals.cpu(), cu.tolist(), resp.tolist())[0])


def test_expand_per_sequence_matches_the_reference_repeat_interleave(dev):
    """expand_as_nested (verl/utils/torch_functional.py:989-1011): the per-sample temperature repeated over the tokens
    of its sequence. Random batches with empty sequences, one sequence, many; known total (no synchronisation) and
    unknown; and offsets that are not a partition are reported."""
    g = torch.Generator().manual_seed(77)
    for B in (1, 2, 7, 300, 5000):
        lens = torch.randint(0, 40, (B,), generator=g)
        lens[torch.rand(B, generator=g) < 0.2] = 0
        if B == 7:
            lens[3] = 5000
        cu = torch.zeros(B + 1, dtype=torch.int64)
        cu[1:] = torch.cumsum(lens, 0)
        vals = torch.rand(B, generator=g) + 0.3
        ref = scoring.expand_as_nested_values(vals, cu)
        got = layout.expand_per_sequence(vals.to(dev), cu.to(dev))
        assert got.dtype == torch.float32 and torch.equal(got.cpu(), ref), B
        got = layout.expand_per_sequence(vals.to(dev), cu.to(dev), total_nnz=int(cu[-1]))
        assert torch.equal(got.cpu(), ref), B
    # no tokens at all
    assert layout.expand_per_sequence(torch.ones(3, device=dev), torch.zeros(4, dtype=torch.int64, device=dev)).numel() == 0
    # with the total known the call does not wait for the device
    vals_d, cu_d, n = vals.to(dev), cu.to(dev), int(cu[-1])
    layout.expand_per_sequence(vals_d, cu_d, n, check="deferred")
    torch.cuda.synchronize(dev)
    torch.cuda.set_sync_debug_mode("error")
    try:
        got = layout.expand_per_sequence(vals_d, cu_d, n, check="deferred")
    finally:
        torch.cuda.set_sync_debug_mode("default")
    errors.check_errors()
    assert torch.equal(got.cpu(), ref)
    # offsets that do not partition the tokens
    for bad in ([1, 3, 6], [0, 4, 3, 6], [0, 3, 5], [0, 3, 9]):
        with pytest.raises(ValueError):
            layout.expand_per_sequence(torch.ones(len(bad) - 1, device=dev), torch.tensor(bad, device=dev), 6)
    with pytest.raises(ValueError):
        layout.expand_per_sequence(torch.ones(3, device=dev), torch.tensor([0, 3, 6], device=dev), 6)
    with pytest.raises(RuntimeError):
        layout.expand_per_sequence(torch.ones(2), torch.tensor([0, 3, 6]), 6)
