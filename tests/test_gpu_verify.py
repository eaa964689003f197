"""The HIP verify kernel (through the C ABI) against the CPU statement of the rule: bit-exact."""

import math

import numpy as np
import pytest
import torch

from verl_amd import spec_rl as sv
from verl_amd import synthetic
from oracle import c_oracle, verify as overify

pytestmark = pytest.mark.gpu


def _same(res, ref, with_draft=False):
    assert np.array_equal(res.accept.cpu().numpy().astype(np.uint8), np.asarray(ref["accept"]).astype(np.uint8))
    for k in ("first_reject", "prefix_len", "near_count"):
        assert np.array_equal(getattr(res, k).cpu().numpy(), np.asarray(ref[k])), k
    if with_draft:
        assert np.array_equal(res.out_ids.cpu().numpy(), np.asarray(ref["out_ids"]))
        assert np.array_equal(res.out_mask.cpu().numpy().astype(np.uint8), np.asarray(ref["out_mask"]).astype(np.uint8))


def _inputs(dev, B, T, seed, drift=0.3, lengths=None):
    g = torch.Generator(device=dev).manual_seed(seed)
    ln = -torch.rand(B, T, generator=g, device=dev) * 5
    lo = ln + torch.randn(B, T, generator=g, device=dev) * drift
    lu = torch.log(torch.rand(B, T, generator=g, device=dev))
    ids = torch.randint(0, 150000, (B, T), generator=g, device=dev)
    if lengths is None:
        lengths = torch.randint(0, T + 1, (B,), generator=torch.Generator().manual_seed(seed))
    mask = synthetic.right_pad_mask(lengths, T, dev)
    return ln, lo, lu, mask, ids


@pytest.mark.parametrize("B,T", [(1, 1), (3, 63), (4, 64), (5, 65), (8, 512), (7, 1000), (2, 5000)])
@pytest.mark.parametrize("off", [0.0, 0.5, -0.5])
def test_padded_matches_oracles(dev, B, T, off):
    ln, lo, lu, mask, ids = _inputs(dev, B, T, seed=B * 1000 + T)
    res = sv.spec_verify(ln, lo, mask, log_u=lu, thresh_offset=off, draft_ids=ids, pad_id=-7)
    _same(res, overify.verify(ln, lo, lu, mask, off, draft_ids=ids, pad_id=-7), with_draft=True)
    _same(res, c_oracle.spec_verify(ln, lo, lu, mask, off, draft_ids=ids, pad_id=-7), with_draft=True)
    if B * T <= 4096:
        _same(res, overify.verify_loops(ln, lo, lu, mask, off, draft_ids=ids, pad_id=-7), with_draft=True)


def test_mask_dtypes_and_no_mask(dev):
    ln, lo, lu, mask, ids = _inputs(dev, 6, 200, seed=5)
    ref = overify.verify(ln, lo, lu, mask, 0.0)
    for m in (mask, mask.long(), mask.float(), mask.to(torch.uint8), mask.int() * 3):
        _same(sv.spec_verify(ln, lo, m, log_u=lu), ref)
    _same(sv.spec_verify(ln, lo, None, log_u=lu), overify.verify(ln, lo, lu, None, 0.0))


def test_masks_with_holes(dev):
    # multi-turn style masks: tool-output tokens inside the response are masked out
    ln, lo, lu, _, ids = _inputs(dev, 9, 333, seed=6)
    g = torch.Generator(device=dev).manual_seed(60)
    mask = torch.rand(9, 333, generator=g, device=dev) < 0.6
    mask[0] = False           # no valid token at all
    mask[1, :] = True
    res = sv.spec_verify(ln, lo, mask, log_u=lu, draft_ids=ids)
    _same(res, c_oracle.spec_verify(ln, lo, lu, mask, 0.0, draft_ids=ids), with_draft=True)
    _same(res, overify.verify_loops(ln, lo, lu, mask, 0.0, draft_ids=ids), with_draft=True)
    assert res.first_reject[0].item() == 0 and res.prefix_len[0].item() == 0


def test_packed_layout_ragged_lengths(dev):
    lengths = torch.tensor([0, 1, 63, 64, 65, 300, 0, 2049, 17, 256])
    cu = synthetic.pack_by_lengths(lengths)
    N = int(cu[-1])
    g = torch.Generator(device=dev).manual_seed(8)
    ln = -torch.rand(N, generator=g, device=dev) * 4
    lo = ln + torch.randn(N, generator=g, device=dev) * 0.2
    lu = torch.log(torch.rand(N, generator=g, device=dev))
    mask = torch.rand(N, generator=g, device=dev) < 0.9
    ids = torch.randint(0, 1000, (N,), generator=g, device=dev)
    for m in (None, mask):
        res = sv.spec_verify(ln, lo, m, log_u=lu, thresh_offset=0.25, cu_seqlens=cu.to(dev), draft_ids=ids, pad_id=1)
        _same(res, c_oracle.spec_verify(ln, lo, lu, m, 0.25, cu_seqlens=cu, draft_ids=ids, pad_id=1), with_draft=True)
        _same(res, overify.verify(ln, lo, lu, m, 0.25, cu_seqlens=cu, draft_ids=ids, pad_id=1), with_draft=True)


def test_exact_rows(dev):
    # hand-computed: d = -1.0 everywhere, log u = -2.0 / -0.5 / -1.0 (boundary)
    ln = torch.full((3, 6), -2.0, device=dev)
    lo = torch.full((3, 6), -1.0, device=dev)
    lu = torch.tensor([[-2.0] * 6, [-2.0, -2.0, -0.5, -2.0, -0.5, -2.0], [-1.0] * 6], device=dev)
    mask = torch.tensor([[1, 1, 1, 1, 0, 0], [1, 1, 1, 1, 1, 1], [1, 1, 1, 0, 0, 0]], device=dev)
    res = sv.spec_verify(ln, lo, mask, log_u=lu, near_eps=1e-6)
    assert res.accept.int().tolist() == [[1, 1, 1, 1, 0, 0], [1, 1, 0, 1, 0, 1], [1, 1, 1, 0, 0, 0]]
    assert res.first_reject.tolist() == [4, 2, 3]
    assert res.prefix_len.tolist() == [4, 2, 3]
    assert res.near_count.tolist() == [0, 0, 3]          # d == tau exactly on the valid tokens of row 2
    # lenience: literal adds log(l) to the threshold, relax subtracts it
    strict = sv.spec_verify(ln, lo, mask, log_u=lu, lenience=math.e, lenience_mode="literal")
    assert strict.first_reject.tolist() == [4, 2, 0]     # tau = log u + 1: rows 0 (=-1, boundary) still accept
    loose = sv.spec_verify(ln, lo, mask, log_u=lu, lenience=math.e, lenience_mode="relax")
    assert loose.first_reject.tolist() == [4, 6, 3]


def test_special_values(dev):
    nan, inf = float("nan"), float("inf")
    ln = torch.tensor([[-1.0, nan, -1.0, -1.0], [-1.0, -1.0, -inf, -1.0], [-1.0, -1.0, -1.0, -1.0]], device=dev)
    lo = torch.full((3, 4), -1.0, device=dev)
    lu = torch.tensor([[-1.0, -1.0, -1.0, -1.0], [-inf, -inf, -inf, -1.0], [-1.0, nan, -inf, -1.0]], device=dev)
    res = sv.spec_verify(ln, lo, None, log_u=lu)
    # NaN d rejects; u = 0 accepts any finite d; d = -inf vs tau = -inf accepts (>=); NaN tau rejects
    assert res.accept.int().tolist() == [[1, 0, 1, 1], [1, 1, 1, 1], [1, 0, 1, 1]]
    assert res.first_reject.tolist() == [1, 4, 1]
    _same(res, c_oracle.spec_verify(ln, lo, lu, None, 0.0))
    _same(res, overify.verify_loops(ln, lo, lu, None, 0.0))


def test_seeded_uniforms_reproduce(dev):
    ln, lo, _, mask, _ = _inputs(dev, 4, 100, seed=12)
    a = sv.spec_verify(ln, lo, mask, seed=1234)
    b = sv.spec_verify(ln, lo, mask, seed=1234)
    c = sv.spec_verify(ln, lo, mask, seed=1235)
    assert torch.equal(a.log_u, b.log_u) and torch.equal(a.accept, b.accept)
    assert not torch.equal(a.log_u, c.log_u)
    _same(a, overify.verify(ln, lo, a.log_u, mask, 0.0))
    with pytest.raises(ValueError):
        sv.spec_verify(ln, lo, mask)
    with pytest.raises(ValueError):
        sv.spec_verify(ln, lo, mask, seed=1, log_u=a.log_u)


def test_truncate_draft_standalone_and_idempotent(dev):
    ln, lo, lu, mask, ids = _inputs(dev, 5, 77, seed=13)
    res = sv.spec_verify(ln, lo, mask, log_u=lu, draft_ids=ids, pad_id=9)
    ids2, mask2 = sv.truncate_draft(ids, mask, res.first_reject, pad_id=9)
    assert torch.equal(ids2, res.out_ids) and torch.equal(mask2, res.out_mask)
    ids3, mask3 = sv.truncate_draft(ids2, mask2, res.first_reject, pad_id=9)
    assert torch.equal(ids3, ids2) and torch.equal(mask3, mask2)


def test_empty_shapes(dev):
    z = torch.empty(0, 5, device=dev)
    res = sv.spec_verify(z, z, None, log_u=z)
    assert res.accept.shape == (0, 5) and res.first_reject.shape == (0,)
    z = torch.empty(3, 0, device=dev)
    res = sv.spec_verify(z, z, None, log_u=z)
    assert res.first_reject.tolist() == [0, 0, 0] and res.prefix_len.tolist() == [0, 0, 0]
    # packed layout whose sequences are all empty: no token tensor has storage
    e = torch.empty(0, device=dev)
    cu = torch.zeros(4, dtype=torch.int64, device=dev)
    res = sv.spec_verify(e, e, None, log_u=e, cu_seqlens=cu, draft_ids=torch.empty(0, dtype=torch.long, device=dev))
    assert res.first_reject.tolist() == [0, 0, 0] and res.near_count.tolist() == [0, 0, 0] and res.out_ids.shape == (0,)
    ids, mask = sv.truncate_draft(torch.empty(0, dtype=torch.long, device=dev), None, res.first_reject, cu_seqlens=cu)
    assert ids.shape == (0,) and mask.shape == (0,)
    lp, h, res = sv.fused_score_verify(torch.empty(0, 100, device=dev), torch.empty(0, dtype=torch.long, device=dev), e,
                                       log_u=e, cu_seqlens=cu)
    assert lp.shape == (0,) and res.prefix_len.tolist() == [0, 0, 0]


def test_c5_imbalance_verify_only_full_size(dev):
    """512 sequences, lengths log-uniform in [32, 16384], Student-t drift: packed layout, whole workload."""
    w = synthetic.WORKLOADS["c5"]
    lengths = synthetic.draw_lengths(w, seed=5002)
    cu = synthetic.pack_by_lengths(lengths)
    N = int(cu[-1])
    g = torch.Generator(device=dev).manual_seed(5000)
    ln = -torch.rand(N, generator=g, device=dev) * 6
    lo = synthetic.drift_old_logprobs(ln, w, seed=5000)
    lu = torch.log(torch.rand(N, generator=g, device=dev))
    off = sv.thresh_offset_from_lenience(w.lenience)
    assert off == 0.5
    res = sv.spec_verify(ln, lo, None, log_u=lu, thresh_offset=off, cu_seqlens=cu.to(dev))
    ref = c_oracle.spec_verify(ln, lo, lu, None, off, cu_seqlens=cu)
    _same(res, ref)
    _same(res, overify.verify(ln, lo, lu, None, off, cu_seqlens=cu))
    assert (res.first_reject.cpu() <= lengths).all()
    assert res.first_reject.float().mean().item() < lengths.float().mean().item()   # early rejections do happen


def _shifted(t, by):
    """The same values in storage that starts `by` elements past an allocation boundary (a view no 16-byte access fits)."""
    raw = torch.empty(t.numel() + by, dtype=t.dtype, device=t.device)
    raw[by:] = t.reshape(-1)
    return raw[by:].view(t.shape)


@pytest.mark.parametrize("layout", ["padded", "packed"])
def test_views_that_start_off_the_16_byte_grid_give_the_same_results(dev, layout):
    # allocator-aligned arrays take the 128-bit kernel, shifted views the element-wise one: same integers from both
    if layout == "padded":
        ln, lo, lu, mask, ids = _inputs(dev, 6, 1111, seed=21)
        mask = mask & (torch.rand(6, 1111, generator=torch.Generator(device=dev).manual_seed(22), device=dev) < 0.8)
        cu = None
    else:
        lengths = torch.tensor([5, 0, 1030, 2, 4097, 63, 1, 777])
        cu = synthetic.pack_by_lengths(lengths)
        N = int(cu[-1])
        g = torch.Generator(device=dev).manual_seed(23)
        ln = -torch.rand(N, generator=g, device=dev) * 4
        lo = ln + torch.randn(N, generator=g, device=dev) * 0.15
        lu = torch.log(torch.rand(N, generator=g, device=dev))
        mask = torch.rand(N, generator=g, device=dev) < 0.85
        ids = torch.randint(0, 5000, (N,), generator=g, device=dev)
    cud = None if cu is None else cu.to(dev)
    ref = c_oracle.spec_verify(ln, lo, lu, mask, -0.1, cu_seqlens=cu, draft_ids=ids, pad_id=3)
    a = sv.spec_verify(ln, lo, mask, log_u=lu, thresh_offset=-0.1, cu_seqlens=cud, draft_ids=ids, pad_id=3)
    _same(a, ref, with_draft=True)
    for by in (1, 2, 3):
        mb = _shifted(mask.bool(), by)      # a bool mask is handed to the kernel as it lies
        b = sv.spec_verify(_shifted(ln, by), _shifted(lo, by), mb, log_u=_shifted(lu, by), thresh_offset=-0.1,
                           cu_seqlens=cud, draft_ids=_shifted(ids, 1), pad_id=3)
        _same(b, ref, with_draft=True)


def test_packed_sequences_around_one_trip_of_the_wide_kernel(dev):
    """The 16-wavefront workgroup holds 16384 tokens (4096 groups of 4) in registers; sequences just below, at and
    above that, at every phase of the 4-token grid, with holes in the mask and a late first rejection."""
    lengths = torch.tensor([16384, 1, 16383, 2, 16385, 3, 16381, 16388, 40000, 0, 7])
    cu = synthetic.pack_by_lengths(lengths)
    N = int(cu[-1])
    g = torch.Generator(device=dev).manual_seed(31)
    ln = -torch.rand(N, generator=g, device=dev) * 4
    lo = ln + torch.randn(N, generator=g, device=dev) * 0.01          # small drift: most tokens accept
    lu = torch.log(torch.rand(N, generator=g, device=dev) * 0.2)       # u < 0.2: thresholds well below zero
    mask = torch.rand(N, generator=g, device=dev) < 0.9
    ids = torch.randint(0, 150000, (N,), generator=g, device=dev)
    # one sequence without any rejection, one rejected at its very last valid token
    lo[cu[2]:cu[3]] = ln[cu[2]:cu[3]] - 1.0
    lo[cu[4]:cu[5]] = ln[cu[4]:cu[5]] - 1.0
    last = int(cu[5]) - 1
    mask[last] = True
    lo[last] = ln[last] + 50.0
    for m in (mask, None):
        res = sv.spec_verify(ln, lo, m, log_u=lu, cu_seqlens=cu.to(dev), draft_ids=ids, pad_id=-1)
        ref = c_oracle.spec_verify(ln, lo, lu, m, 0.0, cu_seqlens=cu, draft_ids=ids, pad_id=-1)
        _same(res, ref, with_draft=True)
        assert res.first_reject[4].item() == 16384 and res.first_reject[2].item() > 16000


# ---- the two-pass form (flat tiles of 1024 tokens + one bit per token of scratch) against the oracles -----------------

def _both_forms(*args, **kw):
    one = sv.spec_verify(*args, two_pass=False, **kw)
    two = sv.spec_verify(*args, two_pass=True, **kw)
    return one, two


@pytest.mark.parametrize("B,T", [(1, 1), (3, 63), (4, 64), (5, 65), (70, 7), (8, 512), (7, 1000), (3, 1024), (2, 5000),
                                 (2, 1025), (9, 2048), (1, 40000)])
def test_two_pass_padded_matches_oracles(dev, B, T):
    ln, lo, lu, mask, ids = _inputs(dev, B, T, seed=B * 1000 + T + 1, drift=0.05)
    g = torch.Generator(device=dev).manual_seed(B + T)
    holes = mask & (torch.rand(B, T, generator=g, device=dev) < 0.85)
    for m in (mask, holes, None):
        one, two = _both_forms(ln, lo, m, log_u=lu, thresh_offset=-0.2, draft_ids=ids, pad_id=-7)
        ref = c_oracle.spec_verify(ln, lo, lu, m, -0.2, draft_ids=ids, pad_id=-7)
        _same(two, ref, with_draft=True)
        _same(one, ref, with_draft=True)
    # without a draft only the per-sequence results and accept are produced
    res = sv.spec_verify(ln, lo, holes, log_u=lu, thresh_offset=-0.2, two_pass=True)
    _same(res, c_oracle.spec_verify(ln, lo, lu, holes, -0.2))


def _packed_case(dev, lengths, seed, drift, keep=0.9, u_scale=1.0):
    cu = synthetic.pack_by_lengths(torch.as_tensor(lengths))
    N = int(cu[-1])
    g = torch.Generator(device=dev).manual_seed(seed)
    ln = -torch.rand(N, generator=g, device=dev) * 4
    lo = ln + torch.randn(N, generator=g, device=dev) * drift
    lu = torch.log(torch.rand(N, generator=g, device=dev) * u_scale)
    mask = torch.rand(N, generator=g, device=dev) < keep
    ids = torch.randint(0, 150000, (N,), generator=g, device=dev)
    return cu, ln, lo, lu, mask, ids


@pytest.mark.parametrize("lengths", [
    [0, 1, 63, 64, 65, 300, 0, 2049, 17, 256],
    [1024, 1024, 2048, 1, 1023, 1, 1024],                 # sequences that start and end on tile borders
    [5000, 0, 0, 3, 0, 9000, 1, 1],                       # empty sequences between long ones
    [1] * 700 + [2] * 300 + [3] * 500 + [40],             # more than 256 sequence starts inside one tile
    [0] * 300 + [5] + [0] * 600 + [2000] + [0] * 4,       # runs of empty sequences (equal offsets)
    [70000, 12, 33000],                                   # sequences over many tiles
    [7],
])
def test_two_pass_packed_matches_oracles(dev, lengths):
    for drift, u_scale in ((0.2, 1.0), (0.003, 0.05)):    # early rejections / hardly any
        cu, ln, lo, lu, mask, ids = _packed_case(dev, lengths, seed=len(lengths) + 77, drift=drift, u_scale=u_scale)
        for m in (mask, None):
            one, two = _both_forms(ln, lo, m, log_u=lu, thresh_offset=0.1, cu_seqlens=cu.to(dev), draft_ids=ids, pad_id=1)
            ref = c_oracle.spec_verify(ln, lo, lu, m, 0.1, cu_seqlens=cu, draft_ids=ids, pad_id=1)
            _same(two, ref, with_draft=True)
            _same(one, ref, with_draft=True)


def test_two_pass_carries_across_tiles(dev):
    """What a tile needs from its neighbours, case by case: a rejection many tiles back, none at all (the prefix ends
    behind the last valid token, many tiles ahead), a valid token only in the very last tile, rejections exactly on the
    first and last token of a tile, a sequence whose only valid tokens lie before a run of masked tiles."""
    L = 10 * 1024 + 5
    lengths = [3, L, L, L, L, L, 100]
    cu = synthetic.pack_by_lengths(torch.tensor(lengths))
    N = int(cu[-1])
    ln = torch.zeros(N, device=dev)
    lo = torch.full((N,), -1.0, device=dev)     # d = +1: every token accepts against log u = 0
    lu = torch.zeros(N, device=dev)
    mask = torch.ones(N, dtype=torch.bool, device=dev)
    ids = torch.arange(N, device=dev)
    s = [int(x) for x in cu]
    lo[s[1] + 2] = 5.0                           # sequence 1: rejected at its third token, then nine tiles of tail
    #                                              sequence 2: no rejection at all
    mask[s[3]:s[4]] = False                      # sequence 3: valid only at its last token
    mask[s[4] - 1] = True
    first_of_tile = (s[4] // 1024 + 3) * 1024    # sequence 4: rejected on the first token of a tile ...
    lo[first_of_tile] = 5.0
    last_of_tile = (s[5] // 1024 + 4) * 1024 - 1  # sequence 5: ... and on the last token of one, valid tokens only before it
    lo[last_of_tile] = 5.0
    mask[last_of_tile + 1:s[6]] = False
    mask[s[5] + 10:last_of_tile - 2000] = False
    one, two = _both_forms(ln, lo, mask, log_u=lu, cu_seqlens=cu.to(dev), draft_ids=ids, pad_id=-1)
    ref = c_oracle.spec_verify(ln, lo, lu, mask, 0.0, cu_seqlens=cu, draft_ids=ids, pad_id=-1)
    _same(two, ref, with_draft=True)
    _same(one, ref, with_draft=True)
    assert two.first_reject.tolist() == [3, 2, L, L, first_of_tile - s[4], last_of_tile - s[5], 100]
    # a sequence without any valid token, between two others, over several tiles
    mask[s[2]:s[3]] = False
    two = sv.spec_verify(ln, lo, mask, log_u=lu, cu_seqlens=cu.to(dev), draft_ids=ids, pad_id=-1, two_pass=True)
    _same(two, c_oracle.spec_verify(ln, lo, lu, mask, 0.0, cu_seqlens=cu, draft_ids=ids, pad_id=-1), with_draft=True)
    assert two.first_reject[2].item() == 0 and (two.out_ids[s[2]:s[3]] == -1).all()


def test_two_pass_is_what_the_library_plans_for_c5(dev):
    w = synthetic.WORKLOADS["c5"]
    lengths = synthetic.draw_lengths(w, seed=5002)
    cu, ln, lo, lu, mask, ids = _packed_case(dev, lengths.tolist(), seed=5001, drift=0.3)
    from verl_amd import _lib
    assert _lib.load().vrl_spec_verify_plan(1, len(lengths), 0, ln.numel()) == 1
    res = sv.spec_verify(ln, lo, mask, log_u=lu, thresh_offset=0.5, cu_seqlens=cu.to(dev), draft_ids=ids)   # planned form
    _same(res, c_oracle.spec_verify(ln, lo, lu, mask, 0.5, cu_seqlens=cu, draft_ids=ids), with_draft=True)
