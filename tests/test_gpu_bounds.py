"""Packed layouts keep their offsets on the device, where the host cannot check them. The kernels hold every span to
the arrays' length: whatever cu_seqlens holds, nothing outside the per-token arrays is read or written, the error
flag carries VRL_FLAG_SEQ_RANGE, and the wrappers turn it into ValueError (the reference asserts
``sequence_offsets[-1] == values.shape[0]``, verl/workers/utils/padding.py:129-130).

Every array sits between guard regions filled with a sentinel; after each call with inconsistent offsets the guards
must be byte for byte what they were."""

import numpy as np
import pytest
import torch

from verl_amd import _lib, errors, layout, spec_rl
from oracle import verify as overify

pytestmark = pytest.mark.gpu

from _guards import BAD_OFFSETS, Arena


@pytest.mark.parametrize("case", sorted(BAD_OFFSETS))
def test_verify_and_truncate_hold_bad_offsets_to_the_arrays(dev, case):
    lib = _lib.load()
    N, B = 100, 3
    g = torch.Generator().manual_seed(5)
    ar = Arena(dev)
    ln = ar.make(N, torch.float32, torch.randn(N, generator=g))
    lo = ar.make(N, torch.float32, torch.randn(N, generator=g))
    lu = ar.make(N, torch.float32, torch.log(torch.rand(N, generator=g)))
    mask = ar.make(N, torch.uint8, torch.ones(N, dtype=torch.uint8))
    ids = ar.make(N, torch.int64, torch.arange(N))
    accept = ar.make(N, torch.uint8)
    out_ids = ar.make(N, torch.int64)
    out_mask = ar.make(N, torch.uint8)
    first = ar.make(B, torch.int32)
    prefix = ar.make(B, torch.int32)
    near = ar.make(B, torch.int32)
    cu = ar.make(B + 1, torch.int64, torch.tensor(BAD_OFFSETS[case], dtype=torch.int64))
    flag = ar.make(1, torch.int32, torch.zeros(1, dtype=torch.int32))
    print(f"[bounds] verify/truncate with cu_seqlens={BAD_OFFSETS[case]} over {N} tokens", flush=True)
    with torch.cuda.device(dev):
        s = _lib.stream_ptr(dev)
        st = lib.vrl_spec_verify(ln.data_ptr(), lo.data_ptr(), lu.data_ptr(), mask.data_ptr(), cu.data_ptr(), B, 0, N, 0.0,
                                 1e-6, accept.data_ptr(), first.data_ptr(), prefix.data_ptr(), near.data_ptr(),
                                 ids.data_ptr(), -1, out_ids.data_ptr(), out_mask.data_ptr(), flag.data_ptr(), None, 0, s)
        assert st == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert int(flag.item()) & _lib.VRL_FLAG_SEQ_RANGE
        assert ar.guards_intact()
        # per-sequence results are those of the spans cut to [0, N]
        cuts = np.clip(np.array(BAD_OFFSETS[case], dtype=np.int64), 0, N)
        for b in range(B):
            length = max(int(cuts[b + 1]) - int(cuts[b]), 0)
            assert 0 <= int(first[b]) <= length and 0 <= int(prefix[b]) <= length
        # the two-pass form (its scratch between guards too): same guarantees
        flag.zero_()
        nbytes = lib.vrl_spec_verify_workspace(N)
        work = ar.make(nbytes, torch.uint8)
        print(f"[bounds] two-pass verify with cu_seqlens={BAD_OFFSETS[case]} over {N} tokens", flush=True)
        st = lib.vrl_spec_verify(ln.data_ptr(), lo.data_ptr(), lu.data_ptr(), mask.data_ptr(), cu.data_ptr(), B, 0, N, 0.0,
                                 1e-6, accept.data_ptr(), first.data_ptr(), prefix.data_ptr(), near.data_ptr(),
                                 ids.data_ptr(), -1, out_ids.data_ptr(), out_mask.data_ptr(), flag.data_ptr(),
                                 work.data_ptr(), nbytes, s)
        assert st == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert int(flag.item()) & _lib.VRL_FLAG_SEQ_RANGE
        assert ar.guards_intact()
        for b in range(B):
            length = max(int(cuts[b + 1]) - int(cuts[b]), 0)
            assert 0 <= int(first[b]) <= length and 0 <= int(prefix[b]) <= length
        flag.zero_()
        st = lib.vrl_truncate_draft(ids.data_ptr(), mask.data_ptr(), cu.data_ptr(), B, 0, N, first.data_ptr(), -1,
                                    out_ids.data_ptr(), out_mask.data_ptr(), flag.data_ptr(), s)
        assert st == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert int(flag.item()) & _lib.VRL_FLAG_SEQ_RANGE
        assert ar.guards_intact()
    # the wrappers raise, in every mode that looks
    cu_t = torch.tensor(BAD_OFFSETS[case], dtype=torch.int64, device=dev)
    with pytest.raises(ValueError, match="partition"):
        spec_rl.spec_verify(ln.clone(), lo.clone(), mask.clone(), log_u=lu.clone(), cu_seqlens=cu_t, draft_ids=ids.clone())
    with pytest.raises(ValueError, match="partition"):
        spec_rl.truncate_draft(ids.clone(), mask.clone(), first.clone(), cu_seqlens=cu_t)
    res = spec_rl.spec_verify(ln.clone(), lo.clone(), mask.clone(), log_u=lu.clone(), cu_seqlens=cu_t, check="deferred")
    with pytest.raises(ValueError, match="partition"):
        errors.check_errors()
    # tokens that no in-range span covers come back as "not accepted", never as uninitialised memory
    covered = np.zeros(N, dtype=bool)
    for b in range(B):
        covered[int(cuts[b]):max(int(cuts[b + 1]), int(cuts[b]))] = True
    assert not res.accept.cpu().numpy()[~covered].any()


@pytest.mark.parametrize("case", sorted(BAD_OFFSETS))
def test_response_slice_and_pack_hold_bad_offsets_to_the_arrays(dev, case):
    lib = _lib.load()
    N, B, T = 100, 3, 16
    g = torch.Generator().manual_seed(6)
    ar = Arena(dev)
    values = ar.make(N, torch.float32, torch.randn(N, generator=g))
    cu = ar.make(B + 1, torch.int64, torch.tensor(BAD_OFFSETS[case], dtype=torch.int64))
    rl = ar.make(B, torch.int64, torch.tensor([4, 7, 9], dtype=torch.int64))
    out = ar.make(B * T, torch.float32)
    out_cu = ar.make(B + 1, torch.int64, torch.tensor([0, 4, 11, 20], dtype=torch.int64))
    packed = ar.make(20, torch.float32)
    flag = ar.make(1, torch.int32, torch.zeros(1, dtype=torch.int32))
    print(f"[bounds] response slice/pack with cu_seqlens={BAD_OFFSETS[case]} over {N} values", flush=True)
    with torch.cuda.device(dev):
        s = _lib.stream_ptr(dev)
        st = lib.vrl_response_slice(values.data_ptr(), 4, cu.data_ptr(), rl.data_ptr(), B, N, T, out.data_ptr(),
                                    flag.data_ptr(), s)
        assert st == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert int(flag.item()) & _lib.VRL_FLAG_SEQ_RANGE
        assert ar.guards_intact()
        assert torch.isfinite(out).all()            # every output element was written (values or zeros)
        flag.zero_()
        st = lib.vrl_response_pack(values.data_ptr(), 4, cu.data_ptr(), rl.data_ptr(), out_cu.data_ptr(), B, N, 20,
                                   packed.data_ptr(), flag.data_ptr(), s)
        assert st == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert int(flag.item()) & _lib.VRL_FLAG_SEQ_RANGE
        assert ar.guards_intact()
        # rows of several elements ((N, 6) bf16: 12 bytes a row, moved in 4-byte units) between guards of their own
        flag.zero_()
        wide = ar.make(N * 6, torch.bfloat16, torch.randn(N * 6, generator=g).bfloat16())
        wide_out = ar.make(B * T * 6, torch.bfloat16)
        wide_packed = ar.make(20 * 6, torch.bfloat16)
        print(f"[bounds] response slice/pack of 12-byte rows with cu_seqlens={BAD_OFFSETS[case]}", flush=True)
        st = lib.vrl_response_slice(wide.data_ptr(), 12, cu.data_ptr(), rl.data_ptr(), B, N, T, wide_out.data_ptr(),
                                    flag.data_ptr(), s)
        assert st == _lib.VRL_OK
        st = lib.vrl_response_pack(wide.data_ptr(), 12, cu.data_ptr(), rl.data_ptr(), out_cu.data_ptr(), B, N, 20,
                                   wide_packed.data_ptr(), flag.data_ptr(), s)
        assert st == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert int(flag.item()) & _lib.VRL_FLAG_SEQ_RANGE
        assert ar.guards_intact()
        assert torch.isfinite(wide_out.float()).all()
        # one value per sequence spread over the tokens: every token written (a value or 0), nothing else
        flag.zero_()
        per_seq = ar.make(B, torch.float32, torch.tensor([0.5, 1.5, 2.5]))
        per_tok = ar.make(N, torch.float32)
        print(f"[bounds] expand per sequence with cu_seqlens={BAD_OFFSETS[case]} over {N} tokens", flush=True)
        st = lib.vrl_expand_per_sequence(per_seq.data_ptr(), cu.data_ptr(), B, N, per_tok.data_ptr(), flag.data_ptr(), s)
        assert st == _lib.VRL_OK
        torch.cuda.synchronize(dev)
        assert int(flag.item()) & _lib.VRL_FLAG_SEQ_RANGE
        assert ar.guards_intact()
        assert bool(torch.isin(per_tok, torch.tensor([0.0, 0.5, 1.5, 2.5], device=dev)).all())
    cu_t = torch.tensor(BAD_OFFSETS[case], dtype=torch.int64, device=dev)
    with pytest.raises(ValueError, match="partition"):
        layout.expand_per_sequence(per_seq.clone(), cu_t, N)
    with pytest.raises(ValueError, match="partition"):
        layout.response_slice(values.clone(), cu_t, rl.clone(), T)
    with pytest.raises(ValueError, match="partition"):
        layout.response_from_packed(values.clone(), cu_t, rl.clone())


def test_fused_score_verify_holds_bad_offsets_to_the_rows(dev):
    N, V, B = 64, 1000, 2
    g = torch.Generator(device=dev).manual_seed(7)
    x = (torch.randn(N, V, generator=g, device=dev) * 2).bfloat16()
    lab = torch.randint(0, V, (N,), generator=g, device=dev)
    old = torch.randn(N, generator=g, device=dev)
    lu = torch.log(torch.rand(N, generator=g, device=dev))
    good = torch.tensor([0, 40, 64], device=dev)
    lp, h, res = spec_rl.fused_score_verify(x, lab, old, log_u=lu, cu_seqlens=good, draft_ids=lab)
    ref = overify.verify(lp, old, lu, None, res.thresh_offset, cu_seqlens=good.cpu(), draft_ids=lab)
    assert np.array_equal(res.accept.cpu().numpy().astype(np.uint8), ref["accept"].numpy())
    for bad in ([0, 40, 65], [0, 40, 63], [1, 40, 64], [0, 50, 40]):
        with pytest.raises(ValueError, match="partition"):
            spec_rl.fused_score_verify(x, lab, old, log_u=lu, cu_seqlens=torch.tensor(bad, device=dev), draft_ids=lab)
    # a bad label and bad offsets in one call: the label error is an IndexError, reported first
    bad_lab = lab.clone()
    bad_lab[3] = V
    with pytest.raises(IndexError):
        spec_rl.fused_score_verify(x, bad_lab, old, log_u=lu, cu_seqlens=torch.tensor([0, 40, 65], device=dev))
