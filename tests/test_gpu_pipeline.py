"""The path end to end, the way verl's engine and driver would walk it on a packed micro-batch
(verl/workers/engine/fsdp/transformer_impl.py:1149-1177, 1353-1418; verl/workers/utils/padding.py:97-141):
roll the labels over the packed axis, score every token with its sample's temperature, slice the response
positions into (B, T), verify the draft. Each stage is checked against the oracle's restatement of the same stage.
Also: the installed shims route GPU tensors to the HIP path, and the entry points can be captured in a graph."""

import contextlib
import sys
import types

import numpy as np
import pytest
import torch

import verl_amd
from verl_amd import _lib, errors, hook, layout, spec_rl
from verl_amd import torch_functional as vf
from oracle import scoring, verify as overify

pytestmark = pytest.mark.gpu


def test_packed_micro_batch_end_to_end(dev):
    g = torch.Generator().manual_seed(42)
    B, V = 7, 20011
    prompt = torch.randint(1, 40, (B,), generator=g)
    resp = torch.randint(1, 90, (B,), generator=g)
    seq = prompt + resp
    cu = torch.zeros(B + 1, dtype=torch.int64)
    cu[1:] = torch.cumsum(seq, 0)
    nnz = int(cu[-1])
    gd = torch.Generator(device=dev).manual_seed(43)
    ids = torch.randint(0, V, (nnz,), generator=gd, device=dev)
    logits = (torch.randn(nnz, V, generator=gd, device=dev) * 2.5).bfloat16()
    temp_per_sample = torch.tensor([0.7, 1.0, 1.3, 0.9, 1.0, 0.6, 1.1], device=dev)
    temp = torch.repeat_interleave(temp_per_sample, seq.to(dev))          # expand_as_nested(...).values()

    labels = layout.roll_labels(ids)                                       # :1177
    assert torch.equal(labels.cpu(), scoring.roll_labels(ids.cpu()))
    lp, ent = vf.fused_logprob_entropy(logits, labels, temp)               # :1357-1399 in one pass
    ref_lp, ref_ent = scoring.score_fp32(logits, labels, temp)
    assert (lp - ref_lp).abs().max().item() <= 2e-3 and (ent - ref_ent).abs().max().item() <= 2e-3

    T = int(resp.max())
    lp_bt = layout.response_slice(lp, cu.to(dev), resp.to(dev), T)         # no_padding_2_padding
    ent_bt = layout.response_slice(ent, cu.to(dev), resp.to(dev), T)
    assert torch.equal(lp_bt.cpu(), scoring.response_slice(lp.cpu(), prompt.tolist(), resp.tolist(), T))
    assert torch.equal(ent_bt.cpu(), scoring.response_slice(ent.cpu(), prompt.tolist(), resp.tolist(), T))
    # position j of row b is the log-prob of response token j of sample b
    b, j = 3, 5 % int(resp[3])
    row = int(cu[b + 1]) - int(resp[b]) - 1 + j
    assert lp_bt[b, j].item() == lp[row].item() and labels[row].item() == ids[row + 1].item()

    mask = (torch.arange(T).unsqueeze(0) < resp.unsqueeze(1)).to(dev)
    draft = torch.zeros(B, T, dtype=torch.int64, device=dev)
    for bb in range(B):
        e, r = int(cu[bb + 1]), int(resp[bb])
        draft[bb, :r] = ids[e - r:e]
    old = lp_bt + torch.randn(B, T, generator=gd, device=dev) * 0.3
    res = spec_rl.spec_verify(lp_bt, old, mask, seed=7, lenience=float(np.exp(0.5)), draft_ids=draft, pad_id=0)
    ref = overify.verify_loops(lp_bt, old, res.log_u, mask, res.thresh_offset, draft_ids=draft, pad_id=0)
    assert np.array_equal(res.accept.cpu().numpy().astype(np.uint8), ref["accept"])
    assert np.array_equal(res.first_reject.cpu().numpy(), ref["first_reject"])
    assert np.array_equal(res.out_ids.cpu().numpy(), ref["out_ids"])
    assert (res.prefix_len.cpu() <= resp).all()


@contextlib.contextmanager
def _stand_in_verl(extra=()):
    """A stand-in ``verl`` package whose torch_functional holds the oracle's restatements, with the hook installed."""
    names = ("verl", "verl.utils", "verl.utils.torch_functional") + tuple(extra)
    mods = {n: types.ModuleType(n) for n in names}
    tf = mods["verl.utils.torch_functional"]
    for name in hook.PATCHED_NAMES:
        setattr(tf, name, getattr(scoring, name))
    saved = {k: sys.modules.get(k) for k in mods}
    sys.modules.update(mods)
    try:
        yield mods
    finally:
        hook.uninstall()
        errors.discard()
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v


def _calls(stats):
    return {k: stats[k] for k in ("hip_calls", "passed_to_verl", "memo_hits")}


def test_installed_shims_send_gpu_tensors_to_the_hip_path(dev):
    with _stand_in_verl() as mods:
        tf = mods["verl.utils.torch_functional"]
        hook.install()
        x = torch.randn(6, 999, device=dev)
        lab = torch.randint(0, 999, (6,), device=dev)
        lp = tf.logprobs_from_logits(x, lab)
        h = tf.entropy_from_logits(x.bfloat16())
        q = tf.calculate_sum_pi_squared_from_logits(x)
        hc = tf.entropy_from_logits_with_chunking(x, chunk_size=4)
        assert _calls(hook.stats()) == {"hip_calls": 4, "passed_to_verl": 0, "memo_hits": 0}
        assert (lp - scoring.logprobs_from_logits(x, lab)).abs().max().item() <= 1e-5
        assert (h - scoring.entropy_from_logits(x.bfloat16().float())).abs().max().item() <= 2e-3
        assert (q - scoring.calculate_sum_pi_squared_from_logits(x)).abs().max().item() <= 1e-6
        assert torch.equal(hc, vf.entropy_from_logits(x))
        with pytest.raises(ValueError):
            tf.entropy_from_logits_with_chunking(x, chunk_size=0)
        tf.entropy_from_logits(x.cpu())                    # the driver's CPU tensors stay with verl's own function
        tf.entropy_from_logits(x.double())
        assert _calls(hook.stats()) == {"hip_calls": 5, "passed_to_verl": 2, "memo_hits": 0}
        xg = x.clone().requires_grad_(True)               # update_actor: gradient through the HIP backward
        tf.logprobs_from_logits(xg * 1.0, lab, inplace_backward=True).sum().backward()
        assert xg.grad is not None and hook.stats()["hip_calls"] == 6
        # the engines wrap the entropy function in torch.compile (fsdp/transformer_impl.py:164-168 in the reference):
        # the shim is run as it is, not traced
        compiled = torch.compile(tf.entropy_from_logits, dynamic=True)
        assert torch.equal(compiled(x), vf.entropy_from_logits(x))
        assert torch.equal(compiled(x[:3]), vf.entropy_from_logits(x[:3]))
        assert hook.stats()["hip_calls"] == 8
        hook.check_errors()


def test_one_pass_serves_entropy_and_logprobs_of_the_same_tensor(dev, monkeypatch):
    """compute_log_prob asks for the entropy and the label log-probs of one logits tensor in two calls
    (fsdp/transformer_impl.py:1364-1376, :1395-1399 in the reference): the second call must not read the logits
    again. What the first call leaves is single-use: only the next call can take it, and only one of the other kind."""
    with _stand_in_verl() as mods:
        tf = mods["verl.utils.torch_functional"]
        hook.install()
        g = torch.Generator(device=dev).manual_seed(8)
        V = 5003
        x = (torch.randn(300, V, generator=g, device=dev) * 3).bfloat16()
        lab = torch.randint(0, V, (300,), generator=g, device=dev)
        want_h, want_lp = vf.entropy_from_logits(x), vf.logprobs_from_logits(x, lab)

        def passes():
            return hook.stats()["forward_passes"]

        n0 = passes()
        with torch.no_grad():
            h = tf.entropy_from_logits(x)                      # the engine's order: entropy, then log-probs
            lp = tf.logprobs_from_logits(x, lab)
        assert passes() == n0 + 1 and hook.stats()["memo_hits"] == 1 and hook.stats()["label_gathers"] >= 1
        # the gather route rounds the logsumexp to fp32 once more than the one-pass route
        assert torch.equal(h, want_h) and (lp - want_lp).abs().max().item() <= 2e-6
        with torch.no_grad():                                   # the other order: log-probs first, entropy is then a lookup
            y = x.clone()
            lp2 = tf.logprobs_from_logits(y, lab)
            h2 = tf.entropy_from_logits_with_chunking(y, chunk_size=128)
        assert passes() == n0 + 2 and hook.stats()["memo_hits"] == 2
        assert torch.equal(lp2, want_lp) and torch.equal(h2, want_h)
        # single use: the pair is complete, so a third call on the same tensor makes its own pass
        with torch.no_grad():
            assert torch.equal(tf.entropy_from_logits(y), want_h)
        assert passes() == n0 + 3 and hook.stats()["memo_hits"] == 2
        # ... and so a write that torch's version counter cannot see, made after the pair, is never served stale
        with torch.no_grad():
            tf.logprobs_from_logits(y, lab)                     # takes what the entropy call above left: pair complete
            y.data[5:7] *= 0.5
            h3 = tf.entropy_from_logits(y)
            lp3 = tf.logprobs_from_logits(y, lab)
        assert not torch.equal(h3[5:7], want_h[5:7]) and torch.equal(h3, vf.entropy_from_logits(y))
        assert (lp3 - vf.logprobs_from_logits(y, lab)).abs().max().item() <= 2e-6
        # two calls of the same kind never share: the second one replaces what the first left
        with torch.no_grad():
            hits = hook.stats()["memo_hits"]
            tf.entropy_from_logits(x)
            n1 = passes()
            tf.entropy_from_logits(x)
            assert passes() == n1 + 1 and hook.stats()["memo_hits"] == hits
        # an in-place write between the two calls of a pair (also through a view) invalidates what was left
        with torch.no_grad():
            y2 = x.clone()
            tf.entropy_from_logits(y2)
            y2[5:7].mul_(0.5)
            n1 = passes()
            lp4 = tf.logprobs_from_logits(y2, lab)
        assert passes() == n1 + 1 and torch.equal(lp4, vf.logprobs_from_logits(y2, lab))
        # any other shim call in between drops it
        with torch.no_grad():
            tf.entropy_from_logits(x)
            tf.calculate_sum_pi_squared_from_logits(x[:4])
            n1 = passes()
            tf.logprobs_from_logits(x, lab)
        assert passes() == n1 + 1
        # another tensor object, even at the same address with the same contents, is never served from the old one
        with torch.no_grad():
            y3 = x.clone()
            tf.entropy_from_logits(y3)
            del y3
            z = x.clone()
            n1 = passes()
            tf.logprobs_from_logits(z, lab)
        assert passes() == n1 + 1
        # a label outside the vocabulary is reported on the gather route too (deferred: no synchronisation in the call)
        with torch.no_grad():
            bad = lab.clone()
            bad[0] = V
            tf.entropy_from_logits(z)
            lp_bad = tf.logprobs_from_logits(z, bad)
        with pytest.raises(IndexError):
            hook.check_errors()
        assert torch.isnan(lp_bad[0]) and (lp_bad[1:] - want_lp[1:]).abs().max().item() <= 2e-6
        # inference-mode tensors carry no version counter: served by the ordinary route
        with torch.inference_mode():
            xi = x.clone()
            n1 = passes()
            hi = tf.entropy_from_logits(xi)
            tf.logprobs_from_logits(xi, lab)
        assert passes() == n1 + 2 and torch.equal(hi, want_h)
        # and it can be switched off
        monkeypatch.setattr(hook, "MEMO", False)
        n1 = passes()
        with torch.no_grad():
            tf.entropy_from_logits(x)
            tf.logprobs_from_logits(x, lab)
        assert passes() == n1 + 2
        hook.check_errors()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_stock_update_actor_sequence_shares_one_forward_and_one_backward_pass(dev, dtype):
    """Under update_actor the engine calls entropy_from_logits and then logprobs_from_logits on the same logits with
    gradients on (fsdp/transformer_impl.py:1364-1399 in the reference; loss.backward() at :739-743). Through the
    installed shims that is one forward pass, one per-row gather and ONE backward pass, and the gradient equals the
    one-call form's bit for bit."""
    with _stand_in_verl() as mods:
        tf = mods["verl.utils.torch_functional"]
        hook.install()
        g = torch.Generator(device=dev).manual_seed(21)
        n, V = 257, 9001
        base = (torch.randn(n, V, generator=g, device=dev) * 3).to(dtype)
        lab = torch.randint(0, V, (n,), generator=g, device=dev)
        w_lp = torch.randn(n, generator=g, device=dev)
        w_h = torch.randn(n, generator=g, device=dev)

        def one_call():
            leaf = base.clone().requires_grad_(True)
            lp, h = vf.fused_logprob_entropy(leaf * 1.0, lab)
            ((lp * w_lp).sum() + (h * w_h).sum()).backward()
            return lp.detach(), h.detach(), leaf.grad

        def stock(order, use_lp=True, use_h=True):
            leaf = base.clone().requires_grad_(True)
            logits = leaf * 1.0
            s0 = hook.stats()
            if order == "entropy_first":
                h = tf.entropy_from_logits(logits)
                lp = tf.logprobs_from_logits(logits=logits, labels=lab, inplace_backward=False)
            else:
                lp = tf.logprobs_from_logits(logits, lab, inplace_backward=False)
                h = tf.entropy_from_logits(logits)
            loss = 0.0
            if use_lp:
                loss = loss + (lp * w_lp).sum()
            if use_h:
                loss = loss + (h * w_h).sum()
            loss.backward()
            s1 = hook.stats()
            delta = {k: s1[k] - s0[k] for k in ("forward_passes", "backward_passes", "memo_hits")}
            return lp.detach(), h.detach(), leaf.grad, delta

        ref_lp, ref_h, ref_grad = one_call()
        for order in ("entropy_first", "logprob_first"):
            lp, h, grad, delta = stock(order)
            assert delta == {"forward_passes": 1, "backward_passes": 1, "memo_hits": 1}, (order, delta)
            assert torch.equal(h, ref_h) and torch.equal(grad, ref_grad), order
            assert (lp - ref_lp).abs().max().item() <= (2e-6 if order == "entropy_first" else 0.0)
        # only one of the two results feeds the loss: still one backward pass, equal to that term's own gradient
        for order in ("entropy_first", "logprob_first"):
            leaf = base.clone().requires_grad_(True)
            (vf.entropy_from_logits(leaf * 1.0) * w_h).sum().backward()
            _, _, grad, delta = stock(order, use_lp=False)
            assert delta["backward_passes"] == 1 and torch.equal(grad, leaf.grad), order
            leaf = base.clone().requires_grad_(True)
            (vf.logprobs_from_logits(leaf * 1.0, lab, inplace_backward=False) * w_lp).sum().backward()
            _, _, grad, delta = stock(order, use_h=False)
            assert delta["backward_passes"] == 1 and torch.equal(grad, leaf.grad), order
        # entropy under activation checkpointing (entropy_checkpointing, :1371-1374): a re-entrant checkpoint runs its
        # forward without gradients, and nothing such a call leaves may serve the differentiable log-prob call
        for use_reentrant in (False, True):
            leaf = base.clone().requires_grad_(True)
            logits = leaf * 1.0
            h = torch.utils.checkpoint.checkpoint(tf.entropy_from_logits, logits, use_reentrant=use_reentrant)
            lp = tf.logprobs_from_logits(logits, lab, inplace_backward=False)
            ((lp * w_lp).sum() + (h * w_h).sum()).backward()
            assert torch.equal(h.detach(), ref_h) and (lp.detach() - ref_lp).abs().max().item() <= 2e-6
            err = (leaf.grad.float() - ref_grad.float()).abs().max().item()
            scale = ref_grad.float().abs().max().item()
            assert err <= (1e-5 if dtype == torch.float32 else 2.0 ** -7) * max(scale, 1.0), (use_reentrant, err)
        hook.check_errors()


def test_a_pair_that_never_completes_pins_nothing(dev):
    """With gradients the first call of a pair leaves a per-row vector that carries its autograd graph, and the graph
    holds the logits. A caller that makes only one call of the pair (entropy without log-probs, or a forward that is
    never followed by a backward) must get the logits' memory back as soon as it lets go of the result, without
    another shim call on the thread."""
    import gc
    import weakref
    with _stand_in_verl() as mods:
        tf = mods["verl.utils.torch_functional"]
        hook.install()
        g = torch.Generator(device=dev).manual_seed(5)
        n, V = 64, 4099
        lab = torch.randint(0, V, (n,), generator=g, device=dev)
        leaf = torch.randn(n, V, generator=g, device=dev).requires_grad_(True)
        for first in ("entropy", "logprob"):
            logits = leaf * 1.0
            alive = weakref.ref(logits)
            res = tf.entropy_from_logits(logits) if first == "entropy" else tf.logprobs_from_logits(logits, lab)
            assert res.requires_grad
            del logits
            gc.collect()
            assert alive() is not None          # held by the result's graph, as with any differentiable op
            del res
            gc.collect()
            assert alive() is None, first       # ... and by nothing else
        # the result is kept (as the engine does) and the pair completes: shared as before
        logits = leaf * 1.0
        s0 = hook.stats()
        h = tf.entropy_from_logits(logits)
        lp = tf.logprobs_from_logits(logits, lab, inplace_backward=False)
        (h.sum() + lp.sum()).backward()
        s1 = hook.stats()
        assert s1["memo_hits"] - s0["memo_hits"] == 1 and s1["backward_passes"] - s0["backward_passes"] == 1
        # the explicit form
        logits = leaf * 1.0
        alive = weakref.ref(logits)
        res = tf.entropy_from_logits(logits)
        hook.clear_memo()
        n0 = hook.stats()["forward_passes"]
        tf.logprobs_from_logits(logits, lab)
        assert hook.stats()["forward_passes"] == n0 + 1     # nothing was left to share
        hook.clear_memo()
        del logits, res
        gc.collect()
        assert alive() is None
        hook.check_errors()


def test_installed_shims_never_synchronise(dev, monkeypatch):
    """The torch.gather the shims replace asserts on the device and returns (verl/utils/torch_functional.py:69): the
    shims must not drain the launch queue either. Fifty calls with every host synchronisation torch offers patched
    to raise, a bad label among them; check_errors() then reports it by waiting on events only."""
    with _stand_in_verl() as mods:
        tf = mods["verl.utils.torch_functional"]
        hook.install()
        g = torch.Generator(device=dev).manual_seed(3)
        V = 20011
        x = (torch.randn(512, V, generator=g, device=dev) * 3).bfloat16()
        x3 = torch.randn(3, 40, V, generator=g, device=dev)[:, 4:36]      # a batch of row slices: one flag for the loop
        lab = torch.randint(0, V, (512,), generator=g, device=dev)
        lab3 = torch.randint(0, V, (3, 32), generator=g, device=dev)
        bad = lab.clone()
        bad[100] = V + 5
        want = vf.logprobs_from_logits(x, lab)
        torch.cuda.synchronize()

        def refuse(*a, **k):
            raise AssertionError("a host synchronisation inside a shim call")

        with monkeypatch.context() as m:
            m.setattr(torch.Tensor, "item", refuse)
            m.setattr(torch.Tensor, "tolist", refuse)
            m.setattr(torch.Tensor, "cpu", refuse)
            m.setattr(torch.cuda, "synchronize", refuse)
            m.setattr(torch.cuda.Stream, "synchronize", refuse)
            outs = []
            with torch.no_grad():
                for i in range(50):
                    tf.entropy_from_logits(x)
                    outs.append(tf.logprobs_from_logits(x, lab))
                    tf.logprobs_from_logits_v2(x3, lab3)
                tf.entropy_from_logits(x)
                outs.append(tf.logprobs_from_logits(x, bad))
            with pytest.raises(IndexError, match="outside"):
                hook.check_errors()                 # waits on the recorded events only, never on the device
        torch.cuda.synchronize()
        assert torch.isnan(outs[50][100])
        assert (outs[49] - want).abs().max().item() <= 2e-6
        hook.check_errors()                      # nothing left, nothing raised


def test_installed_fused_linear_entry_points_serve_gpu_tensors(dev):
    from verl_amd.fused_linear import fused_linear_for_ppo

    class RefModule(torch.nn.Module):
        def __init__(self, chunk_size=512):
            super().__init__()

        def forward(self, hidden_states, vocab_weights, input_ids, temperature=1.0):
            raise AssertionError("GPU tensors must not reach the stand-in reference module")

    def ref_lce(*a, **k):
        raise AssertionError("GPU tensors must not reach the stand-in reference function")

    names = ("verl", "verl.utils", "verl.utils.torch_functional", "verl.utils.experimental",
             "verl.utils.experimental.torch_functional", "verl.utils.kernel", "verl.utils.kernel.linear_cross_entropy")
    mods = {n: types.ModuleType(n) for n in names}
    mods["verl.utils.experimental.torch_functional"].FusedLinearForPPO = RefModule
    mods["verl.utils.kernel.linear_cross_entropy"].linear_cross_entropy = ref_lce
    saved = {k: sys.modules.get(k) for k in mods}
    sys.modules.update(mods)
    try:
        hook.install()
        g = torch.Generator(device=dev).manual_seed(2)
        h = torch.empty(2, 30, 64, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
        w = torch.empty(1000, 64, device=dev).uniform_(-0.5, 0.5, generator=g).bfloat16()
        ids = torch.randint(0, 1000, (2, 30), generator=g, device=dev)
        want = fused_linear_for_ppo(h, w, ids, 1.2)
        mod = mods["verl.utils.experimental.torch_functional"].FusedLinearForPPO()
        got = mod.forward(hidden_states=h, vocab_weights=w, input_ids=ids, temperature=1.2)   # dense_common.py:122-128
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
        lce = mods["verl.utils.kernel.linear_cross_entropy"].linear_cross_entropy
        lp, ent = lce(h, w, ids, 1.2, "none")                                                   # dense_common.py:189-195
        assert torch.equal(lp, want[0].reshape(-1)) and torch.equal(ent, want[1].reshape(-1))
        assert _calls(hook.stats()) == {"hip_calls": 2, "passed_to_verl": 0, "memo_hits": 0}
    finally:
        hook.uninstall()
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v


def test_entry_points_replay_from_a_graph(dev):
    """The C ABI only enqueues kernels (no allocation, memset or synchronisation), so a caller may capture it.
    Replay three times with new inputs written into the same buffers; every replay must equal the eager result."""
    lib = _lib.load()
    B, T, V = 4, 64, 30011
    n = B * T
    gd = torch.Generator(device=dev).manual_seed(5)
    logits = torch.empty(n, V, dtype=torch.bfloat16, device=dev)
    labels = torch.empty(n, dtype=torch.int64, device=dev)
    old = torch.empty(n, device=dev); log_u = torch.empty(n, device=dev)
    mask = torch.ones(n, dtype=torch.uint8, device=dev)
    lp = torch.empty(n, device=dev); h = torch.empty(n, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    accept = torch.empty(n, dtype=torch.uint8, device=dev)
    first = torch.empty(B, dtype=torch.int32, device=dev); prefix = torch.empty_like(first); near = torch.empty_like(first)
    out_ids = torch.empty_like(labels); out_mask = torch.empty_like(mask)

    def fill():
        logits.copy_((torch.randn(n, V, generator=gd, device=dev) * 3).bfloat16())
        labels.copy_(torch.randint(0, V, (n,), generator=gd, device=dev))
        log_u.copy_(torch.log(torch.rand(n, generator=gd, device=dev)))
        ref_lp, _ = vf.fused_logprob_entropy(logits, labels, n_splits=1)
        old.copy_(ref_lp + torch.randn(n, generator=gd, device=dev) * 0.3)

    def call(stream):
        st = lib.vrl_fused_score_verify(
            logits.data_ptr(), _lib.VRL_BF16, n, V, V, labels.data_ptr(), None, lp.data_ptr(), h.data_ptr(), None, None,
            flag.data_ptr(), old.data_ptr(), log_u.data_ptr(), mask.data_ptr(), None, B, T, 0.0, 1e-6, accept.data_ptr(),
            first.data_ptr(), prefix.data_ptr(), near.data_ptr(), labels.data_ptr(), 0, out_ids.data_ptr(),
            out_mask.data_ptr(), stream)
        assert st == 0

    fill()
    call(torch.cuda.current_stream(dev).cuda_stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(torch.cuda.current_stream(dev).cuda_stream)
    for _ in range(3):
        fill()
        call(torch.cuda.current_stream(dev).cuda_stream)
        torch.cuda.synchronize()
        eager = [t.clone() for t in (lp, h, accept, first, prefix, near, out_ids, out_mask)]
        for t in (lp, h, accept, first, prefix, near, out_ids, out_mask):
            t.fill_(0) if t.dtype != torch.float32 else t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(eager, (lp, h, accept, first, prefix, near, out_ids, out_mask)):
            assert torch.equal(a, b)


def test_two_threads_two_streams_are_independent(dev):
    """The library keeps no state between calls: two host threads, each on its own stream with its own
    buffers, get the same results as one thread alone."""
    import threading

    gd = torch.Generator(device=dev).manual_seed(77)
    V = 50021
    xs = [(torch.randn(300, V, generator=gd, device=dev) * 3).bfloat16() for _ in range(2)]
    labs = [torch.randint(0, V, (300,), generator=gd, device=dev) for _ in range(2)]
    expected = [vf.fused_logprob_entropy(x, l, 0.8) for x, l in zip(xs, labs)]
    torch.cuda.synchronize()
    results = [None, None]
    errors = []

    def work(i):
        try:
            s = torch.cuda.Stream(device=dev)
            with torch.cuda.stream(s):
                out = None
                for _ in range(20):
                    out = vf.fused_logprob_entropy(xs[i], labs[i], 0.8)
                s.synchronize()
            results[i] = out
        except Exception as exc:  # surfaced below
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for got, exp in zip(results, expected):
        assert torch.equal(got[0], exp[0]) and torch.equal(got[1], exp[1])
