"""TEST INFRASTRUCTURE — CPU statement of the SPEC-RL draft-verify rule.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this. Nothing under verl_amd/ does.

PARITY UNPINNED BY THE REFERENCE: the reference has no implementation of this
step (its ``recipe/`` submodule is an empty, un-vendored directory,
.gitmodules:1-3; nothing in the tree mentions SPEC-RL or lenience). The rule
below is the one the task statement gives: per response token form
log p_new - log p_old, test it against log(u) + log(lenience), apply the
response mask, take the first rejection per sequence. Tensor conventions
((B, T) fp32 log-probs, response_mask 1 = valid, sequences with no valid token
handled explicitly) follow verl/trainer/ppo/rollout_corr_helper.py:197-233,
262-268 and verl/trainer/ppo/ray_trainer.py:120-135.

What does pin it (tests/test_oracle_verify.py): ``verify_loops`` is a scalar
double loop written from the rule; ``verify`` is the vectorised form used at
size; they are checked against each other on random and hand-built cases, and
against properties the rule fixes (all accepted when d >= 0 and the offset is
<= 0; masked tokens never reject; accept is monotone in the offset;
prefix_len <= number of valid tokens; truncation is idempotent; u = 0 accepts;
NaN rejects), and against hand-computed rows in the style of the reference's
exact-input mask tests (tests/trainer/ppo/test_rollout_corr.py:312-366).

Decisions the rule leaves open, fixed here:
  D1  tau = log(u) + thresh_offset; thresh_offset = +log(lenience) ("literal"
      reading of the task statement) or -log(lenience) ("relax": accept with
      probability min(1, lenience * p_new / p_old)). The offset is one fp32 number.
  D2  comparison is d >= tau (u = 1, d = 0 accepts).
  D3  u = 0 gives log u = -inf: always accepted.
  D4  masked tokens never reject and have accept = 0.
  D5  first_reject = position of the first valid rejected token; with none, one
      past the last valid position (= number of valid tokens for a right-padded mask).
  D6  NaN in d or tau: the comparison is false, the token is rejected.
"""

from __future__ import annotations

import numpy as np
import torch


def _f32(x) -> np.ndarray:
    if isinstance(x, torch.Tensor):
        x = x.detach().cpu().float().numpy()
    return np.asarray(x, dtype=np.float32)


def _spans(shape, cu_seqlens):
    if cu_seqlens is None:
        B, T = shape
        return [(b * T, T) for b in range(B)]
    cu = [int(c) for c in (cu_seqlens.tolist() if hasattr(cu_seqlens, "tolist") else cu_seqlens)]
    return [(cu[b], max(cu[b + 1] - cu[b], 0)) for b in range(len(cu) - 1)]


def verify_loops(logp_new, logp_old, log_u, mask, thresh_offset, near_eps=1e-6, cu_seqlens=None,
                 draft_ids=None, pad_id=0):
    """Scalar statement of the rule: one Python loop over sequences, one over positions.

    Inputs are (B, T) arrays (padded) or 1-D arrays with cu_seqlens (packed).
    Returns a dict of numpy arrays: accept (uint8, input shape), first_reject / prefix_len /
    near_count (int32, (B,)), and out_ids / out_mask when draft_ids is given.
    """
    ln, lo, lu = _f32(logp_new), _f32(logp_old), _f32(log_u)
    shape = ln.shape
    ln, lo, lu = ln.reshape(-1), lo.reshape(-1), lu.reshape(-1)
    mk = None if mask is None else (np.asarray(mask.cpu() if isinstance(mask, torch.Tensor) else mask).reshape(-1) != 0)
    ids = None if draft_ids is None else np.asarray(draft_ids.cpu() if isinstance(draft_ids, torch.Tensor) else draft_ids).reshape(-1).astype(np.int64)
    off = np.float32(thresh_offset)
    eps = np.float32(near_eps)
    spans = _spans(shape, cu_seqlens)
    accept = np.zeros(ln.shape, dtype=np.uint8)
    first = np.zeros(len(spans), dtype=np.int32)
    prefix = np.zeros(len(spans), dtype=np.int32)
    near = np.zeros(len(spans), dtype=np.int32)
    out_ids = None if ids is None else np.empty_like(ids)
    out_mask = None if ids is None else np.zeros(ids.shape, dtype=np.uint8)
    with np.errstate(invalid="ignore"):
        for b, (start, length) in enumerate(spans):
            first_rej = None
            last_valid = 0
            for i in range(length):
                g = start + i
                valid = True if mk is None else bool(mk[g])
                d = np.float32(ln[g] - lo[g])
                tau = np.float32(lu[g] + off)
                ok = bool(d >= tau)
                if valid:
                    last_valid = i + 1
                    if ok:
                        accept[g] = 1
                    elif first_rej is None:
                        first_rej = i
                    if bool(np.abs(np.float32(d - tau)) < eps):
                        near[b] += 1
            f = last_valid if first_rej is None else first_rej
            first[b] = f
            prefix[b] = sum(1 for i in range(f) if (mk is None or mk[start + i]))
            if ids is not None:
                for i in range(length):
                    g = start + i
                    keep = i < f
                    out_ids[g] = ids[g] if keep else pad_id
                    out_mask[g] = (1 if (mk is None or mk[g]) else 0) if keep else 0
    res = {"accept": accept.reshape(shape), "first_reject": first, "prefix_len": prefix, "near_count": near}
    if ids is not None:
        res["out_ids"] = out_ids.reshape(shape)
        res["out_mask"] = out_mask.reshape(shape)
    return res


def verify(logp_new, logp_old, log_u, mask, thresh_offset, near_eps=1e-6, cu_seqlens=None,
           draft_ids=None, pad_id=0):
    """Vectorised form of verify_loops (torch, fp32 on the CPU); same return dict with torch tensors.

    Padded (B, T) inputs are processed as a whole; packed inputs are scattered into a padded
    (B, Lmax) frame first and the per-token outputs gathered back.
    """
    ln = torch.as_tensor(logp_new).detach().cpu().float()
    lo = torch.as_tensor(logp_old).detach().cpu().float()
    lu = torch.as_tensor(log_u).detach().cpu().float()
    shape = tuple(ln.shape)
    mk = None if mask is None else torch.as_tensor(mask).detach().cpu().ne(0)
    ids = None if draft_ids is None else torch.as_tensor(draft_ids).detach().cpu().long()
    off = torch.tensor(float(np.float32(thresh_offset)), dtype=torch.float32)
    eps = torch.tensor(float(np.float32(near_eps)), dtype=torch.float32)

    packed = cu_seqlens is not None
    if packed:
        cu = torch.as_tensor(cu_seqlens).detach().cpu().long()
        lens = (cu[1:] - cu[:-1]).clamp(min=0)
        B = lens.numel()
        T = int(lens.max().item()) if B > 0 else 0
        pos = torch.arange(T).unsqueeze(0).expand(B, T)
        inside = pos < lens.unsqueeze(1)
        src = (cu[:-1].unsqueeze(1) + pos)[inside]

        def frame(x, fill):
            out = torch.full((B, T), fill, dtype=x.dtype)
            out[inside] = x.reshape(-1)[src]
            return out

        ln, lo, lu = frame(ln, 0.0), frame(lo, 0.0), frame(lu, 0.0)
        mk = inside if mk is None else (frame(mk, False) & inside)
        if ids is not None:
            ids = frame(ids, 0)
    else:
        B, T = shape
        inside = torch.ones(B, T, dtype=torch.bool)
        if mk is None:
            mk = inside

    d = ln - lo
    tau = lu + off
    ok = d >= tau
    accept = mk & ok
    rej = mk & ~ok
    pos = torch.arange(T).unsqueeze(0).expand(B, T)
    big = T + 1
    first_rej = torch.where(rej, pos, torch.full_like(pos, big)).min(dim=1).values if T > 0 else torch.full((B,), big)
    last_valid = torch.where(mk, pos + 1, torch.zeros_like(pos)).max(dim=1).values if T > 0 else torch.zeros(B, dtype=torch.long)
    first = torch.where(first_rej == big, last_valid, first_rej)
    before = pos < first.unsqueeze(1)
    prefix = (mk & before).sum(dim=1)
    near = (mk & ((d - tau).abs() < eps)).sum(dim=1)

    def unframe(x):
        if not packed:
            return x
        out = torch.zeros(shape, dtype=x.dtype)
        out.reshape(-1)[src] = x[inside]
        return out

    res = {
        "accept": unframe(accept.to(torch.uint8)),
        "first_reject": first.to(torch.int32),
        "prefix_len": prefix.to(torch.int32),
        "near_count": near.to(torch.int32),
    }
    if ids is not None:
        res["out_ids"] = unframe(torch.where(before, ids, torch.full_like(ids, pad_id)))
        res["out_mask"] = unframe((mk & before).to(torch.uint8))
    return res
