"""SPEC-RL draft verification on MI355X, and the fused score+verify step.

The reference holds no implementation of this step (its ``recipe/`` submodule
is not vendored, .gitmodules:1-3); tensor conventions follow the code that sits
where a caller would put it, verl/trainer/ppo/rollout_corr_helper.py:197-233
(``(B, T)`` fp32 log-probs, ``response_mask`` with 1 = valid) and
verl/trainer/ppo/ray_trainer.py:120-135.

Definition, per response token with ``d = logp_new - logp_old``:
  accept  <=>  valid  and  d >= log(u) + thresh_offset
``thresh_offset = +log(lenience)`` under ``lenience_mode="literal"`` (a lenience
above 1 is stricter) and ``-log(lenience)`` under ``"relax"`` (accept with
probability min(1, lenience * p_new / p_old)). ``u = 0`` always accepts, NaN
never does, masked tokens neither accept nor reject. The first rejected
position of a sequence ends its reusable prefix.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Union

import numpy as np
import torch

from . import _lib
from . import errors as _errors
from .torch_functional import _DTYPE_CODES, _check_logits, _ptr, _rows_2d, _temperature_rows

__all__ = ["VerifyResult", "draw_log_uniforms", "thresh_offset_from_lenience", "spec_verify", "truncate_draft", "fused_score_verify"]

DEFAULT_NEAR_EPS = 1e-6


@dataclass
class VerifyResult:
    accept: torch.Tensor  # bool, same shape as logp_new
    first_reject: torch.Tensor  # int32 (B,): in-sequence position of the first rejection, or end of valid tokens
    prefix_len: torch.Tensor  # int32 (B,): valid tokens before first_reject
    near_count: torch.Tensor  # int32 (B,): valid tokens with |d - tau| < near_eps
    log_u: torch.Tensor  # fp32, the uniforms' logs that were used
    thresh_offset: float
    out_ids: Optional[torch.Tensor] = None  # int64, draft with positions >= first_reject set to pad_id
    out_mask: Optional[torch.Tensor] = None  # bool, mask with positions >= first_reject cleared

    def metrics(self, response_mask: Optional[torch.Tensor] = None) -> dict:
        """spec/* scalars in the style of the reference's rollout_corr/* metrics."""
        n_valid = float(response_mask.ne(0).sum().item()) if response_mask is not None else float(self.accept.numel())
        return {
            "spec/accept_rate": float(self.accept.sum().item()) / max(n_valid, 1.0),
            "spec/mean_prefix_len": float(self.prefix_len.float().mean().item()) if self.prefix_len.numel() else 0.0,
            "spec/reuse_rate": float(self.prefix_len.sum().item()) / max(n_valid, 1.0),
            "spec/near_threshold_count": int(self.near_count.sum().item()),
        }


def thresh_offset_from_lenience(lenience: float = 1.0, lenience_mode: str = "literal") -> float:
    """log(lenience) rounded to fp32, signed by the mode (see module docstring)."""
    if not (lenience > 0.0) or math.isinf(lenience):
        raise ValueError(f"lenience must be a positive finite number, got {lenience}")
    if lenience_mode not in ("literal", "relax"):
        raise ValueError(f"lenience_mode must be 'literal' or 'relax', got {lenience_mode!r}")
    off = float(np.float32(math.log(lenience)))
    return off if lenience_mode == "literal" else -off


def draw_log_uniforms(shape, seed: int, device) -> torch.Tensor:
    """log(u), u ~ U[0,1) drawn from a generator on ``device`` seeded with ``seed``.

    The kernel and whoever checks it must consume this same tensor: a log taken
    elsewhere may round differently and flip a token that sits on the threshold.
    """
    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    u = torch.rand(tuple(shape), generator=g, device=device, dtype=torch.float32)
    return torch.log(u)


def _mask_u8(mask: Optional[torch.Tensor], shape, device) -> Optional[torch.Tensor]:
    if mask is None:
        return None
    if tuple(mask.shape) != tuple(shape):
        raise ValueError(f"response_mask shape {tuple(mask.shape)} does not match {tuple(shape)}")
    mask = mask.to(device)
    if mask.dtype == torch.bool:
        return mask.contiguous().view(torch.uint8)
    return mask.ne(0).contiguous().view(torch.uint8)


def _f32(t: torch.Tensor, name: str, shape, device) -> torch.Tensor:
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} shape {tuple(t.shape)} does not match {tuple(shape)}")
    if not t.is_cuda:
        raise RuntimeError(f"{name} is on {t.device}; verl_amd only runs on the GPU, it has no CPU implementation")
    return t.to(device=device, dtype=torch.float32).contiguous()


def _layout(shape, cu_seqlens: Optional[torch.Tensor], device):
    """-> (B, T, cu) for a padded (B, T) or packed (N,) + cu_seqlens (B+1,) layout."""
    if cu_seqlens is None:
        if len(shape) != 2:
            raise ValueError(f"padded layout needs (B, T) tensors, got shape {tuple(shape)}; pass cu_seqlens for packed tokens")
        return int(shape[0]), int(shape[1]), None
    if len(shape) != 1:
        raise ValueError(f"packed layout needs 1-D token tensors, got shape {tuple(shape)}")
    if cu_seqlens.dim() != 1 or cu_seqlens.numel() < 1:
        raise ValueError("cu_seqlens must be 1-D with B+1 entries")
    cu = cu_seqlens.to(device=device, dtype=torch.int64).contiguous()
    return int(cu.numel() - 1), 0, cu


def _seq_messages(what: str, n_tokens: int, vocab: Optional[int] = None) -> dict:
    """What the kernels' error bits mean for ``what``. The packed offsets live on the device: the kernels hold them
    to the arrays' length (nothing outside is touched) and report through the flag, like the reference's assert at
    verl/workers/utils/padding.py:129-130."""
    msgs = {}
    if vocab is not None:
        msgs[_lib.VRL_FLAG_LABEL_OOB] = (IndexError, f"{what}: a label is outside [0, {vocab})")
    msgs[_lib.VRL_FLAG_SEQ_RANGE] = (ValueError, f"{what}: cu_seqlens is not a partition of the {n_tokens} tokens "
                                     "(it must start at 0, never decrease and end at the number of tokens)")
    return msgs


def _verify_buffers(shape, B, device, draft_ids, want_truncated, packed=False, pad_id=0):
    # packed: tokens that no in-range span covers are not written by the kernel, so they start as "not accepted"
    accept = (torch.zeros if packed else torch.empty)(tuple(shape), dtype=torch.uint8, device=device)
    first = torch.empty(B, dtype=torch.int32, device=device)
    prefix = torch.empty(B, dtype=torch.int32, device=device)
    near = torch.empty(B, dtype=torch.int32, device=device)
    ids = out_ids = out_mask = None
    if want_truncated:
        if tuple(draft_ids.shape) != tuple(shape):
            raise ValueError(f"draft_ids shape {tuple(draft_ids.shape)} does not match {tuple(shape)}")
        ids = draft_ids.to(device=device, dtype=torch.int64).contiguous()
        out_ids = torch.full_like(ids, int(pad_id)) if packed else torch.empty_like(ids)
        out_mask = (torch.zeros if packed else torch.empty)(tuple(shape), dtype=torch.uint8, device=device)
    return accept, first, prefix, near, ids, out_ids, out_mask


def _resolve_log_u(log_u, uniforms, seed, shape, device) -> torch.Tensor:
    given = sum(x is not None for x in (log_u, uniforms, seed))
    if given != 1:
        raise ValueError("give exactly one of log_u, uniforms, seed")
    if log_u is not None:
        return _f32(log_u, "log_u", shape, device)
    if uniforms is not None:
        return torch.log(_f32(uniforms, "uniforms", shape, device))
    return draw_log_uniforms(shape, seed, device)


def spec_verify(
    logp_new: torch.Tensor,
    logp_old: torch.Tensor,
    response_mask: Optional[torch.Tensor] = None,
    *,
    log_u: Optional[torch.Tensor] = None,
    uniforms: Optional[torch.Tensor] = None,
    seed: Optional[int] = None,
    lenience: float = 1.0,
    lenience_mode: str = "literal",
    thresh_offset: Optional[float] = None,
    near_eps: float = DEFAULT_NEAR_EPS,
    cu_seqlens: Optional[torch.Tensor] = None,
    draft_ids: Optional[torch.Tensor] = None,
    pad_id: int = 0,
    check=None,
    two_pass: Optional[bool] = None,
) -> VerifyResult:
    """Verify a draft against new log-probs; see the module docstring for the rule.

    Layouts: padded ``(B, T)`` tensors, or packed 1-D token tensors with
    ``cu_seqlens`` (``B+1`` row offsets that partition the tokens; anything else raises
    ValueError, when and how is ``check``'s business as in verl_amd.errors). With
    ``draft_ids`` the truncated draft and mask come back too.

    ``two_pass`` picks the kernel form: False is one workgroup per sequence, True two flat passes over the tokens whose
    work does not depend on how the tokens are cut into sequences (a scratch tensor of half a byte per token is
    allocated for them); None lets the library choose by shape (``vrl_spec_verify_plan``: large packed batches, and
    padded ones with few long sequences). The results are the same integers.
    """
    _errors.poll()
    if not logp_new.is_cuda:
        raise RuntimeError(f"logp_new is on {logp_new.device}; verl_amd only runs on the GPU, it has no CPU implementation")
    dev = logp_new.device
    shape = tuple(logp_new.shape)
    B, T, cu = _layout(shape, cu_seqlens, dev)
    ln = _f32(logp_new, "logp_new", shape, dev)
    lo = _f32(logp_old, "logp_old", shape, dev)
    lu = _resolve_log_u(log_u, uniforms, seed, shape, dev)
    m8 = _mask_u8(response_mask, shape, dev)
    off = thresh_offset_from_lenience(lenience, lenience_mode) if thresh_offset is None else float(np.float32(thresh_offset))
    accept, first, prefix, near, ids, out_ids, out_mask = _verify_buffers(shape, B, dev, draft_ids,
                                                                         draft_ids is not None, cu is not None, pad_id)
    flag = torch.zeros(1, dtype=torch.int32, device=dev) if cu is not None else None

    if ln.numel() == 0:
        # no token at all (B empty sequences): nothing to launch, every sequence's results are zero
        for t in (first, prefix, near):
            t.zero_()
        return VerifyResult(
            accept=accept.view(torch.bool), first_reject=first, prefix_len=prefix, near_count=near, log_u=lu,
            thresh_offset=off, out_ids=out_ids, out_mask=None if out_mask is None else out_mask.view(torch.bool),
        )
    lib = _lib.load()
    if two_pass is None:
        two_pass = bool(lib.vrl_spec_verify_plan(int(cu is not None), B, T, ln.numel()))
    work = None
    if two_pass and B > 0:
        work = torch.empty(int(lib.vrl_spec_verify_workspace(ln.numel())), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        stream = _lib.stream_ptr(dev)
        st = lib.vrl_spec_verify(
            ln.data_ptr(), lo.data_ptr(), lu.data_ptr(), _ptr(m8), _ptr(cu), B, T, ln.numel(), off, float(near_eps),
            accept.data_ptr(), first.data_ptr(), prefix.data_ptr(), near.data_ptr(),
            _ptr(ids), int(pad_id), _ptr(out_ids), _ptr(out_mask), _ptr(flag), _ptr(work),
            0 if work is None else work.numel(), stream,
        )
    _lib.check("vrl_spec_verify", st)
    if flag is not None and B > 0:
        _errors.report(flag, _seq_messages("spec_verify", ln.numel()), check)
    return VerifyResult(
        accept=accept.view(torch.bool), first_reject=first, prefix_len=prefix, near_count=near, log_u=lu,
        thresh_offset=off, out_ids=out_ids, out_mask=None if out_mask is None else out_mask.view(torch.bool),
    )


def truncate_draft(
    draft_ids: torch.Tensor,
    response_mask: Optional[torch.Tensor],
    first_reject: torch.Tensor,
    *,
    pad_id: int = 0,
    cu_seqlens: Optional[torch.Tensor] = None,
    check=None,
):
    """(ids, mask) with every position >= first_reject[b] set to pad_id / False."""
    _errors.poll()
    if not draft_ids.is_cuda:
        raise RuntimeError(f"draft_ids is on {draft_ids.device}; verl_amd only runs on the GPU, it has no CPU implementation")
    dev = draft_ids.device
    shape = tuple(draft_ids.shape)
    B, T, cu = _layout(shape, cu_seqlens, dev)
    if tuple(first_reject.shape) != (B,):
        raise ValueError(f"first_reject must have shape ({B},), got {tuple(first_reject.shape)}")
    ids = draft_ids.to(dtype=torch.int64).contiguous()
    m8 = _mask_u8(response_mask, shape, dev)
    fr = first_reject.to(device=dev, dtype=torch.int32).contiguous()
    packed = cu is not None
    out_ids = torch.full_like(ids, int(pad_id)) if packed else torch.empty_like(ids)
    out_mask = (torch.zeros if packed else torch.empty)(shape, dtype=torch.uint8, device=dev)
    if ids.numel() == 0:
        return out_ids, out_mask.view(torch.bool)
    flag = torch.zeros(1, dtype=torch.int32, device=dev) if packed else None
    lib = _lib.load()
    with torch.cuda.device(dev):
        stream = _lib.stream_ptr(dev)
        st = lib.vrl_truncate_draft(ids.data_ptr(), _ptr(m8), _ptr(cu), B, T, ids.numel(), fr.data_ptr(), int(pad_id),
                                    out_ids.data_ptr(), out_mask.data_ptr(), _ptr(flag), stream)
    _lib.check("vrl_truncate_draft", st)
    if packed and B > 0:
        _errors.report(flag, _seq_messages("truncate_draft", ids.numel()), check)
    return out_ids, out_mask.view(torch.bool)


def fused_score_verify(
    logits: torch.Tensor,
    labels: torch.Tensor,
    logp_old: torch.Tensor,
    response_mask: Optional[torch.Tensor] = None,
    *,
    temperature: Union[None, float, torch.Tensor] = None,
    log_u: Optional[torch.Tensor] = None,
    uniforms: Optional[torch.Tensor] = None,
    seed: Optional[int] = None,
    lenience: float = 1.0,
    lenience_mode: str = "literal",
    thresh_offset: Optional[float] = None,
    near_eps: float = DEFAULT_NEAR_EPS,
    cu_seqlens: Optional[torch.Tensor] = None,
    draft_ids: Optional[torch.Tensor] = None,
    pad_id: int = 0,
    check_labels=None,
):
    """Score ``logits`` and verify the draft in one call: (log-probs, entropy, VerifyResult).

    ``logits`` is ``(B, T, V)`` (padded) or ``(N, V)`` with ``cu_seqlens``
    (packed); every per-token tensor has the logits' leading shape. ``check_labels`` governs both device-side
    checks, labels inside the vocabulary (IndexError) and packed offsets that partition the rows (ValueError).
    """
    _check_logits(logits, "fused_score_verify")
    _errors.poll()
    if torch.is_grad_enabled() and logits.requires_grad:
        raise NotImplementedError("fused_score_verify is a forward-only step (verification happens under no_grad); "
                                  "use fused_logprob_entropy for the differentiable scores")
    dev = logits.device
    lead = tuple(logits.shape[:-1])
    V = logits.shape[-1]
    B, T, cu = _layout(lead, cu_seqlens, dev)
    x = _rows_2d(logits)
    n = x.shape[0]
    if tuple(labels.shape) != lead:
        raise ValueError(f"labels shape {tuple(labels.shape)} does not match logits leading shape {lead}")
    if labels.dtype.is_floating_point or labels.dtype == torch.bool:
        raise TypeError(f"labels must be an integer tensor, got {labels.dtype}")
    lab = labels.to(device=dev, dtype=torch.int64).reshape(n).contiguous()
    temp = _temperature_rows(temperature, lead, n, dev)
    lo = _f32(logp_old, "logp_old", lead, dev)
    lu = _resolve_log_u(log_u, uniforms, seed, lead, dev)
    m8 = _mask_u8(response_mask, lead, dev)
    off = thresh_offset_from_lenience(lenience, lenience_mode) if thresh_offset is None else float(np.float32(thresh_offset))
    out_lp = torch.empty(n, dtype=torch.float32, device=dev)
    out_h = torch.empty(n, dtype=torch.float32, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    accept, first, prefix, near, ids, out_ids, out_mask = _verify_buffers(lead, B, dev, draft_ids,
                                                                         draft_ids is not None, cu is not None, pad_id)

    if n == 0:
        for t in (first, prefix, near):
            t.zero_()
        res = VerifyResult(
            accept=accept.view(torch.bool), first_reject=first, prefix_len=prefix, near_count=near, log_u=lu,
            thresh_offset=off, out_ids=out_ids, out_mask=None if out_mask is None else out_mask.view(torch.bool),
        )
        return out_lp.reshape(lead), out_h.reshape(lead), res
    lib = _lib.load()
    with torch.cuda.device(dev):
        stream = _lib.stream_ptr(dev)
        st = lib.vrl_fused_score_verify(
            x.data_ptr(), _DTYPE_CODES[x.dtype], n, V, x.stride(0) if n > 1 else V, lab.data_ptr(), _ptr(temp),
            out_lp.data_ptr(), out_h.data_ptr(), None, None, flag.data_ptr(),
            lo.data_ptr(), lu.data_ptr(), _ptr(m8), _ptr(cu), B, T, off, float(near_eps),
            accept.data_ptr(), first.data_ptr(), prefix.data_ptr(), near.data_ptr(),
            _ptr(ids), int(pad_id), _ptr(out_ids), _ptr(out_mask), stream,
        )
    _lib.check("vrl_fused_score_verify", st)
    _errors.report(flag, _seq_messages("fused_score_verify", n, V), check_labels)
    res = VerifyResult(
        accept=accept.view(torch.bool), first_reject=first, prefix_len=prefix, near_count=near, log_u=lu,
        thresh_offset=off, out_ids=out_ids, out_mask=None if out_mask is None else out_mask.view(torch.bool),
    )
    return out_lp.reshape(lead), out_h.reshape(lead), res
