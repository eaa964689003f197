"""Rollout correction (IS weights, rejection masks, off-policy metrics) on MI355X.

Same functions, arguments, errors and metric names as verl/trainer/ppo/rollout_corr_helper.py
(compute_rollout_rejection_mask :197, compute_rollout_correction_weights :522,
compute_rollout_correction_and_rejection_mask :786, compute_offpolicy_metrics :904). The reference runs
~150 small torch kernels and ~80 ``.item()`` synchronisations per call; here one HIP kernel
(vrl_rollout_corr) produces the weights, the mask and a ``(B, 40)`` table of per-sequence partial sums,
one copy brings the table to the host, and every scalar metric is finished there in double precision.
Tensors must be on the GPU; there is no CPU path.
"""

from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch

from . import _lib

__all__ = [
    "compute_rollout_rejection_mask",
    "compute_rollout_correction_weights",
    "compute_rollout_correction_and_rejection_mask",
    "compute_offpolicy_metrics",
    "SUPPORTED_ROLLOUT_RS_OPTIONS",
]

# order = bit positions in the kernel's rs_bits / seq_keep_bits
RS_ORDER = ("token_k1", "token_k2", "token_k3", "seq_sum_k1", "seq_sum_k2", "seq_sum_k3",
            "seq_mean_k1", "seq_mean_k2", "seq_mean_k3", "seq_max_k2", "seq_max_k3")
SUPPORTED_ROLLOUT_RS_OPTIONS = set(RS_ORDER)
_EPS = 1e-8

# columns of the statistics table (enum CorrStat in csrc/rollout_corr_kernels.h)
(N, SUM_OLD, SUM_ROLL, SUM_LR, SUM_K3RAW, SUM_RHO2, SUM_K1, SUM_K2, SUM_K3, MAX_K1, MIN_K1, MAX_K2, MIN_K2, MAX_K3, MIN_K3,
 TOK_HI0, TOK_LO0, TOK_CL0, TOK_CL20, TOK_HI1, TOK_LO1, TOK_CL1, TOK_CL21, TOK_HI2, TOK_LO2, TOK_CL2, TOK_CL22,
 TOK_MASKED0, TOK_MASKED1, TOK_MASKED2, FINAL_MASKED,
 SUM_W, SUM_WRAW, MAX_W, MIN_W, CNT_RAW_HI, CNT_RAW_LO, SUM_WC, SUM_WC2, CNT_OOB, NUM_STATS) = range(41)


# ---- threshold specifications (same grammar and errors as the reference, :92-194) ----------------------------

def _parse_is_threshold(spec):
    if isinstance(spec, bool):
        raise TypeError("rollout_is_threshold must be specified as a float or a string threshold specification, not a boolean.")
    if isinstance(spec, (int, float)):
        upper, lower = float(spec), None
    elif isinstance(spec, str):
        text = spec.strip()
        if not text:
            raise ValueError("rollout_is_threshold must not be an empty string.")
        try:
            if "_" in text:
                lo, up = text.split("_", 1)
                lower, upper = float(lo), float(up)
            else:
                upper, lower = float(text), None
        except ValueError as exc:
            raise ValueError(f"Invalid rollout_is_threshold '{spec}'.") from exc
    else:
        raise TypeError("rollout_is_threshold must be a float or a string threshold specification.")
    if upper <= 0:
        raise ValueError(f"rollout_is_threshold upper bound must be positive, got {upper}.")
    if lower is not None:
        if lower <= 0:
            raise ValueError(f"rollout_is_threshold lower bound must be positive, got {lower}.")
        if lower > upper:
            raise ValueError("rollout_is_threshold lower bound must be <= upper bound.")
    return upper, lower


def _normalize_rs_options(rollout_rs):
    if rollout_rs is None or not isinstance(rollout_rs, str):
        raise ValueError("rollout_rs must be a non-empty string (comma separated for multiple options).")
    out = []
    for opt in (o.strip() for o in rollout_rs.split(",")):
        if not opt:
            continue
        if opt not in SUPPORTED_ROLLOUT_RS_OPTIONS:
            raise ValueError(f"Invalid rollout_rs option: {opt}. Must be one of {sorted(SUPPORTED_ROLLOUT_RS_OPTIONS)}.")
        if opt not in out:
            out.append(opt)
    if not out:
        raise ValueError("rollout_rs must contain at least one valid option.")
    return out


def _parse_rs_thresholds(options, spec):
    if spec is None:
        raise ValueError("rollout_rs_threshold must be provided for rejection sampling.")
    if isinstance(spec, (int, float)) and not isinstance(spec, bool):
        parts = [str(spec)]
    elif isinstance(spec, str):
        parts = [p.strip() for p in spec.split(",") if p.strip()]
    else:
        raise TypeError("rollout_rs_threshold must be a string or numeric value specifying per-option thresholds.")
    if not parts:
        raise ValueError("rollout_rs_threshold must contain at least one threshold value.")
    if len(parts) not in (1, len(options)):
        raise ValueError(f"rollout_rs_threshold expects either one threshold shared by all options or exactly {len(options)} thresholds.")
    if len(parts) == 1:
        parts = parts * len(options)
    out = {}
    for opt, text in zip(options, parts):
        try:
            if opt.endswith("k1"):
                lo_s, up_s = text.split("_", 1) if "_" in text else (str(1.0 / float(text)), text)
                lower, upper = float(lo_s), float(up_s)
            else:
                if "_" in text:
                    raise ValueError(f"rollout_rs_threshold for option '{opt}' must provide a single upper bound without '_'. Received '{text}'.")
                lower, upper = None, float(text)
        except ValueError as exc:
            if "single upper bound" in str(exc):
                raise
            raise ValueError(f"Invalid numeric threshold '{text}' for option '{opt}'.") from exc
        if upper <= 0 or (lower is not None and lower <= 0):
            raise ValueError(f"Thresholds for option '{opt}' must be positive, got {text}.")
        if lower is not None and lower > upper:
            raise ValueError(f"Thresholds for option '{opt}' must be lower <= upper, got {text}.")
        out[opt] = (lower, upper)
    return out


# ---- the launch ---------------------------------------------------------------------------------------------

class _Result:
    __slots__ = ("weights", "keep", "stats", "seq_bits")


def _f32_2d(t, name, shape=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor; verl_amd has no CPU implementation")
    if t.dim() != 2 or (shape is not None and tuple(t.shape) != tuple(shape)):
        raise ValueError(f"{name} shape {tuple(t.shape)} does not match {tuple(shape) if shape else '(B, T)'}")
    return t.detach().to(torch.float32).contiguous()


def _mask_u8(mask, shape, device):
    if tuple(mask.shape) != tuple(shape):
        raise ValueError(f"log_prob shape {tuple(shape)} does not match response_mask shape {tuple(mask.shape)}.")
    m = mask.to(device)
    return (m if m.dtype == torch.bool else m.ne(0)).contiguous().view(torch.uint8)


def _launch(old, roll, mask8, *, is_mode=0, icepop=False, is_upper=1.0, is_lower=0.0, is_lower_metric=0.0,
            rs_bounds=None, want_weights=False, want_keep=False) -> _Result:
    B, T = old.shape
    dev = old.device
    lib = _lib.load()
    ns = lib.vrl_rollout_corr_num_stats()
    assert ns == NUM_STATS, (ns, NUM_STATS)
    res = _Result()
    res.weights = torch.empty((B, T), dtype=torch.float32, device=dev) if want_weights else None
    res.keep = torch.empty((B, T), dtype=torch.uint8, device=dev) if want_keep else None
    stats = torch.empty((B, ns), dtype=torch.float32, device=dev)
    bits = torch.empty(B, dtype=torch.int32, device=dev)
    lo = (_lib._c.c_float * len(RS_ORDER))()
    hi = (_lib._c.c_float * len(RS_ORDER))()
    rs_bits = 0
    for name, (lower, upper) in (rs_bounds or {}).items():
        i = RS_ORDER.index(name)
        rs_bits |= 1 << i
        lo[i] = 0.0 if lower is None else lower
        hi[i] = upper
    with torch.cuda.device(dev):
        st = lib.vrl_rollout_corr(old.data_ptr(), roll.data_ptr(), mask8.data_ptr(), B, T, int(is_mode), int(bool(icepop)),
                                  float(is_upper), float(is_lower), float(is_lower_metric), rs_bits,
                                  _lib._c.cast(lo, _lib._c.c_void_p), _lib._c.cast(hi, _lib._c.c_void_p),
                                  None if res.weights is None else res.weights.data_ptr(),
                                  None if res.keep is None else res.keep.data_ptr(), stats.data_ptr(), bits.data_ptr(),
                                  _lib.stream_ptr(dev))
    _lib.check("vrl_rollout_corr", st)
    table = torch.cat([stats, bits.to(torch.float32).unsqueeze(1)], dim=1).cpu().numpy()  # the one copy to the host
    res.stats = table[:, :ns].astype(np.float64)
    res.seq_bits = table[:, ns].astype(np.int64)
    return res


# ---- metrics from the per-sequence table -----------------------------------------------------------------------

def _std_unbiased(x):
    return float(np.std(x, ddof=1)) if x.size > 1 else 0.0


def _rs_bounds_as_compared(options, specs):
    """name -> (lower, upper) exactly as the kernel compares them, in fp32 (log of the ratio bounds for k1)."""
    out = {}
    for opt in options:
        lower, upper = specs[opt]
        if opt.endswith("k1"):
            out[opt] = (float(np.float32(math.log(lower))), float(np.float32(math.log(upper))))
        else:
            out[opt] = (None, float(np.float32(upper)))
    return out


def _rs_metrics(S, seq_bits, options, bounds):
    n = S[:, N]
    ntot = n.sum()
    valid = n > 0
    nvalid = int(valid.sum())
    m = {}
    sums = {"k1": S[:, SUM_K1], "k2": S[:, SUM_K2], "k3": S[:, SUM_K3]}
    maxs = {"k1": S[:, MAX_K1], "k2": S[:, MAX_K2], "k3": S[:, MAX_K3]}
    mins = {"k1": S[:, MIN_K1], "k2": S[:, MIN_K2], "k3": S[:, MIN_K3]}
    for opt in options:
        kind = opt[-2:]
        j = ("k1", "k2", "k3").index(kind)
        is_k1 = kind == "k1"
        lower, upper = bounds[opt]
        lower_m = lower if is_k1 else 0.0
        pre = f"rollout_rs_{opt}"
        if opt.startswith("token"):
            m[f"{pre}_mean"] = sums[kind].sum() / (ntot + _EPS)
            m[f"{pre}_max"] = maxs[kind][valid].max()
            m[f"{pre}_min"] = mins[kind][valid].min()
            m[f"{pre}_fraction_high"] = S[:, TOK_HI0 + 4 * j].sum() / (ntot + _EPS)
            m[f"{pre}_fraction_low"] = S[:, TOK_LO0].sum() / (ntot + _EPS) if is_k1 else 0.0
            mean_c = S[:, TOK_CL0 + 4 * j].sum() / (ntot + _EPS)
            var = S[:, TOK_CL20 + 4 * j].sum() / (ntot + _EPS) - mean_c**2
            sv = (sums[kind] / (n + _EPS))[valid]
            masked_tokens = S[:, TOK_MASKED0 + j]
            seq_dropped = masked_tokens > 0
        else:
            if opt.startswith("seq_sum"):
                s = sums[kind]
            elif opt.startswith("seq_mean"):
                s = sums[kind].astype(np.float32) / (n.astype(np.float32) + np.float32(_EPS))  # as the kernel divides
                s = s.astype(np.float64)
            else:
                s = np.where(valid, maxs[kind], 0.0)
            sv = s[valid]
            m[f"{pre}_mean"] = (n * s).sum() / (ntot + _EPS)
            m[f"{pre}_max"] = sv.max()
            m[f"{pre}_min"] = sv.min()
            m[f"{pre}_fraction_high"] = float((sv > upper).mean())
            m[f"{pre}_fraction_low"] = float((sv < lower_m).mean()) if is_k1 else 0.0
            c = np.clip(s, lower_m, upper)
            mean_c = (n * c).sum() / (ntot + _EPS)
            var = (n * c * c).sum() / (ntot + _EPS) - mean_c**2
            passed = ((seq_bits >> RS_ORDER.index(opt)) & 1).astype(bool)
            masked_tokens = np.where(passed, 0.0, n)
            seq_dropped = (~passed) & valid
        m[f"{pre}_std"] = math.sqrt(max(var, 0.0)) if ntot > 1 else 0.0
        m[f"{pre}_seq_mean"] = float(sv.mean())
        m[f"{pre}_seq_std"] = _std_unbiased(sv)
        m[f"{pre}_seq_max"] = float(sv.max())
        m[f"{pre}_seq_min"] = float(sv.min())
        m[f"{pre}_seq_max_deviation"] = float(np.abs(sv).max())
        m[f"{pre}_seq_fraction_high"] = float((sv > upper).mean())
        if is_k1:
            m[f"{pre}_seq_fraction_low"] = float((sv < lower_m).mean())
        m[f"{pre}_masked_fraction"] = masked_tokens.sum() / (ntot + _EPS)
        m[f"{pre}_seq_masked_fraction"] = float((seq_dropped & valid).sum() / nvalid) if nvalid > 0 else 0.0
    m["rollout_rs_masked_fraction"] = S[:, FINAL_MASKED].sum() / (ntot + _EPS)
    m["rollout_rs_seq_masked_fraction"] = float((S[:, FINAL_MASKED] > 0).mean())
    return {k: float(v) for k, v in m.items()}


def _is_metrics(S, rollout_is, upper, lower, icepop):
    n = S[:, N]
    ntot = n.sum()
    lower_m = (1.0 / upper) if lower is None else lower
    m = {}
    m["rollout_is_mean"] = S[:, SUM_W].sum() / (ntot + _EPS)
    if rollout_is == "sequence":
        total = S[:, SUM_LR]
        m["rollout_is_max"] = math.exp(min(total.max(), 20.0))
        m["rollout_is_min"] = math.exp(total.min())
        m["rollout_is_ratio_fraction_high"] = float((total > float(np.log(np.float32(upper)))).mean())
        m["rollout_is_ratio_fraction_low"] = float((total < float(np.log(np.float32(lower_m)))).mean())
    else:
        valid = n > 0
        m["rollout_is_ratio_fraction_high"] = S[:, CNT_RAW_HI].sum() / (ntot + _EPS)
        m["rollout_is_ratio_fraction_low"] = S[:, CNT_RAW_LO].sum() / (ntot + _EPS)
        m["rollout_is_max"] = S[:, MAX_W][valid].max()
        m["rollout_is_min"] = S[:, MIN_W][valid].min()
    mean_c = S[:, SUM_WC].sum() / (ntot + _EPS)
    mean_c2 = S[:, SUM_WC2].sum() / (ntot + _EPS)
    m["rollout_is_std"] = math.sqrt(max(mean_c2 - mean_c**2, 0.0)) if ntot > 1 else 0.0
    m["rollout_is_eff_sample_size"] = 1.0 / (mean_c2 / (mean_c + _EPS) ** 2)
    sm = S[:, SUM_W] / (n + _EPS)
    m["rollout_is_seq_mean"] = float(sm.mean())
    m["rollout_is_seq_std"] = _std_unbiased(sm)
    m["rollout_is_seq_max"] = float(sm.max())
    m["rollout_is_seq_min"] = float(sm.min())
    m["rollout_is_seq_max_deviation"] = float(np.abs(sm - 1.0).max())
    raw_sm = S[:, SUM_WRAW] / (n + _EPS)
    m["rollout_is_seq_fraction_high"] = float((raw_sm > upper).mean())
    m["rollout_is_seq_fraction_low"] = float((raw_sm < lower_m).mean())
    if icepop:
        m["rollout_is_oob_ratio"] = S[:, CNT_OOB].sum() / (ntot + _EPS)
    return {k: float(v) for k, v in m.items()}


def _offpolicy_metrics(S, with_rollout=True):
    n = S[:, N]
    ntot = n.sum()
    mean_train = S[:, SUM_OLD] / (n + _EPS)
    m = {"training_ppl": float(np.exp(-mean_train).mean()), "training_log_ppl": float((-mean_train).mean())}
    if not with_rollout:
        return m
    m["kl"] = -S[:, SUM_LR].sum() / (ntot + _EPS)
    m["k3_kl"] = S[:, SUM_K3RAW].sum() / (ntot + _EPS)
    mean_roll = S[:, SUM_ROLL] / (n + _EPS)
    m["rollout_ppl"] = float(np.exp(-mean_roll).mean())
    m["rollout_log_ppl"] = float((-mean_roll).mean())
    diff = mean_roll - mean_train
    m["log_ppl_diff"] = float(diff.mean())
    m["log_ppl_abs_diff"] = float(np.abs(diff).mean())
    m["log_ppl_diff_max"] = float(diff.max())
    m["log_ppl_diff_min"] = float(diff.min())
    m["ppl_ratio"] = float(np.exp(diff).mean())
    m["chi2_token"] = S[:, SUM_RHO2].sum() / (ntot + _EPS) - 1.0
    m["chi2_seq"] = float(np.exp(2.0 * np.clip(S[:, SUM_LR], -20.0, 20.0)).mean() - 1.0)
    return {k: float(v) for k, v in m.items()}


def _require_valid(S):
    if S[:, N].sum() <= 0:
        raise ValueError("response_mask must contain at least one valid token (1).")


def _apply_keep(response_mask, keep):
    return (response_mask * keep.to(response_mask.dtype)).to(response_mask.dtype)


def _batch_normalize(weights, S, rollout_is, metrics):
    n = S[:, N]
    if rollout_is == "token":
        mean_w = S[:, SUM_W].sum() / (n.sum() + _EPS)
    else:
        valid = n > 0
        mean_w = ((S[:, SUM_W] / (n + _EPS)) * valid).sum() / max(float(valid.sum()), _EPS)
    if mean_w > 1e-8:
        weights = weights / float(mean_w)
        metrics["rollout_is_batch_norm_factor"] = float(mean_w)
    else:
        metrics["rollout_is_batch_norm_factor"] = 1.0
    return weights


# ---- the reference's four functions -------------------------------------------------------------------------------

def compute_rollout_rejection_mask(log_ratio, response_mask, rollout_rs="token_k1", rollout_rs_threshold=None):
    """(modified_response_mask, metrics) — verl/trainer/ppo/rollout_corr_helper.py:197-413."""
    options = _normalize_rs_options(rollout_rs)
    if rollout_rs_threshold is None:
        raise ValueError("rollout_rs_threshold must be provided for rejection sampling.")
    if log_ratio.shape[0] == 0:
        return response_mask, {}
    bounds = _rs_bounds_as_compared(options, _parse_rs_thresholds(options, rollout_rs_threshold))
    lr = _f32_2d(log_ratio, "log_ratio")
    res = _launch(lr, torch.zeros_like(lr), _mask_u8(response_mask, lr.shape, lr.device), rs_bounds=bounds, want_keep=True)
    _require_valid(res.stats)
    return _apply_keep(response_mask, res.keep), _rs_metrics(res.stats, res.seq_bits, options, bounds)


def compute_rollout_correction_weights(log_ratio, response_mask, rollout_is="token", rollout_is_threshold=2.0,
                                       rollout_is_batch_normalize=False):
    """(rollout_is_weights, metrics) — verl/trainer/ppo/rollout_corr_helper.py:522-657."""
    if rollout_is not in ("token", "sequence"):
        raise ValueError(f"Invalid rollout_is: {rollout_is}. Must be one of {{'token', 'sequence'}}.")
    upper, lower = _parse_is_threshold(rollout_is_threshold)
    lr = _f32_2d(log_ratio, "log_ratio")
    res = _launch(lr, torch.zeros_like(lr), _mask_u8(response_mask, lr.shape, lr.device),
                  is_mode=1 if rollout_is == "token" else 2, icepop=lower is not None, is_upper=upper,
                  is_lower=0.0 if lower is None else lower, is_lower_metric=(1.0 / upper) if lower is None else lower,
                  want_weights=True)
    _require_valid(res.stats)
    metrics = _is_metrics(res.stats, rollout_is, upper, lower, lower is not None)
    weights = res.weights
    if rollout_is_batch_normalize:
        weights = _batch_normalize(weights, res.stats, rollout_is, metrics)
    return weights, metrics


def compute_offpolicy_metrics(old_log_prob, rollout_log_prob, response_mask):
    """KL / perplexity / chi-square diagnostics — verl/trainer/ppo/rollout_corr_helper.py:904-1010."""
    old = _f32_2d(old_log_prob, "old_log_prob")
    roll = old if rollout_log_prob is None else _f32_2d(rollout_log_prob, "rollout_log_prob", old.shape)
    res = _launch(old, roll, _mask_u8(response_mask, old.shape, old.device))
    assert res.stats[:, N].sum() > 0, "Expected at least one valid token in response_mask"
    return _offpolicy_metrics(res.stats, rollout_log_prob is not None)


def compute_rollout_correction_and_rejection_mask(old_log_prob, rollout_log_prob, response_mask,
                                                  rollout_is: Optional[str] = None, rollout_is_threshold=2.0,
                                                  rollout_is_batch_normalize: bool = False,
                                                  rollout_rs: Optional[str] = None, rollout_rs_threshold=None):
    """(rollout_is_weights | None, modified_response_mask, metrics with the ``rollout_corr/`` prefix) —
    verl/trainer/ppo/rollout_corr_helper.py:786-901. The weights come back as a tensor; the reference wraps the
    same tensor in a DataProto under the key ``rollout_is_weights``. One kernel launch serves all three parts."""
    if old_log_prob.shape != rollout_log_prob.shape:
        raise ValueError(f"old_log_prob shape {old_log_prob.shape} does not match rollout_log_prob shape {rollout_log_prob.shape}.")
    if old_log_prob.shape != response_mask.shape:
        raise ValueError(f"log_prob shape {old_log_prob.shape} does not match response_mask shape {response_mask.shape}.")
    use_is = rollout_is is not None and rollout_is_threshold is not None
    upper = lower = None
    if use_is:
        if rollout_is not in ("token", "sequence"):
            raise ValueError(f"Invalid rollout_is: {rollout_is}. Must be one of {{'token', 'sequence'}}.")
        upper, lower = _parse_is_threshold(rollout_is_threshold)
    options, bounds = [], None
    if rollout_rs is not None:
        if rollout_rs_threshold is None:
            raise ValueError("rollout_rs_threshold must be explicitly provided when rollout_rs is enabled. "
                             "Set rollout_rs_threshold to the desired threshold value.")
        options = _normalize_rs_options(rollout_rs)
        bounds = _rs_bounds_as_compared(options, _parse_rs_thresholds(options, rollout_rs_threshold))
    old = _f32_2d(old_log_prob, "old_log_prob")
    roll = _f32_2d(rollout_log_prob, "rollout_log_prob", old.shape)
    res = _launch(old, roll, _mask_u8(response_mask, old.shape, old.device),
                  is_mode=0 if not use_is else (1 if rollout_is == "token" else 2), icepop=lower is not None,
                  is_upper=upper or 1.0, is_lower=lower or 0.0,
                  is_lower_metric=0.0 if not use_is else ((1.0 / upper) if lower is None else lower),
                  rs_bounds=bounds, want_weights=use_is, want_keep=bool(options))
    _require_valid(res.stats)
    metrics = {}
    weights = None
    if use_is:
        metrics.update(_is_metrics(res.stats, rollout_is, upper, lower, lower is not None))
        weights = res.weights
        if rollout_is_batch_normalize:
            weights = _batch_normalize(weights, res.stats, rollout_is, metrics)
    new_mask = response_mask.clone()
    if options:
        new_mask = _apply_keep(response_mask, res.keep)
        metrics.update(_rs_metrics(res.stats, res.seq_bits, options, bounds))
    metrics.update(_offpolicy_metrics(res.stats, True))
    return weights, new_mask, {f"rollout_corr/{k}": v for k, v in metrics.items()}
