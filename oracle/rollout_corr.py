"""TEST INFRASTRUCTURE — CPU restatement of verl's rollout-correction step (masks, IS weights, metrics).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this. Nothing under
verl_amd/ does.

Restates, with plain torch ops on (B, T) tensors, what verl/trainer/ppo/rollout_corr_helper.py computes:
  parse_is_threshold            :92-131   _parse_rollout_is_threshold
  parse_rs_thresholds           :134-194  _parse_rollout_rs_thresholds
  rejection_mask                :197-413  compute_rollout_rejection_mask
  rs_metrics                    :416-519  compute_rs_metrics
  correction_weights            :522-657  compute_rollout_correction_weights
  is_metrics                    :660-783  compute_is_metrics
  correction_and_rejection_mask :786-901  compute_rollout_correction_and_rejection_mask (weights returned as a
                                          tensor, not wrapped in a DataProto)
  offpolicy_metrics             :904-1010 compute_offpolicy_metrics
masked_sum / masked_mean are verl/utils/torch_functional.py:273-308.

Pinned by the reference's own exact-value tests (tests/trainer/ppo/test_rollout_corr.py:312-366 mask mode,
:369-394 IcePop, :416-442 raw-weight sequence fraction, :127-166 one run per option) restated in
tests/test_oracle_rollout_corr.py, plus closed forms (log_ratio = 0 gives weights 1, KL 0, chi2 0).
"""

from __future__ import annotations

import math
from typing import Optional

import torch

SAFETY_BOUND = 20.0  # rollout_corr_helper.py:75
RS_OPTIONS = ("token_k1", "token_k2", "token_k3", "seq_sum_k1", "seq_sum_k2", "seq_sum_k3",
              "seq_mean_k1", "seq_mean_k2", "seq_mean_k3", "seq_max_k2", "seq_max_k3")
TOKEN_OPTIONS = ("token_k1", "token_k2", "token_k3")


def masked_sum(values, mask, axis=None):
    kept = torch.where(mask.bool(), values, torch.zeros((), dtype=values.dtype, device=values.device))
    return (kept * mask).sum(axis=axis)


def masked_mean(values, mask, axis=None):
    return masked_sum(values, mask, axis) / (mask.sum(axis=axis) + 1e-8)


def parse_is_threshold(spec):
    if isinstance(spec, bool):
        raise TypeError("rollout_is_threshold must not be a boolean")
    if isinstance(spec, (int, float)):
        upper, lower = float(spec), None
    elif isinstance(spec, str):
        text = spec.strip()
        if not text:
            raise ValueError("rollout_is_threshold must not be empty")
        try:
            if "_" in text:
                lo, up = text.split("_", 1)
                lower, upper = float(lo), float(up)
            else:
                upper, lower = float(text), None
        except ValueError as exc:
            raise ValueError(f"Invalid rollout_is_threshold '{spec}'.") from exc
    else:
        raise TypeError("rollout_is_threshold must be a float or a string")
    if upper <= 0:
        raise ValueError("rollout_is_threshold upper bound must be positive")
    if lower is not None:
        if lower <= 0:
            raise ValueError("rollout_is_threshold lower bound must be positive")
        if lower > upper:
            raise ValueError("rollout_is_threshold lower bound must be <= upper bound")
    return upper, lower


def normalize_rs_options(rollout_rs):
    if rollout_rs is None or not isinstance(rollout_rs, str):
        raise ValueError("rollout_rs must be a non-empty string")
    out = []
    for opt in (o.strip() for o in rollout_rs.split(",")):
        if not opt:
            continue
        if opt not in RS_OPTIONS:
            raise ValueError(f"Invalid rollout_rs option: {opt}")
        if opt not in out:
            out.append(opt)
    if not out:
        raise ValueError("rollout_rs must contain at least one valid option")
    return out


def parse_rs_thresholds(options, spec):
    if spec is None:
        raise ValueError("rollout_rs_threshold must be provided for rejection sampling.")
    if isinstance(spec, (int, float)):
        parts = [str(spec)]
    elif isinstance(spec, str):
        parts = [p.strip() for p in spec.split(",") if p.strip()]
    else:
        raise TypeError("rollout_rs_threshold must be a string or a number")
    if not parts:
        raise ValueError("rollout_rs_threshold must contain at least one value")
    if len(parts) not in (1, len(options)):
        raise ValueError("rollout_rs_threshold needs one value, or one per option")
    if len(parts) == 1:
        parts = parts * len(options)
    out = {}
    for opt, text in zip(options, parts):
        if opt.endswith("k1"):
            lo_s, up_s = text.split("_", 1) if "_" in text else (str(1.0 / float(text)), text)
            try:
                lower, upper = float(lo_s), float(up_s)
            except ValueError as exc:
                raise ValueError(f"Invalid numeric threshold '{text}' for option '{opt}'.") from exc
            if lower <= 0 or upper <= 0:
                raise ValueError(f"Thresholds for option '{opt}' must be positive")
            if lower > upper:
                raise ValueError(f"Thresholds for option '{opt}' must be lower <= upper")
            out[opt] = {"lower": lower, "upper": upper}
        else:
            if "_" in text:
                raise ValueError(f"rollout_rs_threshold for option '{opt}' must be a single upper bound")
            try:
                upper = float(text)
            except ValueError as exc:
                raise ValueError(f"Invalid numeric threshold '{text}' for option '{opt}'.") from exc
            if upper <= 0:
                raise ValueError(f"Threshold for option '{opt}' must be positive")
            out[opt] = {"lower": None, "upper": upper}
    return out


def rs_metrics(option, stat, response_mask, seq_valid, *, level, per_sequence, upper, lower, apply_lower):
    if not response_mask.any():
        raise ValueError("response_mask must contain at least one valid token (1).")
    m = {}
    pre = f"rollout_rs_{option}"
    mb = response_mask.bool()
    seq_values = per_sequence if per_sequence is not None else masked_mean(stat, response_mask, axis=-1)
    if seq_values.dim() > 1:
        seq_values = seq_values.squeeze(-1)
    sv = seq_values[seq_valid]
    m[f"{pre}_mean"] = masked_mean(stat, response_mask).item()
    if level == "sequence" and sv.numel() > 0:
        m[f"{pre}_max"] = sv.max().item()
        m[f"{pre}_min"] = sv.min().item()
        hi = (sv > upper).float().mean().item()
        lo = (sv < lower).float().mean().item() if apply_lower else 0.0
    else:
        m[f"{pre}_max"] = stat.masked_fill(~mb, float("-inf")).max().item()
        m[f"{pre}_min"] = stat.masked_fill(~mb, float("inf")).min().item()
        hi = masked_mean((stat > upper).float(), response_mask).item()
        lo = masked_mean((stat < lower).float(), response_mask).item() if apply_lower else 0.0
    m[f"{pre}_fraction_high"] = hi
    m[f"{pre}_fraction_low"] = lo
    if response_mask.sum() > 1:
        clamped = stat.clamp(min=lower if apply_lower else 0.0, max=upper)
        mean_c = masked_mean(clamped, response_mask)
        var = masked_mean(clamped.square(), response_mask) - mean_c.square()
        m[f"{pre}_std"] = torch.sqrt(torch.clamp(var, min=0.0)).item()
    else:
        m[f"{pre}_std"] = 0.0
    if sv.numel() > 0:
        m[f"{pre}_seq_mean"] = sv.mean().item()
        m[f"{pre}_seq_std"] = sv.std().item() if sv.numel() > 1 else 0.0
        m[f"{pre}_seq_max"] = sv.max().item()
        m[f"{pre}_seq_min"] = sv.min().item()
        m[f"{pre}_seq_max_deviation"] = sv.abs().max().item()
        m[f"{pre}_seq_fraction_high"] = (sv > upper).float().mean().item()
        if apply_lower:
            m[f"{pre}_seq_fraction_low"] = (sv < lower).float().mean().item()
    else:
        for k in ("seq_mean", "seq_std", "seq_max", "seq_min", "seq_max_deviation", "seq_fraction_high", "seq_fraction_low"):
            m[f"{pre}_{k}"] = 0.0
    return m


def rejection_mask(log_ratio, response_mask, rollout_rs="token_k1", rollout_rs_threshold=None):
    options = normalize_rs_options(rollout_rs)
    if rollout_rs_threshold is None:
        raise ValueError("rollout_rs_threshold must be provided for rejection sampling.")
    if log_ratio.shape[0] == 0:
        return response_mask, {}
    specs = parse_rs_thresholds(options, rollout_rs_threshold)
    lr = torch.clamp(log_ratio, min=-SAFETY_BOUND, max=SAFETY_BOUND)
    k = {"k1": -lr, "k2": 0.5 * lr**2, "k3": torch.exp(lr) - 1.0 - lr}
    mb = response_mask.bool()
    seq_valid = response_mask.sum(dim=-1) > 0
    combined = torch.ones_like(response_mask, dtype=log_ratio.dtype)
    metrics = {}

    def seq_max(v):
        filled = v.masked_fill(~mb, float("-inf")).max(dim=-1).values
        return torch.where(filled == float("-inf"), torch.zeros_like(filled), filled)

    for opt in options:
        kind = opt[-2:]
        is_k1 = kind == "k1"
        upper, lower = specs[opt]["upper"], specs[opt]["lower"]
        lo_t = math.log(lower) if is_k1 else None
        up_t = math.log(upper) if is_k1 else upper
        per_seq = None
        if opt in TOKEN_OPTIONS:
            stat = k[kind]
            keep = (stat >= lo_t) & (stat <= up_t) if is_k1 else stat <= up_t
            level = "token"
        else:
            if opt.startswith("seq_sum"):
                s = masked_sum(k[kind], response_mask, axis=-1)
            elif opt.startswith("seq_mean"):
                s = masked_mean(k[kind], response_mask, axis=-1)
            else:
                s = seq_max(k[kind])
            keep_seq = (s >= lo_t) & (s <= up_t) if is_k1 else s <= up_t
            per_seq = s
            keep = keep_seq.unsqueeze(-1).expand_as(mb)
            stat = s.unsqueeze(-1).expand_as(response_mask)
            level = "sequence"
        keep_f = keep.to(log_ratio.dtype)
        combined = combined * keep_f
        seq_keep = (~((~keep) & mb)).all(dim=-1)
        metrics.update(rs_metrics(opt, stat, response_mask, seq_valid, level=level, per_sequence=per_seq,
                                  upper=up_t, lower=lo_t if is_k1 else 0.0, apply_lower=is_k1))
        metrics[f"rollout_rs_{opt}_masked_fraction"] = masked_mean(1 - keep_f, response_mask).item()
        sv = seq_valid.float()
        metrics[f"rollout_rs_{opt}_seq_masked_fraction"] = (
            (((1.0 - seq_keep.to(log_ratio.dtype)) * sv).sum() / sv.sum()).item() if sv.sum() > 0 else 0.0)
    metrics["rollout_rs_masked_fraction"] = masked_mean(1 - combined, response_mask).item()
    final_keep = (combined > 0.5) & mb
    metrics["rollout_rs_seq_masked_fraction"] = (~final_keep & mb).any(dim=-1).float().mean().item()
    return (response_mask * combined).to(response_mask.dtype), metrics


def is_metrics(weights, raw, log_ratio_for_metrics, response_mask, rollout_is, upper, lower=None):
    if not response_mask.any():
        raise ValueError("response_mask must contain at least one valid token (1).")
    m = {}
    lower = 1.0 / upper if lower is None else lower
    log_up = torch.log(torch.tensor(upper, device=weights.device))
    log_lo = torch.log(torch.tensor(lower, device=weights.device))
    if rollout_is == "sequence":
        m["rollout_is_max"] = torch.exp(torch.clamp(log_ratio_for_metrics.max(), max=SAFETY_BOUND)).item()
        m["rollout_is_min"] = torch.exp(log_ratio_for_metrics.min()).item()
        m["rollout_is_mean"] = masked_mean(weights, response_mask).item()
        m["rollout_is_ratio_fraction_high"] = (log_ratio_for_metrics > log_up).float().mean().item()
        m["rollout_is_ratio_fraction_low"] = (log_ratio_for_metrics < log_lo).float().mean().item()
    else:
        m["rollout_is_mean"] = masked_mean(weights, response_mask).item()
        m["rollout_is_ratio_fraction_high"] = masked_mean((raw > upper).float(), response_mask).item()
        m["rollout_is_ratio_fraction_low"] = masked_mean((raw < lower).float(), response_mask).item()
        mb = response_mask.bool()
        m["rollout_is_max"] = weights.masked_fill(~mb, float("-inf")).max().item()
        m["rollout_is_min"] = weights.masked_fill(~mb, float("inf")).min().item()
    clamped = weights.clamp(min=0.0, max=upper)
    if response_mask.sum() > 1:
        mean_c = masked_mean(clamped, response_mask)
        var = masked_mean(clamped.square(), response_mask) - mean_c.square()
        m["rollout_is_std"] = torch.sqrt(torch.clamp(var, min=0.0)).item()
    else:
        m["rollout_is_std"] = 0.0
    normed = clamped / (masked_mean(clamped, response_mask) + 1e-8)
    m["rollout_is_eff_sample_size"] = 1.0 / masked_mean(normed.square(), response_mask).item()
    if weights.dim() > 1:
        sm = masked_mean(weights, response_mask, axis=-1)
        m["rollout_is_seq_mean"] = sm.mean().item()
        m["rollout_is_seq_std"] = sm.std().item() if sm.numel() > 1 else 0.0
        m["rollout_is_seq_max"] = sm.max().item()
        m["rollout_is_seq_min"] = sm.min().item()
        m["rollout_is_seq_max_deviation"] = (sm - 1.0).abs().max().item()
        raw_sm = masked_mean(raw, response_mask, axis=-1)
        m["rollout_is_seq_fraction_high"] = (raw_sm > upper).float().mean().item()
        m["rollout_is_seq_fraction_low"] = (raw_sm < lower).float().mean().item()
    return m


def correction_weights(log_ratio, response_mask, rollout_is="token", rollout_is_threshold=2.0,
                       rollout_is_batch_normalize=False):
    if rollout_is not in ("token", "sequence"):
        raise ValueError(f"Invalid rollout_is: {rollout_is}")
    upper, lower = parse_is_threshold(rollout_is_threshold)
    if rollout_is == "token":
        for_metrics = log_ratio
        raw = torch.exp(torch.clamp(log_ratio, min=-SAFETY_BOUND, max=SAFETY_BOUND))
    else:
        total = masked_sum(log_ratio, response_mask, axis=-1).unsqueeze(-1)
        for_metrics = total
        raw = torch.exp(torch.clamp(total, min=-SAFETY_BOUND, max=SAFETY_BOUND)).expand_as(log_ratio)
    raw = raw * response_mask
    if lower is None:
        weights = raw.clamp(max=upper)
    else:
        weights = torch.where((raw >= lower) & (raw <= upper), raw, torch.zeros_like(raw))
    metrics = is_metrics(weights, raw, for_metrics, response_mask, rollout_is, upper, lower)
    if lower is not None:
        metrics["rollout_is_oob_ratio"] = masked_mean(((raw < lower) | (raw > upper)).float(), response_mask).item()
    weights = weights.detach()
    if rollout_is_batch_normalize:
        if rollout_is == "token":
            mean_w = masked_mean(weights, response_mask)
        else:
            sw = masked_mean(weights, response_mask, axis=-1)
            sm = (response_mask.sum(dim=-1) > 0).to(weights.dtype)
            mean_w = (sw * sm).sum() / sm.sum().clamp_min(1e-8)
        if mean_w > 1e-8:
            weights = weights / mean_w
            metrics["rollout_is_batch_norm_factor"] = mean_w.item()
        else:
            metrics["rollout_is_batch_norm_factor"] = 1.0
    return weights, metrics


def offpolicy_metrics(old_log_prob, rollout_log_prob, response_mask):
    assert response_mask.any()
    m = {}
    mean_train = masked_mean(old_log_prob, response_mask, axis=-1)
    m["training_ppl"] = torch.exp(-mean_train).mean().item()
    m["training_log_ppl"] = (-mean_train).mean().item()
    if rollout_log_prob is None:
        return m
    m["kl"] = masked_mean(rollout_log_prob - old_log_prob, response_mask).item()
    lr = old_log_prob - rollout_log_prob
    m["k3_kl"] = masked_mean(torch.exp(lr) - lr - 1, response_mask).item()
    mean_roll = masked_mean(rollout_log_prob, response_mask, axis=-1)
    m["rollout_ppl"] = torch.exp(-mean_roll).mean().item()
    m["rollout_log_ppl"] = (-mean_roll).mean().item()
    diff = mean_roll - mean_train
    m["log_ppl_diff"] = diff.mean().item()
    m["log_ppl_abs_diff"] = diff.abs().mean().item()
    m["log_ppl_diff_max"] = diff.max().item()
    m["log_ppl_diff_min"] = diff.min().item()
    m["ppl_ratio"] = torch.exp(diff).mean().item()
    rho = torch.exp(torch.clamp(lr, min=-SAFETY_BOUND, max=SAFETY_BOUND))
    m["chi2_token"] = (masked_mean(rho.square(), response_mask) - 1.0).item()
    total = torch.clamp(masked_sum(lr, response_mask, axis=-1), min=-SAFETY_BOUND, max=SAFETY_BOUND)
    m["chi2_seq"] = (torch.exp(2.0 * total).mean() - 1.0).item()
    return m


def correction_and_rejection_mask(old_log_prob, rollout_log_prob, response_mask, rollout_is: Optional[str] = None,
                                  rollout_is_threshold=2.0, rollout_is_batch_normalize=False,
                                  rollout_rs: Optional[str] = None, rollout_rs_threshold=None):
    if not response_mask.any():
        raise ValueError("response_mask must contain at least one valid token (1).")
    if old_log_prob.shape != rollout_log_prob.shape or old_log_prob.shape != response_mask.shape:
        raise ValueError("shape mismatch between log-probs and response_mask")
    lr = old_log_prob - rollout_log_prob
    metrics = {}
    weights = None
    if rollout_is is not None and rollout_is_threshold is not None:
        weights, im = correction_weights(lr, response_mask, rollout_is, rollout_is_threshold, rollout_is_batch_normalize)
        metrics.update(im)
    new_mask = response_mask.clone()
    if rollout_rs is not None:
        if rollout_rs_threshold is None:
            raise ValueError("rollout_rs_threshold must be explicitly provided when rollout_rs is enabled.")
        new_mask, rm = rejection_mask(lr, response_mask, rollout_rs, rollout_rs_threshold)
        metrics.update(rm)
    metrics.update(offpolicy_metrics(old_log_prob, rollout_log_prob, response_mask))
    return weights, new_mask, {f"rollout_corr/{k}": v for k, v in metrics.items()}
