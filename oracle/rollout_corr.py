"""Oracle for the rollout-correction weights and the off-policy diagnostics (CPU torch).

Test infrastructure only; see ``oracle/__init__.py``.
"""

from __future__ import annotations

import math

import torch

from .masked import masked_mean, masked_sum

SAFETY_BOUND = 20.0  # verl/trainer/ppo/rollout_corr_helper.py:75


@torch.no_grad()
def offpolicy_metrics(old_log_prob, rollout_log_prob, response_mask):
    """compute_offpolicy_metrics, verl/trainer/ppo/rollout_corr_helper.py:835-937: perplexities of the two
    policies per sequence, the k1 / k3 estimates of KL(rollout || training), and the chi-square divergences
    at token and sequence level."""
    assert response_mask.any(), "Expected at least one valid token in response_mask"
    out = {}
    train = masked_mean(old_log_prob, response_mask, axis=-1)
    out["training_ppl"] = torch.exp(-train).mean().item()
    out["training_log_ppl"] = (-train).mean().item()
    if rollout_log_prob is None:
        return out
    d = old_log_prob - rollout_log_prob
    out["kl"] = masked_mean(rollout_log_prob - old_log_prob, response_mask).item()
    out["k3_kl"] = masked_mean(torch.exp(d) - d - 1, response_mask).item()
    roll = masked_mean(rollout_log_prob, response_mask, axis=-1)
    out["rollout_ppl"] = torch.exp(-roll).mean().item()
    out["rollout_log_ppl"] = (-roll).mean().item()
    gap = roll - train
    out["log_ppl_diff"] = gap.mean().item()
    out["log_ppl_abs_diff"] = gap.abs().mean().item()
    out["log_ppl_diff_max"] = gap.max().item()
    out["log_ppl_diff_min"] = gap.min().item()
    out["ppl_ratio"] = torch.exp(gap).mean().item()
    rho = torch.exp(d.clamp(-SAFETY_BOUND, SAFETY_BOUND))
    out["chi2_token"] = (masked_mean(rho.square(), response_mask) - 1.0).item()
    seq = masked_sum(d, response_mask, axis=-1).clamp(-SAFETY_BOUND, SAFETY_BOUND)
    out["chi2_seq"] = (torch.exp(2.0 * seq).mean() - 1.0).item()
    return out


@torch.no_grad()
def is_metrics(weights, log_ratio_for_metrics, response_mask, level, threshold):
    """compute_is_metrics, rollout_corr_helper.py:601-712, on the masked, not yet truncated weights."""
    if not response_mask.any():
        raise ValueError("response_mask must contain at least one valid token (1).")
    out = {}
    lower = 1.0 / threshold
    if level == "sequence":
        log_hi = torch.log(torch.tensor(threshold))
        log_lo = torch.log(torch.tensor(lower))
        out["rollout_is_max"] = torch.exp(log_ratio_for_metrics.max().clamp(max=SAFETY_BOUND)).item()
        out["rollout_is_min"] = torch.exp(log_ratio_for_metrics.min()).item()
        out["rollout_is_mean"] = masked_mean(weights, response_mask).item()
        out["rollout_is_ratio_fraction_high"] = (log_ratio_for_metrics > log_hi).float().mean().item()
        out["rollout_is_ratio_fraction_low"] = (log_ratio_for_metrics < log_lo).float().mean().item()
    else:
        out["rollout_is_mean"] = masked_mean(weights, response_mask).item()
        out["rollout_is_ratio_fraction_high"] = masked_mean((weights > threshold).float(), response_mask).item()
        out["rollout_is_ratio_fraction_low"] = masked_mean((weights < lower).float(), response_mask).item()
        valid = response_mask.bool()
        out["rollout_is_max"] = weights.masked_fill(~valid, float("-inf")).max().item()
        out["rollout_is_min"] = weights.masked_fill(~valid, float("inf")).min().item()
    clamped = weights.clamp(min=lower, max=threshold)
    mean_c = masked_mean(clamped, response_mask)
    if response_mask.sum() > 1:
        var = masked_mean(clamped.square(), response_mask) - mean_c.square()
        out["rollout_is_std"] = torch.sqrt(var.clamp(min=0.0)).item()
    else:
        out["rollout_is_std"] = 0.0
    out["rollout_is_eff_sample_size"] = 1.0 / masked_mean((clamped / (mean_c + 1e-8)).square(), response_mask).item()
    seq = masked_mean(weights, response_mask, axis=-1)
    out["rollout_is_seq_mean"] = seq.mean().item()
    out["rollout_is_seq_std"] = seq.std().item() if seq.numel() > 1 else 0.0
    out["rollout_is_seq_max"] = seq.max().item()
    out["rollout_is_seq_min"] = seq.min().item()
    out["rollout_is_seq_max_deviation"] = (seq - 1.0).abs().max().item()
    out["rollout_is_seq_fraction_high"] = (seq > threshold).float().mean().item()
    out["rollout_is_seq_fraction_low"] = (seq < lower).float().mean().item()
    return out


@torch.no_grad()
def rollout_correction_weights(log_ratio, response_mask, level="token", threshold=2.0, batch_normalize=False):
    """compute_rollout_correction_weights, rollout_corr_helper.py:481-598 (single process): importance weights
    ``exp(clamp(log_ratio))`` per token, or ``exp(clamp(sum of the row's log ratios))`` per sequence, times
    the mask; metrics from the untruncated weights; truncation at ``threshold``; optional division by the
    batch mean.  Returns ``(weights, metrics)``."""
    if level not in ("token", "sequence"):
        raise ValueError(f"Invalid rollout_is: {level}. Must be one of {{'token', 'sequence'}}.")
    if threshold <= 0:
        raise ValueError(f"rollout_is_threshold must be positive, got {threshold}.")
    if level == "token":
        for_metrics = log_ratio
        weights = torch.exp(log_ratio.clamp(-SAFETY_BOUND, SAFETY_BOUND))
    else:
        for_metrics = masked_sum(log_ratio, response_mask, axis=-1).unsqueeze(-1)
        weights = torch.exp(for_metrics.clamp(-SAFETY_BOUND, SAFETY_BOUND)).expand_as(log_ratio)
    weights = weights * response_mask
    metrics = is_metrics(weights, for_metrics, response_mask, level, threshold)
    weights = weights.clamp(max=threshold)
    if batch_normalize:
        if level == "token":
            mean = masked_mean(weights, response_mask)
        else:
            per_seq = masked_mean(weights, response_mask, axis=-1)
            alive = (response_mask.sum(dim=-1) > 0).to(weights.dtype)
            mean = (per_seq * alive).sum() / alive.sum().clamp_min(1e-8)
        if mean > 1e-8:
            weights = weights / mean
            metrics["rollout_is_batch_norm_factor"] = mean.item()
        else:
            metrics["rollout_is_batch_norm_factor"] = 1.0
    return weights, metrics


def rollout_correction_brute_force_fp64(old, roll, mask, level, threshold):
    """Scalar double-precision loops from the definitions (importance ratio, truncation, effective sample size
    ``(sum c)^2 / (n sum c^2)``, chi-square ``E[rho^2] - 1``, perplexity ``exp(-mean log p)``): a subset of the
    metrics above plus the truncated weights, to pin them."""
    B, L = len(old), len(old[0])
    bound = lambda x: max(-SAFETY_BOUND, min(SAFETY_BOUND, x))  # noqa: E731
    w = [[0.0] * L for _ in range(B)]
    n = 0
    tot = {"kl": 0.0, "k3": 0.0, "rho2": 0.0, "c": 0.0, "c2": 0.0, "w": 0.0}
    seq = {"train_ppl": 0.0, "roll_ppl": 0.0, "ratio": 0.0, "rho2": 0.0}
    lower = 1.0 / threshold
    for i in range(B):
        toks = [t for t in range(L) if mask[i][t] != 0]
        dsum = sum(old[i][t] - roll[i][t] for t in toks)
        for t in toks:
            d = old[i][t] - roll[i][t]
            wi = math.exp(bound(d)) if level == "token" else math.exp(bound(dsum))
            w[i][t] = min(wi, threshold)
            c = min(max(wi, lower), threshold)
            n += 1
            tot["kl"] -= d
            tot["k3"] += math.exp(d) - d - 1
            tot["rho2"] += math.exp(bound(d)) ** 2
            tot["c"] += c
            tot["c2"] += c * c
            tot["w"] += wi
        k = max(len(toks), 1e-8)
        mt = sum(old[i][t] for t in toks) / k
        mr = sum(roll[i][t] for t in toks) / k
        seq["train_ppl"] += math.exp(-mt) / B
        seq["roll_ppl"] += math.exp(-mr) / B
        seq["ratio"] += math.exp(mr - mt) / B
        seq["rho2"] += math.exp(2 * bound(dsum)) / B
    metrics = {"kl": tot["kl"] / n, "k3_kl": tot["k3"] / n, "chi2_token": tot["rho2"] / n - 1,
               "chi2_seq": seq["rho2"] - 1, "training_ppl": seq["train_ppl"], "rollout_ppl": seq["roll_ppl"],
               "ppl_ratio": seq["ratio"], "rollout_is_mean": tot["w"] / n,
               "rollout_is_eff_sample_size": tot["c"] ** 2 / (n * tot["c2"]),
               "rollout_is_std": math.sqrt(max(tot["c2"] / n - (tot["c"] / n) ** 2, 0.0))}
    return w, metrics


# ---- rejection sampling (hard trust region) -----------------------------------------------------------------
RS_OPTIONS = ("token_k1", "token_k2", "token_k3", "seq_sum_k1", "seq_sum_k2", "seq_sum_k3", "seq_mean_k1",
              "seq_mean_k2", "seq_mean_k3", "seq_max_k2", "seq_max_k3")  # rollout_corr_helper.py:77-89


def parse_rs_thresholds(options, spec):
    """_parse_rollout_rs_thresholds, rollout_corr_helper.py:94-160: one threshold for all options or one per option;
    a k1 option takes ``lower_upper`` (or ``upper`` alone, lower = 1 / upper), the others a single upper bound.
    Returns ``{option: (lower or None, upper)}``."""
    if spec is None:
        raise ValueError("rollout_rs_threshold must be provided for rejection sampling.")
    if isinstance(spec, (int, float)):
        parts = [str(spec)]
    elif isinstance(spec, str):
        parts = [p.strip() for p in spec.split(",") if p.strip()]
    else:
        raise TypeError("rollout_rs_threshold must be a string or numeric value specifying per-option thresholds.")
    if not parts:
        raise ValueError("rollout_rs_threshold must contain at least one threshold value.")
    if len(parts) not in (1, len(options)):
        raise ValueError("rollout_rs_threshold expects either one threshold shared by all options or exactly "
                         f"{len(options)} thresholds to match the provided rollout_rs options.")
    if len(parts) == 1:
        parts = parts * len(options)
    out = {}
    for option, part in zip(options, parts):
        try:
            if option.endswith("k1"):
                lo, hi = part.split("_", 1) if "_" in part else (str(1.0 / float(part)), part)
                lo, hi = float(lo), float(hi)
            else:
                if "_" in part:
                    raise ValueError(f"rollout_rs_threshold for option '{option}' must provide a single upper bound "
                                     f"without '_'. Received '{part}'.")
                lo, hi = None, float(part)
        except ValueError as exc:
            if "single upper bound" in str(exc):
                raise
            raise ValueError(f"Invalid numeric threshold '{part}' for option '{option}'.") from exc
        if hi <= 0 or (lo is not None and lo <= 0):
            raise ValueError(f"Thresholds for option '{option}' must be positive, got {part}.")
        out[option] = (lo, hi)
    return out


@torch.no_grad()
def rs_metrics(option, stat, response_mask, seq_valid, level, per_sequence, upper, lower, apply_lower):
    """compute_rs_metrics, rollout_corr_helper.py:360-478."""
    if not response_mask.any():
        raise ValueError("response_mask must contain at least one valid token (1).")
    p = f"rollout_rs_{option}"
    out = {}
    valid = response_mask.bool()
    seq = per_sequence if per_sequence is not None else masked_mean(stat, response_mask, axis=-1)
    seq = seq[seq_valid]
    by_sequence = level == "sequence" and seq.numel() > 0
    out[f"{p}_mean"] = masked_mean(stat, response_mask).item()
    if by_sequence:
        out[f"{p}_max"], out[f"{p}_min"] = seq.max().item(), seq.min().item()
        out[f"{p}_fraction_high"] = (seq > upper).float().mean().item()
        out[f"{p}_fraction_low"] = (seq < lower).float().mean().item() if apply_lower else 0.0
    else:
        out[f"{p}_max"] = stat.masked_fill(~valid, float("-inf")).max().item()
        out[f"{p}_min"] = stat.masked_fill(~valid, float("inf")).min().item()
        out[f"{p}_fraction_high"] = masked_mean((stat > upper).float(), response_mask).item()
        out[f"{p}_fraction_low"] = masked_mean((stat < lower).float(), response_mask).item() if apply_lower else 0.0
    if response_mask.sum() > 1:
        c = stat.clamp(min=lower if apply_lower else 0.0, max=upper)
        var = masked_mean(c.square(), response_mask) - masked_mean(c, response_mask).square()
        out[f"{p}_std"] = torch.sqrt(var.clamp(min=0.0)).item()
    else:
        out[f"{p}_std"] = 0.0
    if seq.numel() > 0:
        out[f"{p}_seq_mean"] = seq.mean().item()
        out[f"{p}_seq_std"] = seq.std().item() if seq.numel() > 1 else 0.0
        out[f"{p}_seq_max"] = seq.max().item()
        out[f"{p}_seq_min"] = seq.min().item()
        out[f"{p}_seq_max_deviation"] = seq.abs().max().item()
        out[f"{p}_seq_fraction_high"] = (seq > upper).float().mean().item()
        if apply_lower:
            out[f"{p}_seq_fraction_low"] = (seq < lower).float().mean().item()
    else:
        for key in ("mean", "std", "max", "min", "max_deviation", "fraction_high", "fraction_low"):
            out[f"{p}_seq_{key}"] = 0.0
    return out


@torch.no_grad()
def rollout_rejection_mask(log_ratio, response_mask, rollout_rs="token_k1", rollout_rs_threshold=None):
    """compute_rollout_rejection_mask, rollout_corr_helper.py:163-357: every requested option keeps a token (token
    level) or a whole sequence (sum / mean / max of the token statistic) whose divergence estimate lies inside its
    bounds; the masks multiply.  k1 = -log ratio with bounds ``[log lower, log upper]``, k2 = half the squared log
    ratio, k3 = exp(r) - 1 - r, each with an upper bound; the log ratio is clamped to +-20 first.  Returns
    ``(modified_response_mask, metrics)``."""
    if rollout_rs is None or not isinstance(rollout_rs, str):
        raise ValueError("rollout_rs must be a non-empty string (comma separated for multiple options).")
    if rollout_rs_threshold is None:
        raise ValueError("rollout_rs_threshold must be provided for rejection sampling.")
    if log_ratio.shape[0] == 0:
        return response_mask, {}
    options = []
    for opt in (o.strip() for o in rollout_rs.split(",")):
        if not opt:
            continue
        if opt not in RS_OPTIONS:
            raise ValueError(f"Invalid rollout_rs option: {opt}. Must be one of {sorted(RS_OPTIONS)}.")
        if opt not in options:
            options.append(opt)
    if not options:
        raise ValueError("rollout_rs must contain at least one valid option.")
    bounds = parse_rs_thresholds(options, rollout_rs_threshold)
    d = log_ratio.clamp(-SAFETY_BOUND, SAFETY_BOUND)
    token = {"k1": -d, "k2": 0.5 * d**2, "k3": torch.exp(d) - 1.0 - d}
    valid = response_mask.bool()
    seq_valid = response_mask.sum(dim=-1) > 0
    combined = torch.ones_like(response_mask, dtype=log_ratio.dtype)
    metrics = {}
    for opt in options:
        scope, est = opt.rsplit("_", 1)
        lower, upper = bounds[opt]
        stat = token[est]
        per_sequence = None
        if scope == "seq_sum":
            per_sequence = masked_sum(stat, response_mask, axis=-1)
        elif scope == "seq_mean":
            per_sequence = masked_mean(stat, response_mask, axis=-1)
        elif scope == "seq_max":
            top = stat.masked_fill(~valid, float("-inf")).max(dim=-1).values
            per_sequence = torch.where(top == float("-inf"), torch.zeros_like(top), top)
        if per_sequence is not None:
            stat = per_sequence.unsqueeze(-1).expand_as(response_mask)
        if est == "k1":
            lo, hi, apply_lower = math.log(lower), math.log(upper), True
            keep = (stat >= lo) & (stat <= hi)
        else:
            lo, hi, apply_lower = 0.0, upper, False
            keep = stat <= hi
        combined = combined * keep.to(log_ratio.dtype)
        seq_keep = (~((~keep) & valid)).all(dim=-1)
        metrics.update(rs_metrics(opt, stat, response_mask, seq_valid, "token" if scope == "token" else "sequence",
                                  per_sequence, hi, lo, apply_lower))
        metrics[f"rollout_rs_{opt}_masked_fraction"] = masked_mean(1 - keep.to(log_ratio.dtype), response_mask).item()
        alive = seq_valid.float()
        metrics[f"rollout_rs_{opt}_seq_masked_fraction"] = (
            (((1.0 - seq_keep.to(log_ratio.dtype)) * alive).sum() / alive.sum()).item() if alive.sum() > 0 else 0.0)
    metrics["rollout_rs_masked_fraction"] = masked_mean(1 - combined, response_mask).item()
    final_keep = (combined > 0.5) & valid
    metrics["rollout_rs_seq_masked_fraction"] = ((~final_keep) & valid).any(dim=-1).float().mean().item()
    return (response_mask * combined).to(response_mask.dtype), metrics
