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
