"""Oracle for the trainer-side callers of the path: the KL penalty on rewards and its controllers,
and the per-step data metrics (CPU torch).

Test infrastructure only; see ``oracle/__init__.py``.
"""

from __future__ import annotations

import numpy as np
import torch

from .losses import kl_penalty
from .masked import masked_mean, masked_sum


@torch.no_grad()
def apply_kl_penalty(token_level_scores, old_log_probs, ref_log_prob, response_mask, beta, kind="kl"):
    """verl/trainer/ppo/ray_trainer.py:86-101 without the DataProto plumbing: returns
    ``(token_level_rewards, current_kl)`` with ``current_kl`` a Python float."""
    kld = kl_penalty(old_log_probs, ref_log_prob, kind) * response_mask
    rewards = token_level_scores - beta * kld
    current_kl = torch.mean(masked_mean(kld, response_mask, axis=-1), dim=0).item()
    return rewards, current_kl


def adaptive_kl_update(value, current_kl, n_steps, target, horizon):
    """AdaptiveKLController.update, verl/trainer/ppo/core_algos.py:163-173: the coefficient is multiplied
    by ``1 + clip(kl / target - 1, -0.2, 0.2) * n_steps / horizon``."""
    return value * (1 + float(np.clip(current_kl / target - 1, -0.2, 0.2)) * n_steps / horizon)


def compute_rewards(token_level_scores, old_log_prob, ref_log_prob, kl_ratio):
    """verl/trainer/ppo/core_algos.py:1009-1022."""
    return token_level_scores - (old_log_prob - ref_log_prob) * kl_ratio


@torch.no_grad()
def compute_data_metrics(batch, use_critic=True):
    """verl/trainer/ppo/metric_utils.py:81-225 on a plain mapping of tensors (``batch[name]``); the
    optional multi-turn entries of ``non_tensor_batch`` (:212-223) are host numpy reductions and are
    left to the caller."""
    width = batch["responses"].shape[-1]
    attention = batch["attention_mask"]
    prompt_length = attention[:, :-width].sum(-1).float()           # _compute_response_info, :67-70
    response_length = attention[:, -width:].sum(-1).float()
    max_prompt_length = attention[:, :-width].size(-1)
    valid = batch["response_mask"].bool()
    alive = response_length != 0
    if int(alive.sum()) == 0:
        raise ValueError("All samples are aborted, this should not happen.")
    score = batch["token_level_scores"].sum(-1)[alive]
    reward = batch["token_level_rewards"].sum(-1)[alive]
    adv = batch["advantages"][valid]
    ret = batch["returns"][valid]

    def triple(prefix, x):
        return {f"{prefix}/mean": x.mean().item(), f"{prefix}/max": x.max().item(), f"{prefix}/min": x.min().item()}

    out = {}
    out.update(triple("critic/score", score))
    out.update(triple("critic/rewards", reward))
    out.update(triple("critic/advantages", adv))
    out.update(triple("critic/returns", ret))
    if use_critic:
        val = batch["values"][valid]
        out.update(triple("critic/values", val))
        out["critic/vf_explained_var"] = (1.0 - torch.var(ret - val) / (torch.var(ret) + 1e-5)).item()
    for prefix, x, cap in (("response_length", response_length, width),
                           ("response_length_non_aborted", response_length[alive], width),
                           ("prompt_length", prompt_length, max_prompt_length)):
        out.update(triple(prefix, x))
        out[f"{prefix}/clip_ratio"] = (x == cap).float().mean().item()
    out["response/aborted_ratio"] = (~alive).float().mean().item()
    return out


def pad_to_response_window(values, indices, batch, seqlen, response_length):
    """``pad_input`` (scatter the per-token values to their flat positions in a zero ``(batch * seqlen)``
    buffer) followed by the slice ``[:, -response_length - 1:-1]``, verl/workers/actor/dp_actor.py:316-344."""
    full = torch.zeros(batch * seqlen, dtype=values.dtype)
    full = full.index_put((indices,), values)
    return full.view(batch, seqlen)[:, -response_length - 1:-1]


@torch.no_grad()
def variance_proxy_metrics(batch, gradient_norm=None):
    """compute_variance_proxy_metrics, verl/trainer/ppo/metric_utils.py:306-412, on a plain mapping: with
    W(tau) = sum_t (1 - 2 pi_t + sum pi^2) and the mean advantage per trajectory, proxy 2 = E[A^2 W] (with
    importance weights: E[rho^2 A^2 W_original]), proxy 1 = the squared gradient norm handed in, proxy 3 =
    (proxy 2 - proxy 1) / (N - 1) floored at 0."""
    out = {}
    if "sum_pi_squared" not in batch or "old_log_probs" not in batch or "advantages" not in batch:
        return out
    w = 1 - 2 * torch.exp(batch["old_log_probs"]) + batch["sum_pi_squared"]
    mask = batch["response_mask"]
    isw = batch.get("rollout_is_weights", None)
    if isw is not None:
        w = w * isw**2
    adv = masked_mean(batch["advantages"], mask, axis=-1)
    w_sum = masked_sum(w, mask, axis=-1)
    proxy1 = gradient_norm**2 if gradient_norm is not None else None
    if isw is not None:
        rho = masked_mean(isw, mask, axis=-1)
        w_orig = masked_sum(w / torch.clamp(isw**2, min=1e-10), mask, axis=-1).clamp(min=0.0)
        proxy2 = (rho**2 * adv**2 * w_orig).mean()
    else:
        proxy2 = (adv**2 * w_sum.clamp(min=0.0)).mean()
    proxy3 = None
    if proxy1 is not None and adv.shape[0] > 1:
        proxy3 = max(0.0, ((proxy2 - proxy1) / (adv.shape[0] - 1)).item())
    out["variance_proxy/proxy1_signal_strength"] = proxy1 if proxy1 is not None else 0.0
    out["variance_proxy/proxy2_total_power"] = proxy2.item()
    out["variance_proxy/proxy3_pure_noise"] = proxy3 if proxy3 is not None else 0.0
    out["variance_proxy/expected_a_squared"] = (adv**2).mean().item()
    out["variance_proxy/expected_w"] = w_sum.mean().item()
    return out


@torch.no_grad()
def pf_ppo_weights(token_level_scores, reweight_method="pow", weight_pow=2.0):
    """The resampling probabilities of compute_pf_ppo_reweight_data, verl/trainer/ppo/core_algos.py:1921-1954,
    written sequence by sequence: weight from the sequence's total score, plus 1e-8, floored at 1e-8, normalised the
    way ``torch.multinomial`` normalises.  (The draw itself is a call of ``torch.multinomial`` and has no restatement.)"""
    scores = [float(row.sum()) for row in token_level_scores]
    best, worst = max(scores), min(scores)
    weights = []
    for sc in scores:
        if reweight_method == "pow":
            w = abs(sc) ** weight_pow
        elif reweight_method == "max_min":
            w = 1.0 if sc in (best, worst) else 0.0
        elif reweight_method == "max_random":
            w = 0.4 if sc == best else 0.1
        else:
            raise ValueError(f"Unsupported reweight_method: {reweight_method}")
        weights.append(max(w + 1e-8, 1e-8))
    total = sum(weights)
    return torch.tensor([w / total for w in weights], dtype=torch.float64)
