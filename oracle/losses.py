"""Oracle for loss aggregation, the clipped / dual-clip policy loss, the clipped
value loss and the KL estimators (CPU torch, differentiable through autograd).

Test infrastructure only; see ``oracle/__init__.py``.
"""

from __future__ import annotations

import torch

from .masked import clip_by_value, masked_mean, masked_sum


def agg_loss(loss_mat, loss_mask, loss_agg_mode, dp_size=1, batch_num_tokens=None,
             global_batch_size=None, loss_scale_factor=None):
    """Four aggregation modes, verl/trainer/ppo/core_algos.py:1025-1080.

    ``token-mean`` divides by ``mask.sum()`` with NO epsilon (:1055-1058); the two
    ``seq-mean`` modes drop fully masked rows through a 0/1 row mask
    (:1059-1071); ``seq-mean-token-sum-norm`` divides by the row length unless a
    factor is given (:1072-1076).
    """
    if loss_agg_mode == "token-mean":
        if batch_num_tokens is None:
            batch_num_tokens = loss_mask.sum()
        return masked_sum(loss_mat, loss_mask) / batch_num_tokens * dp_size
    if loss_agg_mode == "seq-mean-token-sum":
        row = torch.sum(loss_mat * loss_mask, dim=-1)
        keep = (torch.sum(loss_mask, dim=-1) > 0).float()
        if global_batch_size is None:
            global_batch_size = keep.sum()
        return masked_sum(row, keep) / global_batch_size * dp_size
    if loss_agg_mode == "seq-mean-token-mean":
        cnt = torch.sum(loss_mask, dim=-1)
        row = torch.sum(loss_mat * loss_mask, dim=-1) / (cnt + 1e-8)
        keep = (cnt > 0).float()
        if global_batch_size is None:
            global_batch_size = keep.sum()
        return masked_sum(row, keep) / global_batch_size * dp_size
    if loss_agg_mode == "seq-mean-token-sum-norm":
        row = torch.sum(loss_mat * loss_mask, dim=-1)
        if loss_scale_factor is None:
            loss_scale_factor = loss_mask.shape[-1]
        return torch.sum(row) / loss_scale_factor
    raise ValueError(f"Invalid loss_agg_mode: {loss_agg_mode}")


def policy_loss_vanilla(old_log_prob, log_prob, advantages, response_mask, loss_agg_mode="token-mean",
                        clip_ratio_low=0.2, clip_ratio_high=0.2, clip_ratio_c=3.0,
                        rollout_is_weights=None, global_batch_info=None):
    """PPO clipped objective with the dual-clip floor for negative advantages.

    Follows verl/trainer/ppo/core_algos.py:1159-1250 with the config fields
    passed as plain numbers.  Returns ``(pg_loss, pg_clipfrac, ppo_kl,
    pg_clipfrac_lower)`` as tensors (the reference turns the last three into
    Python floats with ``.item()`` at :1245-1249).
    """
    assert clip_ratio_c > 1.0
    k = torch.clamp(log_prob - old_log_prob, min=-20.0, max=20.0)
    ratio = torch.exp(k)
    ppo_kl = masked_mean(-k, response_mask)
    l1 = -advantages * ratio
    l2 = -advantages * torch.clamp(ratio, 1 - clip_ratio_low, 1 + clip_ratio_high)
    c1 = torch.maximum(l1, l2)
    pg_clipfrac = masked_mean(torch.gt(l2, l1).float(), response_mask)
    l3 = -advantages * clip_ratio_c
    c2 = torch.min(l3, c1)
    pg_clipfrac_lower = masked_mean(torch.gt(c1, l3) * (advantages < 0).float(), response_mask)
    losses = torch.where(advantages < 0, c2, c1)
    if rollout_is_weights is not None:
        losses = losses * rollout_is_weights
    pg_loss = agg_loss(losses, response_mask, loss_agg_mode, **(global_batch_info or {}))
    return pg_loss, pg_clipfrac, ppo_kl, pg_clipfrac_lower


def value_loss(vpreds, returns, values, response_mask, cliprange_value, loss_agg_mode="token-mean"):
    """Clipped value loss, verl/trainer/ppo/core_algos.py:1799-1838."""
    clipped = clip_by_value(vpreds, values - cliprange_value, values + cliprange_value)
    e1 = (vpreds - returns) ** 2
    e2 = (clipped - returns) ** 2
    vf_loss = 0.5 * agg_loss(torch.max(e1, e2), response_mask, loss_agg_mode)
    vf_clipfrac = masked_mean(torch.gt(e2, e1).float(), response_mask)
    return vf_loss, vf_clipfrac


def kl_penalty_forward(logprob, ref_logprob, kind):
    """KL estimators k1 / abs / k2 / k3, verl/trainer/ppo/core_algos.py:1868-1902."""
    if kind in ("kl", "k1"):
        return logprob - ref_logprob
    if kind == "abs":
        return (logprob - ref_logprob).abs()
    if kind in ("mse", "k2"):
        return 0.5 * (logprob - ref_logprob).square()
    if kind in ("low_var_kl", "k3"):
        d = torch.clamp(ref_logprob - logprob, min=-20, max=20)
        return torch.clamp(torch.exp(d) - d - 1, min=-10, max=10)
    raise NotImplementedError(kind)


def kl_penalty(logprob, ref_logprob, kind):
    """verl/trainer/ppo/core_algos.py:1841-1866, as written: the forward score is evaluated with
    the name as given, so a "+"-suffixed name already fails in ``kl_penalty_forward``; the
    straight-through combination below is what the remaining lines do for a forward score."""
    forward_score = kl_penalty_forward(logprob, ref_logprob, kind)
    if not kind.endswith("+") or kind in ("mse", "k2"):
        return forward_score
    return kl_straight_through(logprob, ref_logprob, forward_score)


def kl_straight_through(logprob, ref_logprob, forward_score):
    """core_algos.py:1861-1866: value of ``forward_score``, gradient of k2."""
    backward_score = 0.5 * (logprob - ref_logprob).square()
    return backward_score - backward_score.detach() + forward_score.detach()


# ---- other registered policy losses ------------------------------------------------------------
def policy_loss_gspo(old_log_prob, log_prob, advantages, response_mask, clip_ratio_low=0.2, clip_ratio_high=0.2,
                     rollout_is_weights=None, global_batch_info=None):
    """GSPO, verl/trainer/ppo/core_algos.py:1253-1326: sequence-level ratio from the masked mean of the
    token log-ratios (length clamped to >= 1), token-level gradient through ``log_prob - log_prob.detach()``,
    log-ratio clamped at 10, clipped objective, always "seq-mean-token-mean".  Returns
    ``(pg_loss, pg_clipfrac, ppo_kl, pg_clipfrac_lower = 0)``."""
    d = log_prob - old_log_prob
    lengths = torch.sum(response_mask, dim=-1).clamp(min=1)
    seq = torch.sum(d * response_mask, dim=-1) / lengths
    log_ratio = torch.clamp(log_prob - log_prob.detach() + seq.detach().unsqueeze(-1), max=10.0)
    ratio = torch.exp(log_ratio)
    l1 = -advantages * ratio
    l2 = -advantages * torch.clamp(ratio, 1 - clip_ratio_low, 1 + clip_ratio_high)
    losses = torch.maximum(l1, l2)
    if rollout_is_weights is not None:
        losses = losses * rollout_is_weights
    pg_loss = agg_loss(losses, response_mask, "seq-mean-token-mean", **(global_batch_info or {}))
    pg_clipfrac = masked_mean(torch.gt(l2, l1).float(), response_mask)
    ppo_kl = masked_mean(-d, response_mask)
    return pg_loss, pg_clipfrac, ppo_kl, torch.tensor(0.0)


def policy_loss_sapo(old_log_prob, log_prob, advantages, response_mask, tau_pos, tau_neg,
                     rollout_is_weights=None, global_batch_info=None):
    """SAPO, core_algos.py:1329-1411: gate ``sigmoid(tau (ratio - 1)) 4 / tau`` with tau chosen by the sign of
    the advantage, always "seq-mean-token-mean".  Returns ``(pg_loss, 0, ppo_kl, 0)``."""
    tp = torch.as_tensor(tau_pos, dtype=advantages.dtype)
    tn = torch.as_tensor(tau_neg, dtype=advantages.dtype)
    k = torch.clamp(log_prob - old_log_prob, min=-20.0, max=20.0)
    ratio = torch.exp(k)
    taus = torch.where(advantages > 0, tp, tn)
    gates = torch.sigmoid(taus * (ratio - 1.0)) * (4.0 / taus)
    losses = -gates * advantages
    if rollout_is_weights is not None:
        losses = losses * rollout_is_weights
    pg_loss = agg_loss(losses, response_mask, "seq-mean-token-mean", **(global_batch_info or {}))
    return pg_loss, torch.tensor(0.0), masked_mean(-k, response_mask), torch.tensor(0.0)


def policy_loss_gpg(log_prob, advantages, response_mask, loss_agg_mode="token-mean", rollout_is_weights=None,
                    global_batch_info=None):
    """GPG, core_algos.py:1414-1447: ``agg_loss(-log_prob * advantages)``; the reference returns no metrics."""
    losses = -log_prob * advantages
    if rollout_is_weights is not None:
        losses = losses * rollout_is_weights
    return agg_loss(losses, response_mask, loss_agg_mode, **(global_batch_info or {}))


def policy_loss_cispo(old_log_prob, log_prob, advantages, response_mask, loss_agg_mode="token-mean",
                      clip_ratio_low=0.2, clip_ratio_high=0.2, rollout_is_weights=None, global_batch_info=None):
    """CISPO, core_algos.py:1721-1779: ``-sg(clamp(ratio)) * A * log_prob``; pg_clipfrac counts the tokens whose
    ratio the clamp changed.  Returns ``(pg_loss, pg_clipfrac, ppo_kl, 0)``."""
    k = torch.clamp(log_prob - old_log_prob, min=-20.0, max=20.0)
    ratio = torch.exp(k)
    clipped = torch.clamp(ratio, 1 - clip_ratio_low, 1 + clip_ratio_high)
    losses = -clipped.detach() * advantages * log_prob
    pg_clipfrac = masked_mean((ratio != clipped).float(), response_mask)
    if rollout_is_weights is not None:
        losses = losses * rollout_is_weights
    pg_loss = agg_loss(losses, response_mask, loss_agg_mode, **(global_batch_info or {}))
    return pg_loss, pg_clipfrac, masked_mean(-k, response_mask), torch.tensor(0.0)


def policy_loss_reinforce(rollout_log_prob, log_prob, advantages, response_mask, loss_agg_mode="seq-mean-token-sum",
                          rollout_is_weights=None, global_batch_info=None):
    """REINFORCE with optional importance weights, verl/trainer/ppo/core_algos.py:1984-2061: returns
    ``(pg_loss, ppo_kl)`` with the KL measured against the rollout policy."""
    losses = -advantages * log_prob
    if rollout_is_weights is not None:
        losses = losses * rollout_is_weights
    pg_loss = agg_loss(losses, response_mask, loss_agg_mode, **(global_batch_info or {}))
    return pg_loss, masked_mean(-(log_prob - rollout_log_prob), response_mask)


def policy_loss_geo_mean(old_log_prob, log_prob, advantages, response_mask, clip_ratio_low=0.2, clip_ratio_high=0.2,
                         rollout_is_weights=None):
    """GMPO, verl/trainer/ppo/core_algos.py:1635-1718: token log-ratios clipped to ``[-low, high]`` on the side
    that the sign of the advantage makes pessimistic, their masked mean exponentiated into one ratio per
    sequence, times the masked mean advantage; importance weights enter as their geometric mean per sequence;
    plain mean over the sequences.  Returns ``(pg_loss, pg_clipfrac, ppo_kl, pg_clipfrac_lower)``."""
    x = log_prob - old_log_prob
    sgn = torch.sign(advantages)
    clamped = torch.clamp(x, -clip_ratio_low, clip_ratio_high)
    x_min = sgn * torch.min(sgn * x, sgn * clamped)
    lengths = response_mask.sum(dim=-1)
    ratio = torch.exp((x_min * response_mask).sum(dim=-1) / (lengths + 1e-8))
    adv = (advantages * response_mask).sum(dim=-1) / (lengths + 1e-8)
    losses = -adv * ratio
    if rollout_is_weights is not None:
        losses = losses * torch.exp((torch.log(rollout_is_weights + 1e-10) * response_mask).sum(dim=-1) / (lengths + 1e-8))
    clipped = torch.ne(x, clamped)
    return (torch.mean(losses), masked_mean((clipped * (advantages > 0)).float(), response_mask),
            masked_mean(-x, response_mask), masked_mean((clipped * (advantages < 0)).float(), response_mask))


def policy_loss_kl_cov(old_log_prob, log_prob, advantages, response_mask, loss_agg_mode="token-mean",
                       kl_cov_ratio=0.0002, ppo_kl_coef=1.0, rollout_is_weights=None, global_batch_info=None):
    """KL-Cov, verl/trainer/ppo/core_algos.py:1555-1632: the unclipped surrogate ``-A ratio`` everywhere, plus
    ``ppo_kl_coef |log ratio|`` on the ``max(1, int(n kl_cov_ratio))`` valid tokens with the largest covariance
    ``(A - mean A)(log_prob - mean log_prob)`` (plain means over the valid tokens).  Returns
    ``(pg_loss, ppo_kl_abs, selected)`` with ``selected`` the boolean matrix of penalised tokens."""
    x = log_prob - old_log_prob
    ratio = torch.exp(x)
    base = -advantages * ratio
    with_kl = base + ppo_kl_coef * x.abs()
    valid = response_mask > 0
    selected = torch.zeros_like(valid)
    adv_v = advantages[valid].detach().reshape(-1)
    lp_v = log_prob[valid].detach().reshape(-1)
    if min(kl_cov_ratio, adv_v.numel()) != 0:
        cov = (adv_v - adv_v.mean()) * (lp_v - lp_v.mean())
        k = max(1, int(cov.numel() * kl_cov_ratio))
        top = torch.topk(cov, k, largest=True).indices
        flat = torch.nonzero(valid.reshape(-1), as_tuple=True)[0][top]
        selected.view(-1)[flat] = True
    losses = torch.where(selected, with_kl, base)
    if rollout_is_weights is not None:
        losses = losses * rollout_is_weights
    pg_loss = agg_loss(losses, response_mask, loss_agg_mode, **(global_batch_info or {}))
    return pg_loss, masked_mean(x.abs(), response_mask), selected


def clip_cov_candidates(old_log_prob, log_prob, advantages, response_mask, clip_ratio_low, clip_ratio_high,
                        clip_cov_lb=1.0, clip_cov_ub=5.0, clip_cov_ratio=0.0002):
    """The deterministic part of Clip-Cov's selection, core_algos.py:1502-1516: ``(candidates, clip_num)`` with
    ``candidates`` the valid, not already clipped tokens whose covariance ``(A - masked_mean A)(log_prob -
    masked_mean log_prob)`` lies strictly between the two bounds, and ``clip_num = max(int(ratio M), 1)``."""
    ratio = torch.exp(log_prob - old_log_prob)
    l1 = -advantages * ratio
    l2 = -advantages * torch.clamp(ratio, 1 - clip_ratio_low, 1 + clip_ratio_high)
    clipped = (l2 > l1) & (response_mask > 0)
    cov = (advantages - masked_mean(advantages, response_mask)) * (log_prob - masked_mean(log_prob.detach(), response_mask))
    cov = cov.detach().clone()
    cov[response_mask == 0] = -torch.inf
    cov[clipped] = -torch.inf
    clip_num = max(int(clip_cov_ratio * response_mask.sum().item()), 1)
    return (cov < clip_cov_ub) & (cov > clip_cov_lb) & (response_mask > 0), clip_num


def policy_loss_clip_cov(old_log_prob, log_prob, advantages, response_mask, loss_agg_mode="token-mean",
                         clip_ratio_low=0.2, clip_ratio_high=0.2, clip_cov_lb=1.0, clip_cov_ub=5.0,
                         clip_cov_ratio=0.0002, rollout_is_weights=None, global_batch_info=None, dropped=None):
    """Clip-Cov, core_algos.py:1450-1552: the clipped surrogate, with ``min(clip_num, #candidates)`` of the
    candidates above, drawn uniformly at random, contributing neither loss nor gradient.  ``dropped`` (a boolean
    matrix) replaces the random draw.  Returns ``(pg_loss, pg_clipfrac, ppo_kl, dropped)``."""
    x = log_prob - old_log_prob
    ratio = torch.exp(x)
    l1 = -advantages * ratio
    l2 = -advantages * torch.clamp(ratio, 1 - clip_ratio_low, 1 + clip_ratio_high)
    if dropped is None:
        cand, clip_num = clip_cov_candidates(old_log_prob, log_prob, advantages, response_mask, clip_ratio_low,
                                             clip_ratio_high, clip_cov_lb, clip_cov_ub, clip_cov_ratio)
        idx = torch.nonzero(cand)
        dropped = torch.zeros_like(cand)
        if len(idx) > 0:
            idx = idx[torch.randperm(len(idx))[: min(clip_num, len(idx))]]
            dropped[idx[:, 0], idx[:, 1]] = True
    corr = (~dropped).to(l1.dtype)
    losses = torch.maximum(l1, l2) * corr
    if rollout_is_weights is not None:
        losses = losses * rollout_is_weights
    pg_loss = agg_loss(losses, response_mask, loss_agg_mode, **(global_batch_info or {}))
    return pg_loss, masked_mean((corr == 0).float(), response_mask), masked_mean(-x, response_mask), dropped
