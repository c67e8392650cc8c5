"""Oracle for the advantage estimators on the path: GAE and GRPO (CPU torch).

Test infrastructure only; see ``oracle/__init__.py``.
"""

from __future__ import annotations

from collections import defaultdict

import numpy as np
import torch

from .masked import masked_whiten


@torch.no_grad()
def gae_raw(token_level_rewards, values, response_mask, gamma, lam):
    """The recurrence of verl/trainer/ppo/core_algos.py:244-260 without the final
    whitening: returns ``(raw_advantages, returns)``."""
    nv = 0
    g = 0
    cols = []
    L = token_level_rewards.shape[-1]
    for t in range(L - 1, -1, -1):
        m = response_mask[:, t]
        delta = token_level_rewards[:, t] + gamma * nv - values[:, t]
        g_new = delta + gamma * lam * g
        nv = values[:, t] * m + (1 - m) * nv
        g = g_new * m + (1 - m) * g
        cols.append(g)
    adv = torch.stack(cols[::-1], dim=1)
    return adv, adv + values


@torch.no_grad()
def gae_advantage_return(token_level_rewards, values, response_mask, gamma, lam):
    """Reverse GAE recurrence with carried state on masked steps, then whiten.

    Follows verl/trainer/ppo/core_algos.py:214-262 step for step, including the
    arithmetic form of the two selects (``x*m + (1-m)*carry``), ``returns`` from
    the RAW advantages (:260) and ``masked_whiten`` last (:261).
    """
    adv, returns = gae_raw(token_level_rewards, values, response_mask, gamma, lam)
    adv = masked_whiten(adv, response_mask)
    return adv, returns


def gae_brute_force_fp64(rewards, values, mask, gamma, lam):
    """Scalar double-precision recurrence over Python lists, written from the
    textbook definition with select-by-branch instead of arithmetic selects; used
    to pin ``gae_advantage_return`` before whitening."""
    B = len(rewards)
    L = len(rewards[0])
    adv = [[0.0] * L for _ in range(B)]
    for b in range(B):
        nv, g = 0.0, 0.0
        for t in range(L - 1, -1, -1):
            if mask[b][t] != 0:
                delta = rewards[b][t] + gamma * nv - values[b][t]
                g = delta + gamma * lam * g
                nv = values[b][t]
            adv[b][t] = g
    return adv


def grpo_outcome_advantage(token_level_rewards, response_mask, index, epsilon=1e-6,
                           norm_adv_by_std_in_grpo=True):
    """Loop form, verl/trainer/ppo/core_algos.py:266-330.

    Score = unmasked row sum (:303); groups keyed by ``index[i]`` with Python
    equality (:312); singleton group -> mean 0, std 1 (:314-316); else
    ``torch.mean`` / unbiased ``torch.std`` (:318-320); epsilon added to the std
    (:325).  Returns the same tensor twice (:330).
    """
    scores = token_level_rewards.sum(dim=-1)
    members = defaultdict(list)
    mean_of, std_of = {}, {}
    with torch.no_grad():
        for i in range(scores.shape[0]):
            members[index[i]].append(scores[i])
        for key, vals in members.items():
            if len(vals) == 1:
                mean_of[key] = torch.tensor(0.0)
                std_of[key] = torch.tensor(1.0)
            elif len(vals) > 1:
                stacked = torch.stack(vals)
                mean_of[key] = torch.mean(stacked)
                std_of[key] = torch.std(stacked)
            else:
                raise ValueError(f"no score in prompt index: {key}")
        for i in range(scores.shape[0]):
            if norm_adv_by_std_in_grpo:
                scores[i] = (scores[i] - mean_of[index[i]]) / (std_of[index[i]] + epsilon)
            else:
                scores[i] = scores[i] - mean_of[index[i]]
        out = scores.unsqueeze(-1) * response_mask
    return out, out


def as_torch_index(index):
    """Labels -> contiguous int64 ids.  Follows verl/utils/groupwise.py:91-160 for
    the cases the path meets: integer arrays pass through, near-integer floats are
    rounded, numeric strings are coerced, everything else is factorised with
    ``np.unique(return_inverse=True)``."""
    if isinstance(index, torch.Tensor):
        t = index.reshape(-1)
        if not t.dtype.is_floating_point:
            return t.to(torch.long)
        t64 = t.to(torch.float64)
        r = torch.round(t64)
        if torch.allclose(t64, r, rtol=0.0, atol=1e-6):
            return r.to(torch.long)
        arr = np.array([str(x.item()) for x in t], dtype=object)
    else:
        try:
            arr = np.asarray(index)
        except Exception:
            arr = np.array(list(index), dtype=object)
        arr = arr.reshape(-1)
        if arr.dtype != object and np.issubdtype(arr.dtype, np.integer):
            return torch.from_numpy(arr.astype(np.int64, copy=False))
        if arr.dtype != object and np.issubdtype(arr.dtype, np.floating):
            a64 = arr.astype(np.float64, copy=False)
            r = np.rint(a64)
            if np.allclose(a64, r, rtol=0.0, atol=1e-6):
                return torch.from_numpy(r.astype(np.int64))
        try:
            return torch.from_numpy(arr.astype(np.int64))
        except Exception:
            pass
        if arr.dtype != object:
            arr = arr.astype(object)
    try:
        _, inv = np.unique(arr, return_inverse=True)
    except Exception:
        _, inv = np.unique(np.array([str(x) for x in arr], dtype=object), return_inverse=True)
    return torch.from_numpy(inv.astype(np.int64, copy=False))


@torch.no_grad()
def group_mean_std(scores, gidx, eps=1e-6):
    """Per-group mean / std / count by ``index_add_`` of 1, x, x^2.

    Follows verl/utils/groupwise.py:163-223: var = (S2 - S1^2/n)/max(n-1,1),
    std = sqrt(clamp(var, min=eps)); singleton (n<=1) -> mean 0, std 1.
    """
    scores = scores.reshape(-1).to(torch.float32)
    gidx = gidx.reshape(-1).to(torch.long)
    if scores.numel() != gidx.numel():
        raise ValueError(f"scores and gidx length mismatch: {scores.numel()} vs {gidx.numel()}")
    G = int(gidx.max().item()) + 1 if gidx.numel() > 0 else 0
    if G == 0:
        e = torch.empty(0, dtype=torch.float32)
        return e, e, e
    cnt = torch.zeros(G).index_add_(0, gidx, torch.ones_like(scores))
    s1 = torch.zeros(G).index_add_(0, gidx, scores)
    s2 = torch.zeros(G).index_add_(0, gidx, scores * scores)
    mean = s1 / cnt.clamp_min(1.0)
    var = (s2 - s1 * s1 / cnt.clamp_min(1.0)) / (cnt - 1.0).clamp_min(1.0)
    std = torch.sqrt(torch.clamp(var, min=eps))
    single = cnt <= 1.0
    mean = torch.where(single, torch.zeros_like(mean), mean)
    std = torch.where(single, torch.ones_like(std), std)
    return mean, std, cnt


@torch.no_grad()
def grpo_vectorized_outcome_advantage(token_level_rewards, response_mask, index, epsilon=1e-6,
                                      norm_adv_by_std_in_grpo=True):
    """Vectorised twin, verl/trainer/ppo/core_algos.py:333-357."""
    scores = token_level_rewards.sum(dim=-1)
    g = as_torch_index(index)
    mean_g, std_g, _ = group_mean_std(scores, g, eps=epsilon)
    if norm_adv_by_std_in_grpo:
        a = (scores - mean_g[g]) / (std_g[g] + epsilon)
    else:
        a = scores - mean_g[g]
    out = a.unsqueeze(-1) * response_mask
    return out, out


# ---- other outcome estimators of the registry -------------------------------------------------
def _group_members(scores, index):
    members = defaultdict(list)
    for i in range(scores.shape[0]):
        members[index[i]].append(i)
    return members


def _group_means(scores, members):
    """Mean per group, 0 for a single-member group (core_algos.py:446-452, :505-511)."""
    mean_of = {}
    for key, rows in members.items():
        if len(rows) == 1:
            mean_of[key] = torch.tensor(0.0)
        elif len(rows) > 1:
            mean_of[key] = torch.mean(torch.stack([scores[i] for i in rows]))
        else:
            raise ValueError(f"no score in prompt index: {key}")
    return mean_of


@torch.no_grad()
def rloo_outcome_advantage(token_level_rewards, response_mask, index):
    """Leave-one-out baseline, loop form (core_algos.py:479-528): with n members in the group
    ``s n/(n-1) - mean n/(n-1)``; a single-member group keeps its score."""
    scores = token_level_rewards.sum(dim=-1)
    members = _group_members(scores, index)
    mean_of = _group_means(scores, members)
    out = scores.clone()
    for i in range(scores.shape[0]):
        n = len(members[index[i]])
        if n > 1:
            out[i] = scores[i] * n / (n - 1) - mean_of[index[i]] * n / (n - 1)
    out = out.unsqueeze(-1) * response_mask
    return out, out


@torch.no_grad()
def rloo_vectorized_outcome_advantage(token_level_rewards, response_mask, index):
    """Vectorised twin (core_algos.py:720-753): ``(c s - group_sum) / max(c - 1, 1) * (c > 1)``."""
    scores = token_level_rewards.sum(dim=-1)
    inv = torch.from_numpy(np.unique(index, return_inverse=True)[1])
    c = torch.bincount(inv)[inv].to(scores.dtype)
    adv = ((c * scores - torch.bincount(inv, weights=scores)[inv]) / (c - 1).clamp_min(1)) * (c > 1)
    adv = adv.unsqueeze(-1) * response_mask
    return adv, adv


@torch.no_grad()
def reinforce_plus_plus_baseline_outcome_advantage(token_level_rewards, response_mask, index):
    """core_algos.py:421-474: score minus the group mean, tiled over the response and masked, then
    ``masked_whiten(.) * mask``."""
    length = token_level_rewards.shape[-1]
    scores = token_level_rewards.sum(dim=-1)
    members = _group_members(scores, index)
    mean_of = _group_means(scores, members)
    out = scores.clone()
    for i in range(scores.shape[0]):
        out[i] = scores[i] - mean_of[index[i]]
    out = out.unsqueeze(-1).tile([1, length]) * response_mask
    out = masked_whiten(out, response_mask) * response_mask
    return out, out


@torch.no_grad()
def opo_outcome_advantage(token_level_rewards, response_mask, index):
    """core_algos.py:531-579: baseline = length-weighted mean score of the group, 0 for a single member."""
    lengths = response_mask.sum(dim=-1)
    scores = token_level_rewards.sum(dim=-1)
    members = _group_members(scores, index)
    out = scores.clone()
    for key, rows in members.items():
        if len(rows) == 1:
            baseline = torch.tensor(0.0)
        else:
            s = torch.stack([scores[i] for i in rows])
            n = torch.stack([lengths[i] for i in rows])
            baseline = (n * s).sum() / n.sum()
        for i in rows:
            out[i] = scores[i] - baseline
    out = out.unsqueeze(-1) * response_mask
    return out, out


@torch.no_grad()
def gpg_outcome_advantage(token_level_rewards, response_mask, index, f_norm=1.0):
    """core_algos.py:657-717: ``alpha (s - mean) / f_norm`` with ``alpha = batch / max(#{s != 0}, 1)``
    (the ``alpha`` argument of the reference is overwritten, :697-698)."""
    scores = token_level_rewards.sum(dim=-1)
    bsz = scores.shape[0]
    alpha = bsz / torch.count_nonzero(scores).clamp(min=1)
    members = _group_members(scores, index)
    mean_of = _group_means(scores, members)
    out = scores.clone()
    for i in range(bsz):
        out[i] = alpha * (scores[i] - mean_of[index[i]]) / f_norm
    out = out.unsqueeze(-1) * response_mask
    return out, out


@torch.no_grad()
def reinforce_plus_plus_outcome_advantage(token_level_rewards, response_mask, gamma):
    """core_algos.py:582-618: discounted return that restarts after a masked step, then
    ``masked_whiten(returns) * mask``; returns ``(advantages, returns)``."""
    returns = torch.zeros_like(token_level_rewards)
    running = 0
    for t in reversed(range(token_level_rewards.shape[1])):
        running = token_level_rewards[:, t] + gamma * running
        returns[:, t] = running
        running = running * response_mask[:, t]
    advantages = masked_whiten(returns, response_mask) * response_mask
    return advantages, returns


@torch.no_grad()
def remax_outcome_advantage(token_level_rewards, reward_baselines, response_mask):
    """core_algos.py:621-654: reverse cumulative sum of the masked rewards minus the per-response
    baseline on the mask."""
    returns = (token_level_rewards * response_mask).flip(dims=[-1]).cumsum(dim=-1).flip(dims=[-1])
    advantages = returns - reward_baselines.unsqueeze(-1) * response_mask
    return advantages, returns


@torch.no_grad()
def grpo_passk_outcome_advantage(token_level_rewards, response_mask, index, epsilon=1e-6, norm_by_std=True):
    """Pass@k, core_algos.py:360-418: per group the two largest scores (``torch.topk``); the response holding
    the largest gets ``max - second max`` (divided by the group's unbiased std plus epsilon when
    ``norm_by_std``), every other response 0; a group of fewer than two responses raises ``ValueError``."""
    scores = token_level_rewards.sum(dim=-1)
    advantages = torch.zeros_like(scores)
    members = _group_members(scores, index)
    for key, rows in members.items():
        rewards = torch.stack([scores[i] for i in rows])
        if rewards.numel() < 2:
            raise ValueError(f"Pass@k requires at least 2 samples per group. Got {rewards.numel()} for group {key}.")
        topk, topk_idx = torch.topk(rewards, 2)
        advantage = topk[0] - topk[1]
        if norm_by_std:
            advantage = advantage / (torch.std(rewards) + epsilon)
        advantages[rows[topk_idx[0].item()]] = advantage
    advantages = advantages.unsqueeze(-1) * response_mask
    return advantages, advantages


def _otb_streams(token_level_rewards, response_mask, old_log_probs, sum_pi_squared, rollout_is_weights):
    """core_algos.py:809-822 (= :924-938): reward to go and the cumulative path-variance proxy."""
    returns = (token_level_rewards * response_mask).flip(dims=[-1]).cumsum(dim=-1).flip(dims=[-1])
    w = 1 - 2 * torch.exp(old_log_probs) + sum_pi_squared
    if rollout_is_weights is not None:
        w = w * (rollout_is_weights**2)
    return returns, (w * response_mask).cumsum(dim=-1)


def _otb_zero_tail(baselines, rows, lengths):
    """core_algos.py:858-868 (= :983-993): when exactly one trajectory of the group is the longest, its
    baseline is 0 from the second-longest length on."""
    ordered = sorted(int(lengths[i]) for i in rows)
    longest, second = ordered[-1], ordered[-2]
    holders = [i for i in rows if int(lengths[i]) == longest]
    if len(holders) == 1 and longest > second:
        baselines[holders[0], second:] = 0.0


@torch.no_grad()
def optimal_token_baseline_advantage(token_level_rewards, response_mask, index, old_log_probs, sum_pi_squared,
                                     rollout_is_weights=None, handle_zero_tail=False, epsilon=1e-8):
    """core_algos.py:756-873: per prompt group and column, baseline = sum(G W m) / (sum(W m) + eps) over the
    group's trajectories (none for a group of one); advantages = (G - baseline) * mask; returns
    ``(advantages, returns)``."""
    returns, w_cum = _otb_streams(token_level_rewards, response_mask, old_log_probs, sum_pi_squared,
                                  rollout_is_weights)
    members = defaultdict(list)
    for i in range(token_level_rewards.shape[0]):
        members[index[i]].append(i)
    baselines = torch.zeros_like(returns)
    lengths = response_mask.sum(dim=-1)
    for rows in members.values():
        if len(rows) == 1:
            continue
        sel = torch.tensor(rows)
        num = (returns[sel] * w_cum[sel] * response_mask[sel]).sum(dim=0)
        den = (w_cum[sel] * response_mask[sel]).sum(dim=0) + epsilon
        baselines[sel] = (num / den).unsqueeze(0).expand(len(rows), -1)
        if handle_zero_tail:
            _otb_zero_tail(baselines, rows, lengths)
    return (returns - baselines) * response_mask, returns


@torch.no_grad()
def multi_turn_optimal_token_baseline_advantage(token_level_rewards, response_mask, index, old_log_probs,
                                                sum_pi_squared, rollout_is_weights=None, handle_zero_tail=True,
                                                epsilon=1e-8):
    """core_algos.py:876-1004: as above, but every trajectory's valid tokens are first packed to the left
    (the k-th valid token of each trajectory shares baseline column k), trajectories with no valid token
    leave their group, and the advantages are scattered back to the valid positions."""
    returns, w_cum = _otb_streams(token_level_rewards, response_mask, old_log_probs, sum_pi_squared,
                                  rollout_is_weights)
    B = returns.shape[0]
    lengths = response_mask.sum(dim=-1).long()
    width = int(lengths.max().item()) if B > 0 else 0
    packed_w = w_cum.new_zeros((B, width))
    packed_g = torch.zeros_like(packed_w)
    valid = response_mask.bool()
    for i in range(B):
        n = int(lengths[i])
        packed_w[i, :n] = w_cum[i, valid[i]]
        packed_g[i, :n] = returns[i, valid[i]]
    members = defaultdict(list)
    for i in range(B):
        if int(lengths[i]) > 0:
            members[index[i]].append(i)
    baselines = torch.zeros_like(packed_g)
    for rows in members.values():
        if len(rows) == 1:
            continue
        sel = torch.tensor(rows)
        b_star = (packed_g[sel] * packed_w[sel]).sum(dim=0) / (packed_w[sel].sum(dim=0) + epsilon)
        baselines[sel] = b_star.to(baselines.dtype)
        if handle_zero_tail:
            _otb_zero_tail(baselines, rows, lengths)
    packed_adv = packed_g - baselines
    advantages = torch.zeros_like(returns)
    for i in range(B):
        n = int(lengths[i])
        if n > 0:
            advantages[i, valid[i]] = packed_adv[i, :n]
    return advantages * response_mask, returns


def otb_brute_force_fp64(rewards, mask, index, old_log_probs, sum_pi_squared, is_weights=None, packed=False,
                         zero_tail=False, epsilon=1e-8):
    """Scalar double-precision loops over Python lists written from the definition of the optimal token
    baseline, B_k = sum_i G_ik W_ik / (sum_i W_ik + eps) with k the column (``packed=False``) or the rank of
    the token among its trajectory's valid tokens (``packed=True``); pins the two functions above."""
    import math
    B, L = len(rewards), len(rewards[0])
    G = [[0.0] * L for _ in range(B)]
    W = [[0.0] * L for _ in range(B)]
    slot = [[-1] * L for _ in range(B)]  # baseline column of each valid token
    n_valid = [0] * B
    for i in range(B):
        acc = 0.0
        for t in range(L - 1, -1, -1):
            acc += rewards[i][t] * mask[i][t]
            G[i][t] = acc
        acc = 0.0
        for t in range(L):
            w = 1.0 - 2.0 * math.exp(old_log_probs[i][t]) + sum_pi_squared[i][t]
            if is_weights is not None:
                w *= is_weights[i][t] ** 2
            acc += w * mask[i][t]
            W[i][t] = acc
            if mask[i][t] != 0:
                slot[i][t] = n_valid[i] if packed else t
                n_valid[i] += 1
    groups = defaultdict(list)
    for i in range(B):
        if not packed or n_valid[i] > 0:
            groups[index[i]].append(i)
    adv = [[0.0] * L for _ in range(B)]
    for rows in groups.values():
        num = defaultdict(float)
        den = defaultdict(float)
        for i in rows:
            for t in range(L):
                if slot[i][t] >= 0:
                    num[slot[i][t]] += G[i][t] * W[i][t] * mask[i][t]
                    den[slot[i][t]] += W[i][t] * mask[i][t]
        no_baseline_from = {i: L + 1 for i in rows}
        if zero_tail and len(rows) > 1:
            ordered = sorted(n_valid[i] for i in rows)
            if ordered[-1] > ordered[-2]:
                holder = [i for i in rows if n_valid[i] == ordered[-1]]
                no_baseline_from[holder[0]] = ordered[-2]
        for i in rows:
            for t in range(L):
                k = slot[i][t]
                if k < 0:
                    continue
                b = 0.0
                if len(rows) > 1 and k < no_baseline_from[i]:
                    b = num[k] / (den[k] + epsilon)
                adv[i][t] = (G[i][t] - b) * mask[i][t]
    return adv, G
