"""Oracle for the trainer-side callers of the path: the KL penalty on rewards and its controllers,
and the per-step data metrics (CPU torch).

Test infrastructure only; see ``oracle/__init__.py``.
"""

from __future__ import annotations

import numpy as np
import torch

from .losses import kl_penalty
from .masked import masked_mean


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
