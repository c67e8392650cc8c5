"""The two trainer-side callers of the per-token policy math, mirrored from the reference's
verl/trainer/ppo/ray_trainer.py: ``apply_kl_penalty`` (:70-109) and ``compute_advantage`` (:129-222).

``data`` is anything shaped like the reference's ``DataProto``: ``data.batch`` maps names to tensors
(a ``TensorDict`` or a plain ``dict``) and ``data.non_tensor_batch`` maps names to numpy arrays.
Nothing else of the trainer lives here.
"""
from __future__ import annotations

from typing import Any, Optional

from . import core_algos
from .core_algos import AdvantageEstimator


def _batch_size(data) -> int:
    size = getattr(data.batch, "batch_size", None)
    if size is not None and not callable(size):
        return int(size[0])
    return int(data.batch["response_mask"].shape[0])


def apply_kl_penalty(data, kl_ctrl, kl_penalty: str = "kl"):
    """Subtract ``beta * KL(old || ref)`` from the token-level scores (reference ray_trainer.py:70-109).

    Reads ``response_mask``, ``token_level_scores``, ``old_log_probs`` and ``ref_log_prob`` from
    ``data.batch``, writes ``token_level_rewards``, updates ``kl_ctrl`` with the batch's mean
    per-sequence KL, and returns ``(data, metrics)`` with the reference's two metric names.  The
    penalty, the subtraction and the KL statistic are one kernel launch; the only host sync is the
    read of the statistic that the controller needs.
    """
    beta = kl_ctrl.value
    rewards, current_kl = core_algos.kl_penalised_rewards(
        data.batch["token_level_scores"], data.batch["old_log_probs"], data.batch["ref_log_prob"],
        data.batch["response_mask"], beta, kl_penalty)
    current_kl = current_kl.item()
    kl_ctrl.update(current_kl=current_kl, n_steps=_batch_size(data))
    data.batch["token_level_rewards"] = rewards
    return data, {"actor/reward_kl_penalty": current_kl, "actor/reward_kl_penalty_coeff": beta}


def compute_response_mask(data):
    """The last ``responses.size(1)`` columns of ``attention_mask`` (reference ray_trainer.py:112-126)."""
    response_length = data.batch["responses"].size(1)
    return data.batch["attention_mask"][:, -response_length:]


def compute_advantage(data, adv_estimator, gamma: float = 1.0, lam: float = 1.0, num_repeat: int = 1,
                      norm_adv_by_std_in_grpo: bool = True, config: Optional[Any] = None):
    """Fill ``data.batch["advantages"]`` and ``data.batch["returns"]`` with the chosen estimator
    (reference ray_trainer.py:129-222): GAE and GRPO are called with their own argument lists, every
    other estimator through the registry with ``token_level_rewards``, ``response_mask``, ``config``
    and whichever of ``uid`` / ``reward_baselines`` the batch holds.

    One difference from the reference: the optimal-token-baseline estimators also receive
    ``old_log_probs`` here (they require it; the reference's dispatcher does not pass it).  With
    ``config.use_pf_ppo`` the batch is resampled after GAE as there (:172-177) and the resampled
    object is what is returned.
    """
    if "response_mask" not in data.batch.keys():
        data.batch["response_mask"] = compute_response_mask(data)
    if adv_estimator == AdvantageEstimator.GAE:
        advantages, returns = core_algos.compute_gae_advantage_return(
            token_level_rewards=data.batch["token_level_rewards"], values=data.batch["values"],
            response_mask=data.batch["response_mask"], gamma=gamma, lam=lam)
        if config is not None and config.get("use_pf_ppo", False):
            data.batch["advantages"] = advantages
            data.batch["returns"] = returns
            return core_algos.compute_pf_ppo_reweight_data(data, config.pf_ppo.get("reweight_method"),
                                                           config.pf_ppo.get("weight_pow"))
    elif adv_estimator == AdvantageEstimator.GRPO:
        advantages, returns = core_algos.compute_grpo_outcome_advantage(
            token_level_rewards=data.batch["token_level_rewards"], response_mask=data.batch["response_mask"],
            index=data.non_tensor_batch["uid"], norm_adv_by_std_in_grpo=norm_adv_by_std_in_grpo)
    else:
        fn = core_algos.get_adv_estimator_fn(adv_estimator)
        kwargs = {"token_level_rewards": data.batch["token_level_rewards"],
                  "response_mask": data.batch["response_mask"], "config": config}
        if "uid" in data.non_tensor_batch:
            kwargs["index"] = data.non_tensor_batch["uid"]
        if "reward_baselines" in data.batch:
            kwargs["reward_baselines"] = data.batch["reward_baselines"]
        if adv_estimator in (AdvantageEstimator.OPTIMAL_TOKEN_BASELINE,
                             AdvantageEstimator.TIR_OPTIMAL_TOKEN_BASELINE):
            assert "sum_pi_squared" in data.batch, (
                "Step-dependent optimal baseline requires sum_pi_squared from actor. "
                "Please set actor.calculate_sum_pi_squared=True in config."
            )
            kwargs["sum_pi_squared"] = data.batch["sum_pi_squared"]
            kwargs["old_log_probs"] = data.batch["old_log_probs"]
            kwargs["rollout_is_weights"] = data.batch.get("rollout_is_weights", None)
        advantages, returns = fn(**kwargs)
    data.batch["advantages"] = advantages
    data.batch["returns"] = returns
    return data
