"""CPU oracle for the per-token policy-math path.  TEST INFRASTRUCTURE ONLY.

This package restates, in plain CPU PyTorch, the arithmetic of the reference's
own PyTorch implementation of the path (file:line citations are on each
function).  It exists so that the HIP kernels can be checked against it.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker or as the timed CPU
baseline.  Nothing under ``verl_amd/`` imports it: the product path has no CPU
fallback and raises when the HIP library is missing.

Parity status: every function here is pinned by ``tests/test_oracle_*.py``
against the reference-held vectors (masked_mean cases, group_mean_std known
answer, GAE multi-turn fixture, GRPO loop==vectorised grids), against
closed forms, fp64 brute-force scalar loops and torch.autograd.  No function is
"parity unpinned".
"""

from .head import (  # noqa: F401
    head_fp32_ground_truth,
    fused_linear_for_ppo_fwd,
    fused_linear_for_ppo_bwd,
    fused_linear_for_ppo_chunked,
    head_grads_closed_form,
    head_fwd_bwd_chunked_fp32,
)
from .masked import (  # noqa: F401
    clip_by_value,
    entropy_from_logits,
    logprobs_from_logits,
    masked_sum,
    masked_mean,
    masked_var,
    masked_whiten,
    sum_pi_squared_from_logits,
)
from .advantages import (  # noqa: F401
    gae_advantage_return,
    gae_raw,
    grpo_outcome_advantage,
    grpo_vectorized_outcome_advantage,
    as_torch_index,
    group_mean_std,
    rloo_outcome_advantage,
    rloo_vectorized_outcome_advantage,
    reinforce_plus_plus_baseline_outcome_advantage,
    opo_outcome_advantage,
    gpg_outcome_advantage,
    reinforce_plus_plus_outcome_advantage,
    remax_outcome_advantage,
    grpo_passk_outcome_advantage,
    optimal_token_baseline_advantage,
    multi_turn_optimal_token_baseline_advantage,
    otb_brute_force_fp64,
)
from .losses import (  # noqa: F401
    agg_loss,
    policy_loss_vanilla,
    value_loss,
    kl_penalty_forward,
    kl_penalty,
    kl_straight_through,
    policy_loss_gspo,
    policy_loss_sapo,
    policy_loss_gpg,
    policy_loss_cispo,
    policy_loss_reinforce,
    policy_loss_geo_mean,
    policy_loss_kl_cov,
    policy_loss_clip_cov,
    clip_cov_candidates,
)
from .trainer import (  # noqa: F401
    apply_kl_penalty,
    adaptive_kl_update,
    compute_rewards,
    compute_data_metrics,
    pad_to_response_window,
    variance_proxy_metrics,
    pf_ppo_weights,
)
from .rollout_corr import (  # noqa: F401
    offpolicy_metrics,
    is_metrics,
    rollout_correction_weights,
    rollout_correction_brute_force_fp64,
    rollout_rejection_mask,
    parse_rs_thresholds,
    RS_OPTIONS,
)
