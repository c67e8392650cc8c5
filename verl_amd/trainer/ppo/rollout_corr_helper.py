"""Rollout-correction importance weights and off-policy diagnostics, mirrored from the reference's
verl/trainer/ppo/rollout_corr_helper.py: ``compute_rollout_correction_weights`` (:481-598, with
``compute_is_metrics`` :601-712), ``compute_offpolicy_metrics`` (:835-937) and the unified
``compute_rollout_correction_and_rejection_mask`` (:715-832).

One kernel launch reads the log-probabilities and the mask once and produces the weights and all
metrics; the host reads the metric vector with a single copy.  Rejection sampling (``rollout_rs``)
is not provided: asking for it raises ``NotImplementedError``.
"""
from __future__ import annotations

import types
from typing import Any, Optional

import torch

from ... import _cabi

SAFETY_BOUND = 20.0

_LEVELS = {None: 0, "token": 1, "sequence": 2}
# metric vector slot -> name, in the order of the VAMD_RC_* constants of include/verl_amd.h
_OFFPOLICY = ("training_ppl", "training_log_ppl", "kl", "k3_kl", "rollout_ppl", "rollout_log_ppl", "log_ppl_diff",
              "log_ppl_abs_diff", "log_ppl_diff_max", "log_ppl_diff_min", "ppl_ratio", "chi2_token", "chi2_seq")
_IS = ("rollout_is_mean", "rollout_is_max", "rollout_is_min", "rollout_is_ratio_fraction_high",
       "rollout_is_ratio_fraction_low", "rollout_is_std", "rollout_is_eff_sample_size", "rollout_is_seq_mean",
       "rollout_is_seq_std", "rollout_is_seq_max", "rollout_is_seq_min", "rollout_is_seq_max_deviation",
       "rollout_is_seq_fraction_high", "rollout_is_seq_fraction_low", "rollout_is_batch_norm_factor")
_SLOTS = _OFFPOLICY + _IS + ("_valid_tokens",)


def _run(old_log_prob, rollout_log_prob, response_mask, level, threshold, batch_normalize):
    """One pass: ``(weights or None, {name: float})`` with every slot of the metric vector."""
    with torch.no_grad():
        dev = _cabi.compute_device(old_log_prob, response_mask)
        old = _cabi.as_f32(old_log_prob, dev)
        if old.dim() == 1:
            old = old.view(1, -1)
        assert old.dim() == 2, f"expected (batch, length) log-probabilities, got {tuple(old_log_prob.shape)}"
        roll = None
        if rollout_log_prob is not None:
            roll = _cabi.as_f32(rollout_log_prob, dev).view(old.shape)
        mask, code = _cabi.mask_code(response_mask.detach().to(dev))
        mask = mask.view(old.shape)
        rows, cols = old.shape
        weights = torch.empty_like(old) if level else None
        out = torch.empty(len(_SLOTS), dtype=torch.float64, device=dev)
        Lb = _cabi.lib()
        ws = _cabi.workspace(Lb.vamd_rollout_correction_workspace_bytes(rows, cols), dev)
        with torch.cuda.device(dev):
            _cabi.check(Lb.vamd_rollout_correction(old.data_ptr(), _cabi.ptr(roll), mask.data_ptr(), code, rows, cols,
                                                   level, float(threshold or 0.0), int(bool(batch_normalize)),
                                                   _cabi.ptr(weights), out.data_ptr(), ws.data_ptr(), ws.numel(),
                                                   _cabi.stream_ptr(dev)))
        values = dict(zip(_SLOTS, out.cpu().tolist()))       # the one host sync
        if weights is not None:
            weights = weights.view(old_log_prob.shape).to(old_log_prob.device)
        return weights, values


def _check_level(rollout_is, rollout_is_threshold):
    valid = {"token", "sequence"}
    if rollout_is not in valid:
        raise ValueError(f"Invalid rollout_is: {rollout_is}. Must be one of {valid}.")
    if rollout_is_threshold <= 0:
        raise ValueError(f"rollout_is_threshold must be positive, got {rollout_is_threshold}.")


def _is_metrics(values, batch_normalize):
    names = _IS if batch_normalize else _IS[:-1]
    return {k: values[k] for k in names}


def compute_rollout_correction_weights(log_ratio: torch.Tensor, response_mask: torch.Tensor,
                                       rollout_is: str = "token", rollout_is_threshold: float = 2.0,
                                       rollout_is_batch_normalize: bool = False):
    """Truncated importance weights ``pi_train / pi_rollout`` from their log ratio, per token or per sequence,
    zero outside the mask, with the reference's ``rollout_is_*`` metrics (computed before truncation).
    Returns ``(rollout_is_weights, metrics)``; the weights carry no gradient.  Raises ``ValueError`` for an
    unknown level, a non-positive threshold, or a mask without a valid token."""
    _check_level(rollout_is, rollout_is_threshold)
    weights, values = _run(log_ratio, torch.zeros_like(log_ratio), response_mask, _LEVELS[rollout_is],
                           rollout_is_threshold, rollout_is_batch_normalize)
    if values["_valid_tokens"] == 0:
        raise ValueError("response_mask must contain at least one valid token (1).")
    return weights, _is_metrics(values, rollout_is_batch_normalize)


def compute_offpolicy_metrics(old_log_prob: torch.Tensor, rollout_log_prob: Optional[torch.Tensor],
                              response_mask: torch.Tensor) -> dict[str, Any]:
    """Perplexities of the training and rollout policies, the k1 / k3 estimates of KL(rollout || training)
    and the token- and sequence-level chi-square divergences (reference :835-937).  Without
    ``rollout_log_prob`` only ``training_ppl`` and ``training_log_ppl`` are returned."""
    _, values = _run(old_log_prob, rollout_log_prob, response_mask, 0, None, False)
    assert values["_valid_tokens"] > 0, "Expected at least one valid token in response_mask"
    names = _OFFPOLICY if rollout_log_prob is not None else _OFFPOLICY[:2]
    return {k: values[k] for k in names}


def compute_rollout_correction_and_rejection_mask(old_log_prob: torch.Tensor, rollout_log_prob: torch.Tensor,
                                                  response_mask: torch.Tensor, rollout_is: Optional[str] = None,
                                                  rollout_is_threshold: Optional[float] = 2.0,
                                                  rollout_is_batch_normalize: bool = False,
                                                  rollout_rs: Optional[str] = None,
                                                  rollout_rs_threshold=None):
    """Importance weights and off-policy metrics of one batch in a single pass (reference :715-832).

    Returns ``(weights_proto, modified_response_mask, metrics)``: ``weights_proto.batch["rollout_is_weights"]``
    holds the weights (``weights_proto`` is ``None`` when ``rollout_is`` is ``None``), the mask is a copy of
    ``response_mask`` (no rejection is applied), and every metric name is prefixed with ``rollout_corr/``.
    ``rollout_rs`` other than ``None`` raises ``NotImplementedError``.
    """
    if old_log_prob.shape != rollout_log_prob.shape:
        raise ValueError(
            f"old_log_prob shape {old_log_prob.shape} does not match rollout_log_prob shape {rollout_log_prob.shape}."
        )
    if old_log_prob.shape != response_mask.shape:
        raise ValueError(
            f"log_prob shape {old_log_prob.shape} does not match response_mask shape {response_mask.shape}."
        )
    if rollout_rs is not None:
        raise NotImplementedError("rejection sampling (rollout_rs) is not part of verl_amd")
    use_is = rollout_is is not None and rollout_is_threshold is not None
    if use_is:
        _check_level(rollout_is, rollout_is_threshold)
    weights, values = _run(old_log_prob, rollout_log_prob, response_mask, _LEVELS[rollout_is] if use_is else 0,
                           rollout_is_threshold, rollout_is_batch_normalize)
    if values["_valid_tokens"] == 0:
        raise ValueError("response_mask must contain at least one valid token (1).")
    metrics = _is_metrics(values, rollout_is_batch_normalize) if use_is else {}
    metrics.update({k: values[k] for k in _OFFPOLICY})
    proto = types.SimpleNamespace(batch={"rollout_is_weights": weights}) if use_is else None
    return proto, response_mask.clone(), {f"rollout_corr/{k}": v for k, v in metrics.items()}
