"""Rollout-correction importance weights and off-policy diagnostics, mirrored from the reference's
verl/trainer/ppo/rollout_corr_helper.py: ``compute_rollout_correction_weights`` (:481-598, with
``compute_is_metrics`` :601-712), ``compute_offpolicy_metrics`` (:835-937) and the unified
``compute_rollout_correction_and_rejection_mask`` (:715-832).

One kernel launch reads the log-probabilities and the mask once and produces the weights and all
metrics; the host reads the metric vector with a single copy.  Rejection sampling
(``compute_rollout_rejection_mask``, :163-357) is two streaming passes around a host step on a
``[batch]``-sized table, where the sequence-level options are decided.
"""
from __future__ import annotations

import ctypes
import math
import types
from typing import Any, Optional

import numpy as np
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
        mask, code = _cabi.mask_code(_cabi.on_device(response_mask, dev))
        mask = mask.view(old.shape)
        rows, cols = old.shape
        weights = torch.empty_like(old) if level else None
        out = torch.empty(len(_SLOTS), dtype=torch.float64, device=dev)
        Lb = _cabi.lib()
        ws = _cabi.workspace(Lb.vamd_rollout_correction_workspace_bytes(rows, cols), dev)
        with _cabi.device_guard(dev):
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
    holds the weights (``weights_proto`` is ``None`` when ``rollout_is`` is ``None``), the mask is
    ``response_mask`` with the tokens / sequences that ``rollout_rs`` rejects set to 0 (a copy when ``rollout_rs``
    is ``None``), and every metric name is prefixed with ``rollout_corr/``.
    """
    if old_log_prob.shape != rollout_log_prob.shape:
        raise ValueError(
            f"old_log_prob shape {old_log_prob.shape} does not match rollout_log_prob shape {rollout_log_prob.shape}."
        )
    if old_log_prob.shape != response_mask.shape:
        raise ValueError(
            f"log_prob shape {old_log_prob.shape} does not match response_mask shape {response_mask.shape}."
        )
    use_is = rollout_is is not None and rollout_is_threshold is not None
    if use_is:
        _check_level(rollout_is, rollout_is_threshold)
    weights, values = _run(old_log_prob, rollout_log_prob, response_mask, _LEVELS[rollout_is] if use_is else 0,
                           rollout_is_threshold, rollout_is_batch_normalize)
    if values["_valid_tokens"] == 0:
        raise ValueError("response_mask must contain at least one valid token (1).")
    metrics = _is_metrics(values, rollout_is_batch_normalize) if use_is else {}
    modified_response_mask = response_mask.clone()
    if rollout_rs is not None:
        if rollout_rs_threshold is None:
            raise ValueError(
                "rollout_rs_threshold must be explicitly provided when rollout_rs is enabled. "
                "Set rollout_rs_threshold to the desired threshold value."
            )
        modified_response_mask, rs_metrics = _rejection(old_log_prob, rollout_log_prob, response_mask, rollout_rs,
                                                        rollout_rs_threshold)
        metrics.update(rs_metrics)
    metrics.update({k: values[k] for k in _OFFPOLICY})
    proto = types.SimpleNamespace(batch={"rollout_is_weights": weights}) if use_is else None
    return proto, modified_response_mask, {f"rollout_corr/{k}": v for k, v in metrics.items()}


# ---- rejection sampling ------------------------------------------------------------------------------------------
SUPPORTED_ROLLOUT_RS_OPTIONS: set[str] = {
    "token_k1", "token_k2", "token_k3", "seq_sum_k1", "seq_sum_k2", "seq_sum_k3", "seq_mean_k1", "seq_mean_k2",
    "seq_mean_k3", "seq_max_k2", "seq_max_k3",
}
TOKEN_LEVEL_ROLLOUT_RS_OPTIONS: set[str] = {"token_k1", "token_k2", "token_k3"}
_ESTIMATOR = {"k1": 0, "k2": 1, "k3": 2}


def _parse_rollout_rs_thresholds(options: list[str], threshold_spec) -> dict[str, dict[str, Optional[float]]]:
    """One threshold shared by all options or one per option (comma separated); ``*k1`` options take
    ``lower_upper`` ratio bounds (``upper`` alone means ``lower = 1 / upper``), the others one upper bound
    (reference :94-160)."""
    if threshold_spec is None:
        raise ValueError("rollout_rs_threshold must be provided for rejection sampling.")
    if isinstance(threshold_spec, (int, float)):
        raw = [str(threshold_spec)]
    elif isinstance(threshold_spec, str):
        raw = [part.strip() for part in threshold_spec.split(",") if part.strip()]
    else:
        raise TypeError("rollout_rs_threshold must be a string or numeric value specifying per-option thresholds.")
    if not raw:
        raise ValueError("rollout_rs_threshold must contain at least one threshold value.")
    if len(raw) not in (1, len(options)):
        raise ValueError(
            f"rollout_rs_threshold expects either one threshold shared by all options or exactly "
            f"{len(options)} thresholds to match the provided rollout_rs options."
        )
    if len(raw) == 1:
        raw = raw * len(options)
    out: dict[str, dict[str, Optional[float]]] = {}
    for option, spec in zip(options, raw):
        two_sided = option.endswith("k1")
        if not two_sided and "_" in spec:
            raise ValueError(
                f"rollout_rs_threshold for option '{option}' must provide a single upper bound "
                f"without '_'. Received '{spec}'."
            )
        try:
            if two_sided and "_" in spec:
                lower, upper = (float(x) for x in spec.split("_", 1))
            else:
                upper = float(spec)
                lower = 1.0 / upper if two_sided else None
        except ValueError as exc:
            raise ValueError(f"Invalid numeric threshold '{spec}' for option '{option}'.") from exc
        if upper <= 0 or (lower is not None and lower <= 0):
            raise ValueError(f"Thresholds for option '{option}' must be positive, got {spec}.")
        out[option] = {"lower": lower, "upper": upper}
    return out


def _records(flat: torch.Tensor, slots: int, chunks: int, rows: int) -> np.ndarray:
    return flat.cpu().numpy().reshape(slots, chunks, rows)


def _sequence_summary(prefix, seq, upper, lower, two_sided, out):
    """The ``_seq_*`` metrics over the sequences that have tokens (reference :455-478)."""
    if seq.size > 0:
        out[f"{prefix}_seq_mean"] = float(seq.mean())
        out[f"{prefix}_seq_std"] = float(seq.std(ddof=1)) if seq.size > 1 else 0.0
        out[f"{prefix}_seq_max"] = float(seq.max())
        out[f"{prefix}_seq_min"] = float(seq.min())
        out[f"{prefix}_seq_max_deviation"] = float(np.abs(seq).max())
        out[f"{prefix}_seq_fraction_high"] = float((seq > upper).mean())
        if two_sided:
            out[f"{prefix}_seq_fraction_low"] = float((seq < lower).mean())
    else:
        for key in ("mean", "std", "max", "min", "max_deviation", "fraction_high", "fraction_low"):
            out[f"{prefix}_seq_{key}"] = 0.0


def _rejection(old_log_prob, rollout_log_prob, response_mask, rollout_rs, rollout_rs_threshold):
    if rollout_rs is None or not isinstance(rollout_rs, str):
        raise ValueError("rollout_rs must be a non-empty string (comma separated for multiple options).")
    if rollout_rs_threshold is None:
        raise ValueError("rollout_rs_threshold must be provided for rejection sampling.")
    if old_log_prob.shape[0] == 0:
        return response_mask, {}
    options: list[str] = []
    for opt in (o.strip() for o in rollout_rs.split(",")):
        if not opt:
            continue
        if opt not in SUPPORTED_ROLLOUT_RS_OPTIONS:
            raise ValueError(
                f"Invalid rollout_rs option: {opt}. Must be one of {sorted(SUPPORTED_ROLLOUT_RS_OPTIONS)}."
            )
        if opt not in options:
            options.append(opt)
    if not options:
        raise ValueError("rollout_rs must contain at least one valid option.")
    bounds = _parse_rollout_rs_thresholds(options, rollout_rs_threshold)

    with torch.no_grad():
        dev = _cabi.compute_device(old_log_prob, response_mask)
        old = _cabi.as_f32(old_log_prob, dev)
        if old.dim() == 1:
            old = old.view(1, -1)
        roll = _cabi.as_f32(rollout_log_prob, dev).view(old.shape)
        mask, code = _cabi.mask_code(_cabi.on_device(response_mask, dev))
        mask = mask.view(old.shape)
        rows, cols = old.shape
        Lb = _cabi.lib()
        chunks = int(Lb.vamd_rollout_rs_chunks(cols))
        stream = _cabi.stream_ptr(dev)
        # pass 1: per-sequence sums and maxima of the three estimates
        rec = torch.empty(6 * chunks * rows, dtype=torch.float64, device=dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_rollout_rs_row_stats(old.data_ptr(), roll.data_ptr(), mask.data_ptr(), code, rows, cols,
                                                     rec.data_ptr(), stream))
        table = _records(rec, 6, chunks, rows)                 # host sync 1
        count = table[0].sum(axis=0)
        total = float(count.sum())
        if total == 0:
            raise ValueError("response_mask must contain at least one valid token (1).")
        sums = {"k1": table[1].sum(axis=0), "k2": table[2].sum(axis=0), "k3": table[3].sum(axis=0)}
        tops = {"k2": table[4].max(axis=0), "k3": table[5].max(axis=0)}
        alive = count > 0
        n32 = count.astype(np.float32)
        denom = float(np.float32(total) + np.float32(1e-8))    # masked_mean over the batch
        f32 = np.float32

        def per_sequence(scope, est):
            if scope == "seq_sum":
                return sums[est].astype(f32)
            if scope == "seq_max":
                return np.where(np.isneginf(tops[est]), 0.0, tops[est]).astype(f32)
            return sums[est].astype(f32) / (n32 + f32(1e-8))   # seq_mean, and the per-sequence mean of a token option

        row_keep = np.ones(rows, dtype=bool)
        plan = []                                              # (option, scope, est, lower, upper, two_sided, keep or None)
        token_opts = []
        for opt in options:
            scope, est = opt.rsplit("_", 1)
            two_sided = est == "k1"
            lower = math.log(bounds[opt]["lower"]) if two_sided else 0.0
            upper = math.log(bounds[opt]["upper"]) if two_sided else bounds[opt]["upper"]
            keep = None
            if scope != "token":
                seq = per_sequence(scope, est)
                keep = (seq >= f32(lower)) & (seq <= f32(upper)) if two_sided else seq <= f32(upper)
                row_keep &= keep
            else:
                token_opts.append((opt, est, lower, upper))
            plan.append((opt, scope, est, lower, upper, two_sided, keep))
        # pass 2: the new mask and the token-level counts
        n_tok = len(token_opts)
        new_mask = torch.empty_like(mask)
        rec2 = torch.empty((1 + 8 * n_tok) * chunks * rows, dtype=torch.float64, device=dev)
        keep_dev = torch.from_numpy(row_keep.astype(np.uint8)).to(dev)
        est_arr = (ctypes.c_int * 3)(*[_ESTIMATOR[t[1]] for t in token_opts], *([0] * (3 - n_tok)))
        lo_arr = (ctypes.c_float * 3)(*[t[2] for t in token_opts], *([0.0] * (3 - n_tok)))
        hi_arr = (ctypes.c_float * 3)(*[t[3] for t in token_opts], *([0.0] * (3 - n_tok)))
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_rollout_rs_apply(old.data_ptr(), roll.data_ptr(), mask.data_ptr(), code, rows, cols,
                                                 keep_dev.data_ptr(), n_tok, ctypes.addressof(est_arr),
                                                 ctypes.addressof(lo_arr), ctypes.addressof(hi_arr),
                                                 new_mask.data_ptr(), rec2.data_ptr(), stream))
        table2 = _records(rec2, 1 + 8 * n_tok, chunks, rows)   # host sync 2

    metrics: dict[str, float] = {}
    n_alive = float(alive.sum())
    for opt, scope, est, lower, upper, two_sided, keep in plan:
        p = f"rollout_rs_{opt}"
        if scope == "token":
            j = [t[0] for t in token_opts].index(opt)
            t = table2[1 + 8 * j:1 + 8 * (j + 1)]
            seq = per_sequence("seq_mean", est)[alive]
            metrics[f"{p}_mean"] = float(t[0].sum()) / denom
            metrics[f"{p}_max"] = float(t[1].max())
            metrics[f"{p}_min"] = float(-t[2].max())
            metrics[f"{p}_fraction_high"] = float(t[3].sum()) / denom
            metrics[f"{p}_fraction_low"] = float(t[4].sum()) / denom if two_sided else 0.0
            mean_c, mean_c2 = float(t[5].sum()) / denom, float(t[6].sum()) / denom
            rejected_rows = t[7].sum(axis=0)
            masked_fraction = float(rejected_rows.sum()) / denom
            seq_rejected = (rejected_rows > 0) & alive
        else:
            full = per_sequence(scope, est).astype(np.float64)
            seq = full[alive]
            metrics[f"{p}_mean"] = float((full * count).sum()) / denom
            metrics[f"{p}_max"] = float(seq.max())
            metrics[f"{p}_min"] = float(seq.min())
            metrics[f"{p}_fraction_high"] = float((seq > upper).mean())
            metrics[f"{p}_fraction_low"] = float((seq < lower).mean()) if two_sided else 0.0
            c = np.clip(full, lower if two_sided else 0.0, upper)
            mean_c, mean_c2 = float((c * count).sum()) / denom, float((c * c * count).sum()) / denom
            masked_fraction = float(count[~keep].sum()) / denom
            seq_rejected = ~keep & alive
        metrics[f"{p}_std"] = math.sqrt(max(mean_c2 - mean_c * mean_c, 0.0)) if total > 1 else 0.0
        _sequence_summary(p, seq.astype(np.float64), upper, lower, two_sided, metrics)
        metrics[f"{p}_masked_fraction"] = masked_fraction
        metrics[f"{p}_seq_masked_fraction"] = float(seq_rejected.sum()) / n_alive if n_alive > 0 else 0.0
    dropped = table2[0].sum(axis=0)
    metrics["rollout_rs_masked_fraction"] = float(dropped.sum()) / denom
    metrics["rollout_rs_seq_masked_fraction"] = float((dropped > 0).mean())
    out_mask = new_mask.view(response_mask.shape).to(response_mask.device)
    if out_mask.dtype != response_mask.dtype:
        out_mask = out_mask.to(response_mask.dtype)
    return out_mask, metrics


def compute_rollout_rejection_mask(log_ratio: torch.Tensor, response_mask: torch.Tensor, rollout_rs: str = "token_k1",
                                   rollout_rs_threshold=None):
    """Hard trust-region mask from divergence estimates of the log ratio (reference :163-357): each comma
    separated option of ``rollout_rs`` keeps a token (``token_k{1,2,3}``) or a whole sequence
    (``seq_sum_*``, ``seq_mean_*``, ``seq_max_k{2,3}``) whose estimate lies inside its bounds; the options
    multiply.  Returns ``(modified_response_mask, metrics)`` with the reference's ``rollout_rs_*`` metric names."""
    return _rejection(log_ratio, torch.zeros_like(log_ratio), response_mask, rollout_rs, rollout_rs_threshold)


def compute_rollout_correction_and_add_to_batch(batch, rollout_corr_config):
    """Run the rollout correction on ``batch.batch["old_log_probs" / "rollout_log_probs" / "response_mask"]``
    with the settings of ``rollout_corr_config`` (``rollout_is``, ``rollout_is_threshold``,
    ``rollout_is_batch_normalize``, ``rollout_rs``, ``rollout_rs_threshold``): ``response_mask`` is always
    replaced by the mask after rejection, ``rollout_is_weights`` is added when ``rollout_is`` is set
    (reference :940-994).  Returns ``(batch, metrics)``."""
    proto, modified_response_mask, metrics = compute_rollout_correction_and_rejection_mask(
        old_log_prob=batch.batch["old_log_probs"], rollout_log_prob=batch.batch["rollout_log_probs"],
        response_mask=batch.batch["response_mask"], rollout_is=rollout_corr_config.get("rollout_is", None),
        rollout_is_threshold=rollout_corr_config.get("rollout_is_threshold", 2.0),
        rollout_is_batch_normalize=rollout_corr_config.get("rollout_is_batch_normalize", False),
        rollout_rs=rollout_corr_config.get("rollout_rs", None),
        rollout_rs_threshold=rollout_corr_config.get("rollout_rs_threshold", None))
    batch.batch["response_mask"] = modified_response_mask
    if proto is not None:
        batch.batch["rollout_is_weights"] = proto.batch["rollout_is_weights"]
    return batch, metrics


def compute_rollout_corr_metrics_from_logprobs(log_prob: torch.Tensor, rollout_log_prob: torch.Tensor,
                                               response_mask: torch.Tensor) -> dict[str, float]:
    """The off-policy diagnostics of the current policy against the rollout policy, with the ``rollout_corr/``
    prefix (reference :997-1031)."""
    return {f"rollout_corr/{k}": v for k, v in compute_offpolicy_metrics(log_prob, rollout_log_prob, response_mask).items()}

