"""``compute_data_metrics`` of the reference (verl/trainer/ppo/metric_utils.py:81-225) as one kernel
launch and one device-to-host copy instead of ~30 masked reductions with a ``.item()`` each, and
``compute_variance_proxy_metrics`` (:306-412) as one pass that leaves per-trajectory sums for the host.

``batch`` is anything shaped like the reference's ``DataProto``: ``batch.batch`` maps names to
tensors, ``batch.non_tensor_batch`` maps names to numpy arrays.
"""
from __future__ import annotations

import math
from typing import Any

import numpy as np
import torch

from ... import _cabi

# output slot -> metric name, in the order of the VAMD_DM_* constants of include/verl_amd.h
_SLOTS = (
    "critic/score/mean", "critic/score/max", "critic/score/min",
    "critic/rewards/mean", "critic/rewards/max", "critic/rewards/min",
    "critic/advantages/mean", "critic/advantages/max", "critic/advantages/min",
    "critic/returns/mean", "critic/returns/max", "critic/returns/min",
    "critic/values/mean", "critic/values/max", "critic/values/min",
    "critic/vf_explained_var",
    "response_length/mean", "response_length/max", "response_length/min", "response_length/clip_ratio",
    "response_length_non_aborted/mean", "response_length_non_aborted/max", "response_length_non_aborted/min",
    "response_length_non_aborted/clip_ratio",
    "response/aborted_ratio",
    "prompt_length/mean", "prompt_length/max", "prompt_length/min", "prompt_length/clip_ratio",
    "_valid_tokens", "_non_aborted",
)
_CRITIC_ONLY = ("critic/values/mean", "critic/values/max", "critic/values/min", "critic/vf_explained_var")


def compute_data_metrics(batch, use_critic: bool = True) -> dict[str, Any]:
    """Score / reward / advantage / return / value statistics and prompt / response length statistics of
    one training batch, with the reference's metric names.

    Reads ``token_level_scores``, ``token_level_rewards``, ``advantages``, ``returns``, ``responses`` (for
    its width), ``attention_mask``, ``response_mask`` and, with ``use_critic``, ``values``.  Sequence
    scores and rewards are unmasked row sums over the rows whose response length (from
    ``attention_mask``) is not zero; advantages, returns and values are taken where ``response_mask`` is
    set.  Raises ``ValueError`` when every sample is aborted, as the reference does, and
    ``RuntimeError`` when no token is valid (the reference's ``torch.max`` of an empty selection).
    """
    b = batch.batch
    scores = b["token_level_scores"]
    dev = _cabi.compute_device(scores, b["response_mask"], b["attention_mask"])
    width = b["responses"].shape[-1]
    sc = _cabi.as_f32(scores, dev)
    rows = sc.shape[0]
    assert sc.dim() == 2 and sc.shape[1] == width, f"token_level_scores {tuple(sc.shape)} vs response width {width}"
    tensors = [sc] + [_cabi.as_f32(b[k], dev) for k in ("token_level_rewards", "advantages", "returns")]
    values = _cabi.as_f32(b["values"], dev) if use_critic else None
    for t in tensors + ([values] if use_critic else []):
        assert t.shape == sc.shape
    mask, mcode = _cabi.mask_code(b["response_mask"].detach().to(dev))
    attention, acode = _cabi.mask_code(b["attention_mask"].detach().to(dev))
    assert tuple(mask.shape) == tuple(sc.shape) and attention.shape[0] == rows and attention.shape[1] >= width
    prompt = attention.shape[1] - width
    out = torch.empty(len(_SLOTS), dtype=torch.float64, device=dev)
    Lb = _cabi.lib()
    ws = _cabi.workspace(Lb.vamd_data_metrics_workspace_bytes(rows, width), dev)
    with _cabi.device_guard(dev):
        _cabi.check(Lb.vamd_data_metrics(tensors[0].data_ptr(), tensors[1].data_ptr(), tensors[2].data_ptr(),
                                         tensors[3].data_ptr(), _cabi.ptr(values), mask.data_ptr(), mcode,
                                         attention.data_ptr(), acode, rows, prompt, width, out.data_ptr(),
                                         ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
    got = dict(zip(_SLOTS, out.cpu().tolist()))          # the one host sync of the function
    if got.pop("_non_aborted") == 0:
        raise ValueError("All samples are aborted, this should not happen.")
    if got.pop("_valid_tokens") == 0:
        raise RuntimeError("max(): Expected reduction dim to be specified for input.numel() == 0. "
                           "Specify the reduction dim with the 'dim' argument.")
    if not use_critic:
        for key in _CRITIC_ONLY:
            del got[key]
    metrics = {k: (float("nan") if math.isnan(v) else float(v)) for k, v in got.items()}
    extra = getattr(batch, "non_tensor_batch", None) or {}
    for name in ("__num_turns__", "tool_call_counts"):   # host numpy arrays, :212-223
        if name in extra:
            label = "num_turns" if name == "__num_turns__" else name
            metrics[f"{label}/min"] = extra[name].min()
            metrics[f"{label}/max"] = extra[name].max()
            metrics[f"{label}/mean"] = extra[name].mean()
    return metrics


def compute_variance_proxy_metrics(batch, gradient_norm: float = None) -> dict[str, float]:
    """Gradient-variance proxies from the score-norm proxy ``W(tau) = sum_t (1 - 2 pi_t + sum pi^2)`` (reference
    :306-412): ``proxy2_total_power = E[A^2 W]`` with ``A`` the trajectory's mean advantage (with
    ``rollout_is_weights`` in the batch: ``E[rho^2 A^2 W_original]``), ``proxy1_signal_strength =
    gradient_norm^2``, ``proxy3_pure_noise = max(0, (proxy2 - proxy1) / (N - 1))``, plus ``expected_a_squared``
    and ``expected_w``.  Returns ``{}`` unless ``sum_pi_squared``, ``old_log_probs`` and ``advantages`` are in
    the batch."""
    b = batch.batch
    if "sum_pi_squared" not in b or "old_log_probs" not in b or "advantages" not in b:
        return {}
    adv_t = b["advantages"]
    dev = _cabi.compute_device(adv_t, b["response_mask"])
    adv = _cabi.as_f32(adv_t, dev)
    if adv.dim() == 1:
        adv = adv.view(1, -1)
    lp = _cabi.as_f32(b["old_log_probs"], dev).view(adv.shape)
    pi2 = _cabi.as_f32(b["sum_pi_squared"], dev).view(adv.shape)
    isw = _cabi.as_f32(b["rollout_is_weights"], dev).view(adv.shape) if "rollout_is_weights" in b else None
    mask, code = _cabi.mask_code(b["response_mask"].detach().to(dev))
    rows, cols = adv.shape
    Lb = _cabi.lib()
    chunks = int(Lb.vamd_rollout_rs_chunks(cols))
    rec = torch.empty(5 * chunks * rows, dtype=torch.float64, device=dev)
    with _cabi.device_guard(dev):
        _cabi.check(Lb.vamd_variance_proxy_rows(adv.data_ptr(), lp.data_ptr(), pi2.data_ptr(), _cabi.ptr(isw),
                                                mask.data_ptr(), code, rows, cols, rec.data_ptr(),
                                                _cabi.stream_ptr(dev)))
    t = rec.cpu().numpy().reshape(5, chunks, rows).sum(axis=1)      # the one host sync
    f32 = np.float32
    n = t[0].astype(f32) + f32(1e-8)                                # masked_mean's denominator
    a = t[1].astype(f32) / n
    w_sum = t[2].astype(f32)
    proxy1 = gradient_norm**2 if gradient_norm is not None else None
    if isw is not None:
        rho = t[3].astype(f32) / n
        proxy2 = float((rho**2 * a**2 * np.maximum(t[4].astype(f32), 0)).mean())
    else:
        proxy2 = float((a**2 * np.maximum(w_sum, 0)).mean())
    proxy3 = None
    if proxy1 is not None and rows > 1:
        proxy3 = max(0.0, (proxy2 - proxy1) / (rows - 1))
    return {
        "variance_proxy/proxy1_signal_strength": proxy1 if proxy1 is not None else 0.0,
        "variance_proxy/proxy2_total_power": proxy2,
        "variance_proxy/proxy3_pure_noise": proxy3 if proxy3 is not None else 0.0,
        "variance_proxy/expected_a_squared": float((a**2).mean()),
        "variance_proxy/expected_w": float(w_sum.mean()),
    }

