"""PPO / GRPO policy math on MI355X.

Drop-ins for the functions of ``verl.trainer.ppo.core_algos`` that sit on the per-token hot path:
the two registries, GAE, GRPO (loop and vectorised forms), ``agg_loss``, the vanilla clipped /
dual-clip policy loss and the clipped value loss.  Signatures, return tuples, error types and
messages follow the reference (verl/trainer/ppo/core_algos.py); the arithmetic runs in
``libverl_amd.so``.  Inputs may be CPU tensors (the trainer computes advantages on the driver):
they are staged to the current GPU and results come back on the input's device.
"""
from __future__ import annotations

import collections

from enum import Enum
import warnings
from typing import Any, Callable, Optional

import numpy as np
import torch

from ... import _cabi
from ...utils import torch_functional as verl_F
from ...utils.groupwise import as_torch_index, contiguous_group_ids, group_mean_std  # noqa: F401

PolicyLossFn = Callable[..., tuple[torch.Tensor, dict[str, Any]]]

POLICY_LOSS_REGISTRY: dict[str, PolicyLossFn] = {}


def register_policy_loss(name: str) -> Callable[[PolicyLossFn], PolicyLossFn]:
    """Decorator: ``POLICY_LOSS_REGISTRY[name] = fn`` (reference core_algos.py:53-67)."""

    def decorator(func: PolicyLossFn) -> PolicyLossFn:
        POLICY_LOSS_REGISTRY[name] = func
        return func

    return decorator


def get_policy_loss_fn(name):
    """Look a policy loss up by name; unknown names raise ``ValueError`` with the reference's
    message (core_algos.py:70-85)."""
    loss_name = name
    if loss_name not in POLICY_LOSS_REGISTRY:
        raise ValueError(
            f"Unsupported loss mode: {loss_name}. Supported modes are: {list(POLICY_LOSS_REGISTRY.keys())}"
        )
    return POLICY_LOSS_REGISTRY[loss_name]


class AdvantageEstimator(str, Enum):
    """Names of the reference's advantage estimators (core_algos.py:88-109); every one is registered below."""

    GAE = "gae"
    GRPO = "grpo"
    REINFORCE_PLUS_PLUS = "reinforce_plus_plus"
    REINFORCE_PLUS_PLUS_BASELINE = "reinforce_plus_plus_baseline"
    REMAX = "remax"
    RLOO = "rloo"
    OPO = "opo"
    GRPO_PASSK = "grpo_passk"
    GPG = "gpg"
    RLOO_VECTORIZED = "rloo_vectorized"
    GRPO_VECTORIZED = "grpo_vectorized"
    OPTIMAL_TOKEN_BASELINE = "optimal_token_baseline"
    TIR_OPTIMAL_TOKEN_BASELINE = "tir_optimal_token_baseline"


ADV_ESTIMATOR_REGISTRY: dict[str, Any] = {}


def register_adv_est(name_or_enum) -> Any:
    """Decorator registering an advantage estimator; re-registering a name with a different
    function raises ``ValueError`` (reference core_algos.py:115-133)."""

    def decorator(fn):
        name = name_or_enum.value if isinstance(name_or_enum, Enum) else name_or_enum
        if name in ADV_ESTIMATOR_REGISTRY and ADV_ESTIMATOR_REGISTRY[name] != fn:
            raise ValueError(
                f"Adv estimator {name} has already been registered: {ADV_ESTIMATOR_REGISTRY[name]} vs {fn}"
            )
        ADV_ESTIMATOR_REGISTRY[name] = fn
        return fn

    return decorator


def get_adv_estimator_fn(name_or_enum):
    """Reference core_algos.py:136-149."""
    name = name_or_enum.value if isinstance(name_or_enum, Enum) else name_or_enum
    if name not in ADV_ESTIMATOR_REGISTRY:
        raise ValueError(f"Unknown advantage estimator simply: {name}")
    return ADV_ESTIMATOR_REGISTRY[name]


class AdaptiveKLController:
    """KL coefficient that tracks a target KL (reference core_algos.py:152-173): ``update`` multiplies
    ``value`` by ``1 + clip(current_kl / target - 1, -0.2, 0.2) * n_steps / horizon``."""

    def __init__(self, init_kl_coef, target_kl, horizon):
        self.value = init_kl_coef
        self.target = target_kl
        self.horizon = horizon

    def update(self, current_kl, n_steps):
        error = min(max(current_kl / self.target - 1, -0.2), 0.2)
        self.value *= 1 + error * n_steps / self.horizon


class FixedKLController:
    """Constant KL coefficient (reference core_algos.py:176-189); ``update`` does nothing."""

    def __init__(self, kl_coef):
        self.value = kl_coef

    def update(self, current_kl, n_steps):
        pass


def get_kl_controller(kl_ctrl):
    """Controller for ``kl_ctrl.type`` in {"fixed", "adaptive"} (reference core_algos.py:192-211)."""
    if kl_ctrl.type == "fixed":
        return FixedKLController(kl_coef=kl_ctrl.kl_coef)
    if kl_ctrl.type == "adaptive":
        assert kl_ctrl.horizon > 0, f"horizon must be larger than 0. Got {kl_ctrl.horizon}"
        return AdaptiveKLController(init_kl_coef=kl_ctrl.kl_coef, target_kl=kl_ctrl.target_kl,
                                    horizon=kl_ctrl.horizon)
    raise NotImplementedError


# ---------------------------------------------------------------------------------------------
def _matrix(t: torch.Tensor, dev: torch.device) -> torch.Tensor:
    x = _cabi.as_f32(t, dev)
    if x.dim() == 1:
        x = x.view(1, -1)
    assert x.dim() == 2, f"expected a (batch, length) tensor, got shape {tuple(t.shape)}"
    return x


def _mask_matrix(mask: torch.Tensor, dev: torch.device, shape) -> tuple[torch.Tensor, int]:
    m, code = _cabi.mask_code(_cabi.on_device(mask, dev))
    if m.dim() == 1:
        m = m.view(1, -1)
    assert tuple(m.shape) == tuple(shape), f"mask shape {tuple(mask.shape)} does not match {tuple(shape)}"
    return m, code


_WARNED = set()




def _warn_once(text: str) -> None:
    if text not in _WARNED:
        _WARNED.add(text)
        warnings.warn(text, RuntimeWarning, stacklevel=3)


@register_adv_est(AdvantageEstimator.GAE)
def compute_gae_advantage_return(token_level_rewards: torch.Tensor, values: torch.Tensor,
                                 response_mask: torch.Tensor, gamma, lam):
    """GAE with state carried over masked tokens, then ``masked_whiten`` of the advantages.

    Args / returns as in the reference (core_algos.py:214-262): all ``(bs, response_length)``;
    returns ``(advantages, returns)`` with ``returns = raw advantages + values``.  Runs under
    ``no_grad``.  The recurrence is evaluated as a parallel scan of affine maps, so results agree
    with the sequential fp32 loop to rounding, not bit for bit.
    """
    with torch.no_grad():
        dev = _cabi.compute_device(token_level_rewards, values, response_mask)
        r = _matrix(token_level_rewards, dev)
        v = _matrix(values, dev)
        assert r.shape == v.shape
        m, code = _mask_matrix(response_mask, dev, r.shape)
        B, Lc = r.shape
        adv = torch.empty_like(r)
        ret = torch.empty_like(r)
        mom = torch.empty(5, dtype=torch.float64, device=dev)
        Lb = _cabi.lib()
        ws = _cabi.ticket_workspace(Lb.vamd_gae_workspace_bytes(B, Lc), dev)
        # 1: one launch whose workgroups meet once (the library itself takes the two-launch form when waiting kernels
        # are switched off); 2: two launches, nobody waits.  Once the meeting has timed out in this process (a GPU
        # shared with long-running kernels) the waiting kernels are switched off for the whole library -- GRPO and the
        # sequence-level losses included: a time-out costs about a second of polling, and the conditions that caused it
        # rarely go away between two calls.
        for whiten in (1, 2):
            with _cabi.device_guard(dev):
                _cabi.check(Lb.vamd_gae(r.data_ptr(), v.data_ptr(), m.data_ptr(), code, B, Lc, float(gamma),
                                        float(lam), whiten, adv.data_ptr(), ret.data_ptr(), mom.data_ptr(),
                                        ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
            mom_host = mom.tolist()
            if mom_host[4] == 0.0:
                break
            # the workgroups' bounded wait for each other ran out (a GPU shared with long-running kernels): the
            # advantages were left unwhitened; do it again without waiting
            Lb.vamd_set_waiting_kernels(0)
            _warn_once("vamd_gae: the one-launch estimator timed out waiting for its workgroups; kernels that wait "
                       "inside a launch are switched off from now on (set VAMD_WAITING_KERNELS=0 to make that the "
                       "rule from the start)")
        verl_F._raise_on_tiny_mask(mom_host[0])
        if mom_host[4] != 0.0:
            raise RuntimeError("vamd_gae: the workgroups' bounded wait for the whitening statistics ran out; "
                               "the advantages were left unwhitened")
        out_dev = token_level_rewards.device
        return adv.view(token_level_rewards.shape).to(out_dev), ret.view(token_level_rewards.shape).to(out_dev)


# GRPO and the sequence-level losses recover from a wait that ran out inside their kernels and tell nobody; the
# kernels count such workgroups in their counter buffer, and every _WAITING_CHECK_EVERY-th call looks at the count
# (four bytes read back: a synchronisation, hence not on every call).  A count that has grown switches the waiting
# kernels off for the process, like a time-out of GAE does.
_WAITING_CHECK_EVERY = 64
_WAITING_WATCH = {"calls": 0, "seen": {}}


def _watch_waiting_kernels(ticket_ws: torch.Tensor) -> None:
    _WAITING_WATCH["calls"] += 1
    if _WAITING_WATCH["calls"] % _WAITING_CHECK_EVERY:
        return
    if torch.cuda.is_current_stream_capturing() or not _cabi.lib().vamd_waiting_kernels_enabled():
        return
    count = _cabi.waiting_gave_up(ticket_ws)
    # the first look at a buffer only notes where its count stands; growth after that is what counts
    if count > _WAITING_WATCH["seen"].get(ticket_ws.data_ptr(), count):
        _cabi.lib().vamd_set_waiting_kernels(0)
        _warn_once("workgroups of a kernel that waits inside its launch gave up waiting (a GPU shared with "
                   "long-running kernels); such kernels are switched off from now on (set VAMD_WAITING_KERNELS=0 to "
                   "make that the rule from the start)")
    _WAITING_WATCH["seen"][ticket_ws.data_ptr()] = count


_GROUP_ID_CACHE: "collections.OrderedDict" = collections.OrderedDict()
_GROUP_ID_CACHE_SIZE = 8


def _group_ids_on_device(index, vectorized: bool, dev: torch.device):
    """``contiguous_group_ids(index)`` as a device tensor, and the number of groups.  The trainer hands the same
    ``uid`` array to every estimator call of a step, and factorising the labels plus copying 4 KB to the device
    costs more than the advantage kernel itself, so the last few results are kept, keyed by the labels' content
    (numpy arrays: dtype, shape and raw bytes -- for object arrays the bytes are the addresses of the label
    objects, which the kept array keeps alive).  Anything else is factorised afresh."""
    key = None
    if isinstance(index, np.ndarray):
        # the bytes themselves, not their hash: a dictionary compares keys in full, so two label arrays can never
        # be taken for each other
        key = (index.dtype.str, index.shape, index.tobytes(), bool(vectorized), dev)
        hit = _GROUP_ID_CACHE.get(key)
        if hit is not None:
            _GROUP_ID_CACHE.move_to_end(key)
            return hit[0], hit[1]
    ids, G = contiguous_group_ids(index, vectorized=vectorized)
    ids = ids.to(dev)
    if key is not None:
        _GROUP_ID_CACHE[key] = (ids, G, index)
        while len(_GROUP_ID_CACHE) > _GROUP_ID_CACHE_SIZE:
            _GROUP_ID_CACHE.popitem(last=False)
    return ids, G


def _grpo(token_level_rewards, response_mask, index, epsilon, norm_adv_by_std_in_grpo, std_mode):
    with torch.no_grad():
        dev = _cabi.compute_device(token_level_rewards, response_mask)
        r = _matrix(token_level_rewards, dev)
        m, code = _mask_matrix(response_mask, dev, r.shape)
        B, Lc = r.shape
        ids, G = _group_ids_on_device(index, std_mode == 1, dev)
        if ids.numel() != B:
            raise ValueError(f"index has {ids.numel()} entries for a batch of {B}")
        adv = torch.empty_like(r)
        Lb = _cabi.lib()
        ws = _cabi.ticket_workspace(Lb.vamd_grpo_workspace_bytes(B, Lc, G), dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_grpo_advantage(r.data_ptr(), m.data_ptr(), code, ids.data_ptr(), B, Lc, G,
                                               float(epsilon), int(bool(norm_adv_by_std_in_grpo)), std_mode,
                                               adv.data_ptr(), None, ws.data_ptr(), ws.numel(),
                                               _cabi.stream_ptr(dev)))
        _watch_waiting_kernels(ws)
        out = adv.view(token_level_rewards.shape).to(token_level_rewards.device)
        return out, out


@register_adv_est(AdvantageEstimator.GRPO)
def compute_grpo_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor,
                                   index: np.ndarray, epsilon: float = 1e-6,
                                   norm_adv_by_std_in_grpo: bool = True, config: Optional[Any] = None):
    """Outcome-reward GRPO advantage (reference core_algos.py:266-330).

    Score = unmasked row sum of ``token_level_rewards``; per group ``mean`` and unbiased ``std``
    (a single-member group uses mean 0, std 1); ``(score - mean) / (std + epsilon)`` (or without
    the division) broadcast over the row and multiplied by ``response_mask``.  ``index`` may hold
    any hashable labels.  Returns the same tensor twice, like the reference.
    """
    return _grpo(token_level_rewards, response_mask, index, epsilon, norm_adv_by_std_in_grpo, std_mode=0)


@register_adv_est(AdvantageEstimator.GRPO_VECTORIZED)
def compute_grpo_vectorized_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor,
                                              index: np.ndarray, epsilon: float = 1e-6,
                                              norm_adv_by_std_in_grpo: bool = True, config: Optional[Any] = None):
    """Vectorised twin (reference core_algos.py:333-357): std = sqrt(clamp(var, min=epsilon))."""
    return _grpo(token_level_rewards, response_mask, index, epsilon, norm_adv_by_std_in_grpo, std_mode=1)


# ---- the other outcome estimators of the registry ----------------------------------------------
_ADV = {"grpo": 0, "rloo": 1, "rloo_vectorized": 2, "mean_baseline": 3, "opo": 4, "gpg": 5, "grpo_passk": 6}


def _group_outcome(token_level_rewards, response_mask, index, estimator: str, epsilon=1e-6, f_norm=1.0,
                   whiten_after=False, norm_by_std=True, min_group_size=1):
    """Score per response -> statistic of its prompt group -> one scalar per response -> scalar * mask
    (``vamd_group_outcome_advantage``); ``whiten_after`` adds ``masked_whiten(.) * mask``."""
    with torch.no_grad():
        dev = _cabi.compute_device(token_level_rewards, response_mask)
        r = _matrix(token_level_rewards, dev)
        m, code = _mask_matrix(response_mask, dev, r.shape)
        B, Lc = r.shape
        ids, G = contiguous_group_ids(index, vectorized=estimator == "rloo_vectorized")
        if ids.numel() != B:
            raise ValueError(f"index has {ids.numel()} entries for a batch of {B}")
        if min_group_size > 1:
            counts = torch.bincount(ids, minlength=G)
            small = (counts < min_group_size).nonzero()
            if small.numel():
                where = (ids == small[0, 0]).nonzero()[0, 0].item()
                raise ValueError(f"Pass@k requires at least 2 samples per group. Got {int(counts[small[0, 0]])} "
                                 f"for group {index[where]}.")
        ids = ids.to(dev)
        adv = torch.empty_like(r)
        Lb = _cabi.lib()
        ws = _cabi.ticket_workspace(Lb.vamd_group_outcome_advantage_workspace_bytes(B, Lc, G), dev)
        with _cabi.device_guard(dev):
            s = _cabi.stream_ptr(dev)
            _cabi.check(Lb.vamd_group_outcome_advantage(r.data_ptr(), m.data_ptr(), code, ids.data_ptr(), B, Lc, G,
                                                        _ADV[estimator], float(epsilon), int(bool(norm_by_std)), 0,
                                                        float(f_norm),
                                                        adv.data_ptr(), None, ws.data_ptr(), ws.numel(), s))
            if whiten_after:
                mom = verl_F._moments(adv, m, per_row=False)
                verl_F._raise_on_tiny_mask(float(mom[0].item()))
                stats = torch.empty(4, dtype=torch.float32, device=dev)
                _cabi.check(Lb.vamd_whiten_stats(mom.data_ptr(), 1, stats.data_ptr(), s))
                _cabi.check(Lb.vamd_affine_by_stats_masked(adv.data_ptr(), stats.data_ptr(), m.data_ptr(), code,
                                                           adv.numel(), adv.data_ptr(), s))
        out = adv.view(token_level_rewards.shape).to(token_level_rewards.device)
        return out, out


@register_adv_est(AdvantageEstimator.GRPO_PASSK)
def compute_grpo_passk_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor, index,
                                         epsilon: float = 1e-6, norm_adv_by_std_in_grpo: bool = True,
                                         config: Optional[Any] = None, **kwargs):
    """Pass@k advantage (reference core_algos.py:360-418): only the best response of a prompt group gets a
    non-zero advantage, ``max - second max`` of the group's scores, divided by ``std + epsilon`` when
    ``config.get("norm_adv_by_std_in_grpo", True)`` (the argument of the same name is overridden by the
    config, as there, :388).  Every group needs at least two responses (``ValueError`` otherwise)."""
    assert config is not None
    norm = _cfg_get(config, "norm_adv_by_std_in_grpo", True)
    return _group_outcome(token_level_rewards, response_mask, index, "grpo_passk", epsilon, norm_by_std=norm,
                          min_group_size=2)


@register_adv_est(AdvantageEstimator.REINFORCE_PLUS_PLUS_BASELINE)
def compute_reinforce_plus_plus_baseline_outcome_advantage(token_level_rewards: torch.Tensor,
                                                           response_mask: torch.Tensor, index, epsilon: float = 1e-6,
                                                           config: Optional[Any] = None, **kwargs):
    """REINFORCE++ with a group-mean baseline (reference core_algos.py:421-474): score minus the
    mean of its prompt group (0 for a single member), on the mask, whitened over all valid tokens,
    on the mask again.  Returns one tensor twice."""
    return _group_outcome(token_level_rewards, response_mask, index, "mean_baseline", epsilon, whiten_after=True)


@register_adv_est(AdvantageEstimator.RLOO)
def compute_rloo_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor, index,
                                   epsilon: float = 1e-6, config: Optional[Any] = None, **kwargs):
    """Leave-one-out baseline (reference core_algos.py:479-528); a single-member group keeps its score."""
    return _group_outcome(token_level_rewards, response_mask, index, "rloo", epsilon)


@register_adv_est(AdvantageEstimator.RLOO_VECTORIZED)
def compute_rloo_vectorized_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor, index,
                                              epsilon: float = 1e-6, config: Optional[Any] = None, **kwargs):
    """Vectorised RLOO (reference core_algos.py:720-753); a single-member group gets 0."""
    return _group_outcome(token_level_rewards, response_mask, index, "rloo_vectorized", epsilon)


@register_adv_est(AdvantageEstimator.OPO)
def compute_opo_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor, index,
                                  epsilon: float = 1e-6, config: Optional[Any] = None, **kwargs):
    """Length-weighted group baseline (reference core_algos.py:531-579)."""
    return _group_outcome(token_level_rewards, response_mask, index, "opo", epsilon)


@register_adv_est(AdvantageEstimator.GPG)
def compute_gpg_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor, index,
                                  epsilon: float = 1e-6, f_norm: float = 1.0, alpha: float = 1.0, config=None,
                                  **kwargs):
    """GPG (reference core_algos.py:657-717): ``alpha (score - group mean) / f_norm`` where ``alpha`` is
    recomputed as ``batch / max(#{score != 0}, 1)`` whatever the argument says, as there (:697-698)."""
    return _group_outcome(token_level_rewards, response_mask, index, "gpg", epsilon, f_norm=f_norm)


def _returns_advantage(token_level_rewards, response_mask, mode: int, gamma: float, baselines=None):
    with torch.no_grad():
        dev = _cabi.compute_device(token_level_rewards, response_mask)
        r = _matrix(token_level_rewards, dev)
        m, code = _mask_matrix(response_mask, dev, r.shape)
        B, Lc = r.shape
        base = None
        if baselines is not None:
            base = _cabi.as_f32(baselines, dev).reshape(-1).contiguous()
            assert base.numel() == B, f"reward_baselines has {base.numel()} entries for a batch of {B}"
        adv = torch.empty_like(r)
        ret = torch.empty_like(r)
        mom = torch.empty(4, dtype=torch.float64, device=dev)
        Lb = _cabi.lib()
        ws = _cabi.ticket_workspace(Lb.vamd_returns_advantage_workspace_bytes(B, Lc), dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_returns_advantage(r.data_ptr(), m.data_ptr(), code, _cabi.ptr(base), B, Lc,
                                                  float(gamma), mode, adv.data_ptr(), ret.data_ptr(), mom.data_ptr(),
                                                  ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
        if mode == 1:
            verl_F._raise_on_tiny_mask(float(mom[0].item()))
        shape, out_dev = token_level_rewards.shape, token_level_rewards.device
        return adv.view(shape).to(out_dev), ret.view(shape).to(out_dev)


@register_adv_est(AdvantageEstimator.REINFORCE_PLUS_PLUS)
def compute_reinforce_plus_plus_outcome_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor,
                                                  config: Optional[Any] = None, **kwargs):
    """REINFORCE++ (reference core_algos.py:582-618): discounted return that restarts after a masked
    step, whitened over the valid tokens and masked.  ``config.gamma`` is required, as there.
    Returns ``(advantages, returns)``."""
    assert config is not None
    return _returns_advantage(token_level_rewards, response_mask, 1, float(config.gamma))


@register_adv_est(AdvantageEstimator.REMAX)
def compute_remax_outcome_advantage(token_level_rewards: torch.Tensor, reward_baselines: torch.Tensor,
                                    response_mask: torch.Tensor, config: Optional[Any] = None, **kwargs):
    """ReMax (reference core_algos.py:621-654): reverse cumulative sum of the masked rewards minus the
    greedy-rollout baseline of the response on its mask.  Returns ``(advantages, returns)``."""
    return _returns_advantage(token_level_rewards, response_mask, 0, 1.0, baselines=reward_baselines)


def _optimal_token_baseline(token_level_rewards, response_mask, index, old_log_probs, sum_pi_squared,
                            rollout_is_weights, handle_zero_tail, epsilon, packed):
    """Both optimal-token-baseline estimators (``vamd_otb_advantage``).  The host part is the grouping: the
    rows sorted by prompt, and, for ``handle_zero_tail``, the column from which the longest trajectory of
    a group stands alone."""
    with torch.no_grad():
        dev = _cabi.compute_device(token_level_rewards, response_mask, old_log_probs, sum_pi_squared)
        r = _matrix(token_level_rewards, dev)
        m, code = _mask_matrix(response_mask, dev, r.shape)
        lp = _matrix(old_log_probs, dev)
        q = _matrix(sum_pi_squared, dev)
        assert lp.shape == r.shape and q.shape == r.shape
        isw = None
        if rollout_is_weights is not None:
            isw = _matrix(rollout_is_weights, dev)
            assert isw.shape == r.shape
        B, Lc = r.shape
        ids, _ = contiguous_group_ids(index)
        if ids.numel() != B:
            raise ValueError(f"index has {ids.numel()} entries for a batch of {B}")
        ids = ids.numpy()
        lengths = None
        if packed or handle_zero_tail:
            lengths = verl_F._moments(r, m, per_row=True)[0].cpu().numpy().astype(np.int64)
        rows = np.argsort(ids, kind="stable")
        if packed:  # trajectories without a valid token leave their group
            rows = rows[lengths[rows] > 0]
        sorted_ids = ids[rows]
        starts = np.flatnonzero(np.r_[True, sorted_ids[1:] != sorted_ids[:-1]]) if rows.size else np.zeros(0, np.int64)
        offsets = np.r_[starts, rows.size].astype(np.int64)
        G = len(offsets) - 1
        tail = None
        if handle_zero_tail:
            tail = np.full(B, Lc, dtype=np.int64)
            for g in range(G):
                members = rows[offsets[g]:offsets[g + 1]]
                if members.size < 2:
                    continue
                order = np.argsort(lengths[members], kind="stable")
                longest, second = lengths[members[order[-1]]], lengths[members[order[-2]]]
                if longest > second:
                    tail[members[order[-1]]] = second
            tail = torch.from_numpy(tail).to(dev)
        rows_t = torch.from_numpy(rows.astype(np.int64)).to(dev) if G else None
        offs_t = torch.from_numpy(offsets).to(dev) if G else None
        adv = torch.empty_like(r)
        ret = torch.empty_like(r)
        Lb = _cabi.lib()
        ws = _cabi.workspace(Lb.vamd_otb_advantage_workspace_bytes(B, Lc, int(packed)), dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_otb_advantage(r.data_ptr(), m.data_ptr(), code, lp.data_ptr(), q.data_ptr(),
                                              _cabi.ptr(isw), _cabi.ptr(rows_t), _cabi.ptr(offs_t), _cabi.ptr(tail),
                                              B, Lc, G, int(packed), float(epsilon), adv.data_ptr(), ret.data_ptr(),
                                              ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
        shape, out_dev = token_level_rewards.shape, token_level_rewards.device
        return adv.view(shape).to(out_dev), ret.view(shape).to(out_dev)


@register_adv_est(AdvantageEstimator.OPTIMAL_TOKEN_BASELINE)
def compute_optimal_token_baseline_advantage(token_level_rewards: torch.Tensor, response_mask: torch.Tensor,
                                             index: np.ndarray, old_log_probs: torch.Tensor,
                                             sum_pi_squared: torch.Tensor, rollout_is_weights: torch.Tensor = None,
                                             handle_zero_tail: bool = False, epsilon: float = 1e-8,
                                             config: Optional[Any] = None):
    """Optimal token baseline (reference core_algos.py:756-873): per prompt group and column
    ``B_t = sum(G_t W_t) / (sum(W_t) + epsilon)`` over the group's trajectories, with ``G`` the reward to go
    and ``W`` the running sum of ``1 - 2 pi_t + sum pi^2`` (times the squared importance weights when given);
    ``advantages = (G - B) * mask``, a lone trajectory keeps ``G``.  ``handle_zero_tail`` drops the baseline
    of a group's single longest trajectory beyond the second-longest length.  ``sum_pi_squared`` is what
    ``linear_cross_entropy_with_sum_pi_squared`` returns.  ``config`` is accepted and unused (the trainer's
    dispatcher passes it to every estimator).  Returns ``(advantages, returns)``."""
    return _optimal_token_baseline(token_level_rewards, response_mask, index, old_log_probs, sum_pi_squared,
                                   rollout_is_weights, handle_zero_tail, epsilon, packed=False)


@register_adv_est(AdvantageEstimator.TIR_OPTIMAL_TOKEN_BASELINE)
def compute_multi_turn_optimal_token_baseline_advantage(token_level_rewards: torch.Tensor,
                                                        response_mask: torch.Tensor, index: np.ndarray,
                                                        old_log_probs: torch.Tensor, sum_pi_squared: torch.Tensor,
                                                        rollout_is_weights: torch.Tensor = None,
                                                        handle_zero_tail: bool = True, epsilon: float = 1e-8,
                                                        config: Optional[Any] = None):
    """Optimal token baseline for tool-integrated (multi-turn) rollouts (reference core_algos.py:876-1004):
    the valid tokens of each trajectory are packed together first, so the k-th generated token of every
    trajectory shares a baseline whatever tool output lies in between; trajectories without a valid token
    do not count towards their group.  Returns ``(advantages, returns)``."""
    return _optimal_token_baseline(token_level_rewards, response_mask, index, old_log_probs, sum_pi_squared,
                                   rollout_is_weights, handle_zero_tail, epsilon, packed=True)


# ---------------------------------------------------------------------------------------------
def _agg_mode(loss_agg_mode: str) -> int:
    if loss_agg_mode not in _cabi.AGG_MODES:
        raise ValueError(f"Invalid loss_agg_mode: {loss_agg_mode}")
    return _cabi.AGG_MODES[loss_agg_mode]


def _opt(x) -> float:
    """``None`` -> -1 (the C ABI's "not given"); tensors and numbers -> float."""
    if x is None:
        return -1.0
    return float(x.item()) if isinstance(x, torch.Tensor) else float(x)


class _AggLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, loss_mat, loss_mask, mode, dp_size, bnt, gbs, lsf):
        dev = _cabi.compute_device(loss_mat, loss_mask)
        x = _matrix(loss_mat, dev)
        m, code = _mask_matrix(loss_mask, dev, x.shape)
        rows, cols = x.shape
        Lb = _cabi.lib()
        out = torch.empty((), dtype=torch.float32, device=dev)
        coef = torch.empty(rows, dtype=torch.float32, device=dev)
        ws = _cabi.ticket_workspace(Lb.vamd_agg_loss_workspace_bytes(rows, cols), dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_agg_loss_forward(x.data_ptr(), m.data_ptr(), code, rows, cols, mode, dp_size, bnt,
                                                 gbs, lsf, out.data_ptr(), coef.data_ptr(), ws.data_ptr(),
                                                 ws.numel(), _cabi.stream_ptr(dev)))
        ctx.save_for_backward(coef, m)
        ctx.code = code
        ctx.in_shape = loss_mat.shape
        ctx.in_device = loss_mat.device
        ctx.in_dtype = loss_mat.dtype
        return out.to(loss_mat.device)

    @staticmethod
    def backward(ctx, d_loss):
        coef, m = ctx.saved_tensors
        dev = coef.device
        rows, cols = m.shape
        g = torch.empty((rows, cols), dtype=torch.float32, device=dev)
        d = _cabi.as_f32(d_loss, dev).reshape(1)
        with _cabi.device_guard(dev):
            _cabi.check(_cabi.lib().vamd_agg_loss_backward(d.data_ptr(), coef.data_ptr(), m.data_ptr(), ctx.code,
                                                           rows, cols, g.data_ptr(), _cabi.stream_ptr(dev)))
        g = g.view(ctx.in_shape).to(device=ctx.in_device, dtype=ctx.in_dtype)
        return g, None, None, None, None, None, None


def agg_loss(loss_mat: torch.Tensor, loss_mask: torch.Tensor, loss_agg_mode: str, dp_size: int = 1,
             batch_num_tokens: Optional[int] = None, global_batch_size: Optional[int] = None,
             loss_scale_factor: Optional[int] = None):
    """Aggregate a ``(bs, response_length)`` loss matrix to a scalar (reference
    core_algos.py:1025-1080): ``token-mean``, ``seq-mean-token-sum``, ``seq-mean-token-mean`` or
    ``seq-mean-token-sum-norm``; any other mode raises ``ValueError``.  Differentiable with
    respect to ``loss_mat``."""
    mode = _agg_mode(loss_agg_mode)
    return _AggLoss.apply(loss_mat, loss_mask, mode, float(dp_size), _opt(batch_num_tokens),
                          _opt(global_batch_size), _opt(loss_scale_factor))


# ---------------------------------------------------------------------------------------------
class _NoGradContext:
    """What a loss Function's ``forward`` sees in place of an autograd context when nothing asks for a gradient."""
    needs_input_grad = (False,) * 16

    def save_for_backward(self, *tensors):
        pass

    def mark_non_differentiable(self, *tensors):
        pass


def _apply_loss(fn, differentiable_input, *rest):
    """``fn.apply`` when the one differentiable input requires a gradient; otherwise ``fn.forward`` called directly,
    which skips the Function machinery (argument wrapping, context, output bookkeeping: about 5 us of a 40 us
    call)."""
    if torch.is_grad_enabled() and differentiable_input.requires_grad:
        return fn.apply(differentiable_input, *rest)
    return fn.forward(_NoGradContext(), differentiable_input, *rest)


class _PolicyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_prob, old_log_prob, advantages, response_mask, is_weights, clip_low, clip_high, clip_c,
                mode, dp_size, bnt, gbs, lsf, variant=0, tau_pos=1.0, tau_neg=1.0):
        dev = _cabi.compute_device(log_prob, old_log_prob, advantages, response_mask)
        lp = _matrix(log_prob, dev)
        old = _matrix(old_log_prob, dev)
        adv = _matrix(advantages, dev)
        assert lp.shape == old.shape == adv.shape
        m, code = _mask_matrix(response_mask, dev, lp.shape)
        isw = _matrix(is_weights, dev) if is_weights is not None else None
        rows, cols = lp.shape
        need_grad = ctx.needs_input_grad[0]
        Lb = _cabi.lib()
        # one allocation for the four result floats and the per-row coefficients (16-byte aligned both)
        buf = torch.empty(4 + rows, dtype=torch.float32, device=dev)
        out, coef = buf[:4], buf[4:]
        g = torch.empty_like(lp) if need_grad else None
        ws = _cabi.ticket_workspace(Lb.vamd_policy_loss_variant_workspace_bytes(rows, cols), dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_policy_loss_variant_forward(variant, old.data_ptr(), lp.data_ptr(), adv.data_ptr(),
                                                            m.data_ptr(), code, _cabi.ptr(isw), rows, cols, clip_low,
                                                            clip_high, clip_c, tau_pos, tau_neg, mode, dp_size, bnt,
                                                            gbs, lsf, out.data_ptr(), _cabi.ptr(g), coef.data_ptr(),
                                                            ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
        if variant in (_PL["gspo"], _PL["geo_mean"]):
            _watch_waiting_kernels(ws)
        if need_grad:
            ctx.save_for_backward(g, coef)
        ctx.in_shape = log_prob.shape
        ctx.in_device = log_prob.device
        ctx.in_dtype = log_prob.dtype
        out = out.to(log_prob.device)
        ctx.mark_non_differentiable(out)
        return out[0], out   # a view: the loss and the metrics share the floats the kernel wrote

    @staticmethod
    def backward(ctx, d_loss, _d_out):
        g, coef = ctx.saved_tensors
        dev = g.device
        rows, cols = g.shape
        d = _cabi.as_f32(d_loss, dev).reshape(1)
        res = torch.empty_like(g)
        with _cabi.device_guard(dev):
            _cabi.check(_cabi.lib().vamd_scale_rows(g.data_ptr(), coef.data_ptr(), d.data_ptr(), 1.0, rows, cols,
                                                    res.data_ptr(), _cabi.stream_ptr(dev)))
        res = res.view(ctx.in_shape).to(device=ctx.in_device, dtype=ctx.in_dtype)
        return (res,) + (None,) * 15


def _cfg_get(config, key, default=None):
    getter = getattr(config, "get", None)
    if callable(getter):
        return getter(key, default)
    return getattr(config, key, default)


@register_policy_loss("vanilla")
def compute_policy_loss_vanilla(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                                response_mask: torch.Tensor, loss_agg_mode: str = "token-mean",
                                config: Optional[Any] = None, rollout_is_weights: torch.Tensor | None = None):
    """Clipped PPO objective with the dual-clip floor (reference core_algos.py:1159-1250).

    ``config`` needs ``clip_ratio``, optional ``clip_ratio_low`` / ``clip_ratio_high``,
    ``get("clip_ratio_c", 3.0)`` and a ``global_batch_info`` dict that is forwarded to
    ``agg_loss``.  Returns ``(pg_loss, metrics)`` with ``actor/pg_clipfrac``, ``actor/ppo_kl``
    and ``actor/pg_clipfrac_lower`` as Python floats.  One fused kernel pass produces the loss,
    the three metrics and the gradient with respect to ``log_prob``.
    """
    assert config is not None
    clip_ratio = config.clip_ratio
    low = getattr(config, "clip_ratio_low", None)
    high = getattr(config, "clip_ratio_high", None)
    clip_ratio_low = low if low is not None else clip_ratio
    clip_ratio_high = high if high is not None else clip_ratio
    clip_ratio_c = _cfg_get(config, "clip_ratio_c", 3.0)
    assert clip_ratio_c > 1.0, (
        "The lower bound of the clip_ratio_c for dual-clip PPO should be greater than 1.0,"
        + f" but get the value: {clip_ratio_c}."
    )
    info = dict(getattr(config, "global_batch_info", None) or {})
    mode = _agg_mode(loss_agg_mode)
    pg_loss, out = _apply_loss(
        _PolicyLoss, log_prob, old_log_prob, advantages, response_mask, rollout_is_weights, float(clip_ratio_low),
        float(clip_ratio_high), float(clip_ratio_c), mode, float(info.get("dp_size", 1)),
        _opt(info.get("batch_num_tokens")), _opt(info.get("global_batch_size")), _opt(info.get("loss_scale_factor")))
    vals = out.detach().tolist()
    pg_metrics = {
        "actor/pg_clipfrac": vals[1],
        "actor/ppo_kl": vals[2],
        "actor/pg_clipfrac_lower": vals[3],
    }
    return pg_loss, pg_metrics


_PL = {"vanilla": 0, "gpg": 1, "cispo": 2, "sapo": 3, "gspo": 4, "reinforce": 5, "geo_mean": 6}


def _policy_loss_variant(variant, old_log_prob, log_prob, advantages, response_mask, loss_agg_mode, config,
                         rollout_is_weights, tau_pos=1.0, tau_neg=1.0, needs_clip=True):
    clip_low = clip_high = 0.0
    if needs_clip:
        clip_ratio = config.clip_ratio
        low = getattr(config, "clip_ratio_low", None)
        high = getattr(config, "clip_ratio_high", None)
        clip_low = low if low is not None else clip_ratio
        clip_high = high if high is not None else clip_ratio
    info = dict(getattr(config, "global_batch_info", None) or {})
    pg_loss, out = _apply_loss(
        _PolicyLoss, log_prob, old_log_prob, advantages, response_mask, rollout_is_weights, float(clip_low),
        float(clip_high), 3.0, _agg_mode(loss_agg_mode), float(info.get("dp_size", 1)),
        _opt(info.get("batch_num_tokens")),
        _opt(info.get("global_batch_size")), _opt(info.get("loss_scale_factor")), _PL[variant], float(tau_pos),
        float(tau_neg))
    vals = out.detach().tolist()
    return pg_loss, {"actor/pg_clipfrac": vals[1], "actor/ppo_kl": vals[2], "actor/pg_clipfrac_lower": vals[3]}


@register_policy_loss("gspo")
def compute_policy_loss_gspo(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                             response_mask: torch.Tensor, loss_agg_mode: str = "seq-mean-token-mean",
                             config: Optional[Any] = None, rollout_is_weights: torch.Tensor | None = None):
    """GSPO (reference core_algos.py:1253-1326): the clipped objective on the sequence-level importance
    ratio ``exp(min(mean_t(log_prob - old_log_prob), 10))`` with token-level gradients; always aggregated
    as "seq-mean-token-mean" whatever ``loss_agg_mode`` says, as there (:1307-1309)."""
    assert config is not None
    return _policy_loss_variant("gspo", old_log_prob, log_prob, advantages, response_mask, "seq-mean-token-mean",
                                config, rollout_is_weights)


@register_policy_loss("sapo")
def compute_policy_loss_sapo(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                             response_mask: torch.Tensor, loss_agg_mode: str = "seq-mean-token-mean",
                             config: Optional[Any] = None, rollout_is_weights: torch.Tensor | None = None):
    """SAPO (reference core_algos.py:1329-1411): ``-4/tau sigmoid(tau (ratio - 1)) A`` with ``config.tau_pos``
    for positive and ``config.tau_neg`` for the other advantages; always "seq-mean-token-mean"."""
    assert config is not None
    return _policy_loss_variant("sapo", old_log_prob, log_prob, advantages, response_mask, "seq-mean-token-mean",
                                config, rollout_is_weights, tau_pos=config.tau_pos, tau_neg=config.tau_neg,
                                needs_clip=False)


@register_policy_loss("gpg")
def compute_policy_loss_gpg(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                            response_mask: torch.Tensor, loss_agg_mode: str = "token-mean",
                            config: Optional[Any] = None, rollout_is_weights: torch.Tensor | None = None):
    """GPG (reference core_algos.py:1414-1447): ``agg_loss(-log_prob A)``; returns an empty metrics dict."""
    assert config is not None
    pg_loss, _ = _policy_loss_variant("gpg", old_log_prob, log_prob, advantages, response_mask, loss_agg_mode, config,
                                      rollout_is_weights, needs_clip=False)
    return pg_loss, {}


@register_policy_loss("cispo")
def compute_policy_loss_cispo(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                              response_mask: torch.Tensor, loss_agg_mode: str = "token-mean",
                              config: Optional[Any] = None, rollout_is_weights: torch.Tensor | None = None):
    """CISPO (reference core_algos.py:1721-1779): ``-sg(clip(ratio)) A log_prob``; ``actor/pg_clipfrac`` is the
    share of valid tokens whose ratio was clipped."""
    assert config is not None
    return _policy_loss_variant("cispo", old_log_prob, log_prob, advantages, response_mask, loss_agg_mode, config,
                                rollout_is_weights)


class _CovLoss(torch.autograd.Function):
    """The two covariance-selected losses (``vamd_policy_loss_cov_forward``)."""

    @staticmethod
    def forward(ctx, log_prob, old_log_prob, advantages, response_mask, is_weights, kind, clip_low, clip_high, cov_lb,
                cov_ub, ratio, kl_coef, seed, mode, dp_size, bnt, gbs, lsf, want_selected):
        dev = _cabi.compute_device(log_prob, old_log_prob, advantages, response_mask)
        lp = _matrix(log_prob, dev)
        old = _matrix(old_log_prob, dev)
        adv = _matrix(advantages, dev)
        assert lp.shape == old.shape == adv.shape
        m, code = _mask_matrix(response_mask, dev, lp.shape)
        isw = _matrix(is_weights, dev) if is_weights is not None else None
        rows, cols = lp.shape
        need_grad = ctx.needs_input_grad[0]
        Lb = _cabi.lib()
        out = torch.empty(4, dtype=torch.float32, device=dev)
        coef = torch.empty(rows, dtype=torch.float32, device=dev)
        g = torch.empty_like(lp) if need_grad else None
        selected = torch.empty((rows, cols), dtype=torch.uint8, device=dev) if want_selected else None
        ws = _cabi.workspace(Lb.vamd_policy_loss_cov_workspace_bytes(rows, cols), dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_policy_loss_cov_forward(kind, old.data_ptr(), lp.data_ptr(), adv.data_ptr(),
                                                        m.data_ptr(), code, _cabi.ptr(isw), rows, cols, clip_low,
                                                        clip_high, cov_lb, cov_ub, ratio, kl_coef, seed, mode,
                                                        dp_size, bnt, gbs, lsf, out.data_ptr(), _cabi.ptr(g),
                                                        coef.data_ptr(), _cabi.ptr(selected), ws.data_ptr(),
                                                        ws.numel(), _cabi.stream_ptr(dev)))
        if need_grad:
            ctx.save_for_backward(g, coef)
        ctx.in_shape = log_prob.shape
        ctx.in_device = log_prob.device
        ctx.in_dtype = log_prob.dtype
        out = out.to(log_prob.device)
        if selected is None:
            selected = torch.empty(0, dtype=torch.uint8, device=log_prob.device)
        else:
            selected = selected.view(log_prob.shape).to(log_prob.device)
        ctx.mark_non_differentiable(out, selected)
        return out[0].clone(), out, selected

    @staticmethod
    def backward(ctx, d_loss, _d_out, _d_sel):
        g, coef = ctx.saved_tensors
        dev = g.device
        rows, cols = g.shape
        d = _cabi.as_f32(d_loss, dev).reshape(1)
        res = torch.empty_like(g)
        with _cabi.device_guard(dev):
            _cabi.check(_cabi.lib().vamd_scale_rows(g.data_ptr(), coef.data_ptr(), d.data_ptr(), 1.0, rows, cols,
                                                    res.data_ptr(), _cabi.stream_ptr(dev)))
        return (res.view(ctx.in_shape).to(device=ctx.in_device, dtype=ctx.in_dtype),) + (None,) * 18


def _policy_loss_option(config, name, default):
    """``config.policy_loss.<name>`` (attribute or mapping), ``default`` when absent or ``None``."""
    pl = config.policy_loss
    value = pl.get(name, None) if isinstance(pl, dict) else getattr(pl, name, None)
    return default if value is None else value


def _cov_loss(kind, old_log_prob, log_prob, advantages, response_mask, loss_agg_mode, config, rollout_is_weights,
              clip_low, clip_high, cov_lb, cov_ub, ratio, kl_coef, return_selected):
    info = dict(getattr(config, "global_batch_info", None) or {})
    # the draw of Clip-Cov follows torch's generator, so torch.manual_seed makes a step reproducible
    seed = int(torch.randint(0, 2**62, (1,)).item()) if kind == 1 else 0
    pg_loss, out, selected = _CovLoss.apply(
        log_prob, old_log_prob, advantages, response_mask, rollout_is_weights, kind, float(clip_low), float(clip_high),
        float(cov_lb), float(cov_ub), float(ratio), float(kl_coef), seed, _agg_mode(loss_agg_mode),
        float(info.get("dp_size", 1)), _opt(info.get("batch_num_tokens")), _opt(info.get("global_batch_size")),
        _opt(info.get("loss_scale_factor")), bool(return_selected))
    return pg_loss, out.detach().tolist(), selected


@register_policy_loss("clip_cov")
def compute_policy_loss_clip_cov(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                                 response_mask: torch.Tensor, loss_agg_mode: str = "token-mean",
                                 config: Optional[Any] = None, rollout_is_weights: torch.Tensor | None = None,
                                 return_selected: bool = False):
    """Clip-Cov (reference core_algos.py:1450-1552): the clipped surrogate, except that
    ``min(max(int(clip_cov_ratio * sum(mask)), 1), #candidates)`` tokens drawn uniformly at random from the valid,
    not already clipped tokens whose covariance ``(A - masked_mean A)(log_prob - masked_mean log_prob)`` lies
    strictly between ``clip_cov_lb`` and ``clip_cov_ub`` contribute neither loss nor gradient;
    ``actor/pg_clipfrac`` is their share of the valid tokens.  ``config.policy_loss`` supplies ``clip_cov_ratio``
    (0.0002), ``clip_cov_lb`` (1.0), ``clip_cov_ub`` (5.0).  The draw is made on the device from a seed taken from
    torch's default generator; with ``return_selected=True`` the metrics carry the boolean matrix of dropped tokens
    under ``"selected"``."""
    assert config is not None
    assert config.policy_loss is not None
    ratio = _policy_loss_option(config, "clip_cov_ratio", 0.0002)
    clip_ratio = config.clip_ratio
    low = getattr(config, "clip_ratio_low", None)
    high = getattr(config, "clip_ratio_high", None)
    assert ratio > 0, "clip_ratio should be larger than 0."
    pg_loss, vals, selected = _cov_loss(1, old_log_prob, log_prob, advantages, response_mask, loss_agg_mode, config,
                                        rollout_is_weights, low if low is not None else clip_ratio,
                                        high if high is not None else clip_ratio,
                                        _policy_loss_option(config, "clip_cov_lb", 1.0),
                                        _policy_loss_option(config, "clip_cov_ub", 5.0), ratio, 0.0, return_selected)
    metrics = {"actor/pg_clipfrac": vals[1], "actor/ppo_kl": vals[2]}
    if return_selected:
        metrics["selected"] = selected.bool()
    return pg_loss, metrics


@register_policy_loss("kl_cov")
def compute_policy_loss_kl_cov(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                               response_mask: torch.Tensor, loss_agg_mode: str = "token-mean",
                               config: Optional[Any] = None, rollout_is_weights: torch.Tensor | None = None,
                               return_selected: bool = False):
    """KL-Cov (reference core_algos.py:1555-1632): ``-A ratio`` on every token plus ``ppo_kl_coef |log ratio|`` on
    the ``max(1, int(n * kl_cov_ratio))`` valid tokens with the largest covariance ``(A - mean A)(log_prob - mean
    log_prob)``; ``actor/ppo_kl`` is the masked mean of ``|log ratio|``.  ``config.policy_loss`` supplies
    ``kl_cov_ratio`` (0.0002) and ``ppo_kl_coef`` (1.0).  The top-k runs on the device (the reference moves the
    valid tokens to the CPU for it)."""
    assert config is not None
    assert config.policy_loss is not None
    ratio = _policy_loss_option(config, "kl_cov_ratio", 0.0002)
    assert ratio > 0, "kl_cov_ratio should be larger than 0."
    pg_loss, vals, selected = _cov_loss(0, old_log_prob, log_prob, advantages, response_mask, loss_agg_mode, config,
                                        rollout_is_weights, 0.0, 0.0, 0.0, 0.0, ratio,
                                        _policy_loss_option(config, "ppo_kl_coef", 1.0), return_selected)
    metrics = {"actor/ppo_kl": vals[2]}
    if return_selected:
        metrics["selected"] = selected.bool()
    return pg_loss, metrics


@register_policy_loss("geo_mean")
def compute_policy_loss_geo_mean(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                                 response_mask: torch.Tensor, loss_agg_mode: str = "token-mean",
                                 config: Optional[Any] = None, rollout_is_weights: torch.Tensor | None = None):
    """GMPO (reference core_algos.py:1635-1718): per sequence ``-mean_t(A) * exp(mean_t clipped log-ratio)``, the
    log-ratio clipped to ``[-clip_ratio_low, clip_ratio_high]`` on the side the advantage's sign makes
    pessimistic; importance weights enter as their geometric mean per sequence; the loss is the plain mean over
    the sequences (``loss_agg_mode`` is not used, as there)."""
    assert config is not None
    return _policy_loss_variant("geo_mean", old_log_prob, log_prob, advantages, response_mask, "seq-mean-token-sum",
                                config, rollout_is_weights)


def compute_policy_loss_reinforce(rollout_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                                  response_mask: torch.Tensor, loss_agg_mode: str = "seq-mean-token-sum",
                                  config: Optional[Any] = None, rollout_is_weights: Optional[torch.Tensor] = None):
    """REINFORCE with optional importance weights (reference core_algos.py:1984-2061):
    ``agg_loss(-A log_prob [w])``; ``actor/ppo_kl`` is measured against the rollout policy."""
    assert config is not None, "ActorConfig must be provided for REINFORCE loss"
    pg_loss, metrics = _policy_loss_variant("reinforce", rollout_log_prob, log_prob, advantages, response_mask,
                                            loss_agg_mode, config, rollout_is_weights, needs_clip=False)
    return pg_loss, {"actor/ppo_kl": metrics["actor/ppo_kl"]}


@register_policy_loss("bypass_mode")
def compute_policy_loss_bypass_mode(old_log_prob: torch.Tensor, log_prob: torch.Tensor, advantages: torch.Tensor,
                                    response_mask: torch.Tensor, loss_agg_mode: str = "token-mean",
                                    config: Optional[Any] = None, rollout_is_weights: torch.Tensor | None = None):
    """Bypass mode (reference core_algos.py:2064-2187): ``old_log_prob`` is the rollout policy's; the importance
    weights ``pi_current / pi_rollout`` and the off-policy metrics are computed here from
    ``config.policy_loss["rollout_correction"]`` (``loss_type`` "ppo_clip" or "reinforce", ``rollout_is``,
    ``rollout_is_threshold``, ``rollout_is_batch_normalize``), then the clipped PPO loss (without the weights)
    or the REINFORCE loss (with them) is returned with both sets of metrics.  ``rollout_is_weights`` is
    ignored, as there.  ``rollout_rs`` raises ``NotImplementedError``."""
    from .rollout_corr_helper import compute_rollout_correction_and_rejection_mask

    assert config is not None, "config is required for bypass_mode loss"
    rc = config.policy_loss.get("rollout_correction", None) if hasattr(config, "policy_loss") else None
    if rc is None:
        raise ValueError(
            "rollout_correction config not found in policy_loss. "
            "When using loss_mode='bypass_mode', ensure rollout_correction config is passed."
        )
    loss_type = rc.get("loss_type", "ppo_clip")
    with torch.no_grad():
        proto, effective_mask, rollout_metrics = compute_rollout_correction_and_rejection_mask(
            old_log_prob=log_prob.detach(), rollout_log_prob=old_log_prob, response_mask=response_mask,
            rollout_is=rc.get("rollout_is", None), rollout_is_threshold=rc.get("rollout_is_threshold", 2.0),
            rollout_is_batch_normalize=rc.get("rollout_is_batch_normalize", False),
            rollout_rs=rc.get("rollout_rs", None), rollout_rs_threshold=rc.get("rollout_rs_threshold", None))
    weights = proto.batch["rollout_is_weights"] if proto else None
    if loss_type == "reinforce":
        pg_loss, pg_metrics = compute_policy_loss_reinforce(
            rollout_log_prob=old_log_prob, log_prob=log_prob, advantages=advantages, response_mask=effective_mask,
            loss_agg_mode=loss_agg_mode, config=config, rollout_is_weights=weights)
    elif loss_type == "ppo_clip":
        pg_loss, pg_metrics = compute_policy_loss_vanilla(
            old_log_prob=old_log_prob, log_prob=log_prob, advantages=advantages, response_mask=effective_mask,
            loss_agg_mode=loss_agg_mode, config=config, rollout_is_weights=None)
    else:
        raise ValueError(f"Invalid loss_type: {loss_type}. Must be 'reinforce' or 'ppo_clip'.")
    pg_metrics.update(rollout_metrics)
    return pg_loss, pg_metrics


def compute_policy_loss(old_log_prob, log_prob, advantages, response_mask, cliprange=None, cliprange_low=None,
                        cliprange_high=None, clip_ratio_c=3.0, loss_agg_mode: str = "token-mean"):
    """Deprecated positional form (reference core_algos.py:1083-1156): returns
    ``(pg_loss, pg_clipfrac, ppo_kl, pg_clipfrac_lower)`` as tensors."""
    assert clip_ratio_c > 1.0, (
        "The lower bound of the clip_ratio_c for dual-clip PPO should be greater than 1.0,"
        + f" but get the value: {clip_ratio_c}."
    )
    if cliprange_low is None:
        cliprange_low = cliprange
    if cliprange_high is None:
        cliprange_high = cliprange
    pg_loss, out = _apply_loss(_PolicyLoss, log_prob, old_log_prob, advantages, response_mask, None,
                               float(cliprange_low), float(cliprange_high), float(clip_ratio_c),
                               _agg_mode(loss_agg_mode), 1.0, -1.0, -1.0, -1.0)
    return pg_loss, out[1], out[2], out[3]


# ---------------------------------------------------------------------------------------------
class _ValueLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, vpreds, returns, values, response_mask, cliprange_value, mode):
        dev = _cabi.compute_device(vpreds, returns, values, response_mask)
        vp = _matrix(vpreds, dev)
        ret = _matrix(returns, dev)
        val = _matrix(values, dev)
        assert vp.shape == ret.shape == val.shape
        m, code = _mask_matrix(response_mask, dev, vp.shape)
        rows, cols = vp.shape
        need_grad = ctx.needs_input_grad[0]
        Lb = _cabi.lib()
        buf = torch.empty(4 + rows, dtype=torch.float32, device=dev)   # results and per-row coefficients together
        out, coef = buf[:2], buf[4:]
        g = torch.empty_like(vp) if need_grad else None
        ws = _cabi.ticket_workspace(Lb.vamd_value_loss_workspace_bytes(rows, cols), dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_value_loss_forward(vp.data_ptr(), ret.data_ptr(), val.data_ptr(), m.data_ptr(), code,
                                                   rows, cols, cliprange_value, mode, out.data_ptr(), _cabi.ptr(g),
                                                   coef.data_ptr(), ws.data_ptr(), ws.numel(),
                                                   _cabi.stream_ptr(dev)))
        if need_grad:
            ctx.save_for_backward(g, coef)
        ctx.in_shape = vpreds.shape
        ctx.in_device = vpreds.device
        ctx.in_dtype = vpreds.dtype
        out = out.to(vpreds.device)
        ctx.mark_non_differentiable(out)
        return out[0], out   # a view: the loss and the metrics share the floats the kernel wrote

    @staticmethod
    def backward(ctx, d_loss, _d_out):
        g, coef = ctx.saved_tensors
        dev = g.device
        rows, cols = g.shape
        d = _cabi.as_f32(d_loss, dev).reshape(1)
        res = torch.empty_like(g)
        with _cabi.device_guard(dev):
            _cabi.check(_cabi.lib().vamd_scale_rows(g.data_ptr(), coef.data_ptr(), d.data_ptr(), 0.5, rows, cols,
                                                    res.data_ptr(), _cabi.stream_ptr(dev)))
        res = res.view(ctx.in_shape).to(device=ctx.in_device, dtype=ctx.in_dtype)
        return res, None, None, None, None, None


def compute_value_loss(vpreds: torch.Tensor, returns: torch.Tensor, values: torch.Tensor,
                       response_mask: torch.Tensor, cliprange_value: float, loss_agg_mode: str = "token-mean"):
    """Clipped value loss (reference core_algos.py:1799-1838): returns ``(vf_loss, vf_clipfrac)``,
    ``vf_loss`` differentiable with respect to ``vpreds``."""
    vf_loss, out = _apply_loss(_ValueLoss, vpreds, returns, values, response_mask, float(cliprange_value),
                                    _agg_mode(loss_agg_mode))
    return vf_loss, out[1]


# ---- PF-PPO data reweighting -----------------------------------------------------------------------
@torch.no_grad()
def _pf_ppo_weights(scores: torch.Tensor, reweight_method: str, weight_pow: float) -> torch.Tensor:
    """Resampling weight of every sequence from its total score (reference core_algos.py:1921-1947)."""
    if reweight_method == "pow":
        return torch.pow(torch.abs(scores), weight_pow)
    if reweight_method == "max_min":
        return torch.where((scores == torch.max(scores)) | (scores == torch.min(scores)), 1.0, 0.0)
    if reweight_method == "max_random":
        return torch.where(scores == torch.max(scores), 0.4, 0.1)
    raise ValueError(f"Unsupported reweight_method: {reweight_method}")


def compute_pf_ppo_reweight_data(data, reweight_method: str = "pow", weight_pow: float = 2.0):
    """Resample the batch with replacement, each sequence drawn with a probability proportional to a weight of its
    total ``token_level_scores`` (reference core_algos.py:1905-1980): ``"pow"`` = ``|score| ** weight_pow``,
    ``"max_min"`` = the best and the worst sequences only, ``"max_random"`` = 0.4 for the best against 0.1 for the
    rest; ``1e-8`` is added to every weight.  Every tensor of ``data.batch``, every array or list of
    ``data.non_tensor_batch`` and every ``meta_info`` list as long as the batch is taken at the same drawn indices.
    Returns a new object of the type of ``data``; ``data`` itself is left as it was.  Host-side bookkeeping on whatever
    device the batch lives on (one ``torch.multinomial`` and one gather per tensor); no kernel of the library runs."""
    import copy

    scores = data.batch["token_level_scores"].sum(dim=-1)
    weights = torch.clamp(_pf_ppo_weights(scores, reweight_method, weight_pow) + 1e-8, min=1e-8)
    batch_size = scores.shape[0]
    sample_indices = torch.multinomial(weights, batch_size, replacement=True)
    resampled_batch = {key: tensor[sample_indices] for key, tensor in data.batch.items()}
    picks = sample_indices.cpu().numpy()
    resampled_non_tensor = {}
    for key, array in getattr(data, "non_tensor_batch", {}).items():
        resampled_non_tensor[key] = array[picks] if isinstance(array, np.ndarray) else [array[i] for i in picks]
    resampled_meta = {}
    for key, value in (getattr(data, "meta_info", None) or {}).items():
        resampled_meta[key] = [value[i] for i in picks] if isinstance(value, list) and len(value) == batch_size else value
    out = copy.copy(data)   # the reference deep-copies and then replaces the same three fields
    out.batch = type(data.batch)(resampled_batch)
    try:
        out.batch.batch_size = data.batch.batch_size
    except AttributeError:   # a batch type that derives its size from its tensors
        pass
    out.non_tensor_batch = resampled_non_tensor
    if hasattr(data, "meta_info"):
        out.meta_info = resampled_meta
    return out


# ---- KL penalty -----------------------------------------------------------------------------------
_KL_KINDS = {"kl": 0, "k1": 0, "abs": 1, "mse": 2, "k2": 2, "low_var_kl": 3, "k3": 3}


def _kl_kind(kl_penalty: str) -> int:
    """Estimator code of ``kl_penalty_forward``; every other name (``"full"``, and in this reference
    snapshot every ``"+"``-suffixed name, which reaches ``kl_penalty_forward`` unstripped,
    core_algos.py:1853,1868-1902) raises ``NotImplementedError`` as there."""
    if kl_penalty not in _KL_KINDS:
        raise NotImplementedError
    return _KL_KINDS[kl_penalty]


class _KlPenalty(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logprob, ref_logprob, kind, straight_through):
        dev = _cabi.compute_device(logprob, ref_logprob)
        assert logprob.shape == ref_logprob.shape
        lp = _cabi.as_f32(logprob, dev).contiguous()
        ref = _cabi.as_f32(ref_logprob, dev).contiguous()
        need_grad = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        kld = torch.empty_like(lp)
        g = torch.empty_like(lp) if need_grad else None
        with _cabi.device_guard(dev):
            _cabi.check(_cabi.lib().vamd_kl_penalty(lp.data_ptr(), ref.data_ptr(), lp.numel(), kind,
                                                    int(straight_through), kld.data_ptr(), _cabi.ptr(g),
                                                    _cabi.stream_ptr(dev)))
        if need_grad:
            ctx.save_for_backward(g)
        ctx.meta = [(t.device, t.dtype) for t in (logprob, ref_logprob)]
        return kld.to(logprob.device)

    @staticmethod
    def backward(ctx, d_kld):
        (g,) = ctx.saved_tensors
        d = g * d_kld.to(device=g.device, dtype=torch.float32)
        outs = []
        for need, (device, dtype), sign in zip(ctx.needs_input_grad[:2], ctx.meta, (1.0, -1.0)):
            outs.append((sign * d).to(device=device, dtype=dtype) if need else None)
        return outs[0], outs[1], None, None


def kl_penalty_forward(logprob: torch.Tensor, ref_logprob: torch.Tensor, kl_penalty) -> torch.Tensor:
    """Per-token KL estimate between the policy and the reference policy
    (reference core_algos.py:1868-1902): ``"kl"/"k1"``, ``"abs"``, ``"mse"/"k2"``,
    ``"low_var_kl"/"k3"``; differentiable with respect to both inputs."""
    return _KlPenalty.apply(logprob, ref_logprob, _kl_kind(kl_penalty), False)


def kl_penalty(logprob: torch.Tensor, ref_logprob: torch.Tensor, kl_penalty) -> torch.Tensor:
    """``kl_penalty`` of the reference (core_algos.py:1841-1866).  It evaluates
    ``kl_penalty_forward`` with the name as given before looking at a trailing ``"+"``, so in this
    snapshot the straight-through names raise ``NotImplementedError`` there; the kernel's
    straight-through path (value of the estimator, gradient of k2) is reachable through
    ``compute_kl_loss(..., straight_through=True)``."""
    return kl_penalty_forward(logprob, ref_logprob, kl_penalty)


class _KlLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logprob, ref_logprob, response_mask, kind, straight_through, mode, dp, bnt, gbs, lsf):
        dev = _cabi.compute_device(logprob, ref_logprob, response_mask)
        lp = _matrix(logprob, dev)
        ref = _matrix(ref_logprob, dev)
        assert lp.shape == ref.shape
        m, code = _mask_matrix(response_mask, dev, lp.shape)
        rows, cols = lp.shape
        need_grad = ctx.needs_input_grad[0]
        Lb = _cabi.lib()
        out = torch.empty(1, dtype=torch.float32, device=dev)
        coef = torch.empty(rows, dtype=torch.float32, device=dev)
        g = torch.empty_like(lp) if need_grad else None
        ws = _cabi.ticket_workspace(Lb.vamd_kl_loss_workspace_bytes(rows, cols), dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_kl_loss_forward(lp.data_ptr(), ref.data_ptr(), m.data_ptr(), code, rows, cols, kind,
                                                int(straight_through), mode, dp, bnt, gbs, lsf, out.data_ptr(),
                                                _cabi.ptr(g), coef.data_ptr(), ws.data_ptr(), ws.numel(),
                                                _cabi.stream_ptr(dev)))
        if need_grad:
            ctx.save_for_backward(g, coef)
        ctx.in_shape = logprob.shape
        ctx.in_device = logprob.device
        ctx.in_dtype = logprob.dtype
        return out[0].to(logprob.device)

    @staticmethod
    def backward(ctx, d_loss):
        g, coef = ctx.saved_tensors
        dev = g.device
        rows, cols = g.shape
        d = _cabi.as_f32(d_loss, dev).reshape(1)
        res = torch.empty_like(g)
        with _cabi.device_guard(dev):
            _cabi.check(_cabi.lib().vamd_scale_rows(g.data_ptr(), coef.data_ptr(), d.data_ptr(), 1.0, rows, cols,
                                                    res.data_ptr(), _cabi.stream_ptr(dev)))
        res = res.view(ctx.in_shape).to(device=ctx.in_device, dtype=ctx.in_dtype)
        return (res,) + (None,) * 9


def compute_kl_loss(logprob: torch.Tensor, ref_logprob: torch.Tensor, response_mask: torch.Tensor,
                    kl_penalty: str = "low_var_kl", loss_agg_mode: str = "token-mean", dp_size: int = 1,
                    batch_num_tokens=None, global_batch_size=None, loss_scale_factor=None,
                    straight_through: bool = False) -> torch.Tensor:
    """``agg_loss(kl_penalty(logprob, ref_logprob, kl_penalty), response_mask, loss_agg_mode)`` in one
    pass over the tensors: the ``kl_loss`` term of the actor update (reference
    verl/workers/actor/dp_actor.py:640-646), differentiable with respect to ``logprob``.  No
    single function of the reference does both steps; this one exists so that the pair costs one
    read of the inputs.  ``straight_through=True`` keeps the estimator's value and uses the k2
    gradient, the behaviour the reference documents for the ``"+"`` names."""
    return _KlLoss.apply(logprob, ref_logprob, response_mask, _kl_kind(kl_penalty), bool(straight_through),
                         _agg_mode(loss_agg_mode), float(dp_size), _opt(batch_num_tokens), _opt(global_batch_size),
                         _opt(loss_scale_factor))


def kl_penalised_rewards(token_level_scores: torch.Tensor, old_log_probs: torch.Tensor, ref_log_prob: torch.Tensor,
                         response_mask: torch.Tensor, beta: float, kl_penalty: str = "kl"):
    """The arithmetic of ``apply_kl_penalty`` (reference verl/trainer/ppo/ray_trainer.py:86-101) in one pass:
    ``kld = kl_penalty(old_log_probs, ref_log_prob) * response_mask``, ``token_level_rewards =
    token_level_scores - beta * kld`` and ``current_kl = mean_i masked_mean(kld_i, mask_i)``.  Returns
    ``(token_level_rewards, current_kl)`` with ``current_kl`` a 0-d device tensor (no host sync here)."""
    with torch.no_grad():
        dev = _cabi.compute_device(token_level_scores, old_log_probs, ref_log_prob, response_mask)
        sc = _matrix(token_level_scores, dev)
        lp = _matrix(old_log_probs, dev)
        rf = _matrix(ref_log_prob, dev)
        assert sc.shape == lp.shape == rf.shape
        m, code = _mask_matrix(response_mask, dev, sc.shape)
        rows, cols = sc.shape
        out = torch.empty_like(sc)
        kl = torch.empty(1, dtype=torch.float32, device=dev)
        Lb = _cabi.lib()
        ws = _cabi.ticket_workspace(Lb.vamd_apply_kl_penalty_workspace_bytes(rows, cols), dev)
        with _cabi.device_guard(dev):
            _cabi.check(Lb.vamd_apply_kl_penalty(sc.data_ptr(), lp.data_ptr(), rf.data_ptr(), m.data_ptr(), code,
                                                 rows, cols, _kl_kind(kl_penalty), float(beta), out.data_ptr(),
                                                 kl.data_ptr(), ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
        out_dev = token_level_scores.device
        return out.view(token_level_scores.shape).to(out_dev), kl[0].to(out_dev)


def compute_rewards(token_level_scores, old_log_prob, ref_log_prob, kl_ratio):
    """``token_level_scores - (old_log_prob - ref_log_prob) * kl_ratio`` (reference core_algos.py:1009-1022)."""
    ones = torch.ones(token_level_scores.shape, dtype=torch.uint8, device=token_level_scores.device)
    return kl_penalised_rewards(token_level_scores, old_log_prob, ref_log_prob, ones, kl_ratio, "kl")[0]
