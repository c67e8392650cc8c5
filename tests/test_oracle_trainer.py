"""Pins for oracle/trainer.py and the host-side controller classes of the mirror: worked examples and
the special cases that reduce to other pinned functions."""
import math
import types

import pytest
import torch

import oracle as O


def test_apply_kl_penalty_by_hand():
    scores = torch.tensor([[1.0, 2.0], [3.0, 4.0]])
    ref = torch.zeros(2, 2)
    old = torch.tensor([[0.1, 0.2], [0.3, 0.4]])
    mask = torch.tensor([[1.0, 1.0], [1.0, 0.0]])
    rewards, current_kl = O.apply_kl_penalty(scores, old, ref, mask, beta=0.5, kind="kl")
    assert torch.allclose(rewards, torch.tensor([[0.95, 1.9], [2.85, 4.0]]))
    assert current_kl == pytest.approx((0.15 + 0.3) / 2, rel=1e-6)
    # k2 on the same numbers: 0.5 d^2
    rewards, current_kl = O.apply_kl_penalty(scores, old, ref, mask, beta=2.0, kind="mse")
    assert torch.allclose(rewards, torch.tensor([[1 - 0.01, 2 - 0.04], [3 - 0.09, 4.0]]))
    assert current_kl == pytest.approx((0.0125 + 0.045) / 2, rel=1e-6)
    # an empty response contributes 0 to the batch mean and keeps its scores
    mask0 = torch.tensor([[1.0, 1.0], [0.0, 0.0]])
    rewards, current_kl = O.apply_kl_penalty(scores, old, ref, mask0, beta=0.5, kind="kl")
    assert torch.equal(rewards[1], scores[1]) and current_kl == pytest.approx(0.075, rel=1e-6)


def test_compute_rewards_is_the_unmasked_k1_penalty():
    g = torch.Generator().manual_seed(0)
    s, a, b = (torch.randn(3, 7, generator=g) for _ in range(3))
    want, _ = O.apply_kl_penalty(s, a, b, torch.ones(3, 7), beta=0.3, kind="kl")
    assert torch.allclose(O.compute_rewards(s, a, b, 0.3), want)
    assert O.compute_rewards(s, a, a, 0.3).equal(s)


def test_kl_controllers_worked_example():
    from verl_amd.trainer.ppo import core_algos as CA
    ctl = CA.AdaptiveKLController(init_kl_coef=0.1, target_kl=0.1, horizon=100)
    ctl.update(current_kl=0.2, n_steps=10)          # error clipped to +0.2 -> x 1.02
    assert ctl.value == pytest.approx(0.102)
    ctl.update(current_kl=0.095, n_steps=50)        # error -0.05 -> x 0.975
    assert ctl.value == pytest.approx(0.102 * 0.975)
    ctl.update(current_kl=0.0, n_steps=100)         # error clipped to -0.2 -> x 0.8
    assert ctl.value == pytest.approx(0.102 * 0.975 * 0.8)
    assert O.adaptive_kl_update(0.1, 0.2, 10, 0.1, 100) == pytest.approx(0.102)
    fixed = CA.FixedKLController(0.05)
    fixed.update(current_kl=3.0, n_steps=7)
    assert fixed.value == 0.05
    cfg = types.SimpleNamespace(type="adaptive", kl_coef=0.2, target_kl=0.1, horizon=10)
    assert isinstance(CA.get_kl_controller(cfg), CA.AdaptiveKLController)
    assert isinstance(CA.get_kl_controller(types.SimpleNamespace(type="fixed", kl_coef=0.2)), CA.FixedKLController)
    with pytest.raises(AssertionError):
        CA.get_kl_controller(types.SimpleNamespace(type="adaptive", kl_coef=0.2, target_kl=0.1, horizon=0))
    with pytest.raises(NotImplementedError):
        CA.get_kl_controller(types.SimpleNamespace(type="pid", kl_coef=0.2))
    assert math.isfinite(ctl.value)
