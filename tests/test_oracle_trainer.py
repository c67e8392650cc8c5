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


def test_data_metrics_reference_mock_batch():
    from conftest import load_golden
    case = load_golden()["data_metrics"]
    batch = {k: torch.tensor(case[k]) for k in ("token_level_scores", "token_level_rewards", "advantages", "returns",
                                                 "values", "attention_mask", "response_mask")}
    batch["responses"] = torch.zeros(case["responses_shape"])
    got = O.compute_data_metrics(batch, use_critic=True)
    for key, want in {**case["expected"], **case["expected_by_hand"]}.items():
        assert got[key] == pytest.approx(want, rel=1e-5, abs=1e-5), key
    assert set(got) == set(case["expected"]) | set(case["expected_by_hand"])
    without = O.compute_data_metrics(batch, use_critic=False)
    for key in case["keys_without_critic_absent"]:
        assert key not in without
    assert set(without) == set(got) - {k for k in got if k.startswith("critic/values") or k == "critic/vf_explained_var"}


def test_data_metrics_masks_lengths_and_aborted_rows_by_hand():
    # row 0: prompt 1 of 2, response 3 of 3 but only 2 tokens in response_mask (a tool token in between);
    # row 1: aborted (no response tokens); row 2: full prompt, response 1 of 3
    batch = {
        "attention_mask": torch.tensor([[0, 1, 1, 1, 1], [1, 1, 0, 0, 0], [1, 1, 1, 0, 0]]),
        "response_mask": torch.tensor([[1, 0, 1], [0, 0, 0], [1, 0, 0]]),
        "responses": torch.zeros(3, 3),
        "token_level_scores": torch.tensor([[1.0, 10.0, 2.0], [100.0, 0.0, 0.0], [4.0, 0.0, 0.0]]),
        "token_level_rewards": torch.tensor([[0.5, 0.0, 0.5], [9.0, 9.0, 9.0], [2.0, 0.0, 0.0]]),
        "advantages": torch.tensor([[1.0, 50.0, -2.0], [50.0, 50.0, 50.0], [4.0, 50.0, 50.0]]),
        "returns": torch.tensor([[1.0, -50.0, 2.0], [-50.0, -50.0, -50.0], [6.0, -50.0, -50.0]]),
        "values": torch.tensor([[0.0, 7.0, 2.0], [7.0, 7.0, 7.0], [3.0, 7.0, 7.0]]),
    }
    got = O.compute_data_metrics(batch)
    want = {
        "critic/score/mean": (13.0 + 4.0) / 2, "critic/score/max": 13.0, "critic/score/min": 4.0,   # row 1 is left out
        "critic/rewards/mean": 1.5, "critic/rewards/max": 2.0, "critic/rewards/min": 1.0,
        "critic/advantages/mean": 1.0, "critic/advantages/max": 4.0, "critic/advantages/min": -2.0,
        "critic/returns/mean": 3.0, "critic/returns/max": 6.0, "critic/returns/min": 1.0,
        "critic/values/mean": 5.0 / 3, "critic/values/max": 3.0, "critic/values/min": 0.0,
        # returns - values = (1, 0, 3): var 7/3; returns (1, 2, 6): var 7
        "critic/vf_explained_var": 1.0 - (7.0 / 3) / (7.0 + 1e-5),
        "response_length/mean": 4.0 / 3, "response_length/max": 3.0, "response_length/min": 0.0,
        "response_length/clip_ratio": 1.0 / 3,
        "response_length_non_aborted/mean": 2.0, "response_length_non_aborted/max": 3.0,
        "response_length_non_aborted/min": 1.0, "response_length_non_aborted/clip_ratio": 0.5,
        "response/aborted_ratio": 1.0 / 3,
        "prompt_length/mean": 5.0 / 3, "prompt_length/max": 2.0, "prompt_length/min": 1.0,
        "prompt_length/clip_ratio": 2.0 / 3,
    }
    assert set(got) == set(want)
    for key, value in want.items():
        assert got[key] == pytest.approx(value, rel=1e-5, abs=1e-6), key
    batch["attention_mask"] = torch.tensor([[1, 1, 0, 0, 0]] * 3)
    with pytest.raises(ValueError, match="aborted"):
        O.compute_data_metrics(batch)


def test_pad_to_response_window_by_hand():
    # batch 2, seqlen 5, response 2: the window is columns 2 and 3 of each row
    attention = torch.tensor([[0, 1, 1, 1, 1], [1, 1, 1, 0, 0]])
    indices = attention.flatten().nonzero().flatten()            # 1 2 3 4 | 5 6 7
    values = torch.tensor([10.0, 11.0, 12.0, 13.0, 20.0, 21.0, 22.0], requires_grad=True)
    out = O.pad_to_response_window(values, indices, 2, 5, 2)
    assert out.tolist() == [[11.0, 12.0], [22.0, 0.0]]
    out.backward(torch.tensor([[1.0, 2.0], [3.0, 4.0]]))
    assert values.grad.tolist() == [0.0, 1.0, 2.0, 0.0, 0.0, 0.0, 3.0]


def test_variance_proxy_by_hand():
    # two trajectories; pi = 1/2 and sum pi^2 = 1/2 give w = 1/2 per token
    batch = {"old_log_probs": torch.full((2, 3), math.log(0.5)), "sum_pi_squared": torch.full((2, 3), 0.5),
             "advantages": torch.tensor([[2.0, 2.0, 9.0], [-1.0, -3.0, -2.0]]),
             "response_mask": torch.tensor([[1.0, 1.0, 0.0], [1.0, 1.0, 1.0]])}
    m = O.variance_proxy_metrics(batch, gradient_norm=0.5)
    # A = (2, -2), W = (1, 1.5): E[A^2 W] = (4 + 6) / 2
    assert m["variance_proxy/proxy2_total_power"] == pytest.approx(5.0)
    assert m["variance_proxy/proxy1_signal_strength"] == 0.25
    assert m["variance_proxy/proxy3_pure_noise"] == pytest.approx(4.75)
    assert m["variance_proxy/expected_a_squared"] == pytest.approx(4.0) and m["variance_proxy/expected_w"] == pytest.approx(1.25)
    # importance weights of 2 on the second trajectory: w carries rho^2, the proxy divides it out again and
    # multiplies by the squared mean weight: (1 * 4 * 1 + 4 * 4 * 1.5) / 2
    batch["rollout_is_weights"] = torch.tensor([[1.0, 1.0, 1.0], [2.0, 2.0, 2.0]])
    m = O.variance_proxy_metrics(batch)
    assert m["variance_proxy/proxy2_total_power"] == pytest.approx(14.0)
    assert m["variance_proxy/expected_w"] == pytest.approx((1 + 6) / 2)
    assert m["variance_proxy/proxy1_signal_strength"] == 0.0 and m["variance_proxy/proxy3_pure_noise"] == 0.0
    assert O.variance_proxy_metrics({"advantages": batch["advantages"]}) == {}


def test_pf_ppo_weights_by_hand():
    # sequence scores 2, -1, 0, 2 (no reference test holds a vector for this function: values worked by hand)
    scores = torch.tensor([[1.0, 1.0], [-1.0, 0.0], [0.0, 0.0], [0.5, 1.5]])
    p = O.pf_ppo_weights(scores, "pow", 2.0)            # 4, 1, 0, 4 (+1e-8 each) over 9
    assert p.tolist() == pytest.approx([4 / 9, 1 / 9, 1e-8 / 9, 4 / 9], rel=1e-6, abs=1e-12)
    p = O.pf_ppo_weights(scores, "pow", 1.0)            # |score|
    assert p.tolist() == pytest.approx([2 / 5, 1 / 5, 1e-8 / 5, 2 / 5], rel=1e-6, abs=1e-12)
    p = O.pf_ppo_weights(scores, "max_min", 2.0)        # both best sequences and the worst one
    assert p.tolist() == pytest.approx([1 / 3, 1 / 3, 1e-8 / 3, 1 / 3], rel=1e-6, abs=1e-12)
    p = O.pf_ppo_weights(scores, "max_random", 2.0)     # 0.4 for the best, 0.1 for the rest
    assert p.tolist() == pytest.approx([0.4, 0.1, 0.1, 0.4], rel=1e-6)
    assert p.sum().item() == pytest.approx(1.0)
    with pytest.raises(ValueError, match="Unsupported reweight_method"):
        O.pf_ppo_weights(scores, "softmax", 2.0)
