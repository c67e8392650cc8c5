"""Pins for oracle/rollout_corr.py: the reference test's literal case and key lists, identities that hold
for identical policies and for constant ratios, and an fp64 scalar brute force."""
import math

import pytest
import torch

import oracle as O
from conftest import load_golden

GOLDEN = load_golden()


def test_mask_mode_reference_literals():
    case = GOLDEN["rollout_corr_mask_mode"]
    old, roll, mask = (torch.tensor(case[k]) for k in ("old_log_prob", "rollout_log_prob", "response_mask"))
    w, metrics = O.rollout_correction_weights(old - roll, mask, case["rollout_is"], case["rollout_is_threshold"])
    assert abs(w[0, 0].item() - case["expected_weight_row0"]) <= case["atol"]
    assert abs(w[1, 0].item() - case["expected_weight_row1"]) <= case["atol"]
    assert (w[0] == w[0, 0]).all() and (w[1] == w[1, 0]).all()
    # constant ratios per row: everything is a two-point distribution over exp(-1) and exp(0.5)
    a, b = math.exp(-1.0), math.exp(0.5)
    assert metrics["rollout_is_mean"] == pytest.approx((a + b) / 2, rel=1e-6)
    assert metrics["rollout_is_max"] == pytest.approx(b, rel=1e-6) and metrics["rollout_is_min"] == pytest.approx(a, rel=1e-6)
    assert metrics["rollout_is_ratio_fraction_low"] == pytest.approx(0.5) and metrics["rollout_is_ratio_fraction_high"] == 0
    ca = max(a, 0.5)
    assert metrics["rollout_is_std"] == pytest.approx(abs(b - ca) / 2, rel=1e-5)
    assert metrics["rollout_is_eff_sample_size"] == pytest.approx((ca + b) ** 2 / (2 * (ca * ca + b * b)), rel=1e-5)
    assert metrics["rollout_is_seq_mean"] == pytest.approx((a + b) / 2, rel=1e-6)
    assert metrics["rollout_is_seq_std"] == pytest.approx(abs(b - a) / math.sqrt(2), rel=1e-5)
    assert metrics["rollout_is_seq_max_deviation"] == pytest.approx(max(1 - a, b - 1), rel=1e-5)
    assert metrics["rollout_is_seq_fraction_low"] == pytest.approx(0.5)


def test_metric_names_of_the_reference_tests():
    names = GOLDEN["rollout_corr_metric_names"]
    g = torch.Generator().manual_seed(0)
    old = torch.randn(3, 8, generator=g)
    roll = old + torch.randn(3, 8, generator=g) * 0.2
    mask = torch.ones(3, 8)
    _, m = O.rollout_correction_weights(old - roll, mask, "token", 2.5)
    assert set(names["is_metrics"]) <= set(m)
    assert set(O.offpolicy_metrics(old, roll, mask)) == set(names["offpolicy_metrics"])
    assert set(O.offpolicy_metrics(old, None, mask)) == set(names["offpolicy_metrics_without_rollout"])


def test_identical_policies_give_the_neutral_values():
    g = torch.Generator().manual_seed(1)
    lp = -torch.rand(4, 9, generator=g) * 3
    mask = (torch.rand(4, 9, generator=g) < 0.7).float()
    mask[:, 0] = 1
    m = O.offpolicy_metrics(lp, lp.clone(), mask)
    for key in ("kl", "k3_kl", "chi2_token", "chi2_seq", "log_ppl_diff", "log_ppl_abs_diff"):
        assert m[key] == pytest.approx(0.0, abs=1e-6), key
    assert m["ppl_ratio"] == pytest.approx(1.0) and m["training_ppl"] == pytest.approx(m["rollout_ppl"])
    for level in ("token", "sequence"):
        w, im = O.rollout_correction_weights(torch.zeros(4, 9), mask, level, 2.0, batch_normalize=True)
        assert torch.equal(w, mask)
        assert im["rollout_is_eff_sample_size"] == pytest.approx(1.0) and im["rollout_is_std"] == pytest.approx(0.0, abs=1e-6)
        assert im["rollout_is_batch_norm_factor"] == pytest.approx(1.0)


@pytest.mark.parametrize("level", ["token", "sequence"])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_against_fp64_brute_force(level, seed):
    g = torch.Generator().manual_seed(seed)
    B, L = 5, 11
    old = (-torch.rand(B, L, generator=g, dtype=torch.float64) * 3)
    roll = old + torch.randn(B, L, generator=g, dtype=torch.float64) * (0.5 if level == "token" else 0.15)
    lens = torch.randint(1, L + 1, (B,), generator=g)
    mask = (torch.arange(L)[None, :] < lens[:, None]).double()
    w, im = O.rollout_correction_weights(old - roll, mask, level, 1.5)
    om = O.offpolicy_metrics(old, roll, mask)
    want_w, want = O.rollout_correction_brute_force_fp64(old.tolist(), roll.tolist(), mask.tolist(), level, 1.5)
    assert torch.allclose(w, torch.tensor(want_w, dtype=torch.float64), rtol=1e-12, atol=1e-12)
    got = {**im, **om}
    for key, value in want.items():
        assert got[key] == pytest.approx(value, rel=1e-7, abs=1e-9), key


def test_sequence_level_and_batch_normalisation_by_hand():
    # two sequences: log-ratio sums ln 4 and ln (1/4), lengths 2 and 1, threshold 2
    d = torch.tensor([[math.log(2.0), math.log(2.0), 9.0], [math.log(0.25), 9.0, 9.0]])
    mask = torch.tensor([[1.0, 1.0, 0.0], [1.0, 0.0, 0.0]])
    w, m = O.rollout_correction_weights(d, mask, "sequence", 2.0)
    assert torch.allclose(w, torch.tensor([[2.0, 2.0, 0.0], [0.25, 0.0, 0.0]]))        # 4 truncated to 2
    assert m["rollout_is_max"] == pytest.approx(4.0) and m["rollout_is_min"] == pytest.approx(0.25)
    assert m["rollout_is_mean"] == pytest.approx((4 + 4 + 0.25) / 3)
    assert m["rollout_is_ratio_fraction_high"] == 0.5 and m["rollout_is_ratio_fraction_low"] == 0.5
    assert m["rollout_is_seq_mean"] == pytest.approx((4 + 0.25) / 2)
    w, m = O.rollout_correction_weights(d, mask, "sequence", 2.0, batch_normalize=True)
    assert m["rollout_is_batch_norm_factor"] == pytest.approx((2 + 0.25) / 2)
    assert torch.allclose(w, torch.tensor([[2.0, 2.0, 0.0], [0.25, 0.0, 0.0]]) / 1.125)
    w, m = O.rollout_correction_weights(d, mask, "token", 2.0, batch_normalize=True)
    assert m["rollout_is_batch_norm_factor"] == pytest.approx((2 + 2 + 0.25) / 3)
    with pytest.raises(ValueError):
        O.rollout_correction_weights(d, mask, "geometric", 2.0)
    with pytest.raises(ValueError):
        O.rollout_correction_weights(d, mask, "token", 0.0)
    with pytest.raises(ValueError):
        O.rollout_correction_weights(d, torch.zeros(2, 3), "token", 2.0)
