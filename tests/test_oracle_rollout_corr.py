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


# ---- rejection sampling ---------------------------------------------------------------------------------------
def _rejection_by_loops(d, mask, option, lower, upper):
    """Scalar loops from the definitions: token statistic, its per-sequence sum / mean / max, the keep rule, the new
    mask and the two masked fractions."""
    B, L = len(d), len(d[0])
    scope, est = option.rsplit("_", 1)

    def stat(x):
        x = max(-20.0, min(20.0, x))
        return {"k1": -x, "k2": 0.5 * x * x, "k3": math.exp(x) - 1.0 - x}[est]

    def inside(v):
        if est == "k1":
            return math.log(lower) <= v <= math.log(upper)
        return v <= upper

    new = [[0.0] * L for _ in range(B)]
    rejected_tokens = valid_tokens = rejected_seqs = valid_seqs = 0
    for i in range(B):
        toks = [t for t in range(L) if mask[i][t] != 0]
        vals = [stat(d[i][t]) for t in toks]
        if scope == "token":
            keep = {t: inside(v) for t, v in zip(toks, vals)}
        else:
            agg = {"seq_sum": sum(vals), "seq_mean": sum(vals) / max(len(vals), 1e-8),
                   "seq_max": max(vals) if vals else 0.0}[scope]
            keep = {t: inside(agg) for t in toks}
        for t in toks:
            new[i][t] = 1.0 if keep[t] else 0.0
        valid_tokens += len(toks)
        rejected_tokens += sum(not k for k in keep.values())
        if toks:
            valid_seqs += 1
            rejected_seqs += any(not k for k in keep.values())
    return new, rejected_tokens / valid_tokens, rejected_seqs / valid_seqs


def test_rejection_mask_reference_literals():
    case = GOLDEN["rollout_corr_mask_mode"]
    old, roll, mask = (torch.tensor(case[k]) for k in ("old_log_prob", "rollout_log_prob", "response_mask"))
    new, metrics = O.rollout_rejection_mask(old - roll, mask, case["rollout_rs"], case["rollout_rs_threshold"])
    assert (new[0] == case["expected_modified_mask_row0"]).all() and (new[1] == case["expected_modified_mask_row1"]).all()
    assert abs(metrics["rollout_rs_masked_fraction"] - case["expected_masked_fraction"]) < case["masked_fraction_atol"]
    assert metrics["rollout_rs_seq_masked_fraction"] == 0.5
    # k1 = -(old - rollout): 1.0 on row 0, -0.5 on row 1
    assert metrics["rollout_rs_token_k1_mean"] == pytest.approx(0.25)
    assert metrics["rollout_rs_token_k1_max"] == pytest.approx(1.0) and metrics["rollout_rs_token_k1_min"] == pytest.approx(-0.5)
    assert metrics["rollout_rs_token_k1_fraction_high"] == pytest.approx(0.5) and metrics["rollout_rs_token_k1_fraction_low"] == 0


def test_every_reference_option_runs_and_names_its_metrics():
    spec = GOLDEN["rollout_rs_options"]
    g = torch.Generator().manual_seed(0)
    B, L = spec["shape"]
    old = torch.randn(B, L, generator=g)
    roll = old + torch.randn(B, L, generator=g) * spec["noise_std"]
    mask = torch.ones(B, L)
    for option, threshold in spec["cases"]:
        assert option in O.RS_OPTIONS
        new, metrics = O.rollout_rejection_mask(old - roll, mask, option, threshold)
        assert spec["expected_key_template"].format(option=option) in metrics and new.shape == mask.shape
    chained = spec["chained"]
    _, metrics = O.rollout_rejection_mask(old - roll, mask, chained["rollout_rs"], chained["rollout_rs_threshold"])
    for option in chained["rollout_rs"].split(","):
        assert spec["expected_key_template"].format(option=option) in metrics
    assert len(O.RS_OPTIONS) == len(spec["cases"])


@pytest.mark.parametrize("option,threshold,lower,upper", [
    ("token_k1", "0.8_1.3", 0.8, 1.3), ("token_k2", 0.02, None, 0.02), ("token_k3", 0.03, None, 0.03),
    ("seq_sum_k1", "0.7_1.5", 0.7, 1.5), ("seq_sum_k2", 0.15, None, 0.15), ("seq_sum_k3", 0.2, None, 0.2),
    ("seq_mean_k1", 1.05, 1 / 1.05, 1.05), ("seq_mean_k2", 0.02, None, 0.02), ("seq_mean_k3", 0.02, None, 0.02),
    ("seq_max_k2", 0.08, None, 0.08), ("seq_max_k3", 0.1, None, 0.1)])
def test_rejection_mask_against_scalar_loops(option, threshold, lower, upper):
    g = torch.Generator().manual_seed(len(option))
    B, L = 9, 13
    d = torch.randn(B, L, generator=g, dtype=torch.float64) * 0.25
    d[0, 0] = 30.0                                               # beyond the safety clamp
    mask = (torch.rand(B, L, generator=g) < 0.75).double()
    mask[3] = 0                                                  # an empty sequence
    new, metrics = O.rollout_rejection_mask(d, mask, option, threshold)
    want, tok_frac, seq_frac = _rejection_by_loops(d.tolist(), mask.tolist(), option, lower, upper)
    assert torch.equal(new, torch.tensor(want, dtype=torch.float64))
    assert 0 < tok_frac < 1                                      # the thresholds above split the data
    assert metrics[f"rollout_rs_{option}_masked_fraction"] == pytest.approx(tok_frac, rel=1e-6)
    assert metrics["rollout_rs_masked_fraction"] == pytest.approx(tok_frac, rel=1e-6)
    assert metrics[f"rollout_rs_{option}_seq_masked_fraction"] == pytest.approx(seq_frac, rel=1e-6)
    assert metrics["rollout_rs_seq_masked_fraction"] == pytest.approx(seq_frac * (B - 1) / B, rel=1e-6)  # over all rows


def test_chained_options_multiply_and_bad_specs_raise():
    g = torch.Generator().manual_seed(4)
    d = torch.randn(6, 10, generator=g) * 0.3
    mask = torch.ones(6, 10)
    a, _ = O.rollout_rejection_mask(d, mask, "token_k2", 0.03)
    b, _ = O.rollout_rejection_mask(d, mask, "seq_max_k3", 0.2)
    both, metrics = O.rollout_rejection_mask(d, mask, "token_k2, seq_max_k3,token_k2", "0.03,0.2")   # duplicates are dropped
    assert torch.equal(both, a * b)
    assert metrics["rollout_rs_masked_fraction"] == pytest.approx(1 - (a * b).mean().item(), rel=1e-6)
    long_mask = mask.long()
    assert O.rollout_rejection_mask(d, long_mask, "token_k2", 0.03)[0].dtype == torch.int64
    for rs, thr, err in (("token_k9", 1.0, ValueError), ("token_k1", None, ValueError), ("token_k2", "1_2", ValueError),
                         ("token_k1,token_k2", "1,2,3", ValueError), ("token_k1", "-1_2", ValueError),
                         ("token_k2", "abc", ValueError), ("token_k2", [1.0], TypeError), (None, 1.0, ValueError),
                         (" , ", 1.0, ValueError)):
        with pytest.raises(err):
            O.rollout_rejection_mask(d, mask, rs, thr)
    assert O.parse_rs_thresholds(["token_k1", "seq_sum_k2"], "2.0") == {"token_k1": (0.5, 2.0), "seq_sum_k2": (None, 2.0)}
