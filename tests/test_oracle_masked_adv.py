"""Pins for oracle/masked.py and oracle/advantages.py: the reference-held
vectors (masked_mean cases, group_mean_std known answer, the multi-turn GAE
fixture, the GRPO loop==vectorised grids with the reference's generators),
closed forms and fp64 brute force."""
import math
import random
import uuid

import numpy as np
import pytest
import torch

from oracle import advantages as A
from oracle import masked as M
from conftest import load_golden

GOLDEN = load_golden()


# ---- masked_* ---------------------------------------------------------------------------------
@pytest.mark.parametrize("value,mask,want", [(c["value"], c["mask"], c["expected"])
                                             for c in GOLDEN["masked_mean"]["cases"]])
def test_masked_mean_reference_vectors(value, mask, want):
    # literals of tests/utils/test_torch_functional.py:60-71 (int64 mask, as there)
    got = M.masked_mean(torch.tensor(value), torch.tensor(mask))
    assert torch.allclose(got, torch.tensor(want), equal_nan=True)


@pytest.mark.parametrize("mdtype", [torch.float32, torch.int64, torch.bool])
def test_masked_var_and_whiten_against_torch_var(mdtype):
    g = torch.Generator().manual_seed(0)
    v = torch.randn(7, 33, generator=g) * 3 + 1.5
    m = (torch.rand(7, 33, generator=g) < 0.6)
    sel = v[m]
    mm = m.to(mdtype)
    assert torch.allclose(M.masked_mean(v, mm), sel.mean(), rtol=1e-6)
    assert torch.allclose(M.masked_var(v, mm), sel.var(unbiased=True), rtol=1e-5)
    assert torch.allclose(M.masked_var(v, mm, unbiased=False), sel.var(unbiased=False), rtol=1e-5)
    w = M.masked_whiten(v, mm)
    assert abs(w[m].mean().item()) < 1e-6 and abs(w[m].var(unbiased=True).item() - 1) < 1e-5
    w2 = M.masked_whiten(v, mm, shift_mean=False)
    assert torch.allclose(w2 - w, sel.mean().expand_as(w), atol=1e-6)
    # every element is transformed, masked or not
    assert torch.allclose(w, (v - sel.mean()) * torch.rsqrt(sel.var() + 1e-8), rtol=1e-5, atol=1e-6)


def test_masked_edge_cases():
    v = torch.tensor([[1.0, 2.0], [3.0, 4.0]])
    zero = torch.zeros(2, 2)
    assert M.masked_mean(v, zero).item() == 0.0                     # 0 / 1e-8
    with pytest.raises(ValueError):
        M.masked_var(v, zero)
    with pytest.raises(ValueError):
        M.masked_var(v, torch.tensor([[1.0, 0.0], [0.0, 0.0]]))
    # weighted float mask: where() keeps, then the weight multiplies
    w = torch.tensor([[0.5, 0.0], [2.0, 1.0]])
    assert M.masked_sum(v, w).item() == 0.5 * 1 + 2 * 3 + 4
    assert torch.equal(M.masked_sum(v, torch.ones(2, 2), axis=-1), torch.tensor([3.0, 7.0]))
    assert torch.equal(M.masked_mean(v, torch.tensor([[1, 0], [0, 0]]), axis=-1), torch.tensor([1.0, 0.0]))


def test_entropy_and_logprob_definitions():
    z = torch.tensor([[0.0, 0.0, 0.0, 0.0], [10.0, 0.0, 0.0, 0.0]])
    ent = M.entropy_from_logits(z)
    assert abs(ent[0].item() - math.log(4)) < 1e-6
    p = torch.softmax(z[1].double(), -1)
    assert abs(ent[1].item() - float(-(p * p.log()).sum())) < 1e-5
    lp = M.logprobs_from_logits(z, torch.tensor([2, 0]))
    assert abs(lp[0].item() + math.log(4)) < 1e-6 and abs(lp[1].item() - float(p[0].log())) < 1e-6
    x = torch.tensor([1.0, 5.0, -3.0])
    assert torch.equal(M.clip_by_value(x, torch.tensor([2.0, 2.0, -1.0]), torch.tensor([3.0, 4.0, 0.0])),
                       torch.tensor([2.0, 4.0, -1.0]))


# ---- GAE --------------------------------------------------------------------------------------
def _raw_gae(r, v, m, gamma, lam):
    adv, ret = A.gae_raw(r, v, m, gamma, lam)
    assert torch.equal(ret, adv + v)
    return adv


@pytest.mark.parametrize("B,L", [(1, 1), (3, 7), (3, 64)])
@pytest.mark.parametrize("gamma,lam", [(1.0, 1.0), (1.0, 0.95), (0.95, 0.5)])
def test_gae_against_fp64_brute_force(B, L, gamma, lam):
    g = torch.Generator().manual_seed(B * 100 + L)
    r = torch.randn(B, L, generator=g, dtype=torch.float64)
    v = torch.randn(B, L, generator=g, dtype=torch.float64)
    m = (torch.rand(B, L, generator=g) < 0.7).double()
    if B > 1:
        m[1] = 0                                   # an all-masked row
    got = _raw_gae(r, v, m, gamma, lam)
    want = torch.tensor(A.gae_brute_force_fp64(r.tolist(), v.tolist(), m.tolist(), gamma, lam), dtype=torch.float64)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    got32 = _raw_gae(r.float(), v.float(), m.float(), gamma, lam)
    assert torch.allclose(got32.double(), want, rtol=1e-5, atol=1e-5)


def test_gae_gamma_lambda_one_is_reverse_cumsum_of_rewards():
    g = torch.Generator().manual_seed(1)
    r = torch.randn(4, 50, generator=g, dtype=torch.float64)
    v = torch.randn(4, 50, generator=g, dtype=torch.float64)
    m = torch.ones(4, 50, dtype=torch.float64)
    _, ret = A.gae_advantage_return(r, v, m, 1.0, 1.0)
    assert torch.allclose(ret, torch.flip(torch.cumsum(torch.flip(r, [1]), 1), [1]), atol=1e-12)


def test_gae_multi_turn_fixture_invariance():
    # rewards / mask literals and the torch.equal assertion of
    # tests/trainer/ppo/test_core_algos_on_cpu.py:143-197
    random.seed(0)
    gamma, lam = random.uniform(0.0, 1.0), random.uniform(0.0, 1.0)
    fx = GOLDEN["gae_multi_turn"]
    rewards = torch.tensor(fx["rewards"])
    mask = torch.tensor(fx["response_mask"], dtype=torch.float)

    def values(free):                                   # fixed values on valid tokens, anything elsewhere
        v = torch.zeros(1, rewards.shape[1])
        for k, x in fx["values_at_valid_and_padding"].items():
            v[0, int(k)] = x
        for slot, x in zip(fx["free_value_slots"], free):
            v[0, slot] = x
        return v

    v1 = values([random.uniform(-100.0, 100.0), random.random(), random.uniform(-100.0, 0), random.random()])
    v2 = values([random.random(), random.uniform(-100.0, 100.0), random.random(), random.uniform(0.0, 100.0)])
    a1, r1 = A.gae_advantage_return(rewards, v1, mask, gamma, lam)
    a2, r2 = A.gae_advantage_return(rewards, v2, mask, gamma, lam)
    assert torch.equal(a1, a2) and torch.equal(r1 * mask, r2 * mask)
    # masked positions carry the state of the next valid token; trailing padding is 0 before whitening
    raw, _ = A.gae_raw(rewards, v1, mask, gamma, lam)
    assert raw[0, 0] == raw[0, 1] == raw[0, 2] and raw[0, 5] == raw[0, 6] == raw[0, 7]
    assert raw[0, 9] == 0 and raw[0, 10] == 0


# ---- GRPO -------------------------------------------------------------------------------------
def _make_group_index(batch_size, num_groups):
    counts = [2] * num_groups
    for _ in range(batch_size - 2 * num_groups):
        counts[random.randrange(num_groups)] += 1
    index = []
    for gid, c in enumerate(counts):
        index.extend([gid] * c)
    random.shuffle(index)
    return np.asarray(index, dtype=np.int64)


def _rand_mask(batch_size, seq_len):
    mask = torch.randint(0, 2, (batch_size, seq_len), dtype=torch.int64).float()
    rows = (mask.sum(dim=-1) == 0).nonzero(as_tuple=True)[0]
    if len(rows) > 0:
        mask[rows, -1] = 1.0
    return mask


@pytest.mark.parametrize("batch_size,seq_len,num_groups,seed", GOLDEN["grpo_equivalence_grid"]["cases"])
def test_grpo_loop_equals_vectorised_reference_grid(batch_size, seq_len, num_groups, seed):
    # grid and tolerance of tests/trainer/ppo/test_core_algos_on_cpu.py:262-313
    torch.manual_seed(seed); random.seed(seed); np.random.seed(seed)
    index = _make_group_index(batch_size, num_groups)
    mask = _rand_mask(batch_size, seq_len)
    rewards = torch.randn(batch_size, seq_len) * mask
    a1, r1 = A.grpo_outcome_advantage(rewards, mask, index)
    a2, r2 = A.grpo_vectorized_outcome_advantage(rewards, mask, index)
    assert a1.shape == (batch_size, seq_len) and a1 is r1 and a2 is r2
    assert torch.allclose(a1, a2, rtol=1e-5, atol=1e-6)


def test_group_mean_std_reference_known_answer():
    # tests/utils/test_groupwise.py:51-65
    fx = GOLDEN["group_mean_std"]
    mean_g, std_g, cnt_g = A.group_mean_std(torch.tensor(fx["scores"]), A.as_torch_index(fx["gidx"]))
    assert torch.allclose(mean_g, torch.tensor(fx["expected_mean"]))
    assert torch.allclose(cnt_g, torch.tensor(fx["expected_count"]))
    assert std_g[1].item() == fx["expected_std"][1] and abs(std_g[0].item() - fx["expected_std"][0]) < 1e-6
    e = A.group_mean_std(torch.tensor([]), torch.tensor([], dtype=torch.long))
    assert all(t.numel() == 0 for t in e)


def test_as_torch_index_cases():
    g = A.as_torch_index(["a", "b", "a", "c", "0042", 42])
    assert g.tolist()[4] != g.tolist()[5] and len(torch.unique(g)) == 5
    assert A.as_torch_index(np.array([3, 3, 7])).tolist() == [3, 3, 7]
    assert A.as_torch_index(torch.tensor([1.0, 2.0, 1.0])).tolist() == [1, 2, 1]
    assert A.as_torch_index(["5", "6", "5"]).tolist() == [5, 6, 5]
    ids = [str(uuid.UUID(int=i)) for i in (9, 4, 9, 1)]
    g = A.as_torch_index(np.array(ids, dtype=object))
    assert g[0] == g[2] and len(torch.unique(g)) == 3


def test_grpo_toy_input_by_hand():
    # input of tests/trainer/config/test_algo_config_on_cpu.py:187-197; answer worked by hand:
    # scores (1.5, 3.0 | 0.7, 2.3); unbiased std of a pair = |a-b|/sqrt(2)
    fx = GOLDEN["grpo_toy"]
    rewards = torch.tensor(fx["token_level_rewards"])
    mask = torch.tensor(fx["response_mask"])
    assert torch.allclose(rewards.sum(-1), torch.tensor(fx["scores"]))
    adv, _ = A.grpo_outcome_advantage(rewards, mask, np.array(fx["index"]))
    s0, s1 = 1.5 / math.sqrt(2), 1.6 / math.sqrt(2)
    want = torch.tensor([-0.75 / (s0 + 1e-6), 0.75 / (s0 + 1e-6), -0.8 / (s1 + 1e-6), 0.8 / (s1 + 1e-6)])
    assert torch.allclose(adv, want[:, None].expand(4, 3), rtol=1e-5)
    adv2, _ = A.grpo_outcome_advantage(rewards, mask, np.array([0, 0, 1, 1]), norm_adv_by_std_in_grpo=False)
    assert torch.allclose(adv2[:, 0], torch.tensor(fx["expected_unnormalised"]), rtol=1e-5)


def test_grpo_singletons_strings_equal_scores_and_unmasked_sum():
    rewards = torch.tensor([[1.0, 2.0], [3.0, 0.0], [3.0, 0.0], [5.0, 5.0]])
    mask = torch.tensor([[1.0, 0.0], [1.0, 1.0], [1.0, 1.0], [0.0, 1.0]])
    index = np.array(["u-a", "u-b", "u-b", "u-c"], dtype=object)
    adv, _ = A.grpo_outcome_advantage(rewards, mask, index)
    # singleton: (s - 0)/(1 + eps), score counts the reward at the masked position too
    assert torch.allclose(adv[0], torch.tensor([3.0 / (1 + 1e-6), 0.0]))
    assert torch.equal(adv[1], torch.zeros(2)) and torch.equal(adv[2], torch.zeros(2))   # equal scores -> 0
    assert torch.allclose(adv[3], torch.tensor([0.0, 10.0 / (1 + 1e-6)]))
    adv_v, _ = A.grpo_vectorized_outcome_advantage(rewards, mask, index)
    assert torch.allclose(adv, adv_v, rtol=1e-5, atol=1e-6)


# ---- other outcome estimators ---------------------------------------------------------------------
@pytest.mark.parametrize("batch_size,seq_len,num_groups,seed", GOLDEN["grpo_equivalence_grid"]["cases"])
def test_rloo_loop_equals_vectorised_reference_grid(batch_size, seq_len, num_groups, seed):
    # the same grid, generators and tolerance: tests/trainer/ppo/test_core_algos_on_cpu.py:222-259
    torch.manual_seed(seed); random.seed(seed); np.random.seed(seed)
    index = _make_group_index(batch_size, num_groups)
    mask = _rand_mask(batch_size, seq_len)
    rewards = torch.randn(batch_size, seq_len) * mask
    a1, r1 = A.rloo_outcome_advantage(rewards, mask, index)
    a2, r2 = A.rloo_vectorized_outcome_advantage(rewards, mask, index)
    assert a1.shape == a2.shape == (batch_size, seq_len) and a1 is r1 and a2 is r2
    assert torch.allclose(a1, a2, rtol=1e-5, atol=1e-6)


def _scores_groups():
    rewards = torch.tensor([[1.0, 2.0, 0.0], [0.5, 0.0, 0.0], [4.0, 1.0, 1.0], [0.0, 0.0, 0.0], [2.0, 2.0, 2.0]])
    mask = torch.tensor([[1.0, 1.0, 0.0], [1.0, 0.0, 0.0], [1.0, 1.0, 1.0], [1.0, 1.0, 0.0], [1.0, 1.0, 1.0]])
    index = np.array(["a", "a", "a", "b", "c"], dtype=object)      # sizes 3, 1, 1; scores 3, 0.5, 6 | 0 | 6
    return rewards, mask, index


def test_rloo_is_leave_one_out_mean_and_singleton_rules():
    rewards, mask, index = _scores_groups()
    adv, _ = A.rloo_outcome_advantage(rewards, mask, index)
    s = [3.0, 0.5, 6.0]
    for i in range(3):                                  # s_i minus the mean of the OTHER members
        others = [s[j] for j in range(3) if j != i]
        assert torch.allclose(adv[i], (s[i] - sum(others) / 2) * mask[i], atol=1e-6)
    assert torch.equal(adv[3], torch.zeros(3)) and torch.equal(adv[4], 6.0 * mask[4])   # single member keeps its score
    adv_v, _ = A.rloo_vectorized_outcome_advantage(rewards, mask, index)
    assert torch.allclose(adv_v[:3], adv[:3], atol=1e-6) and torch.equal(adv_v[4], torch.zeros(3))   # ... or gets 0


def test_opo_gpg_and_mean_baseline_by_hand():
    rewards, mask, index = _scores_groups()
    lens = [2.0, 1.0, 3.0]
    bsl = (2 * 3.0 + 1 * 0.5 + 3 * 6.0) / 6.0
    adv, _ = A.opo_outcome_advantage(rewards, mask, index)
    for i, s in enumerate([3.0, 0.5, 6.0]):
        assert torch.allclose(adv[i], (s - bsl) * mask[i], atol=1e-6)
    assert torch.equal(adv[4], 6.0 * mask[4])           # single member: baseline 0
    # GPG: alpha = 5 / #{scores != 0} = 5/4, mean of group a = 19/6, f_norm = 2
    adv, _ = A.gpg_outcome_advantage(rewards, mask, index, f_norm=2.0)
    for i, s in enumerate([3.0, 0.5, 6.0]):
        assert torch.allclose(adv[i], 1.25 * (s - 19.0 / 6.0) / 2.0 * mask[i], atol=1e-6)
    assert torch.allclose(adv[4], 1.25 * 6.0 / 2.0 * mask[4])
    # REINFORCE++ baseline: centred scores on the mask, then masked whitening, then the mask again
    adv, _ = A.reinforce_plus_plus_baseline_outcome_advantage(rewards, mask, index)
    cen = torch.tensor([3.0 - 19 / 6, 0.5 - 19 / 6, 6.0 - 19 / 6, 0.0, 6.0])[:, None] * mask
    sel = cen[mask.bool()]
    want = (cen - sel.mean()) * torch.rsqrt(sel.var(unbiased=True) + 1e-8) * mask
    assert torch.allclose(adv, want, atol=1e-5)
    w = adv[mask.bool()]
    assert abs(w.mean().item()) < 1e-6 and abs(w.var(unbiased=True).item() - 1) < 1e-5


def test_reinforce_plus_plus_and_remax_closed_forms():
    g = torch.Generator().manual_seed(3)
    r = torch.randn(3, 17, generator=g, dtype=torch.float64)
    ones = torch.ones(3, 17, dtype=torch.float64)
    # all-ones mask: plain discounted return  R_t = sum_s gamma^(s-t) r_s
    _, ret = A.reinforce_plus_plus_outcome_advantage(r, ones, 0.9)
    want = torch.zeros_like(r)
    for t in range(17):
        want[:, t] = sum(0.9 ** (s - t) * r[:, s] for s in range(t, 17))
    assert torch.allclose(ret, want, atol=1e-12)
    # a masked step cuts the return: position 9 is the last one that sees anything from the right of it ... no:
    # the running value is zeroed AFTER position 10 was written, so R_9 = r_9 and nothing to the right leaks in
    m = ones.clone(); m[:, 10] = 0
    adv, ret = A.reinforce_plus_plus_outcome_advantage(r, m, 0.9)
    assert torch.allclose(ret[:, 9], r[:, 9]) and torch.allclose(ret[:, 10], want[:, 10])
    assert torch.equal(adv[:, 10], torch.zeros(3, dtype=torch.float64))
    sel = ret[m.bool()]
    assert torch.allclose(adv, (ret - sel.mean()) * torch.rsqrt(sel.var(unbiased=True) + 1e-8) * m, atol=1e-10)
    # gamma = 1, all-ones mask: REINFORCE++ returns == ReMax returns == reverse cumulative sum
    _, r1 = A.reinforce_plus_plus_outcome_advantage(r, ones, 1.0)
    base = torch.tensor([0.5, -1.0, 2.0], dtype=torch.float64)
    adv2, r2 = A.remax_outcome_advantage(r, base, ones)
    cum = torch.flip(torch.cumsum(torch.flip(r, [1]), 1), [1])
    assert torch.allclose(r1, cum, atol=1e-12) and torch.allclose(r2, cum, atol=1e-12)
    assert torch.allclose(adv2, cum - base[:, None], atol=1e-12)
    # ReMax with a mask: masked rewards do not count, masked positions still show the carried sum
    adv3, r3 = A.remax_outcome_advantage(r, base, m)
    assert torch.allclose(r3[:, 10], r3[:, 11]) and torch.allclose(adv3[:, 10], r3[:, 10])


def test_sum_pi_squared_closed_forms():
    z = torch.zeros(2, 50, dtype=torch.float64)
    assert torch.allclose(M.sum_pi_squared_from_logits(z), torch.full((2,), 1 / 50, dtype=torch.float64))   # uniform
    z = torch.tensor([[40.0, 0.0, 0.0]], dtype=torch.float64)
    assert abs(M.sum_pi_squared_from_logits(z).item() - 1.0) < 1e-15                                          # one-hot
    g = torch.Generator().manual_seed(0)
    z = torch.randn(5, 33, generator=g, dtype=torch.float64) * 3
    assert torch.allclose(M.sum_pi_squared_from_logits(z), (torch.softmax(z, -1) ** 2).sum(-1), rtol=1e-12)  # brute force
    assert torch.allclose(M.sum_pi_squared_from_logits(z + 7.5), M.sum_pi_squared_from_logits(z), rtol=1e-12)  # shift


def test_grpo_passk_by_hand():
    rewards, mask, _ = _scores_groups()                               # scores 3, 0.5, 6, 0, 6
    index = np.array(["a", "a", "a", "b", "b"], dtype=object)         # groups {3, 0.5, 6} and {0, 6}
    adv, adv2 = A.grpo_passk_outcome_advantage(rewards, mask, index, norm_by_std=False)
    assert adv is adv2
    assert torch.equal(adv[2], 3.0 * mask[2]) and torch.equal(adv[4], 6.0 * mask[4])      # max - second max
    assert adv[[0, 1, 3]].abs().sum().item() == 0
    adv, _ = A.grpo_passk_outcome_advantage(rewards, mask, index)
    std_a = torch.tensor([3.0, 0.5, 6.0]).std()
    assert torch.allclose(adv[2], 3.0 / (std_a + 1e-6) * mask[2])
    assert torch.allclose(adv[4], 6.0 / (6.0 / math.sqrt(2) + 1e-6) * mask[4])
    tied = rewards.clone(); tied[0] = tied[2]                         # best score held twice: the advantage is 0
    assert A.grpo_passk_outcome_advantage(tied, mask, index)[0][:3].abs().sum().item() == 0
    with pytest.raises(ValueError):
        A.grpo_passk_outcome_advantage(rewards, mask, np.array(["a", "a", "a", "b", "c"], dtype=object))


# ---- optimal token baseline ---------------------------------------------------------------------
def _otb_case(seed, B, L, groups, multi_turn):
    g = torch.Generator().manual_seed(seed)
    rewards = torch.randn(B, L, generator=g, dtype=torch.float64)
    if multi_turn:  # several generation turns with tool output (masked) between them
        mask = (torch.rand(B, L, generator=g) < 0.6).double()
        mask[0] = 0  # a trajectory with no valid token
    else:
        lens = torch.randint(1, L + 1, (B,), generator=g)
        mask = (torch.arange(L)[None, :] < lens[:, None]).double()
    old_lp = -torch.rand(B, L, generator=g, dtype=torch.float64) * 4
    pi2 = torch.rand(B, L, generator=g, dtype=torch.float64)
    isw = 0.5 + torch.rand(B, L, generator=g, dtype=torch.float64)
    index = np.array([f"p{int(i)}" for i in torch.randint(0, groups, (B,), generator=g)], dtype=object)
    return rewards, mask, index, old_lp, pi2, isw


@pytest.mark.parametrize("seed,B,L,groups", [(0, 12, 17, 3), (1, 9, 8, 9), (2, 16, 33, 2)])
@pytest.mark.parametrize("with_isw", [False, True])
@pytest.mark.parametrize("zero_tail", [False, True])
@pytest.mark.parametrize("multi_turn", [False, True])
def test_optimal_token_baseline_against_fp64_brute_force(seed, B, L, groups, with_isw, zero_tail, multi_turn):
    r, m, index, lp, pi2, isw = _otb_case(seed, B, L, groups, multi_turn)
    w = isw if with_isw else None
    want_adv, want_ret = A.otb_brute_force_fp64(r.tolist(), m.tolist(), index.tolist(), lp.tolist(), pi2.tolist(),
                                                None if w is None else w.tolist(), packed=multi_turn,
                                                zero_tail=zero_tail)
    fn = A.multi_turn_optimal_token_baseline_advantage if multi_turn else A.optimal_token_baseline_advantage
    adv, ret = fn(r, m, index, lp, pi2, rollout_is_weights=w, handle_zero_tail=zero_tail)
    assert torch.allclose(ret, torch.tensor(want_ret, dtype=torch.float64), rtol=1e-12, atol=1e-12)
    assert torch.allclose(adv, torch.tensor(want_adv, dtype=torch.float64), rtol=1e-9, atol=1e-9)


def test_optimal_token_baseline_by_hand():
    # two full-length responses of one prompt and a lone response of another; pi = 1/2 and sum pi^2 = 1/2 give
    # w = 1/2 per token, so W = (1/2, 1) on both rows and the baseline is the plain mean of the returns
    r = torch.tensor([[1.0, 2.0], [3.0, 0.0], [5.0, 7.0]])
    m = torch.ones(3, 2)
    lp = torch.full((3, 2), math.log(0.5))
    pi2 = torch.full((3, 2), 0.5)
    index = np.array(["a", "a", "b"], dtype=object)
    adv, ret = A.optimal_token_baseline_advantage(r, m, index, lp, pi2)
    assert ret.tolist() == [[3.0, 2.0], [3.0, 0.0], [12.0, 7.0]]
    assert torch.allclose(adv, torch.tensor([[0.0, 1.0], [0.0, -1.0], [12.0, 7.0]]), atol=1e-6)
    # unequal path variance: row 0 deterministic (w = 0), row 1 as before -> the baseline is row 1's return
    lp0 = lp.clone(); lp0[0] = 0.0
    pi20 = pi2.clone(); pi20[0] = 1.0
    adv, _ = A.optimal_token_baseline_advantage(r, m, index, lp0, pi20)
    assert torch.allclose(adv[:2], torch.tensor([[0.0, 2.0], [0.0, 0.0]]), atol=1e-6)
    # the importance weights enter squared: doubling them on row 1 leaves a one-sided baseline unchanged
    adv2, _ = A.optimal_token_baseline_advantage(r, m, index, lp0, pi20,
                                                 rollout_is_weights=torch.tensor([[1.0, 1.0], [2.0, 2.0], [1.0, 1.0]]))
    assert torch.allclose(adv2[:2], adv[:2], atol=1e-6)
    # zero tail: row 1 shorter -> beyond its length the longest row keeps its return as the advantage
    m2 = torch.tensor([[1.0, 1.0], [1.0, 0.0], [1.0, 1.0]])
    adv3, ret3 = A.optimal_token_baseline_advantage(r, m2, index, lp, pi2, handle_zero_tail=True)
    assert adv3[0, 1].item() == ret3[0, 1].item() == 2.0
    adv4, _ = A.optimal_token_baseline_advantage(r, m2, index, lp, pi2, handle_zero_tail=False)
    assert abs(adv4[0, 1].item()) < 1e-6  # alone in its column: the baseline equals its own return


def test_multi_turn_optimal_token_baseline_packs_valid_tokens():
    # with prefix masks the packed variant is the plain one
    r, m, index, lp, pi2, _ = _otb_case(5, 10, 12, 3, multi_turn=False)
    a, _ = A.optimal_token_baseline_advantage(r, m, index, lp, pi2)
    b, _ = A.multi_turn_optimal_token_baseline_advantage(r, m, index, lp, pi2, handle_zero_tail=False)
    assert torch.allclose(a, b, rtol=1e-12, atol=1e-12)
    # inserting masked columns into the trajectories does not change the advantages of the valid tokens
    L = m.shape[1]
    wide = lambda x: torch.stack([x, torch.zeros_like(x)], dim=-1).reshape(x.shape[0], 2 * L)  # noqa: E731
    c, _ = A.multi_turn_optimal_token_baseline_advantage(wide(r), wide(m), index, wide(lp), wide(pi2),
                                                         handle_zero_tail=False)
    assert torch.allclose(c[:, 0::2], b, rtol=1e-12, atol=1e-12) and (c[:, 1::2] == 0).all()
