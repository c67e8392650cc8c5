"""Pins for oracle/losses.py: scalar Python loops written from the definitions,
the special cases that collapse to closed forms, and the hand-derived gradients
checked against autograd (including exact ties)."""
import math

import pytest
import torch

from oracle import losses as L
from oracle import masked as M


def _case(B=5, T=37, seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    old = torch.randn(B, T, generator=g, dtype=dtype) * 0.5 - 1
    new = old + torch.randn(B, T, generator=g, dtype=dtype) * 0.3
    adv = torch.randn(B, T, generator=g, dtype=dtype)
    mask = (torch.rand(B, T, generator=g) < 0.7).to(dtype)
    mask[1] = 0
    return old, new, adv, mask


def _scalar_policy_loss(old, new, adv, mask, lo, hi, c):
    """Per-element loss and indicator sums by plain Python floats."""
    n = tot = kl = cf = cfl = 0.0
    per_elem = []
    for o, x, a, m in zip(old.flatten().tolist(), new.flatten().tolist(), adv.flatten().tolist(),
                          mask.flatten().tolist()):
        k = min(max(x - o, -20.0), 20.0)
        r = math.exp(k)
        l1 = -a * r
        l2 = -a * min(max(r, 1 - lo), 1 + hi)
        c1 = max(l1, l2)
        l3 = -a * c
        loss = min(l3, c1) if a < 0 else c1
        per_elem.append(loss)
        if m:
            n += m; tot += loss * m; kl += -k * m
            cf += (l2 > l1) * m
            cfl += ((c1 > l3) and (a < 0)) * m
    return per_elem, tot, n, kl, cf, cfl


@pytest.mark.parametrize("seed", [0, 1])
def test_policy_loss_token_mean_against_scalar_loop(seed):
    old, new, adv, mask = _case(seed=seed)
    new[0, :5] = old[0, :5] + 25.0          # beyond the +-20 clamp
    new[2, :5] = old[2, :5] + 2.0           # large ratio: dual clip for A<0
    loss, cf, kl, cfl = L.policy_loss_vanilla(old, new, adv, mask, "token-mean", 0.2, 0.28, 3.0)
    _, tot, n, kls, cfs, cfls = _scalar_policy_loss(old, new, adv, mask, 0.2, 0.28, 3.0)
    assert abs(loss.item() - tot / n) < 1e-12
    assert abs(kl.item() - kls / (n + 1e-8)) < 1e-12
    assert abs(cf.item() - cfs / (n + 1e-8)) < 1e-12
    assert abs(cfl.item() - cfls / (n + 1e-8)) < 1e-12


def test_policy_loss_special_cases():
    old, _, adv, mask = _case(seed=3)
    # on-policy: ratio 1  =>  loss = -sum(A m)/M, kl = 0, nothing clipped
    loss, cf, kl, cfl = L.policy_loss_vanilla(old, old.clone(), adv, mask, "token-mean")
    assert abs(loss.item() + (adv * mask).sum().item() / mask.sum().item()) < 1e-12
    assert kl.item() == 0 and cf.item() == 0 and cfl.item() == 0
    # A >= 0 never dual-clips
    _, _, _, cfl = L.policy_loss_vanilla(old, old + 3.0, adv.abs(), mask, "token-mean")
    assert cfl.item() == 0
    # A < 0 and a huge ratio: every valid token sits on the floor -A*c
    loss, _, _, cfl = L.policy_loss_vanilla(old, old + 5.0, -adv.abs() - 0.1, mask, "token-mean", clip_ratio_c=3.0)
    want = (3.0 * (adv.abs() + 0.1) * mask).sum() / mask.sum()
    assert abs(loss.item() - want.item()) < 1e-12 and abs(cfl.item() - mask.sum().item() / (mask.sum().item() + 1e-8)) < 1e-12
    # rollout importance weights scale the per-token loss
    w = torch.full_like(old, 0.5)
    a = L.policy_loss_vanilla(old, old + 0.1, adv, mask, "token-mean")[0]
    b = L.policy_loss_vanilla(old, old + 0.1, adv, mask, "token-mean", rollout_is_weights=w)[0]
    assert abs(b.item() - 0.5 * a.item()) < 1e-12
    with pytest.raises(AssertionError):
        L.policy_loss_vanilla(old, old, adv, mask, clip_ratio_c=1.0)


def _hand_policy_grad(old, new, adv, mask, lo, hi, c):
    """d loss / d new for token-mean, from the branch analysis (no autograd)."""
    k = new - old
    inside = (k >= -20) & (k <= 20)
    r = torch.exp(k.clamp(-20, 20))
    l1 = -adv * r
    l2 = -adv * r.clamp(1 - lo, 1 + hi)
    clipped_wins = l2 > l1                       # constant branch selected
    unclipped = ~clipped_wins
    c1 = torch.maximum(l1, l2)
    floor_wins = (adv < 0) & (c1 > -adv * c)
    live = unclipped & ~floor_wins & inside
    return torch.where(live, -adv * r, torch.zeros_like(r)) * mask / mask.sum()


def test_policy_loss_gradient_matches_branch_analysis():
    old, new, adv, mask = _case(seed=4)
    new[0, :6] = old[0, :6] + 1.5
    new[3, :6] = old[3, :6] - 1.5
    new = new.clone().requires_grad_()
    loss = L.policy_loss_vanilla(old, new, adv, mask, "token-mean", 0.2, 0.2, 3.0)[0]
    g, = torch.autograd.grad(loss, new)
    assert torch.allclose(g, _hand_policy_grad(old, new.detach(), adv, mask, 0.2, 0.2, 3.0), atol=1e-14)


def test_policy_loss_gradient_on_exact_ties():
    # r == 1 (l1 == l2, both carry d/dlp = -A) and A == 0: torch splits max() ties 50/50, total unchanged
    old = torch.zeros(1, 4, dtype=torch.float64)
    new = torch.zeros(1, 4, dtype=torch.float64, requires_grad=True)
    adv = torch.tensor([[1.0, -2.0, 0.0, 0.5]], dtype=torch.float64)
    mask = torch.ones(1, 4, dtype=torch.float64)
    g, = torch.autograd.grad(L.policy_loss_vanilla(old, new, adv, mask)[0], new)
    assert torch.allclose(g, -adv / 4)


@pytest.mark.parametrize("mode", ["token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm"])
def test_agg_loss_modes_by_loops(mode):
    _, x, _, mask = _case(seed=5)
    got = L.agg_loss(x, mask, mode).item()
    rows = [(sum(v * m for v, m in zip(xr, mr)), sum(mr)) for xr, mr in zip(x.tolist(), mask.tolist())]
    if mode == "token-mean":
        want = sum(s for s, _ in rows) / sum(c for _, c in rows)
    elif mode == "seq-mean-token-sum":
        want = sum(s for s, c in rows if c > 0) / sum(1 for _, c in rows if c > 0)
    elif mode == "seq-mean-token-mean":
        want = sum(s / (c + 1e-8) for s, c in rows if c > 0) / sum(1 for _, c in rows if c > 0)
    else:
        want = sum(s for s, _ in rows) / x.shape[-1]
    assert abs(got - want) < 1e-12
    # global-batch arguments
    if mode == "token-mean":
        assert abs(L.agg_loss(x, mask, mode, dp_size=4, batch_num_tokens=1000).item()
                   - sum(s for s, _ in rows) / 1000 * 4) < 1e-12
    if mode == "seq-mean-token-sum-norm":
        assert abs(L.agg_loss(x, mask, mode, loss_scale_factor=7).item() - sum(s for s, _ in rows) / 7) < 1e-12
    with pytest.raises(ValueError):
        L.agg_loss(x, mask, "nope")


def test_value_loss_against_scalar_loop_and_gradient():
    g = torch.Generator().manual_seed(6)
    B, T, c = 4, 29, 0.5
    values = torch.randn(B, T, generator=g, dtype=torch.float64)
    vpreds = (values + torch.randn(B, T, generator=g, dtype=torch.float64)).requires_grad_()
    returns = values + torch.randn(B, T, generator=g, dtype=torch.float64)
    mask = (torch.rand(B, T, generator=g) < 0.8).double()
    loss, frac = L.value_loss(vpreds, returns, values, mask, c)
    tot = cnt = cf = 0.0
    hand = torch.zeros(B, T, dtype=torch.float64)
    for i in range(B):
        for t in range(T):
            vp, R, v, m = vpreds[i, t].item(), returns[i, t].item(), values[i, t].item(), mask[i, t].item()
            vc = max(min(vp, v + c), v - c)
            e1, e2 = (vp - R) ** 2, (vc - R) ** 2
            tot += max(e1, e2) * m; cnt += m; cf += (e2 > e1) * m
            inside = v - c < vp < v + c
            hand[i, t] = (vp - R) * m if (inside or e1 > e2) else 0.0
    assert abs(loss.item() - 0.5 * tot / cnt) < 1e-12 and abs(frac.item() - cf / (cnt + 1e-8)) < 1e-12
    gr, = torch.autograd.grad(loss, vpreds)
    assert torch.allclose(gr, hand / cnt, atol=1e-14)


def test_kl_estimators():
    a = torch.tensor([-1.0, -2.0, -0.5], dtype=torch.float64)
    b = torch.tensor([-1.5, -1.0, -0.5], dtype=torch.float64)
    assert torch.equal(L.kl_penalty_forward(a, b, "kl"), a - b)
    assert torch.equal(L.kl_penalty_forward(a, b, "abs"), (a - b).abs())
    assert torch.allclose(L.kl_penalty_forward(a, b, "mse"), 0.5 * (a - b) ** 2)
    d = b - a
    assert torch.allclose(L.kl_penalty_forward(a, b, "low_var_kl"), torch.exp(d) - d - 1)
    assert L.kl_penalty_forward(torch.tensor([0.0]), torch.tensor([30.0]), "k3").item() == 10.0   # clamp at 10


def test_kl_penalty_as_written_and_straight_through():
    """kl_penalty hands the name to kl_penalty_forward unchanged (core_algos.py:1853), so "+" names fail there;
    the straight-through combination keeps the forward value and takes the k2 gradient."""
    a = torch.tensor([-1.0, -2.0, -0.5, -3.0], dtype=torch.float64, requires_grad=True)
    b = torch.tensor([-1.5, -1.0, -0.5, 25.0], dtype=torch.float64)
    for name in ("kl", "abs", "mse", "low_var_kl", "k1", "k2", "k3"):
        assert torch.equal(L.kl_penalty(a, b, name), L.kl_penalty_forward(a, b, name))
    for name in ("k1+", "k3+", "abs+", "mse+", "full", "nonsense"):
        with pytest.raises(NotImplementedError):
            L.kl_penalty(a, b, name)
    fwd = L.kl_penalty_forward(a, b, "k3")
    st = L.kl_straight_through(a, b, fwd)
    assert torch.equal(st.detach(), fwd.detach())
    g, = torch.autograd.grad(st.sum(), a)
    assert torch.allclose(g, (a - b).detach())
    # closed-form gradients of the estimators: k1 -> 1, abs -> sign, k2 -> d, k3 -> 1 - exp(ref - lp) inside the clamps
    for name, want in (("k1", torch.ones(4, dtype=torch.float64)), ("abs", torch.tensor([1.0, -1.0, 0.0, -1.0], dtype=torch.float64)),
                       ("k2", (a - b).detach())):
        g, = torch.autograd.grad(L.kl_penalty_forward(a, b, name).sum(), a)
        assert torch.allclose(g, want)
    g, = torch.autograd.grad(L.kl_penalty_forward(a, b, "k3").sum(), a)
    want = 1 - torch.exp((b - a).detach())
    want[3] = 0.0                                   # ref - lp = 28 is clamped to 20: no gradient
    assert torch.allclose(g, want)


def _policy_inputs(seed=0, B=4, Lc=9, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    old = torch.randn(B, Lc, generator=g, dtype=dtype) * 0.5 - 1
    new = (old + torch.randn(B, Lc, generator=g, dtype=dtype) * 0.3).requires_grad_()
    adv = torch.randn(B, Lc, generator=g, dtype=dtype)
    mask = (torch.rand(B, Lc, generator=g) < 0.8).to(dtype)
    mask[:, 0] = 1
    return old, new, adv, mask


def test_policy_loss_variants_closed_forms():
    """Each variant against a scalar loop of its published formula, and its gradient against the hand derivative."""
    old, new, adv, mask = _policy_inputs()
    B, Lc = old.shape
    # GPG: token-mean of -lp A; d/dlp = -A m / M
    loss = L.policy_loss_gpg(new, adv, mask)
    M_ = mask.sum()
    assert torch.allclose(loss, (-(new * adv) * mask).sum() / M_)
    g, = torch.autograd.grad(loss, new)
    assert torch.allclose(g, -adv * mask / M_)
    # CISPO: the clipped ratio is a constant factor
    loss, cf, kl, _ = L.policy_loss_cispo(old, new, adv, mask, clip_ratio_low=0.2, clip_ratio_high=0.3)
    r = torch.exp(new.detach() - old)
    rc = r.clamp(0.8, 1.3)
    assert torch.allclose(loss, (-(rc * adv * new.detach()) * mask).sum() / M_)
    g, = torch.autograd.grad(loss, new)
    assert torch.allclose(g, -rc * adv * mask / M_)
    assert torch.allclose(cf, (((r < 0.8) | (r > 1.3)).double() * mask).sum() / (M_ + 1e-8))
    assert torch.allclose(kl, (-(new.detach() - old) * mask).sum() / (M_ + 1e-8))
    # SAPO: seq-mean-token-mean of -(4/tau) sigmoid(tau (r - 1)) A;  d/dlp = -4 A s (1 - s) r
    loss, _, _, _ = L.policy_loss_sapo(old, new, adv, mask, tau_pos=1.0, tau_neg=1.05)
    tau = torch.where(adv > 0, torch.tensor(1.0, dtype=torch.float64), torch.tensor(1.05, dtype=torch.float64))
    sgm = torch.sigmoid(tau * (r - 1))
    per_tok = -(4 / tau) * sgm * adv
    rows = (per_tok * mask).sum(-1) / (mask.sum(-1) + 1e-8)
    assert torch.allclose(loss, rows.mean())
    g, = torch.autograd.grad(loss, new)
    assert torch.allclose(g, (-4 * adv * sgm * (1 - sgm) * r) * mask / (mask.sum(-1, keepdim=True) + 1e-8) / B)
    # GSPO: one ratio per sequence; with identical advantages along a row and no clipping the row loss is -A s_i
    seq = ((new.detach() - old) * mask).sum(-1) / mask.sum(-1)
    adv_row = adv[:, :1].expand(B, Lc).contiguous()
    loss, cf, kl, low = L.policy_loss_gspo(old, new, adv_row, mask, clip_ratio_low=10.0, clip_ratio_high=10.0)
    assert torch.allclose(loss, (-adv_row[:, 0] * torch.exp(seq)).mean()) and cf.item() == 0 and low.item() == 0
    g, = torch.autograd.grad(loss, new)                # d/dlp_t = -A exp(s_i) m_t / M_i / B : token-level gradient
    assert torch.allclose(g, (-adv_row * torch.exp(seq)[:, None]) * mask / (mask.sum(-1, keepdim=True) + 1e-8) / B)
    # tight clip range: every token of a row with s_i outside the range and the "wrong" sign of A is clipped
    loss, cf, _, _ = L.policy_loss_gspo(old, new, adv, mask, clip_ratio_low=1e-4, clip_ratio_high=1e-4)
    rr = torch.exp(seq)[:, None].expand(B, Lc)
    l1 = -adv * rr; l2 = -adv * rr.clamp(1 - 1e-4, 1 + 1e-4)
    assert torch.allclose(cf, ((l2 > l1).double() * mask).sum() / (M_ + 1e-8))


def test_reinforce_and_geo_mean_closed_forms():
    old, new, adv, mask = _policy_inputs()
    B, Lc = old.shape
    M_ = mask.sum()
    # REINFORCE: seq-mean-token-sum of -lp A w; the KL is measured against the first argument
    w = torch.rand(B, Lc, dtype=torch.float64) + 0.5
    loss, kl = L.policy_loss_reinforce(old, new, adv, mask, "seq-mean-token-sum", rollout_is_weights=w)
    assert torch.allclose(loss, (-(new * adv * w) * mask).sum(-1).mean())
    assert torch.allclose(kl, ((old - new.detach()) * mask).sum() / (M_ + 1e-8))
    g, = torch.autograd.grad(loss, new)
    assert torch.allclose(g, -adv * w * mask / B)
    # GMPO against scalar loops written from the paper's objective: per sequence the geometric mean of the token
    # ratios, each clipped only where clipping lowers the objective, times the mean advantage
    lo, hi = 0.05, 0.1
    loss, cf, kl, cfl = L.policy_loss_geo_mean(old, new, adv, mask, lo, hi, rollout_is_weights=w)
    total, n_up, n_dn, dsum = 0.0, 0, 0, 0.0
    grads = torch.zeros(B, Lc, dtype=torch.float64)
    for i in range(B):
        toks = [t for t in range(Lc) if mask[i, t] != 0]
        logs, a_sum, w_logs, free = 0.0, 0.0, 0.0, []
        for t in toks:
            x = (new[i, t] - old[i, t]).item()
            a = adv[i, t].item()
            c = min(max(x, -lo), hi)
            if a > 0:
                k, is_free = min(x, c), x <= hi
            elif a < 0:
                k, is_free = max(x, c), x >= -lo
            else:
                k, is_free = 0.0, False
            logs += k; a_sum += a; w_logs += math.log(w[i, t].item() + 1e-10); dsum -= x
            n_up += (x != c and a > 0); n_dn += (x != c and a < 0)
            free.append((t, is_free))
        n = len(toks)
        row = -(a_sum / n) * math.exp(logs / n) * math.exp(w_logs / n)
        total += row / B
        for t, is_free in free:
            grads[i, t] = row / n / B if is_free else 0.0
    assert loss.item() == pytest.approx(total, rel=1e-7)      # the reference adds 1e-8 to the lengths
    assert cf.item() == pytest.approx(n_up / M_.item()) and cfl.item() == pytest.approx(n_dn / M_.item())
    assert kl.item() == pytest.approx(dsum / M_.item(), rel=1e-9)
    g, = torch.autograd.grad(loss, new)
    assert torch.allclose(g, grads, rtol=1e-7, atol=1e-12)
    # a wide clip range and one advantage per sequence: loss = -mean_i A_i exp(mean_t log-ratio)
    adv_row = adv[:, :1].expand(B, Lc).contiguous()
    loss, cf, _, cfl = L.policy_loss_geo_mean(old, new.detach(), adv_row, mask, 50.0, 50.0)
    seq = ((new.detach() - old) * mask).sum(-1) / mask.sum(-1)
    assert torch.allclose(loss, (-adv_row[:, 0] * torch.exp(seq)).mean()) and cf.item() == 0 and cfl.item() == 0


def test_kl_cov_and_clip_cov_against_scalar_loops():
    old, new, adv, mask = _policy_inputs(seed=3, B=6, Lc=40)
    B, Lc = old.shape
    toks = [(i, t) for i in range(B) for t in range(Lc) if mask[i, t] != 0]
    n = len(toks)
    # KL-Cov: 5 % of the valid tokens, those with the largest covariance, carry the extra |log ratio| term
    loss, kl_abs, selected = L.policy_loss_kl_cov(old, new, adv, mask, "token-mean", kl_cov_ratio=0.05, ppo_kl_coef=0.7)
    ma = sum(adv[i, t].item() for i, t in toks) / n
    ml = sum(new[i, t].item() for i, t in toks) / n
    cov = {(i, t): (adv[i, t].item() - ma) * (new[i, t].item() - ml) for i, t in toks}
    k = max(1, int(n * 0.05))
    top = set(sorted(cov, key=cov.get, reverse=True)[:k])
    assert {(i, t) for i, t in toks if selected[i, t]} == top and int(selected.sum()) == k
    total = 0.0
    for i, t in toks:
        x = (new[i, t] - old[i, t]).item()
        total += -adv[i, t].item() * math.exp(x) + (0.7 * abs(x) if (i, t) in top else 0.0)
    assert loss.item() == pytest.approx(total / n, rel=1e-9)
    assert kl_abs.item() == pytest.approx(sum(abs((new[i, t] - old[i, t]).item()) for i, t in toks) / n, rel=1e-7)
    g, = torch.autograd.grad(loss, new)
    i, t = next(iter(top))
    x = (new[i, t] - old[i, t]).item()
    assert g[i, t].item() == pytest.approx((-adv[i, t].item() * math.exp(x) + 0.7 * math.copysign(1, x)) / n, rel=1e-7)
    assert L.policy_loss_kl_cov(old, new.detach(), adv, mask, kl_cov_ratio=1e-9)[2].sum() == 1       # at least one token

    # Clip-Cov: the candidate band and clip_num by loops; the draw replaced by a fixed choice
    cand, clip_num = L.clip_cov_candidates(old, new.detach(), adv, mask, 0.2, 0.25, clip_cov_lb=0.05, clip_cov_ub=2.0,
                                           clip_cov_ratio=0.02)
    want = set()
    for i, t in toks:
        r = math.exp((new[i, t] - old[i, t]).item())
        a = adv[i, t].item()
        clipped = -a * min(max(r, 0.8), 1.25) > -a * r
        if not clipped and 0.05 < cov[(i, t)] < 2.0:
            want.add((i, t))
    # masked_mean adds 1e-8 to the count: the covariances agree to ~1e-9, the band membership exactly for this data
    assert {(i, t) for i, t in toks if cand[i, t]} == want and clip_num == max(int(0.02 * n), 1)
    dropped = torch.zeros_like(cand)
    for i, t in list(want)[:clip_num]:
        dropped[i, t] = True
    loss, cf, kl, _ = L.policy_loss_clip_cov(old, new, adv, mask, "token-mean", 0.2, 0.25, dropped=dropped)
    total = 0.0
    for i, t in toks:
        if dropped[i, t]:
            continue
        r = math.exp((new[i, t] - old[i, t]).item())
        a = adv[i, t].item()
        total += max(-a * r, -a * min(max(r, 0.8), 1.25))
    assert loss.item() == pytest.approx(total / n, rel=1e-9)
    assert cf.item() == pytest.approx(int(dropped.sum()) / n, rel=1e-6)
    g, = torch.autograd.grad(loss, new)
    assert (g[dropped] == 0).all()
    # the random draw picks clip_num candidates, all inside the band
    torch.manual_seed(0)
    _, cf2, _, drawn = L.policy_loss_clip_cov(old, new.detach(), adv, mask, "token-mean", 0.2, 0.25, clip_cov_lb=0.05,
                                              clip_cov_ub=2.0, clip_cov_ratio=0.02)
    assert int(drawn.sum()) == min(clip_num, len(want)) and (cand[drawn]).all()
