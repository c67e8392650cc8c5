"""Seeded random sweep over shapes, aggregation modes, mask types and options of the [B, L] entry points, each case
against the oracle: the parametrised tests pick their shapes by hand, this one lets a generator pick them (chunk
boundaries, single rows, rows of many chunks, empty rows, every mask type)."""
import random
import types

import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

MODES = ["token-mean", "seq-mean-token-sum", "seq-mean-token-mean", "seq-mean-token-sum-norm"]


def _cfg():
    ns = types.SimpleNamespace(clip_ratio=0.2, clip_ratio_low=0.2, clip_ratio_high=0.28, clip_ratio_c=3.0,
                               global_batch_info={})
    ns.get = lambda k, d=None: getattr(ns, k, d)
    return ns


def _close(got, want, what, rtol=1e-5, atol=1e-6):
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    err = (got - want).abs()
    bad = err > atol + rtol * want.abs()
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off, max err {err.max().item():.3e}"


def _loss_close(got, want64, terms_abs_sum, what):
    """A loss is a sum of terms that largely cancel: compare with the float64 evaluation of the oracle, within
    rtol 1e-5 of the result plus the rounding of an fp32 sum of that many terms."""
    tol = 1e-6 + 1e-5 * abs(want64) + 2e-7 * terms_abs_sum
    assert abs(got - want64) <= tol, f"{what}: got {got!r}, want {want64!r} (tolerance {tol:.3e})"


def _cases(seed, count):
    rng = random.Random(seed)
    for i in range(count):
        B = rng.choice([1, 2, 3, 7, 16, 33, 64, 100, 257, 512, 700])
        Lc = rng.choice([1, 5, 64, 100, 1023, 1024, 4095, 4096, 4097, 4100, 8192, 9000, 12292, 17000])
        if B * Lc > 6_000_000:
            Lc = 4096
        yield (i, B, Lc, rng.choice(["policy", "policy", "value", "kl", "grpo", "gspo", "geo", "agg"]), rng.choice(MODES),
               rng.choice(["float32", "bool", "int64", "int32"]), rng.random() < 0.3, rng.random() < 0.7,
               rng.choice(["kl", "abs", "mse", "low_var_kl"]), rng.choice([1, 2, 4, 8]))


@pytest.mark.parametrize("case", list(_cases(20251, 96)), ids=lambda c: f"{c[0]}-{c[3]}-{c[1]}x{c[2]}")
def test_random_case_against_the_oracle(dev, case):
    from verl_amd.trainer.ppo import core_algos as CA
    i, B, Lc, op, mode, mask_dtype, with_isw, with_grad, kl_kind, group_div = case
    mdt = getattr(torch, mask_dtype)
    g = torch.Generator().manual_seed(977 * i + B + Lc)
    lens = torch.randint(1, Lc + 1, (B,), generator=g)
    mask = (torch.arange(Lc)[None, :] < lens[:, None]).float()
    if B > 2:
        mask[1] = 0
    old = torch.randn(B, Lc, generator=g) * 0.5 - 1
    new = old + torch.randn(B, Lc, generator=g) * 0.2
    adv = torch.randn(B, Lc, generator=g)
    isw = (torch.rand(B, Lc, generator=g) + 0.5) if with_isw else None
    md = mask.to(mdt).to(dev)
    nd = new.to(dev).requires_grad_(with_grad)
    no = new.double().requires_grad_(with_grad)                     # the oracle evaluated in float64
    o64, a64, m64 = old.double(), adv.double(), mask.double()
    i64 = None if isw is None else isw.double()
    iswd = None if isw is None else isw.to(dev)
    n_terms = float((adv.abs() * 2 * mask).sum()) + 1.0
    if op == "policy":
        loss, met = CA.compute_policy_loss_vanilla(old.to(dev), nd, adv.to(dev), md, mode, _cfg(), iswd)
        want = O.policy_loss_vanilla(o64, no, a64, m64, mode, 0.2, 0.28, 3.0, i64)
        assert abs(met["actor/pg_clipfrac"] - want[1].item()) < 2e-6 + 4.0 / max(1.0, float(mask.sum()))
        assert abs(met["actor/ppo_kl"] - want[2].item()) < 1e-5 * max(1.0, abs(want[2].item()))
    elif op == "value":
        loss, cf = CA.compute_value_loss(nd, adv.to(dev), old.to(dev), md, 0.3, mode)
        want = O.value_loss(no, a64, o64, m64, 0.3, mode)
        n_terms = float((((new - adv) ** 2) * mask).sum()) + 1.0
    elif op == "kl":
        loss = CA.compute_kl_loss(nd, old.to(dev), md, kl_kind, mode)
        want = (O.agg_loss(O.kl_penalty(no, o64, kl_kind), m64, mode),)
        n_terms = float(mask.sum()) + 1.0
    elif op in ("gspo", "geo"):
        advs = torch.randn(B, 1, generator=g).expand(B, Lc).contiguous()
        if op == "gspo":
            loss, met = CA.compute_policy_loss_gspo(old.to(dev), nd, advs.to(dev), md, "seq-mean-token-mean", _cfg(), iswd)
            want = O.policy_loss_gspo(o64, no, advs.double(), m64, 0.2, 0.28, i64)
        else:
            loss, met = CA.compute_policy_loss_geo_mean(old.to(dev), nd, advs.to(dev), md, "token-mean", _cfg(), iswd)
            want = O.policy_loss_geo_mean(o64, no, advs.double(), m64, 0.2, 0.28, i64)
        n_terms = 4.0 * B
    elif op == "agg":
        loss = CA.agg_loss(nd, md, mode)
        want = (O.agg_loss(no, m64, mode),)
        n_terms = float((new.abs() * mask).sum()) + 1.0
    else:
        groups = max(1, B // group_div)
        rng = random.Random(i)
        index = np.array([rng.randrange(groups) for _ in range(B)])
        got, _ = CA.compute_grpo_outcome_advantage(adv.to(dev), md, index)
        want_adv, _ = O.grpo_outcome_advantage(a64, m64, index)
        # a group whose scores nearly coincide divides rounding noise by a tiny std: held to 2e-3 of the largest value
        assert (got.cpu().double() - want_adv).abs().max().item() <= 2e-3 * max(1.0, want_adv.abs().max().item())
        return
    scale = {"token-mean": 1.0 / max(1.0, float(mask.sum())), "seq-mean-token-sum": 1.0 / max(1, B),
             "seq-mean-token-mean": 1.0 / max(1, B), "seq-mean-token-sum-norm": 1.0 / Lc}[mode]
    _loss_close(loss.item(), want[0].item(), n_terms * scale, f"{op} loss ({mode})")
    if with_grad:
        got_g, want_g = torch.autograd.grad(loss, nd)[0], torch.autograd.grad(want[0], no)[0]
        # an element whose ratio sits within an ulp of a clip boundary may land on either side of it
        err = (got_g.double().cpu() - want_g).abs()
        bad = err > 1e-9 + 2e-5 * want_g.abs() + 2e-7 * want_g.abs().max()
        assert int(bad.sum()) <= 2, f"{op} gradient: {int(bad.sum())} elements off, max err {err.max().item():.3e}"
