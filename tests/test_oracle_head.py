"""Pins for oracle/head.py: closed forms, fp64 cross-checks, autograd vs the
hand-derived gradient, and the reference's own torch<->fused-torch bar
(tests/utils/test_linear_cross_entropy.py:210-216,260-268 in the reference)."""
import math

import pytest
import torch

from oracle import head as H


def _inputs(n, h, v, seed, dtype=torch.float32, scale=0.5):
    g = torch.Generator().manual_seed(seed)
    hidden = (torch.rand(n, h, generator=g) - 0.5) * 2 * scale
    weight = (torch.rand(v, h, generator=g) - 0.5) * 2 * scale
    labels = torch.randint(0, v, (n,), generator=g)
    return hidden.to(dtype), weight.to(dtype), labels


def test_uniform_logits_closed_form():
    # weight == 0  =>  every logit is 0: logprob = -log V, entropy = log V exactly.
    n, h, v = 5, 16, 37
    hidden, _, labels = _inputs(n, h, v, 0)
    lp, ent = H.head_fp32_ground_truth(hidden, torch.zeros(v, h), labels, 1.3)
    assert torch.allclose(lp, torch.full((n,), -math.log(v)), atol=1e-6)
    assert torch.allclose(ent, torch.full((n,), math.log(v)), atol=1e-6)


def test_two_class_closed_form():
    # V = 2, H = 1: z = (h*w0, h*w1)/T, a logistic in d = z1 - z0.
    hidden = torch.tensor([[2.0], [-1.0], [0.25]])
    weight = torch.tensor([[0.5], [-1.5]])
    labels = torch.tensor([0, 1, 1])
    T = 0.7
    lp, ent = H.head_fp32_ground_truth(hidden, weight, labels, T)
    for i in range(3):
        z0 = hidden[i, 0].item() * 0.5 / T
        z1 = hidden[i, 0].item() * -1.5 / T
        lse = math.log(math.exp(z0) + math.exp(z1))
        p0, p1 = math.exp(z0 - lse), math.exp(z1 - lse)
        want_lp = (z0, z1)[labels[i]] - lse
        want_ent = -(p0 * math.log(p0) + p1 * math.log(p1))
        assert abs(lp[i].item() - want_lp) < 1e-6
        assert abs(ent[i].item() - want_ent) < 1e-6


@pytest.mark.parametrize("n,h,v", [(1, 128, 128), (127, 128, 384), (129, 256, 1152)])
def test_fp32_vs_fp64_and_invariants(n, h, v):
    hidden, weight, labels = _inputs(n, h, v, n)
    lp, ent = H.head_fp32_ground_truth(hidden, weight, labels, 1.5)
    z = (hidden.double() @ weight.double().t()) / 1.5
    lse = torch.logsumexp(z, -1)
    lp64 = z.gather(-1, labels[:, None]).squeeze(-1) - lse
    p = torch.softmax(z, -1)
    ent64 = -(p * torch.log(p)).sum(-1)          # Shannon form, not the lse form
    assert torch.allclose(lp.double(), lp64, atol=1e-5)
    assert torch.allclose(ent.double(), ent64, atol=1e-5)
    assert (lp <= 0).all() and (ent >= 0).all() and (ent <= math.log(v) + 1e-5).all()


def test_temperature_is_a_rescale_of_hidden():
    hidden, weight, labels = _inputs(33, 64, 200, 3)
    a = H.head_fp32_ground_truth(hidden, weight, labels, 0.7)
    b = H.head_fp32_ground_truth(hidden / 0.7, weight, labels, 1.0)
    assert torch.allclose(a[0], b[0], atol=1e-5) and torch.allclose(a[1], b[1], atol=1e-5)


def test_label_permutation_equivariance():
    hidden, weight, labels = _inputs(17, 32, 50, 4)
    perm = torch.randperm(50, generator=torch.Generator().manual_seed(1))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(50)
    a = H.head_fp32_ground_truth(hidden, weight, labels, 1.0)
    b = H.head_fp32_ground_truth(hidden, weight[perm], inv[labels], 1.0)
    assert torch.allclose(a[0], b[0], atol=1e-6) and torch.allclose(a[1], b[1], atol=1e-6)


@pytest.mark.parametrize("T", [1.0, 1.5, 0.7])
def test_autograd_matches_hand_derived_gradient(T):
    hidden, weight, labels = _inputs(19, 48, 96, 5, dtype=torch.float64)
    hidden.requires_grad_()
    weight.requires_grad_()
    g = torch.Generator().manual_seed(9)
    g_lp = torch.randn(19, generator=g, dtype=torch.float64)
    g_ent = torch.randn(19, generator=g, dtype=torch.float64)
    h32 = hidden  # ground truth upcasts to fp32; keep fp64 here by calling the pieces
    z = (h32 @ weight.t()) / T
    lp = torch.log_softmax(z, -1).gather(-1, labels[:, None]).squeeze(-1)
    p = torch.softmax(z, -1)
    ent = torch.logsumexp(z, -1) - (p * z).sum(-1)
    dh, dw = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
    dh2, dw2 = H.head_grads_closed_form(hidden.detach(), weight.detach(), labels, T, g_lp, g_ent)
    assert torch.allclose(dh, dh2, atol=1e-10) and torch.allclose(dw, dw2, atol=1e-10)


def test_fused_torch_backend_matches_ground_truth_fwd_and_bwd():
    # the reference's torch<->fused-torch bar: 1e-4 fwd, atol 1e-2 / rtol 1e-4 bwd, fp32 inputs
    n, h, v = 700, 128, 1024
    hidden, weight, labels = _inputs(n, h, v, 6)
    hidden.requires_grad_()
    weight.requires_grad_()
    g = torch.Generator().manual_seed(2)
    g_ent = (torch.rand(n, generator=g) - 0.5)
    g_lp = (torch.rand(n, generator=g) - 0.5) * 2
    lp, ent = H.head_fp32_ground_truth(hidden, weight, labels, 1.5)
    dh, dw = torch.autograd.grad((ent, lp), (hidden, weight), (g_ent, g_lp))
    lp2, ent2, dh2, dw2 = H.fused_linear_for_ppo_chunked(
        hidden.detach(), weight.detach(), labels, 1.5, chunk_size=512, dlogprobs=g_lp, dentropy=g_ent)
    assert torch.allclose(lp, lp2, atol=1e-4, rtol=1e-4)
    assert torch.allclose(ent, ent2, atol=1e-4, rtol=1e-4)
    assert torch.allclose(dh, dh2, atol=1e-4, rtol=1e-4)
    assert torch.allclose(dw, dw2, atol=1e-4, rtol=1e-4)
    # None upstream grads are allowed, one at a time
    _, _, dh3, _ = H.fused_linear_for_ppo_chunked(hidden.detach(), weight.detach(), labels, 1.5,
                                                  dlogprobs=g_lp, dentropy=None)
    dh4, = torch.autograd.grad(H.head_fp32_ground_truth(hidden, weight, labels, 1.5)[0], hidden, g_lp)
    assert torch.allclose(dh3, dh4, atol=1e-4, rtol=1e-4)


def test_gradient_rows_sum_to_zero_over_vocab():
    # sum_j dz_j = 0  =>  d_weight summed over the vocab axis is 0 for every hidden column
    hidden, weight, labels = _inputs(11, 16, 40, 7)
    _, dw = H.head_grads_closed_form(hidden, weight, labels, 1.2, torch.randn(11), torch.randn(11))
    assert dw.sum(0).abs().max() < 1e-9


def test_chunked_fp32_closed_form_matches_autograd_and_bounds_bf16_dlogits():
    n, h, v = 300, 64, 520
    hidden, weight, labels = _inputs(n, h, v, 8)
    g = torch.Generator().manual_seed(3)
    g_lp, g_ent = torch.randn(n, generator=g), torch.randn(n, generator=g) * 0.1
    hr, wr = hidden.clone().requires_grad_(), weight.clone().requires_grad_()
    lp, ent = H.head_fp32_ground_truth(hr, wr, labels, 0.9)
    dh, dw = torch.autograd.grad((lp, ent), (hr, wr), (g_lp, g_ent))
    lp2, ent2, dh2, dw2, e_dh, e_dw = H.head_fwd_bwd_chunked_fp32(hidden, weight, labels, 0.9, g_lp, g_ent, chunk=128)
    assert torch.allclose(lp, lp2, atol=1e-5) and torch.allclose(ent, ent2, atol=1e-5)
    assert torch.allclose(dh, dh2, atol=1e-5) and torch.allclose(dw, dw2, atol=1e-5)
    # the L1 scales really bound what rounding d_logits to bf16 does to the two GEMMs
    dh3, dw3 = H.fused_linear_for_ppo_bwd(g_lp, g_ent, hidden, weight, labels, 0.9)          # fp32, no rounding
    z = (hidden @ weight.t()) / 0.9
    p = z.softmax(-1)
    dz = (g_lp[:, None] * (torch.zeros_like(z).scatter_(-1, labels[:, None], 1) - p)
          - g_ent[:, None] * p * (z - (p * z).sum(-1, keepdim=True))) / 0.9
    dzr = dz.bfloat16().float()
    assert ((dzr @ weight - dh).abs() <= 2.0 ** -8 * e_dh + 1e-6).all()
    assert ((dzr.t() @ hidden - dw).abs() <= 2.0 ** -8 * e_dw + 1e-6).all()
    assert torch.allclose(dh3, dh, atol=1e-5)
