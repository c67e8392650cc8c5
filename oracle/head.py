"""Oracle for the fused vocab-projection log-prob / entropy head (CPU torch).

Test infrastructure only; see ``oracle/__init__.py``.

Two restatements are kept, because the reference holds two:

* ``head_fp32_ground_truth`` follows the stock-torch ground truth the
  reference's own test compares every implementation against
  (tests/utils/test_linear_cross_entropy.py:48-61): inputs upcast to fp32,
  ``matmul``, ``/T``, ``softmax``, ``logsumexp``, ``cross_entropy`` negated.
  Gradients come from ``torch.autograd.grad`` exactly as that test takes them
  (:229-231).  This is what the HIP head is held to (max-abs 2e-3).
* ``fused_linear_for_ppo_*`` follow the reference's chunked PyTorch backend
  (verl/utils/experimental/torch_functional.py:20-72 for the per-chunk math,
  :75-176 for the 512-token chunk loop), which is also the CPU baseline that
  ``bench.py`` times.
"""

from __future__ import annotations

from typing import Optional

import torch


def head_fp32_ground_truth(hidden, weight, labels, temperature: float = 1.0):
    """fp32 log-prob and entropy of ``labels`` under ``softmax(hidden @ weight.T / T)``.

    Follows tests/utils/test_linear_cross_entropy.py:48-61.  ``hidden`` is
    ``[N, H]``, ``weight`` ``[V, H]``, ``labels`` ``[N]`` int64.  Returns fp32
    ``(logprobs[N], entropy[N])`` that stay attached to the autograd graph of
    ``hidden`` / ``weight``.
    """
    h32 = hidden.to(torch.float32)
    w32 = weight.to(torch.float32)
    z = torch.matmul(h32, w32.transpose(0, 1))
    z = z / temperature
    p = torch.nn.functional.softmax(z, dim=-1)
    lse = torch.logsumexp(z, dim=-1)
    mean_z = torch.sum(p * z, dim=-1)
    entropy = lse - mean_z
    nll = torch.nn.functional.cross_entropy(z, labels, reduction="none")
    return torch.neg(nll), entropy


def fused_linear_for_ppo_fwd(hidden, weight, labels, temperature: float = 1.0):
    """One chunk of the reference's torch backend, forward.

    Follows verl/utils/experimental/torch_functional.py:20-37: the GEMM and the
    division by T run in the input dtype, softmax runs in fp32, and the two
    outputs are cast back to the input dtype.
    """
    z = (hidden @ weight.t()) / temperature
    out_dtype = z.dtype
    z = z.to(torch.float32)
    p = z.softmax(dim=-1)
    logp = z.log_softmax(dim=-1)
    tok = logp.gather(-1, labels.unsqueeze(-1)).squeeze(-1)
    ent = torch.logsumexp(z, dim=-1) - torch.sum(p * z, dim=-1)
    return tok.to(out_dtype), ent.to(out_dtype)


def fused_linear_for_ppo_bwd(
    dlogprobs: Optional[torch.Tensor],
    dentropy: Optional[torch.Tensor],
    hidden,
    weight,
    labels,
    temperature: float = 1.0,
):
    """One chunk of the reference's torch backend, backward.

    Follows verl/utils/experimental/torch_functional.py:40-72: recompute the
    logits, build ``dlogits`` from the two upstream grads (either may be
    ``None``), cast to the input dtype, divide by T, two GEMMs.
    """
    z = (hidden @ weight.t()) / temperature
    out_dtype = z.dtype
    z = z.to(torch.float32)
    p = z.softmax(dim=-1)
    dz = 0
    if dlogprobs is not None:
        onehot = torch.zeros_like(z).scatter_(-1, labels.unsqueeze(-1), 1)
        dz = dz + dlogprobs.to(torch.float32).unsqueeze(-1) * (onehot - p)
    if dentropy is not None:
        logp = z.log_softmax(dim=-1)
        ent = torch.logsumexp(z, dim=-1) - torch.sum(p * z, dim=-1)
        dz = dz + p * (logp + ent.unsqueeze(-1)) * (-dentropy.unsqueeze(-1))
    dz = dz.to(out_dtype) / temperature
    return dz @ weight, dz.t() @ hidden


def fused_linear_for_ppo_chunked(hidden, weight, labels, temperature=1.0, chunk_size=512,
                                 dlogprobs=None, dentropy=None):
    """The reference's chunk loop (verl/utils/experimental/torch_functional.py:75-176).

    Forward only when both upstream grads are ``None``; otherwise also returns
    ``(d_hidden, d_weight)`` accumulated over chunks in the input dtype, as the
    reference does (``dhidden[chunk] += h``, ``dweight += v``).
    """
    n = hidden.shape[0]
    logprobs = hidden.new_zeros(n)
    entropy = hidden.new_zeros(n)
    want_grad = dlogprobs is not None or dentropy is not None
    d_hidden = torch.zeros_like(hidden) if want_grad else None
    d_weight = torch.zeros_like(weight) if want_grad else None
    for lo in range(0, n, chunk_size):
        hi = min(lo + chunk_size, n)
        lp, en = fused_linear_for_ppo_fwd(hidden[lo:hi], weight, labels[lo:hi], temperature)
        logprobs[lo:hi] = lp
        entropy[lo:hi] = en
        if want_grad:
            dh, dw = fused_linear_for_ppo_bwd(
                None if dlogprobs is None else dlogprobs[lo:hi],
                None if dentropy is None else dentropy[lo:hi],
                hidden[lo:hi], weight, labels[lo:hi], temperature)
            d_hidden[lo:hi] += dh
            d_weight += dw
    if want_grad:
        return logprobs, entropy, d_hidden, d_weight
    return logprobs, entropy


def head_grads_closed_form(hidden, weight, labels, temperature, dlogprobs, dentropy,
                           dtype=torch.float64):
    """Closed-form gradients of the head, evaluated in ``dtype`` (fp64 by default).

    d/dz_j = g_lp (1[j=y] - p_j) - g_H p_j (z_j - sum_k p_k z_k), then /T; the
    entropy term is the derivation written out in
    tests/utils/test_special_linear_cross_entropy_tp.py:142-161.  Used to
    cross-check ``torch.autograd.grad`` of ``head_fp32_ground_truth``.
    """
    h = hidden.to(dtype)
    w = weight.to(dtype)
    z = (h @ w.t()) / temperature
    p = z.softmax(dim=-1)
    mean_z = (p * z).sum(-1, keepdim=True)
    onehot = torch.zeros_like(z).scatter_(-1, labels.unsqueeze(-1), 1)
    g_lp = dlogprobs.to(dtype).unsqueeze(-1)
    g_h = dentropy.to(dtype).unsqueeze(-1)
    dz = (g_lp * (onehot - p) - g_h * p * (z - mean_z)) / temperature
    return dz @ w, dz.t() @ h


@torch.no_grad()
def head_fwd_bwd_chunked_fp32(hidden, weight, labels, temperature, dlogprobs, dentropy, chunk=1024):
    """fp32 forward outputs, closed-form gradients (the same formula as
    ``head_grads_closed_form``, which is pinned against autograd) and, for each gradient, the
    L1 magnitude of the products that form it:

        E_dh = |dz| @ |W| ,   E_dw = |dz|^T @ |hidden| .

    Both reference implementations round ``d_logits`` to the input dtype before the two GEMMs
    (verl/utils/experimental/torch_functional.py:65, verl/utils/kernel/kernels.py:1664), so a
    bf16 implementation can differ from the fp32 ground truth by up to 2**-8 * E (half an ulp,
    8 significant bits, per product); tests use E to state that bound.  Works on any device; tokens are processed
    in chunks so that ``[chunk, vocab]`` is the largest temporary.
    """
    w32 = weight.to(torch.float32)
    aw = w32.abs()
    dw = torch.zeros_like(w32)
    e_dw = torch.zeros_like(w32)
    lps, ents, dhs, e_dhs = [], [], [], []
    for lo in range(0, hidden.shape[0], chunk):
        hi = min(lo + chunk, hidden.shape[0])
        h32 = hidden[lo:hi].to(torch.float32)
        lab = labels[lo:hi]
        z = (h32 @ w32.t()) / temperature
        lse = torch.logsumexp(z, dim=-1, keepdim=True)
        p = torch.exp(z - lse)
        mean_z = (p * z).sum(-1, keepdim=True)
        lps.append(z.gather(-1, lab.unsqueeze(-1)).squeeze(-1) - lse.squeeze(-1))
        ents.append((lse - mean_z).squeeze(-1))
        g_lp = dlogprobs[lo:hi].to(torch.float32).unsqueeze(-1)
        g_en = dentropy[lo:hi].to(torch.float32).unsqueeze(-1)
        dz = -(g_lp * p) - g_en * p * (z - mean_z)
        dz.scatter_add_(-1, lab.unsqueeze(-1), g_lp)
        dz /= temperature
        dhs.append(dz @ w32)
        dw += dz.t() @ h32
        dz.abs_()
        e_dhs.append(dz @ aw)
        e_dw += dz.t() @ h32.abs()
    return torch.cat(lps), torch.cat(ents), torch.cat(dhs), dw, torch.cat(e_dhs), e_dw
