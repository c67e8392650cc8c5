"""Oracle for the unfused per-token definitions and the masked reductions (CPU torch).

Test infrastructure only; see ``oracle/__init__.py``.  Each function keeps the
operation ORDER of the reference line by line, because the epsilons and the
``where``-then-multiply in ``masked_sum`` decide the results on edge inputs
(NaN outside the mask, empty masks, weighted float masks).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def clip_by_value(x, lo, hi):
    """max(min(x, hi), lo) with tensor bounds (verl/utils/torch_functional.py:203-221)."""
    return torch.max(torch.min(x, hi), lo)


def entropy_from_logits(logits):
    """lse(z) - sum softmax(z) z (verl/utils/torch_functional.py:224-238)."""
    p = F.softmax(logits, dim=-1)
    return torch.logsumexp(logits, dim=-1) - torch.sum(p * logits, dim=-1)


def logprobs_from_logits(logits, labels):
    """log_softmax + gather (verl/utils/torch_functional.py:148-163, the
    ``logprobs_from_logits_naive`` definition that ``_v2`` :166-200 is
    algebraically equal to)."""
    logp = F.log_softmax(logits, dim=-1)
    return torch.gather(logp, -1, labels.unsqueeze(-1)).squeeze(-1)


def masked_sum(values, mask, axis=None):
    """verl/utils/torch_functional.py:266-284: zero what the mask excludes, THEN weight by the mask."""
    kept = torch.where(mask.bool(), values, 0.0)
    return (kept * mask).sum(axis=axis)


def masked_mean(values, mask, axis=None):
    """verl/utils/torch_functional.py:287-301: masked_sum / (mask.sum + 1e-8)."""
    return masked_sum(values, mask, axis) / (mask.sum(axis=axis) + 1e-8)


def masked_var(values, mask, unbiased=True):
    """verl/utils/torch_functional.py:304-319: two-pass variance, Bessel factor M/(M-1)."""
    mean = masked_mean(values, mask)
    var = masked_mean((values - mean) ** 2, mask)
    if unbiased:
        m = mask.sum()
        if m == 0:
            raise ValueError("At least one element in the mask has to be 1.")
        if m == 1:
            raise ValueError("The sum of the mask is one, which can cause a division by zero.")
        var = var * (m / (m - 1))
    return var


def masked_whiten(values, mask, shift_mean=True):
    """verl/utils/torch_functional.py:322-339: (v - mean) * rsqrt(var + 1e-8) on EVERY element."""
    mean, var = masked_mean(values, mask), masked_var(values, mask)
    out = (values - mean) * torch.rsqrt(var + 1e-8)
    if not shift_mean:
        out = out + mean
    return out


def sum_pi_squared_from_logits(logits):
    """``sum_j softmax(logits)_j ** 2`` as ``exp(logsumexp(2 z) - 2 logsumexp(z))``,
    verl/utils/torch_functional.py:680-694."""
    return torch.exp(torch.logsumexp(2.0 * logits, dim=-1) - 2.0 * torch.logsumexp(logits, dim=-1))
