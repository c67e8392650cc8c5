"""Masked reductions on MI355X: drop-ins for ``masked_sum`` / ``masked_mean`` / ``masked_var`` /
``masked_whiten`` of the reference (verl/utils/torch_functional.py:266-339).

Inputs may live on the CPU (they are staged to the current GPU and the result is returned on
the CPU) or on a GPU.  Values are computed in fp32 with fp64 accumulation of the partial sums.
"""
from __future__ import annotations

import torch

from .. import _cabi


def _as_matrix(values: torch.Tensor, mask: torch.Tensor, dev: torch.device):
    assert values.shape == mask.shape, f"values {tuple(values.shape)} and mask {tuple(mask.shape)} differ"
    v = _cabi.as_f32(values, dev)
    m, code = _cabi.mask_code(mask.detach().to(dev))
    cols = v.shape[-1] if v.dim() >= 1 and v.numel() > 0 else 1
    rows = v.numel() // max(cols, 1)
    return v.view(rows, cols), m.view(rows, cols), code


def _moments(values: torch.Tensor, mask: torch.Tensor, per_row: bool) -> torch.Tensor:
    """Device fp64 tensor of (sum m, sum where(m,v,0) m, sum where(m,v,0)^2 m, count) —
    ``[4]`` or ``[rows, 4]``.  ``values`` / ``mask`` are 2-D device tensors."""
    dev = values.device
    rows, cols = values.shape
    L = _cabi.lib()
    out = torch.empty((rows, 4) if per_row else (4,), dtype=torch.float64, device=dev)
    mk, code = _cabi.mask_code(mask)
    ws = _cabi.ticket_workspace(L.vamd_masked_moments_workspace_bytes(rows, cols), dev)
    with torch.cuda.device(dev):
        _cabi.check(L.vamd_masked_moments(values.data_ptr(), mk.data_ptr(), code, rows, cols, int(per_row),
                                          out.data_ptr(), ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
    return out.t() if per_row else out


def _reduce(values, mask, axis, mean: bool):
    if values.requires_grad:
        raise NotImplementedError("verl_amd masked reductions are forward-only; detach the input or use agg_loss")
    if values.numel() == 0:
        raise ValueError("masked reduction of an empty tensor")
    ndim = values.dim()
    if axis is not None and not (axis in (-1, ndim - 1) or (ndim == 1 and axis == 0)):
        raise NotImplementedError("verl_amd masked reductions support axis=None and the last axis")
    dev = _cabi.compute_device(values, mask)
    v, m, _ = _as_matrix(values, mask, dev)
    mom = _moments(v, m, per_row=axis is not None and ndim > 1)
    s = mom[1].to(torch.float32)
    if mean:
        s = s / (mom[0].to(torch.float32) + 1e-8)
    if axis is not None and ndim > 1:
        s = s.view(values.shape[:-1])
    return s.to(values.device)


def masked_sum(values: torch.Tensor, mask: torch.Tensor, axis=None) -> torch.Tensor:
    """sum(where(mask.bool(), values, 0) * mask) (reference torch_functional.py:266-284)."""
    return _reduce(values, mask, axis, mean=False)


def masked_mean(values: torch.Tensor, mask: torch.Tensor, axis=None) -> torch.Tensor:
    """masked_sum / (mask.sum + 1e-8) (reference torch_functional.py:287-301)."""
    return _reduce(values, mask, axis, mean=True)


def _global_moments(values, mask):
    dev = _cabi.compute_device(values, mask)
    v, m, _ = _as_matrix(values, mask, dev)
    return v, _moments(v, m, per_row=False), dev


def _raise_on_tiny_mask(mask_sum: float) -> None:
    # reference torch_functional.py:309-316
    if mask_sum == 0:
        raise ValueError("At least one element in the mask has to be 1.")
    if mask_sum == 1:
        raise ValueError("The sum of the mask is one, which can cause a division by zero.")


def masked_var(values: torch.Tensor, mask: torch.Tensor, unbiased: bool = True) -> torch.Tensor:
    """Two-pass masked variance with Bessel's factor (reference torch_functional.py:304-319)."""
    _, mom, _ = _global_moments(values, mask)
    s0, s1, s2, _ = (x for x in mom.to("cpu").tolist())
    mean = torch.tensor(s1, dtype=torch.float32) / (torch.tensor(s0, dtype=torch.float32) + 1e-8)
    md = float(mean)
    var = torch.tensor(s2 - 2.0 * md * s1 + md * md * s0, dtype=torch.float32) / (
        torch.tensor(s0, dtype=torch.float32) + 1e-8)
    if unbiased:
        _raise_on_tiny_mask(s0)
        var = var * torch.tensor(s0 / (s0 - 1.0), dtype=torch.float32)
    return var.to(values.device)


def masked_whiten(values: torch.Tensor, mask: torch.Tensor, shift_mean: bool = True) -> torch.Tensor:
    """(values - mean) * rsqrt(var + 1e-8) on every element (reference torch_functional.py:322-339)."""
    v, mom, dev = _global_moments(values, mask)
    _raise_on_tiny_mask(float(mom[0].item()))
    L = _cabi.lib()
    stats = torch.empty(4, dtype=torch.float32, device=dev)
    out = torch.empty_like(v)
    with torch.cuda.device(dev):
        s = _cabi.stream_ptr(dev)
        _cabi.check(L.vamd_whiten_stats(mom.data_ptr(), int(shift_mean), stats.data_ptr(), s))
        _cabi.check(L.vamd_affine_by_stats(v.data_ptr(), stats.data_ptr(), v.numel(), out.data_ptr(), s))
    return out.view(values.shape).to(values.device)
