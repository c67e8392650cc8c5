"""Group-wise helpers on MI355X: drop-ins for ``as_torch_index`` and ``group_mean_std`` of the
reference (verl/utils/groupwise.py:91-223).

Label factorisation (arbitrary hashables -> contiguous int64 ids) is host work, as in the
reference; the per-group statistics run in ``libverl_amd.so``.
"""
from __future__ import annotations

from typing import Any, Optional

import numpy as np
import torch

from .. import _cabi

__all__ = ["as_torch_index", "group_mean_std"]


def _labels_to_numpy(x: Any) -> np.ndarray:
    try:
        arr = np.asarray(x)
    except Exception:
        try:
            arr = np.array(list(x), dtype=object)
        except Exception:
            arr = np.array([x], dtype=object)
    return arr.reshape(-1)


def _factorise(arr: np.ndarray) -> np.ndarray:
    try:
        _, inv = np.unique(arr, return_inverse=True)
    except Exception:  # unorderable mixed types: compare their string forms
        _, inv = np.unique(np.array([str(v) for v in arr], dtype=object), return_inverse=True)
    return inv.astype(np.int64, copy=False)


def as_torch_index(index: Any, device: torch.device | str | None = None) -> torch.Tensor:
    """Group labels -> 1-D ``torch.long`` ids, following the reference's rules
    (verl/utils/groupwise.py:91-160): integer tensors / arrays pass through unchanged, floats
    within 1e-6 of integers are rounded, numeric strings are coerced, anything else (UUID strings,
    mixed types) is factorised with ``np.unique(return_inverse=True)``.  The result stays on the
    CPU unless ``device`` is given."""
    target = torch.device(device) if device is not None else torch.device("cpu")
    if isinstance(index, torch.Tensor):
        flat = index.reshape(-1)
        if flat.dtype in (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8, torch.bool):
            return flat.to(device=target, dtype=torch.long)
        if flat.dtype.is_floating_point:
            f64 = flat.to(torch.float64)
            rounded = torch.round(f64)
            if torch.allclose(f64, rounded, rtol=0.0, atol=1e-6):
                return rounded.to(device=target, dtype=torch.long)
        arr = np.array([str(v.item()) for v in flat], dtype=object)
    else:
        arr = _labels_to_numpy(index)
        if arr.dtype != object and np.issubdtype(arr.dtype, np.integer):
            return torch.from_numpy(arr.astype(np.int64, copy=False)).to(target)
        if arr.dtype != object and np.issubdtype(arr.dtype, np.floating):
            a64 = arr.astype(np.float64, copy=False)
            rounded = np.rint(a64)
            if np.allclose(a64, rounded, rtol=0.0, atol=1e-6):
                return torch.from_numpy(rounded.astype(np.int64)).to(target)
        try:
            return torch.from_numpy(arr.astype(np.int64)).to(target)
        except Exception:
            pass
        if arr.dtype != object:
            arr = arr.astype(object)
    return torch.from_numpy(_factorise(arr)).to(target)


def contiguous_group_ids(index: Any) -> tuple[torch.Tensor, int]:
    """Ids remapped to 0..G-1 (CPU int64) and G.  Membership is what matters downstream, so
    integer labels that ``as_torch_index`` passes through are factorised here as well."""
    ids = as_torch_index(index).cpu().numpy()
    uniq, inv = np.unique(ids, return_inverse=True)
    return torch.from_numpy(inv.astype(np.int64, copy=False).reshape(-1)), int(len(uniq))


@torch.no_grad()
def group_mean_std(scores: torch.Tensor, gidx: torch.Tensor, eps: float = 1e-6,
                   device: Optional[torch.device | str] = None):
    """Per-group ``(mean, std, count)`` as fp32 ``[G]`` tensors, G = max id + 1.

    ``std = sqrt(clamp(unbiased var, min=eps))``; groups with at most one member get mean 0 and
    std 1 (reference verl/utils/groupwise.py:163-223).  Results are returned on ``device`` if
    given, else on the device of ``scores``.
    """
    scores = scores.reshape(-1)
    gidx = gidx.reshape(-1)
    if scores.numel() != gidx.numel():
        raise ValueError(f"scores and gidx length mismatch: {scores.numel()} vs {gidx.numel()}")
    out_dev = torch.device(device) if device is not None else scores.device
    if gidx.numel() == 0:
        e = torch.empty(0, dtype=torch.float32, device=out_dev)
        return e, e, e
    G = int(gidx.max().item()) + 1
    if int(gidx.min().item()) < 0:
        raise ValueError("group ids must be non-negative")
    dev = _cabi.compute_device(scores, gidx)
    s = _cabi.as_f32(scores, dev)
    g = gidx.to(device=dev, dtype=torch.long).contiguous()
    mean = torch.empty(G, dtype=torch.float32, device=dev)
    std = torch.empty(G, dtype=torch.float32, device=dev)
    cnt = torch.empty(G, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        _cabi.check(_cabi.lib().vamd_group_mean_std(s.data_ptr(), g.data_ptr(), s.numel(), G, float(eps),
                                                    mean.data_ptr(), std.data_ptr(), cnt.data_ptr(),
                                                    _cabi.stream_ptr(dev)))
    return mean.to(out_dev), std.to(out_dev), cnt.to(out_dev)
