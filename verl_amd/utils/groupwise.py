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


_INT_TENSORS = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8, torch.bool)


def _flat_labels(index: Any) -> tuple[np.ndarray, bool]:
    """1-D numpy view of the labels and whether they came from a torch tensor (the reference treats non-integral
    float TENSORS as opaque labels but hands non-integral float ARRAYS to numpy's integer cast)."""
    if isinstance(index, torch.Tensor):
        t = index.detach().reshape(-1).cpu()
        if t.dtype.is_floating_point:
            t = t.to(torch.float64)
        return t.numpy(), True
    try:
        arr = np.asarray(index)
    except Exception:
        try:
            arr = np.array(list(index), dtype=object)
        except Exception:
            arr = np.array([index], dtype=object)
    return arr.reshape(-1), False


def _ids_if_numeric(arr: np.ndarray, from_torch: bool) -> Optional[np.ndarray]:
    """int64 ids when the labels ARE numbers: integers and booleans as they are, floats within 1e-6 of an integer
    rounded, and -- for non-tensor input -- anything numpy can cast to int64 (numeric strings such as "0042")."""
    if arr.dtype != object and (np.issubdtype(arr.dtype, np.integer) or arr.dtype == np.bool_):
        return arr.astype(np.int64, copy=False)
    if arr.dtype != object and np.issubdtype(arr.dtype, np.floating):
        nearest = np.rint(arr.astype(np.float64, copy=False))
        if np.allclose(arr, nearest, rtol=0.0, atol=1e-6):
            return nearest.astype(np.int64)
    if from_torch:
        return None
    try:
        return arr.astype(np.int64)
    except Exception:
        return None


def _ids_by_sorted_rank(arr: np.ndarray, from_torch: bool) -> np.ndarray:
    """Rank of each label among the sorted distinct labels (``np.unique``), on their string forms when the labels
    cannot be ordered against each other or came from a float tensor."""
    labels = np.array([str(v) for v in arr.tolist()], dtype=object) if from_torch else arr.astype(object, copy=False)
    try:
        inverse = np.unique(labels, return_inverse=True)[1]
    except Exception:
        inverse = np.unique(np.array([str(v) for v in labels], dtype=object), return_inverse=True)[1]
    return np.asarray(inverse, dtype=np.int64).reshape(-1)


def as_torch_index(index: Any, device: torch.device | str | None = None) -> torch.Tensor:
    """Group labels -> 1-D ``torch.long`` ids with the results of the reference's ``as_torch_index``
    (verl/utils/groupwise.py:91-160): numeric labels keep their value, every other kind of label (UUID strings,
    mixed types) gets its rank among the distinct labels.  The result stays on the CPU unless ``device`` is given."""
    arr, from_torch = _flat_labels(index)
    ids = _ids_if_numeric(arr, from_torch)
    if ids is None:
        ids = _ids_by_sorted_rank(arr, from_torch)
    out = torch.from_numpy(np.ascontiguousarray(ids))
    return out if device is None else out.to(torch.device(device))


def contiguous_group_ids(index: Any, vectorized: bool = False) -> tuple[torch.Tensor, int]:
    """Labels -> ids ``0..G-1`` (CPU int64) and ``G``.  Group membership is decided
    by Python equality of the labels, as in the reference's ``id2score[index[i]]`` dictionaries
    (verl/trainer/ppo/core_algos.py:305-312); nothing downstream depends on which id a group gets.
    ``vectorized``: membership as the reference's vectorised estimators see it, i.e. equality of the
    ``as_torch_index`` values (there the labels "0042" and 42 are one group)."""
    if vectorized:
        index = as_torch_index(index)
    if isinstance(index, torch.Tensor):
        index = index.detach().reshape(-1).cpu().numpy()
    if isinstance(index, np.ndarray) and index.dtype.kind in "iub":
        # plain integers: equality is integer equality, and numpy factorises them without a Python loop (the ids then
        # follow the sorted labels instead of their first appearance, which no caller can tell apart)
        uniq, inverse = np.unique(index.reshape(-1), return_inverse=True)
        return torch.from_numpy(np.ascontiguousarray(inverse.reshape(-1), dtype=np.int64)), int(uniq.size)
    labels = index.reshape(-1).tolist() if isinstance(index, np.ndarray) else list(index)
    table: dict = {}
    ids = [table.setdefault(k, len(table)) for k in labels]
    return torch.tensor(ids, dtype=torch.int64), len(table)


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
    with _cabi.device_guard(dev):
        _cabi.check(_cabi.lib().vamd_group_mean_std(s.data_ptr(), g.data_ptr(), s.numel(), G, float(eps),
                                                    mean.data_ptr(), std.data_ptr(), cnt.data_ptr(),
                                                    _cabi.stream_ptr(dev)))
    return mean.to(out_dev), std.to(out_dev), cnt.to(out_dev)
