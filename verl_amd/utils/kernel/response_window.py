"""Remove-padding outputs of the head -> the ``(batch, response_length)`` window the PPO math works on.

The reference rebuilds a padded ``(batch, seqlen)`` tensor per output with ``pad_input`` and slices the
columns ``[-response_length - 1, -1)`` (verl/workers/actor/dp_actor.py:316-344).  ``pad_to_response_window``
writes the window directly, for up to three per-token tensors in one launch, and is differentiable with
respect to the first two.
"""
from __future__ import annotations

import torch

from ... import _cabi


class _ResponseWindow(torch.autograd.Function):
    @staticmethod
    def forward(ctx, indices, batch, seqlen, response_length, a, b, c):
        dev = _cabi.compute_device(a, indices)
        idx = indices.detach().to(device=dev, dtype=torch.long).contiguous().view(-1)
        vals = [None if t is None else _cabi.as_f32(t, dev).view(-1) for t in (a, b, c)]
        nnz = idx.numel()
        for t in vals:
            assert t is None or t.numel() == nnz, f"{t.numel()} values for {nnz} token positions"
        outs = [None if t is None else torch.empty((batch, response_length), dtype=torch.float32, device=dev)
                for t in vals]
        with _cabi.device_guard(dev):
            _cabi.check(_cabi.lib().vamd_response_window_scatter(
                _cabi.ptr(vals[0]), _cabi.ptr(vals[1]), _cabi.ptr(vals[2]), idx.data_ptr(), nnz, batch, seqlen,
                response_length, _cabi.ptr(outs[0]), _cabi.ptr(outs[1]), _cabi.ptr(outs[2]), _cabi.stream_ptr(dev)))
        ctx.save_for_backward(idx)
        ctx.geometry = (batch, seqlen, response_length)
        ctx.like = [None if t is None else (t.shape, t.dtype, t.device) for t in (a, b, c)]
        return tuple(None if o is None else o.to(a.device) for o in outs)

    @staticmethod
    def backward(ctx, da, db, dc):
        (idx,) = ctx.saved_tensors
        batch, seqlen, width = ctx.geometry
        dev = idx.device
        nnz = idx.numel()
        grads = [da, db, dc]
        res = [None, None, None]
        todo = [k for k in range(3) if grads[k] is not None and ctx.like[k] is not None and ctx.needs_input_grad[4 + k]]
        for first in range(0, len(todo), 2):
            pair = todo[first:first + 2]
            src = [_cabi.as_f32(grads[k], dev).view(batch, width) for k in pair] + [None]
            dst = [torch.empty(nnz, dtype=torch.float32, device=dev) for _ in pair] + [None]
            with _cabi.device_guard(dev):
                _cabi.check(_cabi.lib().vamd_response_window_gather(
                    _cabi.ptr(src[0]), _cabi.ptr(src[1]), idx.data_ptr(), nnz, batch, seqlen, width,
                    _cabi.ptr(dst[0]), _cabi.ptr(dst[1]), _cabi.stream_ptr(dev)))
            for k, d in zip(pair, dst):
                shape, dtype, device = ctx.like[k]
                res[k] = d.view(shape).to(device=device, dtype=dtype)
        return (None, None, None, None, *res)


def pad_to_response_window(indices: torch.Tensor, batch: int, seqlen: int, response_length: int,
                           log_probs: torch.Tensor, entropy: torch.Tensor | None = None,
                           sum_pi_squared: torch.Tensor | None = None):
    """``pad_input(x.unsqueeze(-1), indices, batch, seqlen).squeeze(-1)[:, -response_length - 1:-1]`` for each
    given per-token tensor ``(total_nnz,)``; positions without a token hold 0.  ``indices`` are the flat
    positions of the tokens in the padded ``(batch, seqlen)`` layout, ascending (what ``unpad_input`` returns).
    Returns a tuple with one fp32 ``(batch, response_length)`` tensor per input that is not ``None``."""
    outs = _ResponseWindow.apply(indices, int(batch), int(seqlen), int(response_length), log_probs, entropy,
                                 sum_pi_squared)
    return tuple(o for o in outs if o is not None)
