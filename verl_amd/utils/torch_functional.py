"""Drop-ins for the tensor helpers of the reference's ``verl/utils/torch_functional.py`` on MI355X:

* the per-token definitions on materialised logits the actor uses when the fused head is off --
  ``logprobs_from_logits`` / ``_v2`` / ``_naive`` (reference :72-100, :148-200), ``entropy_from_logits`` /
  ``entropy_from_logits_with_chunking`` (:224-263) -- as one online-softmax pass per row
  (``vamd_row_softmax_stats``) with an elementwise backward (``vamd_row_softmax_backward``), and ``clip_by_value``
  (:203-221);
* the masked reductions ``masked_sum`` / ``masked_mean`` / ``masked_var`` / ``masked_whiten`` (:266-339).

Inputs of the masked reductions may live on the CPU (they are staged to the current GPU and the result is
returned on the CPU) or on a GPU.  Values are computed in fp32 with fp64 accumulation of the partial sums.
"""
from __future__ import annotations

import math

import torch

from .. import _cabi

_ROW_DTYPES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}   # VAMD_DT_*


def _logit_rows(logits: torch.Tensor):
    """``logits`` as a 2-D ``[rows, vocab]`` view with unit stride along the vocabulary, and its row pitch."""
    assert logits.is_cuda, "the logits must live on the GPU: there is no CPU fallback"
    assert logits.dtype in _ROW_DTYPES, f"logits must be fp32, bf16 or fp16, got {logits.dtype}"
    assert logits.dim() >= 1 and logits.numel() > 0
    vocab = logits.shape[-1]
    rows = logits.reshape(-1, vocab)
    if rows.stride(-1) != 1 or (rows.shape[0] > 1 and rows.stride(0) < vocab):
        rows = rows.contiguous()
    return rows, (rows.stride(0) if rows.shape[0] > 1 else vocab)


def _row_stats(rows, ld, labels, want_logprobs: bool, want_entropy: bool, want_mean_z: bool):
    n, vocab = rows.shape
    dev = rows.device
    f = lambda want: torch.empty(n, dtype=torch.float32, device=dev) if want else None
    logprobs, entropy, lse, mean_z = f(want_logprobs), f(want_entropy), f(True), f(want_mean_z)
    with _cabi.device_guard(dev):
        _cabi.check(_cabi.lib().vamd_row_softmax_stats(
            rows.data_ptr(), _ROW_DTYPES[rows.dtype], n, vocab, ld, _cabi.ptr(labels), _cabi.ptr(logprobs),
            _cabi.ptr(entropy), lse.data_ptr(), _cabi.ptr(mean_z), _cabi.stream_ptr(dev)))
    return logprobs, entropy, lse, mean_z


def _row_backward(rows, ld, labels, lse, mean_z, d_logprobs, d_entropy, in_place: bool):
    n, vocab = rows.shape
    dev = rows.device
    out = rows if in_place else torch.empty((n, vocab), dtype=rows.dtype, device=dev)
    ld_out = ld if in_place else vocab
    g = lambda t: None if t is None else t.detach().reshape(-1).to(device=dev, dtype=torch.float32).contiguous()
    d_logprobs, d_entropy = g(d_logprobs), g(d_entropy)
    with _cabi.device_guard(dev):
        _cabi.check(_cabi.lib().vamd_row_softmax_backward(
            rows.data_ptr(), _ROW_DTYPES[rows.dtype], n, vocab, ld, _cabi.ptr(labels), lse.data_ptr(),
            _cabi.ptr(mean_z), _cabi.ptr(d_logprobs), _cabi.ptr(d_entropy), out.data_ptr(), ld_out,
            _cabi.stream_ptr(dev)))
    return out


class _LogProbsFromLogits(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, inplace_backward: bool):
        assert labels.shape == logits.shape[:-1], f"labels {tuple(labels.shape)} do not match logits {tuple(logits.shape)}"
        rows, ld = _logit_rows(logits)
        lab = labels.reshape(-1).to(device=rows.device, dtype=torch.int64).contiguous()
        logprobs, _, lse, _ = _row_stats(rows, ld, lab, True, False, False)
        ctx.save_for_backward(rows, lab, lse)
        ctx.ld, ctx.shape = ld, logits.shape
        # writing the gradient over the logits needs the rows to BE the caller's storage
        ctx.in_place = (bool(inplace_backward) and rows.data_ptr() == logits.data_ptr() and logits.is_contiguous()
                        and not (logits.is_leaf and logits.requires_grad))   # never overwrite a parameter
        return logprobs.to(logits.dtype).view(logits.shape[:-1])

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, g):
        rows, lab, lse = ctx.saved_tensors
        if ctx.in_place:
            # the logits are about to become their own gradient: a second pass over this node would read gradients
            # where it expects logits
            if getattr(ctx, "logits_overwritten", False):
                raise RuntimeError("logprobs_from_logits(inplace_backward=True) wrote the gradient over the logits in "
                                   "its first backward pass and cannot run a second one; pass inplace_backward=False "
                                   "to keep the logits")
            ctx.logits_overwritten = True
        d = _row_backward(rows, ctx.ld, lab, lse, None, g, None, ctx.in_place)
        return d.view(ctx.shape), None, None


class _EntropyFromLogits(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, fp32_output: bool):
        rows, ld = _logit_rows(logits)
        _, entropy, lse, mean_z = _row_stats(rows, ld, None, False, True, True)
        ctx.save_for_backward(rows, lse, mean_z)
        ctx.ld, ctx.shape = ld, logits.shape
        if not fp32_output:
            entropy = entropy.to(logits.dtype)
        return entropy.view(logits.shape[:-1])

    @staticmethod
    def backward(ctx, g):
        rows, lse, mean_z = ctx.saved_tensors
        d = _row_backward(rows, ctx.ld, None, lse, mean_z, None, g, False)
        return d.view(ctx.shape), None


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = True) -> torch.Tensor:
    """Log-probability of ``labels`` under ``softmax(logits)``, shape ``logits.shape[:-1]``, dtype of ``logits``
    (reference torch_functional.py:72-100).  With ``inplace_backward`` (the default, as in the reference) the
    backward pass WRITES THE GRADIENT OVER THE LOGITS' STORAGE, as the reference's flash-attn path does
    (``cross_entropy_loss(..., inplace_backward=True)``); the reference does so only where flash-attn is
    installed, this function always.  Pass ``False`` when the logits are read again after the backward pass or
    the graph is backpropagated twice (a second pass raises instead of differentiating gradients)."""
    return _LogProbsFromLogits.apply(logits, labels, inplace_backward)


def logprobs_from_logits_naive(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """``log_softmax`` + gather (reference torch_functional.py:148-163)."""
    return _LogProbsFromLogits.apply(logits, labels, False)


def logprobs_from_logits_v2(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """``logits[label] - logsumexp(logits)`` row by row (reference torch_functional.py:166-200); fp32 arithmetic for
    every input dtype, one rounding to the dtype of ``logits`` at the end."""
    return _LogProbsFromLogits.apply(logits, labels, False)


def entropy_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """``logsumexp(logits) - sum(softmax(logits) * logits)`` (reference torch_functional.py:224-238), dtype of
    ``logits``."""
    return _EntropyFromLogits.apply(logits, False)


def entropy_from_logits_with_chunking(logits: torch.Tensor, chunk_size: int = 2048) -> torch.Tensor:
    """The same in fp32 whatever the dtype of ``logits`` (reference torch_functional.py:241-263).  ``chunk_size``
    is accepted for the signature: the kernel walks a row at a time and holds no ``[chunk, vocab]`` temporaries."""
    return _EntropyFromLogits.apply(logits, True)


class _ClipByValue(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, tensor_min, tensor_max):
        dev = _cabi.compute_device(x, tensor_min, tensor_max)
        to = lambda t: torch.as_tensor(t, dtype=torch.float32, device=dev)
        shape = torch.broadcast_shapes(*(tuple(torch.as_tensor(t).shape) for t in (x, tensor_min, tensor_max)))
        xs, lo, hi = (to(t).expand(shape).contiguous() for t in (x, tensor_min, tensor_max))
        out = torch.empty_like(xs)
        if xs.numel():
            with _cabi.device_guard(dev):
                _cabi.check(_cabi.lib().vamd_clip_by_value(xs.data_ptr(), lo.data_ptr(), hi.data_ptr(), xs.numel(),
                                                           out.data_ptr(), _cabi.stream_ptr(dev)))
        ctx.save_for_backward(xs, lo, hi)
        ctx.meta = [(tuple(t.shape), t.dtype, t.device) if isinstance(t, torch.Tensor) else None
                    for t in (x, tensor_min, tensor_max)]
        dtypes = [t.dtype for t in (x, tensor_min, tensor_max) if isinstance(t, torch.Tensor)]
        dtype = torch.float32
        if dtypes:   # what torch.max(torch.min(x, hi), lo) would return for same-rank tensors
            dtype = dtypes[0]
            for d in dtypes[1:]:
                dtype = torch.promote_types(dtype, d)
            if not dtype.is_floating_point:
                dtype = torch.float32
        return out.to(device=x.device if isinstance(x, torch.Tensor) else dev, dtype=dtype)

    @staticmethod
    def backward(ctx, g):
        xs, lo, hi = ctx.saved_tensors
        dev = xs.device
        gs = g.detach().to(device=dev, dtype=torch.float32).expand(xs.shape).contiguous()
        need = ctx.needs_input_grad
        outs = [torch.empty_like(xs) if need[i] and ctx.meta[i] is not None else None for i in range(3)]
        if xs.numel() and any(o is not None for o in outs):
            with _cabi.device_guard(dev):
                _cabi.check(_cabi.lib().vamd_clip_by_value_backward(
                    xs.data_ptr(), lo.data_ptr(), hi.data_ptr(), gs.data_ptr(), xs.numel(), _cabi.ptr(outs[0]),
                    _cabi.ptr(outs[1]), _cabi.ptr(outs[2]), _cabi.stream_ptr(dev)))
        res = []
        for o, meta in zip(outs, ctx.meta):
            if o is None:
                res.append(None)
            else:
                shape, dtype, device = meta
                res.append(o.sum_to_size(shape).to(device=device, dtype=dtype))
        return tuple(res)


def clip_by_value(x: torch.Tensor, tensor_min: torch.Tensor, tensor_max: torch.Tensor) -> torch.Tensor:
    """``max(min(x, tensor_max), tensor_min)`` with tensor bounds that broadcast against ``x`` (reference
    torch_functional.py:203-221), differentiable in all three arguments with torch's tie rule."""
    return _ClipByValue.apply(x, tensor_min, tensor_max)


def _as_matrix(values: torch.Tensor, mask: torch.Tensor, dev: torch.device):
    assert values.shape == mask.shape, f"values {tuple(values.shape)} and mask {tuple(mask.shape)} differ"
    v = _cabi.as_f32(values, dev)
    m, code = _cabi.mask_code(_cabi.on_device(mask, dev))
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
    with _cabi.device_guard(dev):
        _cabi.check(L.vamd_masked_moments(values.data_ptr(), mk.data_ptr(), code, rows, cols, int(per_row),
                                          out.data_ptr(), ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
    return out.t() if per_row else out


def _normalise_axis(axis, ndim: int):
    """``None`` or the sorted tuple of reduced dimensions."""
    if axis is None:
        return None
    dims = (axis,) if isinstance(axis, int) else tuple(axis)
    dims = tuple(sorted(d % ndim for d in dims)) if ndim else ()
    assert len(set(dims)) == len(dims), f"duplicate dimension in axis={axis}"
    return dims


def _reduce_geometry(values, dims):
    """(perm, kept_shape, rows, cols) that turn ``values`` into the [kept, reduced] matrix of a reduction."""
    ndim = values.dim()
    if dims is None:
        # all elements: keep the tensor's own [leading, last] matrix shape, which spreads the launch over rows
        cols = values.shape[-1] if ndim else 1
        return None, (), values.numel() // cols, cols
    kept = tuple(d for d in range(ndim) if d not in dims)
    perm = kept + dims
    if perm == tuple(range(ndim)):
        perm = None                      # the reduced dimensions are already the trailing ones
    kept_shape = tuple(values.shape[d] for d in kept)
    return perm, kept_shape, math.prod(kept_shape), math.prod(values.shape[d] for d in dims)


def _masked_reduce_forward(values, mask, dims, mean: bool, want_denom: bool):
    """One launch: fp32 masked sum or mean over ``dims`` (and the mean's denominator for the backward pass)."""
    dev = _cabi.compute_device(values, mask)
    perm, kept_shape, rows, cols = _reduce_geometry(values, dims)
    v = _cabi.as_f32(values, dev)
    m = _cabi.on_device(mask, dev)
    if perm is not None:
        v, m = v.permute(perm), m.permute(perm)
    v = v.reshape(rows, cols)
    m, code = _cabi.mask_code(m.reshape(rows, cols))
    if not v.is_contiguous():
        v = v.contiguous()
    per_row = dims is not None
    out = torch.empty(rows if per_row else 1, dtype=torch.float32, device=dev)
    denom = torch.empty_like(out) if (mean and want_denom) else None
    L = _cabi.lib()
    ws = _cabi.ticket_workspace(L.vamd_masked_moments_workspace_bytes(rows, cols), dev)
    with _cabi.device_guard(dev):
        _cabi.check(L.vamd_masked_reduce(v.data_ptr(), m.data_ptr(), code, rows, cols, int(per_row), None,
                                         None if mean else out.data_ptr(), out.data_ptr() if mean else None,
                                         _cabi.ptr(denom), None, 1, ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
    out_dtype = torch.result_type(values, mask)
    if not out_dtype.is_floating_point:
        out_dtype = torch.float32
    res = out.view(kept_shape)
    if res.dtype != out_dtype or res.device != values.device:
        res = res.to(device=values.device, dtype=out_dtype)
    return res, m, denom, (perm, tuple(values.shape), rows, cols, values.dtype, values.device)


class _MaskedReduce(torch.autograd.Function):
    """``masked_sum`` / ``masked_mean`` over any set of dimensions.  The reduced dimensions are moved last and the
    tensor is seen as ``[kept, reduced]``, which the row-wise moments kernel reduces; the gradient is
    ``mask * upstream`` (``/ (mask.sum + 1e-8)`` for the mean), one row-scaling kernel."""

    @staticmethod
    def forward(ctx, values, mask, dims, mean: bool):
        res, m, denom, geometry = _masked_reduce_forward(values, mask, dims, mean, want_denom=True)
        ctx.save_for_backward(m, denom)
        ctx.geometry = geometry
        return res

    @staticmethod
    def backward(ctx, g):
        m, denom = ctx.saved_tensors
        perm, shape, rows, cols, dtype, device = ctx.geometry
        dev = m.device
        coef = g.detach().to(device=dev, dtype=torch.float32).reshape(-1)   # one per kept row, or one in all
        if denom is not None:
            coef = coef / denom
        coef = coef.expand(rows).contiguous()
        weights = m if m.dtype == torch.float32 else m.to(torch.float32)   # d masked_sum / d values = mask
        one = torch.ones(1, dtype=torch.float32, device=dev)
        res = torch.empty((rows, cols), dtype=torch.float32, device=dev)
        with _cabi.device_guard(dev):
            _cabi.check(_cabi.lib().vamd_scale_rows(weights.data_ptr(), coef.data_ptr(), one.data_ptr(), 1.0, rows,
                                                    cols, res.data_ptr(), _cabi.stream_ptr(dev)))
        if perm is None:
            res = res.view(shape)
        else:
            inverse = [0] * len(perm)
            for i, d in enumerate(perm):
                inverse[d] = i
            res = res.view([shape[d] for d in perm]).permute(inverse)
        return res.to(device=device, dtype=dtype), None, None, None


def _reduce(values, mask, axis, mean: bool):
    assert values.shape == mask.shape, f"values {tuple(values.shape)} and mask {tuple(mask.shape)} differ"
    dims = _normalise_axis(axis, values.dim())
    if values.numel() == 0:   # a sum over nothing is 0, and 0 / (0 + 1e-8) is 0
        kept = () if dims is None else tuple(s for d, s in enumerate(values.shape) if d not in dims)
        return torch.zeros(kept, dtype=torch.float32, device=values.device)
    if values.requires_grad and torch.is_grad_enabled():
        return _MaskedReduce.apply(values, mask, dims, mean)
    return _masked_reduce_forward(values, mask, dims, mean, want_denom=False)[0]   # nothing to record: no autograd node


def masked_sum(values: torch.Tensor, mask: torch.Tensor, axis=None) -> torch.Tensor:
    """sum(where(mask.bool(), values, 0) * mask) over ``axis`` (an int, a tuple of ints or ``None`` for all
    elements), differentiable in ``values`` (reference torch_functional.py:266-284)."""
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


def _var_from_moments(s0: float, s1: float, s2: float, unbiased: bool) -> torch.Tensor:
    mean = torch.tensor(s1, dtype=torch.float32) / (torch.tensor(s0, dtype=torch.float32) + 1e-8)
    md = float(mean)
    var = torch.tensor(s2 - 2.0 * md * s1 + md * md * s0, dtype=torch.float32) / (
        torch.tensor(s0, dtype=torch.float32) + 1e-8)
    if unbiased:
        _raise_on_tiny_mask(s0)
        var = var * torch.tensor(s0 / (s0 - 1.0), dtype=torch.float32)
    return var


def _affine_masked(v, stats, m, code):
    """``((v - stats[0]) * stats[1] + stats[2]) * mask`` through ``vamd_affine_by_stats_masked``."""
    out = torch.empty_like(v)
    dev = v.device
    with _cabi.device_guard(dev):
        _cabi.check(_cabi.lib().vamd_affine_by_stats_masked(v.data_ptr(), stats.data_ptr(), m.data_ptr(), code,
                                                            v.numel(), out.data_ptr(), _cabi.stream_ptr(dev)))
    return out


def _variance_gradient_terms(s0: float, s1: float, unbiased: bool):
    """With D = sum(mask) + 1e-8 and mean = S1 / D:  d var / d v_k = scale * w_k * (v_k - centre), where
    centre = mean + (S1 - mean S0) / D carries the dependence of the mean on v_k (the second term is what the
    epsilon in D leaves of sum_i w_i (v_i - mean)) and scale = 2 / D times Bessel's factor."""
    d = s0 + 1e-8
    mean = s1 / d
    centre = mean + (s1 - mean * s0) / d
    scale = 2.0 / d * (s0 / (s0 - 1.0) if unbiased else 1.0)
    return mean, centre, scale, d


class _MaskedVar(torch.autograd.Function):
    @staticmethod
    def forward(ctx, values, mask, unbiased: bool):
        v, mom, dev = _global_moments(values, mask)
        s0, s1, s2, _ = mom.to("cpu").tolist()
        var = _var_from_moments(s0, s1, s2, unbiased)
        m, code = _cabi.mask_code(_cabi.on_device(mask, dev).reshape(v.shape))
        ctx.save_for_backward(v, m)
        ctx.meta = (code, s0, s1, unbiased, tuple(values.shape), values.dtype, values.device)
        return var.to(values.device)

    @staticmethod
    def backward(ctx, g):
        v, m = ctx.saved_tensors
        code, s0, s1, unbiased, shape, dtype, device = ctx.meta
        _, centre, scale, _ = _variance_gradient_terms(s0, s1, unbiased)
        gs = g.detach().to(device=v.device, dtype=torch.float32).reshape(1)
        stats = torch.cat([gs.new_tensor([centre]), gs * scale, gs.new_zeros(2)])
        return _affine_masked(v, stats, m, code).view(shape).to(device=device, dtype=dtype), None, None


def masked_var(values: torch.Tensor, mask: torch.Tensor, unbiased: bool = True) -> torch.Tensor:
    """Masked variance with Bessel's factor (reference torch_functional.py:304-319), differentiable in
    ``values``.  The reference centres by the mean in a second fp32 pass; here one pass accumulates count, sum and
    sum of squares in fp64 and the variance is ``(S2 - 2 mean S1 + mean^2 S0) / S0`` evaluated in fp64.  With
    fp32 inputs the cancellation costs a relative error of about ``(mean / std)^2 * 1e-16``: below fp32
    resolution while ``|mean| / std`` stays under about 1e4."""
    if values.requires_grad and torch.is_grad_enabled():
        return _MaskedVar.apply(values, mask, unbiased)
    _, mom, _ = _global_moments(values, mask)
    s0, s1, s2, _ = mom.to("cpu").tolist()
    return _var_from_moments(s0, s1, s2, unbiased).to(values.device)


def _masked_whiten_forward(values, mask, shift_mean: bool):
    dev = _cabi.compute_device(values, mask)
    v, m, code = _as_matrix(values, mask, dev)
    rows, cols = v.shape
    L = _cabi.lib()
    mom = torch.empty(4, dtype=torch.float64, device=dev)
    stats = torch.empty(4, dtype=torch.float32, device=dev)
    out = torch.empty_like(v)
    ws = _cabi.ticket_workspace(L.vamd_masked_moments_workspace_bytes(rows, cols), dev)
    with _cabi.device_guard(dev):
        s = _cabi.stream_ptr(dev)
        _cabi.check(L.vamd_masked_reduce(v.data_ptr(), m.data_ptr(), code, rows, cols, 0, mom.data_ptr(), None, None,
                                         None, stats.data_ptr(), int(shift_mean), ws.data_ptr(), ws.numel(), s))
        _cabi.check(L.vamd_affine_by_stats(v.data_ptr(), stats.data_ptr(), v.numel(), out.data_ptr(), s))
    return out, v, m, code, mom, stats


class _MaskedWhiten(torch.autograd.Function):
    """Gradient of ``out_j = (v_j - mean) r [+ mean]`` with ``r = rsqrt(var + 1e-8)``, mean and var taken over the
    mask: ``d_k = g_k r + w_k [(1[not shift] - r) G0 / D - r^3 G1 (d var / d v_k) / 2]`` with ``G0 = sum g`` and
    ``G1 = sum g (v - mean)`` over every element.  G0 and ``sum g v`` come from one masked-moments launch that
    takes ``g`` as the weights; the bracket is one ``vamd_affine_by_stats_masked`` pass."""

    @staticmethod
    def forward(ctx, values, mask, shift_mean: bool):
        out, v, m, code, mom, stats = _masked_whiten_forward(values, mask, shift_mean)
        s0, s1 = mom[:2].tolist()
        _raise_on_tiny_mask(s0)
        ctx.save_for_backward(v, m, stats)
        ctx.meta = (code, s0, s1, shift_mean, tuple(values.shape), values.dtype, values.device)
        return out.view(values.shape).to(values.device)

    @staticmethod
    def backward(ctx, g):
        v, m, stats = ctx.saved_tensors
        code, s0, s1, shift_mean, shape, dtype, device = ctx.meta
        dev = v.device
        mean, centre, scale, d = _variance_gradient_terms(s0, s1, True)
        gs = g.detach().to(device=dev, dtype=torch.float32).reshape(v.shape).contiguous()
        gm = _moments(v, gs, per_row=False)            # sum g, sum g v (g as weights), in fp64 on the device
        r = stats[1].to(torch.float64)
        g0, g1 = gm[0], gm[1] - mean * gm[0]
        slope = -0.5 * r * r * r * g1 * scale            # multiplies w_k (v_k - centre)
        const = ((0.0 if shift_mean else 1.0) - r) * g0 / d
        st = torch.stack([torch.full_like(slope, centre), slope, const, torch.zeros_like(slope)]).to(torch.float32)
        res = _affine_masked(v, st, m, code)
        res.add_(gs * stats[1])
        return res.view(shape).to(device=device, dtype=dtype), None, None


def masked_whiten(values: torch.Tensor, mask: torch.Tensor, shift_mean: bool = True) -> torch.Tensor:
    """(values - mean) * rsqrt(var + 1e-8) on every element (reference torch_functional.py:322-339): one launch for
    the masked moments and the statistics, one for the elementwise pass.  Differentiable in ``values``."""
    if values.requires_grad and torch.is_grad_enabled():
        return _MaskedWhiten.apply(values, mask, shift_mean)
    out, _, _, _, mom, _ = _masked_whiten_forward(values, mask, shift_mean)
    _raise_on_tiny_mask(mom[0].item())   # the reference raises here too; the pass above is already queued
    return out.view(values.shape).to(values.device)
