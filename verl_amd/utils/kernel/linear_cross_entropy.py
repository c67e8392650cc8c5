"""Fused vocab-projection log-prob / entropy head on MI355X.

Drop-in for ``verl.utils.kernel.linear_cross_entropy`` (reference
verl/utils/kernel/linear_cross_entropy.py:38-119): same class name, ``forward`` / ``backward``
signatures, argument checks and return tuple.  The arithmetic runs in ``libverl_amd.so``
(``vamd_lce_forward`` / ``vamd_lce_backward``): bf16 MFMA logits tiles with an in-register online
softmax.  The ``[tokens, vocab]`` logits are never materialised: the backward pass recomputes them
tile by tile, as the reference does.  Opt-in trade for a 288 GB part: with
``VAMD_LCE_LOGITS_CACHE_GB=<budget>`` in the environment (default 0 = off), a forward pass that a
backward pass will follow keeps the logits in fp32 when ``4 * tokens * vocab`` bytes fit the budget,
and the backward pass then skips its logits-recompute GEMM (a quarter of the step's matrix work).
Results are the same either way up to one fp32 rounding of the logits.
"""
from __future__ import annotations

import os
import typing

import torch
import torch.distributed as dist

from ... import _cabi


def get_entropy_reduction_enum_number(reduction: str) -> int:
    """"none" -> 0, "sum" -> 1, "mean" -> 2; anything else raises ``ValueError``
    (reference verl/utils/kernel/kernels.py:110-126)."""
    table = {"none": 0, "sum": 1, "mean": 2}
    if reduction not in table:
        raise ValueError(f"Invalid reduction: {reduction}")
    return table[reduction]


def _check_inputs(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor) -> None:
    # the assertions of efficient_entropy_forward (reference kernels.py:574-593)
    assert hidden.is_cuda and weight.is_cuda and labels.is_cuda
    assert weight.device == hidden.device and labels.device == hidden.device
    assert hidden.dim() == 2 and weight.dim() == 2 and labels.dim() == 1
    assert hidden.is_contiguous() and weight.is_contiguous() and labels.is_contiguous()
    assert hidden.shape[0] == labels.shape[0] and hidden.shape[1] == weight.shape[1]
    assert hidden.shape[1] % 128 == 0
    assert hidden.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16, (
        f"the MI355X head computes on bf16 inputs, got {hidden.dtype} / {weight.dtype}"
    )


def logits_cache_budget_bytes() -> int:
    """Largest fp32 logits cache the autograd path may allocate: ``VAMD_LCE_LOGITS_CACHE_GB`` GiB, default 0
    (no cache: the backward pass recomputes the logits)."""
    return int(float(os.environ.get("VAMD_LCE_LOGITS_CACHE_GB", "0")) * (1 << 30))


def efficient_entropy_forward(hidden, weight, labels, reduction: int = 0, temperature: float = 1.0,
                              dist_process_group=None, logits_cache: torch.Tensor | None = None,
                              sum_pi_squared: torch.Tensor | None = None):
    """Host side of the forward kernels (reference kernels.py:563-753).

    Returns ``(logprobs, entropy, lse, mean_z)``; the last two are the per-token statistics the
    backward pass needs (log-sum-exp and softmax-weighted mean of the scaled logits).
    ``logits_cache``: optional fp32 ``[tokens, vocab]`` tensor that receives the scaled logits.
    ``sum_pi_squared``: optional fp32 ``[tokens]`` tensor that receives ``sum_j softmax(z)_j ** 2``.
    """
    if dist_process_group is not None:
        raise NotImplementedError("vocab-parallel process groups are not supported on this single-GPU path")
    _check_inputs(hidden, weight, labels)
    if labels.dtype != torch.int64:
        labels = labels.to(torch.int64)
    n, h = hidden.shape
    v = weight.shape[0]
    dev = hidden.device
    L = _cabi.lib()
    logprobs = torch.empty((n,), device=dev, dtype=torch.float32)
    entropy = torch.empty((n,), device=dev, dtype=torch.float32)
    lse = torch.empty((n,), device=dev, dtype=torch.float32)
    mean_z = torch.empty((n,), device=dev, dtype=torch.float32)
    if logits_cache is not None:
        assert logits_cache.shape == (n, v) and logits_cache.dtype == torch.float32
        assert logits_cache.is_contiguous() and logits_cache.device == dev
    if sum_pi_squared is not None:
        assert sum_pi_squared.shape == (n,) and sum_pi_squared.dtype == torch.float32
        assert sum_pi_squared.is_contiguous() and sum_pi_squared.device == dev
    ws = _cabi.workspace(L.vamd_lce_forward_workspace_bytes(n, h, v), dev)
    with _cabi.device_guard(dev):
        _cabi.check(L.vamd_lce_forward(hidden.data_ptr(), weight.data_ptr(), labels.data_ptr(), n, h, v,
                                       1.0 / temperature, logprobs.data_ptr(), entropy.data_ptr(), lse.data_ptr(),
                                       mean_z.data_ptr(), _cabi.ptr(logits_cache), _cabi.ptr(sum_pi_squared),
                                       ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
    if reduction == 1:
        logprobs = _sum_f32(logprobs)
    elif reduction == 2:
        logprobs = _sum_f32(logprobs) / n
    return logprobs, entropy, lse, mean_z


def _sum_f32(x: torch.Tensor) -> torch.Tensor:
    """Sum of a 1-D fp32 device tensor through the masked-moments kernel (mask of ones)."""
    from ..torch_functional import _moments

    ones = torch.ones_like(x, dtype=torch.uint8)
    return _moments(x.view(1, -1), ones.view(1, -1), per_row=False)[1].to(torch.float32)


def efficient_entropy_backward(dlogprobs, dentropy, hidden, weight, labels, lse, mean_z, reduction: int = 0,
                               temperature: float = 1.0, dist_process_group=None, d_entropy_scalar: float = 0.0,
                               d_weight_out: torch.Tensor | None = None, vocab_chunk: int = 0,
                               logits_cache: torch.Tensor | None = None,
                               d_weight_acc32: torch.Tensor | None = None, acc32_step: str | None = None,
                               need_d_hidden: bool = True, need_d_weight: bool = True):
    """Host side of the backward kernels (reference kernels.py:1512-1723).

    ``dlogprobs`` / ``dentropy`` may be ``None`` (no contribution).  ``d_entropy_scalar`` adds a
    constant upstream entropy gradient for every token without materialising it.
    ``logits_cache``: the tensor the forward call filled, if any (skips the recompute GEMM).
    Token-chunked callers sum the weight gradient of several calls, in one of two ways:
    ``d_weight_out`` (bf16) alone is ADDED to in bf16, one rounding of the running sum per call, like
    ``weight.grad +=`` in bf16 training; with ``d_weight_acc32`` (fp32 ``[vocab, hidden]``) the sum is kept
    in fp32 and ``acc32_step`` says which call this is: ``"first"`` (store), ``"middle"`` (add) or ``"last"``
    (add, then write the sum, rounded once, to ``d_weight_out`` or a fresh tensor).
    ``need_d_hidden`` / ``need_d_weight``: ``False`` for an input that requires no gradient (a frozen ``lm_head``,
    detached hidden states): its gradient GEMM is not run and ``None`` is returned in its place, as the reference's
    torch backend allocates and accumulates only the gradients its inputs require
    (verl/utils/experimental/torch_functional.py:150-156, :184-187).
    Returns ``(d_hidden, d_weight)`` in ``hidden.dtype``; ``d_weight`` is ``None`` for the "first" and
    "middle" steps of an fp32 accumulation.
    """
    if dist_process_group is not None:
        raise NotImplementedError("vocab-parallel process groups are not supported on this single-GPU path")
    _check_inputs(hidden, weight, labels)
    n, h = hidden.shape
    v = weight.shape[0]
    dev = hidden.device
    if dlogprobs is not None:
        if reduction == 0:
            assert dlogprobs.shape == (n,)
        else:
            assert dlogprobs.dim() == 0
            scale = 1.0 if reduction == 1 else 1.0 / n
            dlogprobs = (dlogprobs.to(torch.float32) * scale).expand(n)
        assert dlogprobs.is_cuda and dlogprobs.device == dev
        dlogprobs = dlogprobs.to(torch.float32).contiguous()
    if dentropy is not None:
        assert dentropy.shape == (n,)
        assert dentropy.is_cuda and dentropy.device == dev
        dentropy = dentropy.to(torch.float32).contiguous()
        assert d_entropy_scalar == 0.0, "pass the entropy gradient either as a tensor or as a scalar"
    assert lse.shape == (n,) and mean_z.shape == (n,)
    if logits_cache is not None:
        assert logits_cache.shape == (n, v) and logits_cache.dtype == torch.float32
        assert logits_cache.is_contiguous() and logits_cache.device == dev
    if labels.dtype != torch.int64:
        labels = labels.to(torch.int64)
    L = _cabi.lib()
    if not (need_d_hidden or need_d_weight):
        return None, None
    d_hidden = torch.empty_like(hidden) if need_d_hidden else None
    if not need_d_weight:
        assert d_weight_out is None and d_weight_acc32 is None, "no weight gradient was asked for"
        mode, d_weight = _cabi.DW_NONE, None
    elif d_weight_acc32 is not None:
        assert acc32_step in ("first", "middle", "last"), "acc32_step must be 'first', 'middle' or 'last'"
        assert d_weight_acc32.shape == weight.shape and d_weight_acc32.dtype == torch.float32
        assert d_weight_acc32.is_contiguous() and d_weight_acc32.device == dev
        mode = {"first": _cabi.DW_F32_STORE, "middle": _cabi.DW_F32_ADD, "last": _cabi.DW_F32_ADD_FINISH}[acc32_step]
        d_weight = (d_weight_out if d_weight_out is not None else torch.empty_like(weight)) if acc32_step == "last" else None
    else:
        assert acc32_step is None, "acc32_step needs d_weight_acc32"
        mode = _cabi.DW_ADD_BF16 if d_weight_out is not None else _cabi.DW_STORE
        d_weight = d_weight_out if d_weight_out is not None else torch.empty_like(weight)
    if d_weight is not None:
        assert d_weight.shape == weight.shape and d_weight.dtype == weight.dtype and d_weight.is_contiguous()
    ws = _cabi.workspace(L.vamd_lce_backward_workspace_bytes(n, h, v, vocab_chunk), dev)
    with _cabi.device_guard(dev):
        _cabi.check(L.vamd_lce_backward(hidden.data_ptr(), weight.data_ptr(), labels.data_ptr(), n, h, v,
                                        1.0 / temperature, lse.data_ptr(), mean_z.data_ptr(), _cabi.ptr(dlogprobs),
                                        _cabi.ptr(dentropy), float(d_entropy_scalar), _cabi.ptr(logits_cache),
                                        _cabi.ptr(d_hidden), _cabi.ptr(d_weight), mode, _cabi.ptr(d_weight_acc32),
                                        int(vocab_chunk), ws.data_ptr(), ws.numel(), _cabi.stream_ptr(dev)))
    return d_hidden, d_weight


_ACTIVE_PROBE_REST = 15
_ACTIVE_PROBE = {"rest": 0}   # calls left during which active_token_index() does not look at the gradients


def active_token_index(dlogprobs, dentropy, n_tokens: int):
    """Indices of the tokens whose upstream gradients are not both zero, or ``None`` when the backward pass should
    run over every token.

    In an actor update the head sees prompt and response tokens alike, and the loss masks the prompt tokens out: their
    ``d_logits`` rows are exactly zero, so they add nothing to ``d_weight`` and their ``d_hidden`` rows are zero.
    Running the backward kernels over the other tokens only gives the same gradients for a fraction of the work (the
    reference's kernels run over all of them).  The count is read on the host, so this is skipped under stream
    capture; ``VAMD_LCE_SKIP_ZERO_GRAD_TOKENS=0`` switches it off; nothing is gained, and nothing done, when more
    than nine tokens in ten are active.  Reading the count stalls the launch queue for about 0.1 ms, so after a call
    that found nearly every token active the next fifteen calls do not look."""
    if os.environ.get("VAMD_LCE_SKIP_ZERO_GRAD_TOKENS", "1") == "0":
        return None
    if torch.cuda.is_current_stream_capturing():
        return None
    if _ACTIVE_PROBE["rest"] > 0:
        _ACTIVE_PROBE["rest"] -= 1
        return None
    active = None
    for g in (dlogprobs, dentropy):
        if g is not None and g.dim() == 1 and g.shape[0] == n_tokens:
            nz = g != 0           # NaN counts as active
            active = nz if active is None else active.logical_or_(nz)
        elif g is not None:
            return None           # a scalar upstream gradient reaches every token
    if active is None:
        return None
    n_active = int(active.sum())  # the one host synchronisation of this path
    if 10 * n_active > 9 * n_tokens:
        _ACTIVE_PROBE["rest"] = _ACTIVE_PROBE_REST
        return None
    return active.nonzero().squeeze(1)


def backward_over_active_tokens(idx, dlogprobs, dentropy, hidden, weight, labels, lse, mean_z, temperature,
                                need_d_hidden: bool, need_d_weight: bool):
    """``efficient_entropy_backward`` over the rows ``idx`` of its per-token arguments; ``d_hidden`` comes back with
    zero rows for the tokens left out.  ``d_hidden`` rows are the same bits as over all tokens (a row depends on its
    own token only); ``d_weight`` sums the same non-zero terms in a different grouping."""
    d_hidden = torch.zeros_like(hidden) if need_d_hidden else None
    if idx.numel() == 0:
        return d_hidden, (torch.zeros_like(weight) if need_d_weight else None)
    take = lambda t: None if t is None else t.index_select(0, idx)
    dh, d_weight = efficient_entropy_backward(take(dlogprobs), take(dentropy), take(hidden), weight, take(labels),
                                              take(lse), take(mean_z), 0, temperature,
                                              need_d_hidden=need_d_hidden, need_d_weight=need_d_weight)
    if need_d_hidden:
        d_hidden.index_copy_(0, idx, dh)
    return d_hidden, d_weight


@torch.no_grad()
def linear_cross_entropy_with_sum_pi_squared(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor,
                                             temperature: float = 1.0):
    """``(logprobs, entropy, sum_pi_squared)`` of the head in one pass, without gradients: what the
    rollout-statistics pass of the actor needs when the optimal-token-baseline estimator is on
    (reference verl/workers/actor/dp_actor.py:280-287 computes ``sum_pi_squared`` from materialised
    logits with ``calculate_sum_pi_squared_from_logits``, verl/utils/torch_functional.py:680-694, and
    refuses to combine it with its fused kernels, dp_actor.py:107-111).  Outputs are flat fp32
    ``(num_tokens,)`` tensors."""
    if hidden.dim() != 2:
        hidden = hidden.view(-1, hidden.shape[-1])
    if labels.dim() != 1:
        labels = labels.view(-1)
    pi2 = torch.empty((hidden.shape[0],), device=hidden.device, dtype=torch.float32)
    logprobs, entropy, _, _ = efficient_entropy_forward(hidden, weight, labels, 0, temperature, sum_pi_squared=pi2)
    return logprobs, entropy, pi2


class LinearCrossEntropy(torch.autograd.Function):
    """``linear_cross_entropy(hidden, weight, labels, temperature, reduction, group)``.

    hidden ``(..., hidden_size)`` bf16 -> flattened to ``(num_tokens, hidden_size)``;
    weight ``(vocab_size, hidden_size)`` bf16; labels ``(...)`` -> ``(num_tokens,)``.
    Returns fp32 ``(logprobs, entropy)`` (``logprobs`` is a scalar for ``reduction`` "sum" /
    "mean").  For 2-D ``hidden`` (the remove-padding path) they are ``(num_tokens,)`` like the
    reference's fused op (verl/utils/kernel/linear_cross_entropy.py:40-87).  For ``hidden`` with
    leading batch dimensions they keep those dimensions, like the reference's torch backend
    (verl/utils/experimental/torch_functional.py:119-121): the padded caller slices them as
    ``[:, -response_length - 1 : -1]`` (verl/workers/actor/dp_actor.py:362-363), which the flat
    shape of the reference's fused op cannot serve, and the remove-padding caller's
    ``squeeze(0)`` (:254) accepts either.
    """

    @staticmethod
    def forward(ctx, hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor,
                temperature: typing.Optional[float] = 1.0, reduction: typing.Optional[str] = "none",
                dist_process_group: typing.Optional[dist.ProcessGroup] = None, grad_mode: bool = True):
        # grad_mode: whether autograd was recording when the caller invoked the op.  Inside forward() grad mode is
        # always off and ctx.needs_input_grad only mirrors requires_grad, so the wrapper below passes it in.
        assert isinstance(temperature, float), f"temperature must be a float, but got {type(temperature)}"
        assert isinstance(reduction, str), f"reduction must be a str, but got {type(reduction)}"
        REDUCTION = get_entropy_reduction_enum_number(reduction.lower())
        original_hidden_shape = hidden.shape
        if len(hidden.shape) != 2:
            hidden = hidden.view(-1, hidden.shape[-1])
        if len(labels.shape) != 1:
            labels = labels.view(-1)
        cache = None
        n_tokens, vocab = hidden.shape[0], weight.shape[0]
        backward_follows = grad_mode and (ctx.needs_input_grad[0] or ctx.needs_input_grad[1])
        if backward_follows and vocab % 8 == 0 and 4 * n_tokens * vocab <= logits_cache_budget_bytes():
            cache = torch.empty((n_tokens, vocab), device=hidden.device, dtype=torch.float32)
        logprobs, entropy, lse, mean_z = efficient_entropy_forward(
            hidden, weight, labels, REDUCTION, temperature, dist_process_group, logits_cache=cache)
        ctx.save_for_backward(hidden, weight, labels, lse, mean_z, cache)
        ctx.original_hidden_shape = original_hidden_shape
        ctx.REDUCTION = REDUCTION
        ctx.dist_process_group = dist_process_group
        ctx.temperature = temperature
        if len(original_hidden_shape) != 2:
            entropy = entropy.view(original_hidden_shape[:-1])
            if REDUCTION == 0:
                logprobs = logprobs.view(original_hidden_shape[:-1])
        return logprobs, entropy

    @staticmethod
    def backward(ctx, dlogprobs: torch.Tensor, dentropy: torch.Tensor):
        hidden, weight, labels, lse, mean_z, cache = ctx.saved_tensors
        if dentropy is not None:
            dentropy = dentropy.reshape(-1)
        if dlogprobs is not None and ctx.REDUCTION == 0:
            dlogprobs = dlogprobs.reshape(-1)
        need_dh, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        idx = None
        if cache is None and ctx.REDUCTION == 0 and (need_dh or need_dw):
            idx = active_token_index(dlogprobs, dentropy, hidden.shape[0])
        if idx is not None:   # tokens the loss masked out are left out of the backward kernels
            d_hidden, d_weight = backward_over_active_tokens(idx, dlogprobs, dentropy, hidden, weight, labels, lse,
                                                             mean_z, ctx.temperature, need_dh, need_dw)
        else:
            d_hidden, d_weight = efficient_entropy_backward(
                dlogprobs, dentropy, hidden, weight, labels, lse, mean_z, ctx.REDUCTION, ctx.temperature,
                ctx.dist_process_group, logits_cache=cache, need_d_hidden=need_dh, need_d_weight=need_dw)
        if d_hidden is not None:
            d_hidden = d_hidden.view(ctx.original_hidden_shape)
        return (d_hidden, d_weight, None, None, None, None, None)


def linear_cross_entropy(hidden: torch.Tensor, weight: torch.Tensor, labels: torch.Tensor,
                         temperature: typing.Optional[float] = 1.0, reduction: typing.Optional[str] = "none",
                         dist_process_group: typing.Optional[dist.ProcessGroup] = None):
    """``LinearCrossEntropy.apply`` with the reference's positional signature
    (verl/utils/kernel/linear_cross_entropy.py:119).  A forward pass under ``torch.no_grad()`` (the actor's
    ``compute_log_prob``) keeps nothing for a backward pass, whatever ``requires_grad`` says."""
    return LinearCrossEntropy.apply(hidden, weight, labels, temperature, reduction, dist_process_group,
                                    torch.is_grad_enabled())
