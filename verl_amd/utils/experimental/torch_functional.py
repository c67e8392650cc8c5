"""``FusedLinearForPPO`` on MI355X: the drop-in for what the reference selects with
``fused_kernel_options.impl_backend: torch`` (verl/utils/experimental/torch_functional.py:75-216).

Same class names, ``forward(hidden_states, vocab_weights, input_ids, temperature)`` signature and output
contract as the reference -- outputs in the dtype of ``hidden_states`` (:37), ``[B, S]`` for 3-D input
(:119-121), upstream gradients that may be ``None`` (:85, :132-133), gradients only for the inputs that
require them (:150-156) -- computed by the HIP head (``vamd_lce_forward`` / ``vamd_lce_backward``) instead of a
Python loop over 512-token chunks of materialised logits.  ``chunk_size`` is accepted and ignored: the
kernels tile tokens and vocabulary themselves and never hold a ``[chunk, vocab]`` logits tensor.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernel.linear_cross_entropy import (active_token_index, backward_over_active_tokens,
                                           efficient_entropy_backward, efficient_entropy_forward)


class FusedLinearForPPOFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden_states: torch.Tensor, vocab_weights: torch.Tensor, input_ids: torch.Tensor,
                temperature: float = 1.0, chunk_size: int = 512):
        ctx.set_materialize_grads(False)
        orig_ndim = hidden_states.ndim
        assert orig_ndim in (2, 3), f"Invalid hidden_states shape, received {hidden_states.shape}"
        orig_batch_size = -1
        if orig_ndim == 3:
            assert input_ids.ndim == 2, f"input_ids shape doesn't match, {hidden_states.shape} {input_ids.shape}"
            orig_batch_size = hidden_states.shape[0]
            hidden_states = hidden_states.flatten(0, 1)
            input_ids = input_ids.flatten(0, 1)
        hidden_states = hidden_states.contiguous()
        vocab_weights = vocab_weights.contiguous()
        input_ids = input_ids.contiguous()
        log_probs, entropy, lse, mean_z = efficient_entropy_forward(hidden_states, vocab_weights, input_ids, 0,
                                                                    float(temperature))
        # the reference casts both outputs back to the dtype of the logits, i.e. of the inputs (:37)
        log_probs = log_probs.to(hidden_states.dtype)
        entropy = entropy.to(hidden_states.dtype)
        if orig_ndim == 3:
            log_probs = log_probs.view(orig_batch_size, -1)
            entropy = entropy.view(orig_batch_size, -1)
        ctx.save_for_backward(hidden_states, vocab_weights, input_ids, lse, mean_z)
        ctx.orig_batch_size = orig_batch_size
        ctx.orig_ndim = orig_ndim
        ctx.temperature = float(temperature)
        ctx.chunk_size = chunk_size
        return log_probs, entropy

    @staticmethod
    def backward(ctx, dlog_probs: Optional[torch.Tensor], dentropy: Optional[torch.Tensor]):
        assert dlog_probs is not None or dentropy is not None
        hidden_states, vocab_weights, input_ids, lse, mean_z = ctx.saved_tensors
        if dlog_probs is not None:
            dlog_probs = dlog_probs.reshape(-1)
        if dentropy is not None:
            dentropy = dentropy.reshape(-1)
        # only the gradient GEMMs whose inputs require a gradient are run (reference :150-156, :184-187), and only over
        # the tokens whose upstream gradients are not both zero (prompt tokens, which the loss masks out)
        need_dh, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        idx = active_token_index(dlog_probs, dentropy, hidden_states.shape[0]) if (need_dh or need_dw) else None
        if idx is not None:
            dhidden_states, dvocab_weights = backward_over_active_tokens(
                idx, dlog_probs, dentropy, hidden_states, vocab_weights, input_ids, lse, mean_z, ctx.temperature,
                need_dh, need_dw)
        else:
            dhidden_states, dvocab_weights = efficient_entropy_backward(
                dlog_probs, dentropy, hidden_states, vocab_weights, input_ids, lse, mean_z, 0, ctx.temperature,
                need_d_hidden=need_dh, need_d_weight=need_dw)
        if dhidden_states is not None and ctx.orig_ndim == 3:
            dhidden_states = dhidden_states.view(ctx.orig_batch_size, -1, hidden_states.shape[-1])
        return dhidden_states, dvocab_weights, None, None, None


class FusedLinearForPPO(torch.nn.Module):
    def __init__(self, chunk_size: int = 512):
        super().__init__()
        self.chunk_size = chunk_size

    def forward(self, hidden_states: torch.Tensor, vocab_weights: torch.Tensor, input_ids: torch.Tensor,
                temperature: float = 1.0):
        input_ids = input_ids.to(torch.int64)
        return FusedLinearForPPOFunction.apply(hidden_states, vocab_weights, input_ids, temperature, self.chunk_size)
