"""Model ``forward`` replacements that end in the HIP log-prob / entropy head instead of ``lm_head`` + logits:
the counterparts of ``forward_with_triton_backend`` / ``forward_with_torch_backend`` and of the selection in
``patch_forward_with_backends`` (reference verl/models/transformers/dense_common.py:71-193,
verl/models/transformers/monkey_patch.py:234-283).

The decoder runs as the model defines it (``self.model(...)``); the labels are the input ids rolled by one
position (dense_common.py:172-175); the head returns ``log_probs`` and ``entropy`` without ever forming logits.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

import torch


@dataclass
class CausalLMOutputForPPO:
    """The fields the actor reads (``log_probs``, ``entropy``, reference dense_common.py:23-26) plus the decoder
    outputs that are passed through."""
    log_probs: Optional[torch.Tensor] = None
    entropy: Optional[torch.Tensor] = None
    past_key_values: Any = None
    hidden_states: Any = None
    attentions: Any = None
    loss: Optional[torch.Tensor] = None
    logits: Optional[torch.Tensor] = None


def _decoder_outputs(self, input_ids, attention_mask, position_ids, past_key_values, inputs_embeds, use_cache,
                     output_attentions, output_hidden_states, return_dict, cache_position):
    config = getattr(self, "config", None)
    if output_attentions is None:
        output_attentions = getattr(config, "output_attentions", None)
    if output_hidden_states is None:
        output_hidden_states = getattr(config, "output_hidden_states", None)
    return self.model(input_ids=input_ids, attention_mask=attention_mask, position_ids=position_ids,
                      past_key_values=past_key_values, inputs_embeds=inputs_embeds, use_cache=use_cache,
                      output_attentions=output_attentions, output_hidden_states=output_hidden_states,
                      return_dict=return_dict, cache_position=cache_position)


def _rolled_labels(labels, input_ids, who: str):
    if labels is not None:
        return torch.roll(labels, shifts=-1, dims=-1)
    if input_ids is not None:
        return torch.roll(input_ids, shifts=-1, dims=-1)
    raise RuntimeError(f"To use {who}, either labels or input_ids must be provided.")


def _ppo_output(outputs, log_probs, entropy):
    return CausalLMOutputForPPO(log_probs=log_probs, entropy=entropy,
                                past_key_values=getattr(outputs, "past_key_values", None),
                                hidden_states=getattr(outputs, "hidden_states", None),
                                attentions=getattr(outputs, "attentions", None))


def forward_with_hip_backend(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None,
                             inputs_embeds=None, labels=None, use_cache=None, output_attentions=None,
                             output_hidden_states=None, return_dict=None, cache_position=None, logits_to_keep=0,
                             temperature: float = 1.0, **loss_kwargs):
    """``forward_with_triton_backend`` (dense_common.py:133-193) with the HIP head: same arguments, same
    ``CausalLMOutputForPPO`` with ``log_probs`` / ``entropy`` shaped like ``input_ids``."""
    from verl_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy

    outputs = _decoder_outputs(self, input_ids, attention_mask, position_ids, past_key_values, inputs_embeds,
                               use_cache, output_attentions, output_hidden_states, return_dict, cache_position)
    hidden_states = outputs[0]
    if not return_dict:
        raise NotImplementedError("forward_with_hip_backend has to return_dict")
    rolled = _rolled_labels(labels, input_ids, "forward_with_hip_backend")
    log_probs, entropy = linear_cross_entropy(hidden_states.contiguous(), self.lm_head.weight, rolled.contiguous(),
                                              float(temperature), "none")
    return _ppo_output(outputs, log_probs, entropy)


def forward_with_torch_backend(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None,
                               inputs_embeds=None, labels=None, use_cache=None, output_attentions=None,
                               output_hidden_states=None, return_dict=None, cache_position=None, logits_to_keep=0,
                               temperature: float = 1.0, **loss_kwargs):
    """``forward_with_torch_backend`` (dense_common.py:71-130): the ``FusedLinearForPPO`` contract (outputs in the
    dtype of the hidden states) on the HIP head."""
    from verl_amd.utils.experimental.torch_functional import FusedLinearForPPO

    outputs = _decoder_outputs(self, input_ids, attention_mask, position_ids, past_key_values, inputs_embeds,
                               use_cache, output_attentions, output_hidden_states, None, cache_position)
    hidden_states = outputs[0]
    if not return_dict:
        raise NotImplementedError("forward_with_torch_backend has to return_dict")
    rolled = _rolled_labels(labels, input_ids, "forward_with_torch_backend")
    log_probs, entropy = FusedLinearForPPO().forward(hidden_states=hidden_states, vocab_weights=self.lm_head.weight,
                                                     input_ids=rolled, temperature=temperature)
    return _ppo_output(outputs, log_probs, entropy)


# the reference's own name for the fused-kernel forward resolves to the HIP head here
forward_with_triton_backend = forward_with_hip_backend


def patch_forward_with_backends(model, use_fused_kernels: bool = False, fused_kernels_backend: str = None):
    """Select the model's ``forward`` as monkey_patch.py:234-283 does.  ``"hip"`` and ``"triton"`` (the value
    existing configurations carry) give the HIP head with fp32 flat-or-batched outputs; ``"torch"`` gives the
    ``FusedLinearForPPO`` contract.  Other values leave the model untouched, as in the reference."""
    if not use_fused_kernels or fused_kernels_backend not in ["hip", "triton", "torch"]:
        print(f"Skipping monkey patch for {model.__class__.__name__} as use_fused_kernels is "
              f"{use_fused_kernels} or fused_kernels_backend is {fused_kernels_backend}")
        return
    if fused_kernels_backend == "torch":
        model.__class__.forward = forward_with_torch_backend
    else:
        model.__class__.forward = forward_with_hip_backend
    print(f"Using the HIP head ({fused_kernels_backend} contract) for fused kernels in {model.__class__.__name__}")
