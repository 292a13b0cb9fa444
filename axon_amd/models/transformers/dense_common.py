"""``forward_with_hip_backend`` — the LM-head face of a dense causal LM on this path.

Mirror of ``forward_with_triton_backend`` / ``forward_with_torch_backend``
(axon/models/transformers/dense_common.py:71-235), the functions the reference patches onto Hugging Face
model classes when ``impl_backend`` is "triton" or "torch": run the body model, choose the labels
(``pre_rolled_labels`` > ``roll(labels, -1)`` > ``roll(input_ids, -1)``, :187-196), call the fused head, return
an output object with ``.log_probs`` and ``.entropy``.  A model with ``final_logit_softcapping`` needs no
fallback here: the cap is applied inside the kernels.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from axon_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy, linear_cross_entropy_rows

try:  # the reference's output type extends the Hugging Face one (dense_common.py:23-26)
    from transformers.modeling_outputs import CausalLMOutputWithPast as _Base
except Exception:  # pragma: no cover - transformers is optional for this mirror
    @dataclass
    class _Base:  # type: ignore[no-redef]
        loss: Any = None
        logits: Any = None
        past_key_values: Any = None
        hidden_states: Any = None
        attentions: Any = None


@dataclass
class CausalLMOutputForPPO(_Base):
    log_probs: torch.FloatTensor | None = None
    entropy: torch.FloatTensor | None = None


def select_rolled_labels(pre_rolled_labels, labels, input_ids, backend: str = "forward_with_hip_backend"):
    """Next-token labels in the reference's order of precedence (dense_common.py:187-196)."""
    if pre_rolled_labels is not None:
        return pre_rolled_labels
    if labels is not None:
        return torch.roll(labels, shifts=-1, dims=-1)
    if input_ids is not None:
        return torch.roll(input_ids, shifts=-1, dims=-1)
    raise RuntimeError(f"To use {backend}, either labels or input_ids must be provided.")


def final_logit_softcapping(config):
    """``final_logit_softcapping`` of the text config, if the model has one (dense_common.py:204-208)."""
    if hasattr(config, "get_text_config"):
        return getattr(config.get_text_config(), "final_logit_softcapping", None)
    return getattr(config, "final_logit_softcapping", None)


def forward_with_hip_backend(
    self,
    input_ids=None,
    attention_mask=None,
    position_ids=None,
    past_key_values=None,
    inputs_embeds=None,
    labels=None,
    use_cache=None,
    output_attentions=None,
    output_hidden_states=None,
    return_dict=None,
    cache_position=None,
    logits_to_keep=0,
    temperature: float = 1.0,
    **loss_kwargs,
):
    """Same signature and behaviour as ``forward_with_triton_backend`` (dense_common.py:147-235); bind it with
    ``types.MethodType`` or assign it as the class's ``forward`` the way ``patch_forward_with_backends`` does."""
    output_attentions = output_attentions if output_attentions is not None else self.config.output_attentions
    output_hidden_states = (
        output_hidden_states if output_hidden_states is not None else self.config.output_hidden_states
    )
    outputs = self.model(
        input_ids=input_ids,
        attention_mask=attention_mask,
        position_ids=position_ids,
        past_key_values=past_key_values,
        inputs_embeds=inputs_embeds,
        use_cache=use_cache,
        output_attentions=output_attentions,
        output_hidden_states=output_hidden_states,
        return_dict=return_dict,
        cache_position=cache_position,
    )
    hidden_states = outputs[0]
    if not return_dict:
        raise NotImplementedError("forward_with_hip_backend has to return_dict")

    rolled_labels = select_rolled_labels(loss_kwargs.pop("pre_rolled_labels", None), labels, input_ids)
    # optional, no counterpart in the reference: rows (positions of hidden_states) the caller will not look at
    head_row_mask = loss_kwargs.pop("head_row_mask", None)
    if head_row_mask is not None:
        log_probs, entropy = linear_cross_entropy_rows(
            hidden_states, self.lm_head.weight, rolled_labels, head_row_mask, float(temperature),
            final_logit_softcapping(self.config),
        )
    else:
        log_probs, entropy = linear_cross_entropy(
            hidden_states.contiguous(), self.lm_head.weight, rolled_labels.contiguous(), float(temperature), "none",
            None, final_logit_softcapping(self.config),
        )
    return CausalLMOutputForPPO(
        log_probs=log_probs,
        entropy=entropy,
        past_key_values=getattr(outputs, "past_key_values", None),
        hidden_states=getattr(outputs, "hidden_states", None),
        attentions=getattr(outputs, "attentions", None),
    )
