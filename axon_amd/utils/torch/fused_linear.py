"""``FusedLinearForPPO`` — the reference's torch-backend face of the fused LM head.

Same constructor and ``forward`` signature as axon/utils/torch/fused_linear.py:219-241;
the work is done by the same HIP kernels as ``linear_cross_entropy``.  ``chunk_size``
is accepted and ignored (the kernels tile on their own).  Outputs are fp32; the
reference rounds them to the input dtype (fused_linear.py:46), which
``round_outputs_to_input_dtype=True`` (an extra constructor argument) reproduces.  ``logit_softcapping``
(Gemma, fused_linear.py:19-23,80-83) is applied inside the kernels.
"""

from __future__ import annotations

import torch

from axon_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy


class FusedLinearForPPO(torch.nn.Module):
    def __init__(self, chunk_size: int = 512, round_outputs_to_input_dtype: bool = False):
        super().__init__()
        self.chunk_size = chunk_size
        self.round_outputs_to_input_dtype = round_outputs_to_input_dtype

    def forward(self, hidden_states, vocab_weights, input_ids, temperature: float = 1.0,
                logit_softcapping: float | None = None):
        assert hidden_states.ndim in (2, 3), f"Invalid hidden_states shape, received {hidden_states.shape}"
        if hidden_states.ndim == 3:
            assert input_ids.ndim == 2, f"input_ids shape doesn't match, {hidden_states.shape} {input_ids.shape}"
        batch_shape = hidden_states.shape[:-1]
        log_probs, entropy = linear_cross_entropy(
            hidden_states.contiguous(), vocab_weights, input_ids.to(torch.int64).contiguous(), float(temperature), "none",
            None, logit_softcapping,
        )
        if self.round_outputs_to_input_dtype:
            log_probs, entropy = log_probs.to(hidden_states.dtype), entropy.to(hidden_states.dtype)
        return log_probs.view(batch_shape), entropy.view(batch_shape)
