"""``FusedLinearForPPO`` — the reference's torch-backend face of the fused LM head.

Same constructor and ``forward`` signature as axon/utils/torch/fused_linear.py:219-241;
the work is done by the same HIP kernels as ``linear_cross_entropy``.  ``chunk_size``
is accepted and ignored (the kernels tile on their own).  Outputs are fp32 (the
reference rounds them to the input dtype, fused_linear.py:46).  ``logit_softcapping``
(Gemma, fused_linear.py:19-23,80-83) is applied inside the kernels.
"""

from __future__ import annotations

import torch

from axon_amd.utils.kernel.linear_cross_entropy import linear_cross_entropy


class FusedLinearForPPO(torch.nn.Module):
    def __init__(self, chunk_size: int = 512):
        super().__init__()
        self.chunk_size = chunk_size

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
        return log_probs.view(batch_shape), entropy.view(batch_shape)
