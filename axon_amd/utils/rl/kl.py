"""KL penalty estimators on the HIP path.

``kl_penalty`` / ``kl_penalty_forward`` keep the signatures and type strings of
axon/utils/rl/kl.py:154-245 ("kl"/"k1", "abs", "mse"/"k2", "low_var_kl"/"k3", the
straight-through variants "k1+"/"k3+"; "full" raises).  One elementwise kernel produces the
estimate and its derivative; the autograd function multiplies the latter by the upstream gradient.
"""

from __future__ import annotations

import torch

from axon_amd import _ops


class _KlPenalty(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logprob, ref_logprob, kl_type, kl_plus):
        out, grad = _ops.kl_penalty(logprob, ref_logprob, kl_type, kl_plus)
        ctx.save_for_backward(grad)
        ctx.in_dtype = logprob.dtype
        return out.to(logprob.dtype)

    @staticmethod
    def backward(ctx, g):
        (grad,) = ctx.saved_tensors
        return (grad * g).to(ctx.in_dtype), None, None, None


def kl_penalty(logprob: torch.Tensor, ref_logprob: torch.Tensor, kl_penalty_type: str = "low_var_kl") -> torch.Tensor:
    """KL estimate per token, differentiable w.r.t. ``logprob`` (kl.py:154-190)."""
    kl_type, plus = _ops.kl_type_of(kl_penalty_type)
    return _KlPenalty.apply(logprob, ref_logprob, kl_type, plus)


def kl_penalty_forward(logprob: torch.Tensor, ref_logprob: torch.Tensor,
                       kl_penalty_type: str = "low_var_kl") -> torch.Tensor:
    """Forward value only (kl.py:193-245): the "+" suffix is ignored."""
    kl_type, _ = _ops.kl_type_of(kl_penalty_type.rstrip("+"))
    return _ops.kl_penalty(logprob, ref_logprob, kl_type, 0)[0].to(logprob.dtype)
