"""Log-probabilities and entropy from materialised logits on the HIP path.

Mirror of ``logprobs_from_logits`` (axon/utils/torch/ops.py:39-102), ``entropy_from_logits`` and
``entropy_from_logits_with_chunking`` (:105-120): what the trainer calls when ``use_fused_kernels`` is off
and the model has written the ``[tokens, vocab]`` logits (axon/utils/fsdp/forward_utils.py:287-304).  One
kernel reads each row once for both quantities; the backward reads it once more and writes the gradient,
over the logits themselves when ``inplace_backward`` is set (the behaviour of the flash-attn cross entropy
the reference prefers, :70-75).  ``logprobs_and_entropy_from_logits`` returns both from a single pass and
has a single backward; the reference runs two functions over the same logits.
"""

from __future__ import annotations

import torch

from axon_amd import _ops

__all__ = ["logprobs_from_logits", "entropy_from_logits", "entropy_from_logits_with_chunking",
           "logprobs_and_entropy_from_logits"]


def _rows(logits):
    flat = logits.reshape(-1, logits.shape[-1])
    if flat.stride(-1) != 1:
        flat = flat.contiguous()
    return flat


class _LogitsHead(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels, want_entropy, inplace_backward):
        flat = _rows(logits)
        lab = labels.reshape(-1).contiguous() if labels is not None else None
        logprob, entropy, lse = _ops.logits_forward(flat, lab, want_entropy)
        ctx.save_for_backward(flat, lab, lse, entropy)
        ctx.shape = logits.shape
        # writing the gradient over the logits is only possible when `flat` is the caller's storage
        ctx.inplace = bool(inplace_backward) and flat.data_ptr() == logits.data_ptr()
        batch = logits.shape[:-1]
        outs = (logprob.view(batch) if logprob is not None else None,
                entropy.view(batch) if entropy is not None else None)
        return outs

    @staticmethod
    def backward(ctx, g_logprob, g_entropy):
        flat, lab, lse, entropy = ctx.saved_tensors
        g_lp = g_logprob.reshape(-1) if g_logprob is not None and lab is not None else None
        g_en = g_entropy.reshape(-1) if g_entropy is not None and entropy is not None else None
        grad = _ops.logits_backward(flat, lab, lse, entropy, g_lp, g_en, inplace=ctx.inplace)
        return grad.view(ctx.shape), None, None, None


def logprobs_and_entropy_from_logits(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = False):
    """``(log_softmax(logits)[labels], entropy)`` of shape ``logits.shape[:-1]``, fp32, from one read of the
    logits."""
    return _LogitsHead.apply(logits, labels, True, inplace_backward)


def logprobs_from_logits(logits: torch.Tensor, labels: torch.Tensor, inplace_backward: bool = True) -> torch.Tensor:
    """Per-token log-probability of ``labels`` (ops.py:39-67), fp32, shape ``logits.shape[:-1]``.  With
    ``inplace_backward`` the backward writes d loss / d logits over the logits' storage."""
    return _LogitsHead.apply(logits, labels, False, inplace_backward)[0]


def entropy_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """``logsumexp(logits) - sum softmax(logits) * logits`` (ops.py:105-109), fp32."""
    return _LogitsHead.apply(logits, None, True, False)[1]


def entropy_from_logits_with_chunking(logits: torch.Tensor, chunk_size: int = 2048) -> torch.Tensor:
    """Same values as ``entropy_from_logits`` (ops.py:112-120); the reference chunks over tokens to bound its
    fp32 temporaries, of which there are none here, so ``chunk_size`` is accepted and not used."""
    return entropy_from_logits(logits)
