"""``linear_cross_entropy`` — fused LM-head log-prob + entropy on MI355X.

Drop-in for axon/utils/kernel/linear_cross_entropy.py:50-131 (``LinearCrossEntropy``
/ ``linear_cross_entropy = LinearCrossEntropy.apply``), the op called from
``forward_with_triton_backend`` (axon/models/transformers/dense_common.py:221-227):

    logprobs, entropy = linear_cross_entropy(hidden, weight, labels, temperature, "none")

* ``hidden`` ``[N, H]`` or ``[1, N, H]``, ``weight`` ``[V, H]``, ``labels`` int32/int64.  The kernels compute in
  bf16 with fp32 accumulation (the trainer runs under bf16 autocast, forward_utils.py:216); fp16 or fp32
  operands are accepted like the reference accepts any float dtype (kernels.py:517-522 asserts layout only),
  are rounded to bf16 first, and receive their gradients in their own dtype.  That is narrower arithmetic than
  the reference's op, which computes in the operands' own dtype, and it costs a bf16 copy of each such operand
  per forward (kept for the backward: 1.2 GB for a 151936 x 4096 fp32 weight) plus the cast of its gradient
  back; a warning says so once per process;
* outputs are flat fp32 ``[N]`` (never reshaped back, like the reference);
* differentiable w.r.t. ``hidden`` and ``weight``; gradients come back in the input dtype;
* ``reduction`` "sum"/"mean" reduce the log-probs as the reference's epilogue does
  (kernels.py:369-378); the trainer path uses "none";
* a ``dist_process_group`` (vocab-parallel head) is refused: one GPU only;
* ``logit_softcapping`` (an extra trailing argument the reference's Triton op does not have; its
  models fall back to the torch path for it, dense_common.py:201-219) applies
  ``cap * tanh(logits / cap)`` before the temperature (fused_linear.py:19-23), forward and backward;
* ``cu_seqlens`` (a second extra trailing argument, int32 ``[S+1]``) selects the token-aligned packed
  layout: ``labels`` is then the packed stream of token ids itself, and the outputs come back aligned
  to token positions (``out[p]`` = log-prob of token ``p`` given its prefix, 0 at the first position of
  every sequence).  That is ``torch.roll(ids, -1)`` before the head and the shift-right after it
  (axon/utils/fsdp/forward_utils.py:131,164-182) done inside the kernels, forward and backward.

The [tokens x vocab] logits are never written to memory: the backward recomputes them chunk by chunk, as
the reference's kernels do (kernels.py:1377-1585).  Opt-in (``axon_amd._ops.LMHEAD_STASH``), a forward that
is going to be differentiated keeps 2 bytes per logit for its backward (each softmax numerator as fp16),
which then decodes the dlogits instead of recomputing the logits: a quarter fewer flops for
tokens x vocab x 2 bytes of memory.
"""

from __future__ import annotations

import torch

from axon_amd import _lib, _ops

_REDUCTIONS = ("none", "sum", "mean")
_warned_rounding = False


def _warn_rounded_to_bf16(hidden_dtype, weight_dtype) -> None:
    global _warned_rounding
    if _warned_rounding:
        return
    _warned_rounding = True
    import warnings

    warnings.warn(f"linear_cross_entropy: hidden ({hidden_dtype}) / weight ({weight_dtype}) are rounded to bfloat16 "
                  "before the head (the kernels compute in bf16 with fp32 accumulation); each call makes a bf16 copy "
                  "of such an operand and casts its gradient back", stacklevel=3)


class LinearCrossEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, labels, temperature=1.0, reduction="none", dist_process_group=None,
                logit_softcapping=None, cu_seqlens=None):
        assert isinstance(temperature, float), f"temperature must be a float, but got {type(temperature)}"
        assert isinstance(reduction, str), f"reduction must be a str, but got {type(reduction)}"
        reduction = reduction.lower()
        if reduction not in _REDUCTIONS:
            raise ValueError(f"Invalid reduction: {reduction}")
        if dist_process_group is not None:
            raise NotImplementedError("vocab-parallel LM head (dist_process_group) is not part of the one-GPU path")
        _lib.require_device(hidden, "linear_cross_entropy")
        assert weight.device == hidden.device and labels.device == hidden.device
        floats = (torch.bfloat16, torch.float16, torch.float32)
        assert hidden.dtype in floats and weight.dtype in floats, "hidden and weight must be bf16, fp16 or fp32"
        assert labels.dtype in (torch.int32, torch.int64), "labels must be int32 or int64"

        shape = hidden.shape
        hidden2 = hidden.reshape(-1, shape[-1])
        labels1 = labels.reshape(-1)
        assert weight.dim() == 2 and hidden2.shape[1] == weight.shape[1]
        assert hidden2.shape[0] == labels1.shape[0]
        assert hidden2.is_contiguous() and weight.is_contiguous() and labels1.is_contiguous()
        ctx.in_dtypes = (hidden.dtype, weight.dtype)
        if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
            _warn_rounded_to_bf16(hidden.dtype, weight.dtype)
        hidden2, weight = hidden2.to(torch.bfloat16), weight.to(torch.bfloat16)  # no copy when already bf16

        inv_t = 1.0 / temperature
        cap = 0.0 if logit_softcapping is None else float(logit_softcapping)
        if not cap >= 0.0:
            raise ValueError(f"logit_softcapping must be positive, got {logit_softcapping}")
        seq_start = None if cu_seqlens is None else _ops.seq_start_flags(cu_seqlens, hidden2.shape[0])
        want_grad = bool(ctx.needs_input_grad[0] or ctx.needs_input_grad[1])
        res = _ops.lmhead_forward(hidden2, weight, labels1, inv_t, timing=_ops.TIMING, softcap=cap,
                                  seq_start=seq_start, stash=want_grad)
        logprobs, entropy, lse, entropy_b = res[:4]
        stash = res[4] if want_grad else None
        ctx.save_for_backward(hidden2, weight, labels1, lse, entropy_b, seq_start, stash)
        ctx.shape, ctx.inv_t, ctx.reduction, ctx.cap = shape, inv_t, reduction, cap
        if reduction == "sum":
            logprobs = logprobs.sum()
        elif reduction == "mean":
            logprobs = logprobs.mean()
        return logprobs, entropy

    @staticmethod
    def backward(ctx, dlogprobs, dentropy):
        hidden2, weight, labels1, lse, entropy_b, seq_start, stash = ctx.saved_tensors
        n = hidden2.shape[0]
        if dlogprobs is None:
            dlogprobs = torch.zeros(n, device=hidden2.device, dtype=torch.float32)
        elif ctx.reduction == "sum":
            dlogprobs = dlogprobs.expand(n)
        elif ctx.reduction == "mean":
            dlogprobs = (dlogprobs / n).expand(n)
        d_hidden, d_weight = _ops.lmhead_backward(
            dlogprobs.reshape(-1), None if dentropy is None else dentropy.reshape(-1), hidden2, weight, labels1, lse,
            entropy_b, ctx.inv_t, timing=_ops.TIMING, softcap=ctx.cap, seq_start=seq_start, stash=stash,
        )
        return (d_hidden.view(ctx.shape).to(ctx.in_dtypes[0]), d_weight.to(ctx.in_dtypes[1]), None, None, None, None,
                None, None)


linear_cross_entropy = LinearCrossEntropy.apply


def linear_cross_entropy_rows(hidden, weight, labels, row_mask, temperature=1.0, logit_softcapping=None):
    """``linear_cross_entropy(..., "none")`` over the rows where ``row_mask`` is not zero only; the other rows
    come back as 0 and receive a zero gradient.  For callers that know which rows nobody will look at (prompt
    positions under a response mask): the reference runs the head over all of them.  One readback."""
    shape = labels.shape
    h2 = hidden.reshape(-1, hidden.shape[-1])
    rows = torch.nonzero(row_mask.reshape(-1)).flatten()
    if row_mask.numel() != h2.shape[0]:
        raise ValueError(f"row_mask has {row_mask.numel()} entries for {h2.shape[0]} rows")
    lp_c, ent_c = linear_cross_entropy(h2.index_select(0, rows), weight, labels.reshape(-1).index_select(0, rows),
                                       float(temperature), "none", None, logit_softcapping)
    zeros = torch.zeros(h2.shape[0], device=lp_c.device, dtype=lp_c.dtype)
    return zeros.index_copy(0, rows, lp_c).view(shape), zeros.index_copy(0, rows, ent_c).view(shape)

