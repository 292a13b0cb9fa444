"""Loss aggregation helpers on the HIP path.

``agg_loss`` keeps the signature of axon/trainer/algos/loss/utils.py:120-187
(two-axis reduction: token_reduce x batch_reduce) and ``masked_mean`` that of
:88-91.  Both are differentiable with respect to their first argument.  The
reductions run in libaxon_amd.so: for ``sum`` / ``token-mean`` one pass over the tokens;
otherwise a row-statistics pass and a single-workgroup pass that folds every denominator
into a per-row multiplier come first.  Scalars are added from per-workgroup partials in a fixed
order (no atomics).
"""

from __future__ import annotations

import torch

from axon_amd import _lib, _ops
from axon_amd.trainer.algos.constants import VALID_BATCH_REDUCE, VALID_TOKEN_REDUCE

__all__ = ["agg_loss", "masked_mean"]


class _WeightedRowSum(torch.autograd.Function):
    """sum_t loss[t] * mask[t] * row_scale[row(t)] with gradient mask*row_scale: the entropy slot of
    ``axon_side_terms`` (one pass for sum / token-mean, a row pass first otherwise)."""

    @staticmethod
    def forward(ctx, loss_mat, mask, rows, token_reduce, batch_reduce, extras):
        prtc, npt, nps, valid = extras
        acc, agg_w, _ = _ops.side_terms(loss_mat, None, None, mask, rows, token_reduce=token_reduce,
                                        batch_reduce=batch_reduce, per_row_token_count=prtc, num_program_tokens=npt,
                                        num_program_steps=nps, valid_count=valid)
        ctx.save_for_backward(agg_w, acc)
        ctx.in_dtype = loss_mat.dtype
        return acc[0].clone()

    @staticmethod
    def backward(ctx, g):
        agg_w, acc = ctx.saved_tensors
        return _ops.scale_f32(agg_w, g, acc[5]).to(ctx.in_dtype), None, None, None, None, None


def agg_loss(
    loss_mat: torch.Tensor,
    loss_mask: torch.Tensor,
    *,
    token_reduce: str = "sum",
    batch_reduce: str = "token-mean",
    num_program_tokens=None,
    num_program_steps=None,
    valid_token_count=None,
    valid_batch_size=None,
    valid_program_count=None,
    per_row_token_count=None,
    cu_seqlens=None,
) -> torch.Tensor:
    """Aggregate a per-token loss to a scalar; extra ``cu_seqlens`` selects the packed layout."""
    if token_reduce not in VALID_TOKEN_REDUCE:
        raise ValueError(f"Invalid token_reduce: {token_reduce!r}. Choose from: {sorted(VALID_TOKEN_REDUCE)}")
    if batch_reduce not in VALID_BATCH_REDUCE:
        raise ValueError(f"Invalid batch_reduce: {batch_reduce!r}. Choose from: {sorted(VALID_BATCH_REDUCE)}")
    if token_reduce == "mean-program":
        assert num_program_tokens is not None, "num_program_tokens required for token_reduce='mean-program'"
    valid = None
    if batch_reduce == "program-mean":
        assert num_program_steps is not None, f"num_program_steps required for batch_reduce='{batch_reduce}'"
        assert valid_program_count is not None, "valid_program_count required for batch_reduce='program-mean'"
        valid = valid_program_count
    elif batch_reduce == "token-mean":
        valid = valid_token_count
    elif batch_reduce == "step-mean":
        valid = valid_batch_size
    _lib.require_device(loss_mat, "agg_loss")
    rows = _ops.rows_of(loss_mat, cu_seqlens)
    return _WeightedRowSum.apply(
        loss_mat, loss_mask, rows, token_reduce, batch_reduce,
        (per_row_token_count, num_program_tokens, num_program_steps, valid),
    )


def masked_mean(values: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """``(values*mask).sum() / max(mask.sum(), 1)`` (loss/utils.py:88-91)."""
    _lib.require_device(values, "masked_mean")
    flat = values.reshape(1, -1)
    return agg_loss(flat, mask.reshape(1, -1), token_reduce="mean", batch_reduce="step-mean", valid_batch_size=1)
