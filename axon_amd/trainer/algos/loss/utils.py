"""Loss aggregation helpers on the HIP path.

``agg_loss`` keeps the signature of axon/trainer/algos/loss/utils.py:120-187
(two-axis reduction: token_reduce x batch_reduce) and ``masked_mean`` that of
:88-91.  Both are differentiable with respect to their first argument.  The
reductions run in libaxon_amd.so: one row-statistics pass, one single-workgroup
pass that folds every denominator into a per-row multiplier, and one
elementwise pass that produces the scalar and its gradient.
"""

from __future__ import annotations

import torch

from axon_amd import _lib, _ops
from axon_amd.trainer.algos.constants import VALID_BATCH_REDUCE, VALID_TOKEN_REDUCE

__all__ = ["agg_loss", "masked_mean"]


class _WeightedRowSum(torch.autograd.Function):
    """sum_t loss[t] * mask[t] * row_scale[row(t)] with gradient mask*row_scale."""

    @staticmethod
    def forward(ctx, loss_mat, mask, rows, tr, br, extras):
        lib = _lib.load()
        dev = loss_mat.device
        x = _ops.f32(loss_mat)
        mk, kind = _ops.mask_arg(mask)
        cnt, _, _ = _ops.row_stats(x, None, mk, rows, want_sum=False)
        scale = torch.empty(rows.n_rows, device=dev, dtype=torch.float32)
        prtc, npt, nps, valid = (_ops._i64_dev(e, dev) for e in extras)
        _lib.check(
            lib.axon_loss_row_scale(_lib.ptr(cnt), None, rows.n_rows, rows.uniform_len, tr, br,
                                    _lib.ptr(prtc if tr == 1 else None), _lib.ptr(npt if tr == 3 else None),
                                    _lib.ptr(nps if br == 2 else None), _lib.ptr(valid), _lib.ptr(scale), None,
                                    _lib.stream_ptr()),
            "axon_loss_row_scale",
        )
        weights = _ops.row_broadcast_mask(scale, mk, rows)  # d out / d loss[t]
        ssum = torch.zeros(1, device=dev, dtype=torch.float32)
        # total = sum_t x[t] * weights[t]: a single row over all slots
        one_row = _ops.Rows(1, rows.n_slots, rows.n_slots, None, rows.shape)
        _lib.check(
            lib.axon_row_stats(_lib.ptr(x), None, _lib.ptr(weights), _lib.MASK_F32, None, 1, one_row.n_slots,
                               one_row.uniform_len, 0, 0.0, None, _lib.ptr(ssum), None, _lib.stream_ptr()),
            "axon_row_stats",
        )
        ctx.save_for_backward(weights)
        ctx.in_dtype = loss_mat.dtype
        return ssum[0]

    @staticmethod
    def backward(ctx, g):
        (weights,) = ctx.saved_tensors
        return (weights * g).to(ctx.in_dtype), None, None, None, None, None


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
        loss_mat, loss_mask, rows, _ops.TOKEN_REDUCE[token_reduce], _ops.BATCH_REDUCE[batch_reduce],
        (per_row_token_count, num_program_tokens, num_program_steps, valid),
    )


def masked_mean(values: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """``(values*mask).sum() / max(mask.sum(), 1)`` (loss/utils.py:88-91)."""
    _lib.require_device(values, "masked_mean")
    flat = values.reshape(1, -1)
    return agg_loss(flat, mask.reshape(1, -1), token_reduce="mean", batch_reduce="step-mean", valid_batch_size=1)
