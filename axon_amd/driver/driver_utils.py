"""``process_mini_batch`` — the loss denominators of a mini-batch (axon/driver/driver_utils.py:436-474).

``agg_loss`` divides by mini-batch-wide counts that the driver writes into the batch before the
micro-batches are cut.  The per-row token counts come from one ragged row-sum launch over the response
mask; the two scalar counts are read back together.
"""

from __future__ import annotations

import torch

from axon_amd import _ops


def process_mini_batch(mini_batch) -> None:
    """Write ``valid_batch_size`` (rows with at least one valid token), ``valid_token_count``,
    ``per_row_token_count`` and, when ``program_uids`` is present, ``valid_program_count`` (distinct
    program uids among valid rows) into ``mini_batch.batch``, each count repeated once per row as int64.
    A batch without ``response_mask`` is left untouched."""
    mask = mini_batch.batch.get("response_mask", None)
    if mask is None:
        return
    home = mask.device
    if not mask.is_cuda:
        if not torch.cuda.is_available():
            _ops.require_device(mask, "process_mini_batch")
        mask = mask.cuda()
    n = len(mini_batch)
    cu = mini_batch.meta_info.get("cu_seqlens", None) if mini_batch.meta_info else None
    values = mask if mask.dtype == torch.float32 else mask.to(torch.float32)
    rows = _ops.rows_of(values, cu)
    _, per_row, _ = _ops.row_stats(values, None, None, rows, want_cnt=False)
    valid = per_row > 0
    n_valid, n_tokens = torch.stack([valid.sum(), per_row.sum(dtype=torch.float64).to(torch.int64)]).tolist()

    mini_batch.batch["valid_batch_size"] = torch.full((n,), int(n_valid), dtype=torch.long, device=home)
    mini_batch.batch["valid_token_count"] = torch.full((n,), int(n_tokens), dtype=torch.long, device=home)
    mini_batch.batch["per_row_token_count"] = per_row.to(device=home, dtype=torch.long)

    program_uids = mini_batch.non_tensor_batch.get("program_uids", None) if mini_batch.non_tensor_batch else None
    if program_uids is not None:
        valid_idx = torch.nonzero(valid, as_tuple=True)[0].tolist()
        count = len({program_uids[i] for i in valid_idx})
        mini_batch.batch["valid_program_count"] = torch.full((n,), count, dtype=torch.long, device=home)
