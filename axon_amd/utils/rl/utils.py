"""``filter_zero_advantage_samples`` — DAPO dynamic sampling (axon/utils/rl/utils.py:23-60)."""

from __future__ import annotations

import torch

from axon_amd import _ops


def filter_zero_advantage_samples(batch):
    """Keep rows with any ``|advantage| > 1e-5``; if none qualifies keep the first uid's group."""
    assert "advantages" in batch.batch
    adv = batch.batch["advantages"]
    if not adv.is_cuda:
        if not torch.cuda.is_available():
            _ops.require_device(adv, "filter_zero_advantage_samples")
        adv = adv.cuda()
    cu = batch.meta_info.get("cu_seqlens", None) if batch.meta_info else None
    rows = _ops.rows_of(adv, cu)
    _, _, flag = _ops.row_stats(adv, None, None, rows, flag_mode=2, threshold=1e-5, want_cnt=False, want_sum=False)
    keep = torch.nonzero(flag, as_tuple=False).squeeze(1).tolist()
    total = len(batch)
    if total - len(keep) > 0:
        print(f"Filtered {total - len(keep)}/{total} samples with zero advantage")
    if keep:
        return batch.select_idxs(keep)
    print("WARNING: All groups have zero advantage! Keeping one group.")
    uids = batch.non_tensor_batch.get("uid", None)
    if uids is None:
        return batch
    first = uids[0]
    return batch.select_idxs([i for i, u in enumerate(uids) if u == first])
