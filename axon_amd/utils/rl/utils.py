"""Driver-side helpers of axon/utils/rl/utils.py: ``filter_zero_advantage_samples`` (DAPO dynamic sampling,
:23-60), ``compute_reward_statistics`` (:63-89) and ``compute_pass_metrics`` (:92-123).  Each forms its per-row
quantity with one ragged row-reduction launch and reads it back once; the grouping by uid is host logic."""

from __future__ import annotations

import numpy as np
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


def _row_scores(batch) -> np.ndarray:
    """Sum of ``token_level_scores`` per row, on the host (one launch, one readback)."""
    scores = batch.batch["token_level_scores"]
    if not scores.is_cuda:
        if not torch.cuda.is_available():
            _ops.require_device(scores, "token_level_scores")
        scores = scores.cuda()
    cu = batch.meta_info.get("cu_seqlens", None) if batch.meta_info else None
    rows = _ops.rows_of(scores, cu)
    _, sums, _ = _ops.row_stats(scores, None, None, rows, want_cnt=False)
    return sums.cpu().numpy()


def compute_reward_statistics(batch):
    """Mean / max / min of the per-program reward over the rows that are not padding and are the last step of
    their program (utils.py:63-89)."""
    sums = _row_scores(batch)
    n = sums.shape[0]
    is_padding = np.asarray(batch.non_tensor_batch.get("is_padding", np.zeros(n, dtype=bool)), dtype=bool)
    is_last = np.asarray(batch.non_tensor_batch.get("is_last_step", np.ones(n, dtype=bool)), dtype=bool)
    valid = ~is_padding & is_last
    if not valid.any():
        return {"reward_mean": 0.0, "reward_max": 0.0, "reward_min": 0.0}
    r = sums[valid]
    return {"batch/reward/mean": float(r.mean(dtype=np.float32)), "batch/reward/max": float(r.max()),
            "batch/reward/min": float(r.min())}


def compute_pass_metrics(batch):
    """``(metrics, uid -> pass rate)`` (utils.py:92-123): a uid solves none / all / part of its samples
    according to their summed scores (pass: >= 1, fail: <= 0); only last steps count when ``is_last_step`` is
    present."""
    sums = _row_scores(batch)
    uids = np.asarray(batch.non_tensor_batch["uid"])
    if "is_last_step" in batch.non_tensor_batch:
        keep = np.asarray(batch.non_tensor_batch["is_last_step"], dtype=bool)
        sums, uids = sums[keep], uids[keep]
    pass_rates, none, full = {}, 0, 0
    for uid in np.unique(uids):
        r = sums[uids == uid]
        pass_rates[uid] = float((r >= 1).astype(np.float32).mean())
        if (r <= 0).all():
            none += 1
        elif (r >= 1).all():
            full += 1
    return {"batch/solve/none": none, "batch/solve/all": full,
            "batch/solve/partial": len(pass_rates) - none - full}, pass_rates
