"""Oracle: GRPO advantage, group statistics and the zero-advantage filter (CPU torch).

Restates axon/utils/rl/advantage.py:106-150 (``group_mean_std``),
axon/trainer/algos/advantages/advantage.py:78-109 (``grpo_advantage_fn``),
axon/trainer/algos/advantages/__init__.py:73-74 (optional clamp) and
axon/utils/rl/utils.py:23-60 (``filter_zero_advantage_samples``).  Group labels are
already integer indices here; label ranking is host logic tested on its own.
"""

from __future__ import annotations

import torch


def group_mean_std(scores, gidx, eps=1e-6):
    """count/s1/s2 by index_add; var = (s2 - s1^2/n)/(n-1); std = sqrt(max(var, eps));
    groups of <= 1 -> (0, 1)."""
    scores = scores.reshape(-1).float()
    gidx = gidx.reshape(-1).long()
    if scores.numel() != gidx.numel():
        raise ValueError("scores and gidx length mismatch")
    if gidx.numel() == 0:
        e = torch.empty(0)
        return e, e, e
    g = int(gidx.max()) + 1
    n = torch.zeros(g).index_add_(0, gidx, torch.ones_like(scores))
    s1 = torch.zeros(g).index_add_(0, gidx, scores)
    s2 = torch.zeros(g).index_add_(0, gidx, scores * scores)
    nn = n.clamp_min(1.0)
    mean = s1 / nn
    var = (s2 - s1 * s1 / nn) / (n - 1.0).clamp_min(1.0)
    std = torch.sqrt(var.clamp(min=eps))
    single = n <= 1.0
    mean = torch.where(single, torch.zeros_like(mean), mean)
    std = torch.where(single, torch.ones_like(std), std)
    return mean, std, n


def grpo_advantage(token_level_rewards, response_mask, gidx, eps=1e-6, norm_adv_by_std=True, clip=False):
    scores = token_level_rewards.sum(-1)
    mean, std, n = group_mean_std(scores, gidx, eps)
    a = scores - mean[gidx]
    if norm_adv_by_std:
        a = a / (std[gidx] + eps)
    a = a * (n[gidx] > 1)
    adv = a.unsqueeze(-1) * response_mask
    return torch.clamp(adv, -1, 1) if clip else adv


def rloo_advantage(token_level_rewards, response_mask, gidx):
    """advantages/advantage.py:112-146: leave-one-out baseline (n*s_i - S_g)/(n-1); singleton groups 0."""
    scores = token_level_rewards.sum(-1)
    c = torch.bincount(gidx)[gidx].to(scores.dtype)
    gsum = torch.bincount(gidx, weights=scores)[gidx]
    a = ((c * scores - gsum) / (c - 1).clamp_min(1)) * (c > 1)
    return a.unsqueeze(-1) * response_mask


def gpg_advantage(token_level_rewards, response_mask, gidx, f_norm=1.0):
    """advantages/advantage.py:336-371: alpha * (score - group mean) / f_norm, alpha = rows / nonzero scores."""
    scores = token_level_rewards.sum(-1)
    alpha = scores.shape[0] / torch.count_nonzero(scores).clamp(min=1).to(scores.dtype)
    c = torch.bincount(gidx)[gidx].to(scores.dtype)
    gsum = torch.bincount(gidx, weights=scores)[gidx]
    gmean = torch.where(c > 1, gsum / c, torch.zeros_like(gsum))
    return (alpha * (scores - gmean) / f_norm).unsqueeze(-1) * response_mask


def zero_advantage_keep_rows(advantages, eps=1e-5):
    """Row indices with any |advantage| > eps (strict), as a python list."""
    return torch.nonzero((advantages.abs() > eps).any(dim=1)).squeeze(1).tolist()


def mini_batch_counts(response_mask, program_uids=None):
    """axon/driver/driver_utils.py:436-474 (``process_mini_batch``): rows with a valid token, valid
    tokens, tokens per row, distinct program uids among valid rows (None without uids)."""
    per_row = response_mask.sum(dim=-1).to(torch.long)
    valid = response_mask.sum(dim=-1) > 0
    programs = None
    if program_uids is not None:
        programs = len({program_uids[i] for i in valid.nonzero(as_tuple=True)[0].tolist()})
    return int(valid.sum().item()), int(response_mask.sum().item()), per_row, programs
