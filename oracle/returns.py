"""Oracle: the return-based and remaining group-based advantage estimators, and the clipped value loss
(CPU torch).  TEST INFRASTRUCTURE ONLY: nothing outside tests/, the smoke check and the benchmark's CPU leg
may import this module.

Restates, from axon/trainer/algos/advantages/advantage.py:
  ``gae_advantage_fn`` :40-75, ``reinforce_plus_plus_advantage_fn`` :149-176,
  ``reinforce_plus_plus_baseline_advantage_fn`` :179-217, ``remax_advantage_fn`` :220-240,
  ``opo_advantage_fn`` :243-280, ``grpo_passk_advantage_fn`` :283-333, ``_chunked_gae_core`` /
  ``chunked_gae_advantage_fn`` :374-540, ``kimi_k1_5_advantage_fn`` :543-626, ``identity_advantage_fn`` :629-645;
from axon/utils/rl/advantage.py: ``masked_mean`` :153-157, ``masked_var`` :160-170, ``masked_whiten`` :173-190;
from axon/trainer/algos/loss/loss.py: ``value_loss_fn`` :547-591 with ``clip_by_value``
(axon/trainer/algos/loss/utils.py:94-101).

Time recurrences run as plain loops from the last token to the first, in fp32, in the reference's operation
order.  Group labels are integer indices already.
"""

from __future__ import annotations

import torch

from oracle.advantage import group_mean_std
from oracle.loss import agg_loss, masked_mean


def masked_var(values, mask, bessel_correction=True):
    """Mean of squared deviations over the mask, times n/(n-1) when n > 1 (rl/advantage.py:161-170)."""
    mask = mask.to(values.dtype)
    n = mask.sum()
    mean = (values * mask).sum() / n.clamp_min(1.0)
    var = ((values - mean) ** 2 * mask).sum() / n.clamp_min(1.0)
    if bessel_correction and n > 1:
        var = var * n / (n - 1)
    return var


def masked_whiten(values, mask, shift_mean=True):
    """rl/advantage.py:173-190."""
    mean, var = masked_mean(values, mask), masked_var(values, mask)
    out = (values - mean) * torch.rsqrt(var + 1e-8)
    return out if shift_mean else out + mean


def gae_raw(rewards, values, mask, gamma, lam):
    """The time loop of advantage.py:57-73 without the whitening: ``(advantages, returns)``."""
    rewards, values, mask = rewards.float(), values.float(), mask.float()
    b, t_len = rewards.shape
    nextv = torch.zeros(b)
    last = torch.zeros(b)
    adv = torch.zeros(b, t_len)
    for t in range(t_len - 1, -1, -1):
        delta = rewards[:, t] + gamma * nextv - values[:, t]
        cand = delta + gamma * lam * last
        m = mask[:, t]
        nextv = values[:, t] * m + (1 - m) * nextv
        last = cand * m + (1 - m) * last
        adv[:, t] = last
    return adv, adv + values


def gae_advantage(rewards, values, mask, gamma=0.99, lam=0.95):
    adv, ret = gae_raw(rewards, values, mask, gamma, lam)
    return masked_whiten(adv, mask.float()), ret


def chunked_gae_advantage(rewards, values, mask, gamma=0.99, lam=0.95):
    """advantage.py:480-540.  The response tokens of a row are gathered, S[i] = delta[i] + gamma*lam*S[i+1] with
    delta[i] = r[i] + gamma*V[i+1] - V[i] and V past the end = 0 runs over the gathered tokens (:406-416; the
    chunk matrices of :428-469 evaluate this same recurrence), and the results are scattered back, zero
    elsewhere, before the whitening."""
    rewards, values, mask = rewards.float(), values.float(), mask.float()
    b, t_len = rewards.shape
    adv = torch.zeros(b, t_len)
    ret = torch.zeros(b, t_len)
    if float((mask > 0).sum(1).max()) == 0:
        return adv, adv
    w = gamma * lam
    for r in range(b):
        idx = torch.where(mask[r] > 0)[0]
        s, nextv = 0.0, 0.0
        for i in reversed(idx.tolist()):
            delta = float(rewards[r, i]) + gamma * nextv - float(values[r, i])
            s = delta + w * s
            nextv = float(values[r, i])
            adv[r, i] = s
            ret[r, i] = s + float(values[r, i])
    return masked_whiten(adv, mask), ret


def reinforce_plus_plus_raw(rewards, mask, gamma):
    rewards, mask = rewards.float(), mask.float()
    b, t_len = rewards.shape
    ret = torch.zeros(b, t_len)
    run = torch.zeros(b)
    for t in range(t_len - 1, -1, -1):
        run = rewards[:, t] + gamma * run
        ret[:, t] = run
        run = run * mask[:, t]  # reset after the end of the response
    return ret


def reinforce_plus_plus_advantage(rewards, mask, gamma=1.0):
    ret = reinforce_plus_plus_raw(rewards, mask, gamma)
    mask = mask.float()
    return masked_whiten(ret, mask) * mask, ret


def _group_count_sum(values, gidx):
    c = torch.bincount(gidx)[gidx].to(values.dtype)
    s = torch.bincount(gidx, weights=values)[gidx].to(values.dtype)
    return c, s


def reinforce_plus_plus_baseline_advantage(rewards, mask, gidx):
    rewards, mask = rewards.float(), mask.float()
    scores = rewards.sum(-1)
    c, s = _group_count_sum(scores, gidx)
    base = torch.where(c > 1, s / c.clamp_min(1), torch.zeros_like(scores))
    spread = (scores - base).unsqueeze(-1) * mask
    return masked_whiten(spread, mask) * mask


def remax_advantage(rewards, mask, baselines):
    rewards, mask = rewards.float(), mask.float()
    ret = (rewards * mask).flip(-1).cumsum(-1).flip(-1)
    return ret - baselines.float().unsqueeze(-1) * mask, ret


def opo_advantage(rewards, mask, gidx):
    rewards, mask = rewards.float(), mask.float()
    lens = mask.sum(-1)
    scores = rewards.sum(-1)
    c, wsum = _group_count_sum(lens * scores, gidx)
    _, lsum = _group_count_sum(lens, gidx)
    base = torch.where(c > 1, wsum / lsum.clamp_min(1), torch.zeros_like(scores))
    return (scores - base).unsqueeze(-1) * mask


def grpo_passk_advantage(rewards, mask, gidx, eps=1e-6, norm_adv_by_std=True):
    rewards, mask = rewards.float(), mask.float()
    scores = rewards.sum(-1)
    adv = torch.zeros_like(scores)
    for g in torch.unique(gidx).tolist():
        rows = torch.where(gidx == g)[0]
        if rows.numel() < 2:
            raise ValueError(f"Pass@k requires at least 2 samples per group. Got {rows.numel()} for group {g}.")
        top, where = torch.topk(scores[rows], 2)
        a = top[0] - top[1]
        if norm_adv_by_std:
            a = a / (torch.std(scores[rows]) + eps)
        adv[rows[where[0]]] = a
    return adv.unsqueeze(-1) * mask


def kimi_length_coef(target, warmup_steps, ramp_steps, global_step):
    """The schedule of advantage.py:579-584."""
    if global_step < warmup_steps:
        return 0.0
    if ramp_steps > 0 and global_step < warmup_steps + ramp_steps:
        return target * (global_step - warmup_steps) / ramp_steps
    return target


def kimi_k1_5_advantage(rewards, mask, gidx, *, length_coef=0.0, correct_threshold=1.0, eps=1e-6,
                        norm_adv_by_std=True):
    rewards, mask = rewards.float(), mask.float()
    scores = rewards.sum(-1)
    lens = mask.sum(-1)
    shaped = scores
    if length_coef > 0.0 and gidx.numel() > 0:
        n_groups = int(gidx.max()) + 1
        lo = torch.full((n_groups,), float("inf")).scatter_reduce_(0, gidx, lens, reduce="amin", include_self=False)
        hi = torch.full((n_groups,), float("-inf")).scatter_reduce_(0, gidx, lens, reduce="amax", include_self=False)
        spread = hi[gidx] - lo[gidx]
        lam = length_coef * (0.5 - (lens - lo[gidx]) / spread.clamp_min(1.0))
        bonus = torch.where(scores >= correct_threshold, lam, torch.minimum(lam, torch.zeros_like(lam)))
        shaped = scores + bonus * (spread > 0).float()
    mean, std, n = group_mean_std(shaped, gidx, eps)
    a = shaped - mean[gidx]
    if norm_adv_by_std:
        a = a / (std[gidx] + eps)
    a = a * (n[gidx] > 1)
    return a.unsqueeze(-1) * mask


def identity_advantage(rewards, mask):
    return rewards.float() * mask.float()


def value_loss(vpreds, values, returns, response_mask, *, cliprange_value=0.5, token_reduce="sum",
               batch_reduce="token-mean", **agg_kwargs):
    """``(loss, metrics)`` of loss.py:547-591; ``vpreds`` may require grad."""
    clipped = torch.maximum(torch.minimum(vpreds, values + cliprange_value), values - cliprange_value)
    l1 = (vpreds - returns) ** 2
    l2 = (clipped - returns) ** 2
    loss = 0.5 * agg_loss(torch.max(l1, l2), response_mask, token_reduce=token_reduce, batch_reduce=batch_reduce,
                          **agg_kwargs)
    metrics = {
        "vf_loss": float(loss.detach()),
        "vf_clipfrac": float(masked_mean(torch.gt(l2, l1).float(), response_mask)),
        "vpred_mean": float(masked_mean(vpreds.detach(), response_mask)),
    }
    return loss, metrics
