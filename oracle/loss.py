"""Oracle: loss aggregation and the PPO / GSPO clipped losses in plain torch (CPU, autograd).

Restates axon/trainer/algos/loss/utils.py:88-251 (``masked_mean``, ``agg_loss``) and
axon/trainer/algos/loss/loss.py:47-180 (``ppo_loss_fn``, ``gspo_loss_fn``; further down ``clip_cov_loss_fn``
:198-280 and ``kl_cov_loss_fn`` :283-352) on plain
tensors (no DataProto), keeping the order of operations so autograd reproduces the
reference's gradient conventions (clamp passes gradient at the bound, maximum/min
split ties evenly).
"""

from __future__ import annotations

import torch

TOKEN_REDUCE = ("sum", "mean", "mean-norm", "mean-program")
BATCH_REDUCE = ("token-mean", "step-mean", "program-mean")


def masked_mean(values, mask):
    """utils.py:88-91."""
    mask = mask.to(values.dtype)
    return (values * mask).sum() / mask.sum().clamp_min(1.0)


def _scalar_count(val, like):
    """utils.py:224-229: element [0] of a count tensor, clamped to >= 1."""
    t = torch.as_tensor(val, dtype=like.dtype)
    if t.dim() > 0:
        t = t[0]
    return t.clamp(min=1)


def agg_loss(loss_mat, loss_mask, *, token_reduce="sum", batch_reduce="token-mean", num_program_tokens=None,
             num_program_steps=None, valid_token_count=None, valid_batch_size=None, valid_program_count=None,
             per_row_token_count=None):
    """utils.py:120-251: (B,T) -> (B,) by token_reduce, then -> scalar by batch_reduce."""
    if token_reduce not in TOKEN_REDUCE:
        raise ValueError(f"Invalid token_reduce: {token_reduce!r}")
    if batch_reduce not in BATCH_REDUCE:
        raise ValueError(f"Invalid batch_reduce: {batch_reduce!r}")
    rows = (loss_mat * loss_mask).sum(-1)
    if token_reduce == "mean":
        d = per_row_token_count if per_row_token_count is not None else loss_mask.sum(-1)
        rows = rows / d.clamp(min=1)
    elif token_reduce == "mean-norm":
        rows = rows / loss_mask.shape[-1]
    elif token_reduce == "mean-program":
        assert num_program_tokens is not None, "num_program_tokens required"
        rows = rows / num_program_tokens.clamp(min=1)
    if batch_reduce == "program-mean":
        assert num_program_steps is not None, "num_program_steps required"
        rows = rows / num_program_steps.clamp(min=1)
    total = rows.sum()
    if batch_reduce == "token-mean":
        d = valid_token_count if valid_token_count is not None else loss_mask.sum().clamp_min(1.0)
        return total / _scalar_count(d, total)
    if batch_reduce == "step-mean":
        if valid_batch_size is not None:
            return total / _scalar_count(valid_batch_size, total)
        return total / (loss_mask.sum(-1) > 0).float().sum().clamp(min=1)
    assert valid_program_count is not None, "valid_program_count required for batch_reduce='program-mean'"
    return total / _scalar_count(valid_program_count, total)


def ppo_loss(log_prob, old_log_prob, advantages, response_mask, *, clip_ratio=0.2, clip_ratio_low=None,
             clip_ratio_high=None, clip_ratio_c=3.0, sampler_is_weights=None, token_reduce="sum",
             batch_reduce="token-mean", **agg_kwargs):
    """loss.py:47-111.  Returns (loss, {pg_clipfrac, ppo_kl, pg_clipfrac_lower})."""
    lo = clip_ratio if clip_ratio_low is None else clip_ratio_low
    hi = clip_ratio if clip_ratio_high is None else clip_ratio_high
    assert clip_ratio_c > 1.0, f"clip_ratio_c must be > 1.0, got {clip_ratio_c}"
    nak = torch.clamp(log_prob - old_log_prob, min=-20.0, max=20.0)
    ratio = torch.exp(nak)
    kl = masked_mean(-nak, response_mask)
    l1 = -advantages * ratio
    l2 = -advantages * torch.clamp(ratio, 1 - lo, 1 + hi)
    c1 = torch.maximum(l1, l2)
    clipfrac = masked_mean(torch.gt(l2, l1).float(), response_mask)
    l3 = -advantages * clip_ratio_c
    c2 = torch.min(l3, c1)
    clipfrac_lower = masked_mean(torch.gt(c1, l3) * (advantages < 0).float(), response_mask)
    per_tok = torch.where(advantages < 0, c2, c1)
    if sampler_is_weights is not None:
        per_tok = per_tok * sampler_is_weights
    loss = agg_loss(per_tok, response_mask, token_reduce=token_reduce, batch_reduce=batch_reduce, **agg_kwargs)
    return loss, {"pg_clipfrac": clipfrac.item(), "ppo_kl": kl.item(), "pg_clipfrac_lower": clipfrac_lower.item()}


def gspo_loss(log_prob, old_log_prob, advantages, response_mask, *, clip_ratio=0.2, clip_ratio_low=None,
              clip_ratio_high=None, sampler_is_weights=None, token_reduce="mean", batch_reduce="token-mean",
              **agg_kwargs):
    """loss.py:114-180: sequence-level geometric-mean ratio with a stop-gradient token term."""
    lo = clip_ratio if clip_ratio_low is None else clip_ratio_low
    hi = clip_ratio if clip_ratio_high is None else clip_ratio_high
    nak = log_prob - old_log_prob
    lens = response_mask.sum(-1).clamp(min=1)
    seq = (nak * response_mask).sum(-1) / lens
    log_s = log_prob - log_prob.detach() + seq.detach().unsqueeze(-1)
    s = torch.exp(torch.clamp(log_s, min=-20.0, max=20.0))
    l1 = -advantages * s
    l2 = -advantages * torch.clamp(s, 1 - lo, 1 + hi)
    per_tok = torch.maximum(l1, l2)
    if sampler_is_weights is not None:
        per_tok = per_tok * sampler_is_weights
    loss = agg_loss(per_tok, response_mask, token_reduce=token_reduce, batch_reduce=batch_reduce, **agg_kwargs)
    clipfrac = masked_mean(torch.gt(l2, l1).float(), response_mask)
    kl = masked_mean(-nak, response_mask)
    return loss, {"pg_clipfrac": clipfrac.item(), "ppo_kl": kl.item(), "pg_clipfrac_lower": 0.0}


def kl_penalty(logprob, ref_logprob, kl_penalty_type="low_var_kl"):
    """axon/utils/rl/kl.py:154-245.  "+" types: forward value of the base type, gradient of k2."""
    base = kl_penalty_type.rstrip("+")
    d = logprob - ref_logprob
    if base in ("kl", "k1"):
        fwd = d
    elif base == "abs":
        fwd = d.abs()
    elif base in ("mse", "k2"):
        fwd = 0.5 * d.square()
    elif base in ("low_var_kl", "k3"):
        k = torch.clamp(ref_logprob - logprob, min=-20, max=20)
        fwd = torch.clamp(torch.exp(k) - k - 1, min=-10, max=10)
    elif base == "full":
        raise NotImplementedError("Full KL divergence requires logits, not just log probs")
    else:
        raise NotImplementedError(f"Unknown KL penalty type: {kl_penalty_type}")
    if not kl_penalty_type.endswith("+") or kl_penalty_type in ("mse", "k2"):
        return fwd
    bwd = 0.5 * d.square()
    return bwd - bwd.detach() + fwd.detach()


def actor_loss(loss_fn, log_prob, entropy, old_log_prob, advantages, response_mask, *, loss_args, ref_log_prob=None,
               side_mask=None, dp_replicas=1, n_micro_batches=1, **agg_kwargs):
    """axon/models/fsdp_models.py:226-276: pg loss - entropy_coef * agg(entropy) + kl_coef * agg(kld), times
    dp_replicas.  ``side_mask``: the mask the side terms aggregate over (the one captured before the
    sampler correction hook); defaults to ``response_mask``."""
    tr = loss_args.get("token_reduce", "sum")
    br = loss_args.get("batch_reduce", "token-mean")
    clip = {k: v for k, v in loss_args.items() if k.startswith("clip")}
    loss, m = loss_fn(log_prob, old_log_prob, advantages, response_mask, token_reduce=tr, batch_reduce=br, **clip,
                      **agg_kwargs)
    metrics = dict(m)
    metrics["pg_loss"] = loss.item() * n_micro_batches
    sm = response_mask if side_mask is None else side_mask
    ent_agg = agg_loss(entropy, sm, token_reduce=tr, batch_reduce=br, **agg_kwargs)
    metrics["entropy"] = ent_agg.item() * n_micro_batches
    metrics["entropy_token_mean"] = agg_loss(entropy, sm, token_reduce="sum", batch_reduce="token-mean").item()
    if loss_args.get("entropy_coef", 0) != 0:
        loss = loss - ent_agg * loss_args["entropy_coef"]
    if loss_args.get("kl_coef", 0) != 0:
        kld = kl_penalty(log_prob, ref_log_prob, loss_args.get("kl_type", "low_var_kl"))
        kl_loss = agg_loss(kld, sm, token_reduce=tr, batch_reduce=br, **agg_kwargs)
        loss = loss + kl_loss * loss_args["kl_coef"]
        metrics["kl_loss"] = kl_loss.item() * n_micro_batches
        metrics["kl_coef"] = loss_args["kl_coef"]
    return loss * dp_replicas, metrics


def reinforce_loss(log_prob, old_log_prob, advantages, response_mask, *, sampler_is_weights=None, token_reduce="sum",
                   batch_reduce="token-mean", **agg_kwargs):
    """loss.py:471-512 (also GPG, :183-197).  Returns (loss, {ppo_kl})."""
    per_tok = -advantages * log_prob
    if sampler_is_weights is not None:
        per_tok = -advantages * log_prob * sampler_is_weights
    loss = agg_loss(per_tok, response_mask, token_reduce=token_reduce, batch_reduce=batch_reduce, **agg_kwargs)
    return loss, {"ppo_kl": masked_mean(-(log_prob - old_log_prob), response_mask).item()}


def cispo_loss(log_prob, old_log_prob, advantages, response_mask, *, clip_ratio=0.2, clip_ratio_low=None,
               clip_ratio_high=None, token_level_mask=False, token_reduce="sum", batch_reduce="token-mean",
               **agg_kwargs):
    """loss.py:411-468: the clipped importance weight is a constant, gradients flow through log_prob only."""
    lo = 1e10 if clip_ratio_low is None else clip_ratio_low
    hi = clip_ratio if clip_ratio_high is None else clip_ratio_high
    nak = torch.clamp(log_prob - old_log_prob, min=-20.0, max=20.0)
    ratio = torch.exp(nak)
    per_tok = -torch.clamp(ratio, 1 - lo, 1 + hi).detach() * advantages * log_prob
    if token_level_mask:
        drop = ((advantages > 0) & (ratio > 1 + hi)) | ((advantages < 0) & (ratio < 1 - lo))
        per_tok = per_tok * (~drop).float()
    loss = agg_loss(per_tok, response_mask, token_reduce=token_reduce, batch_reduce=batch_reduce, **agg_kwargs)
    clipfrac = masked_mean(((ratio > 1 + hi) | (ratio < 1 - lo)).float(), response_mask)
    return loss, {"pg_clipfrac": clipfrac.item(), "ppo_kl": masked_mean(-nak, response_mask).item()}


def geo_mean_loss(log_prob, old_log_prob, advantages, response_mask, *, clip_ratio=0.2, clip_ratio_low=None,
                  clip_ratio_high=None, sampler_is_weights=None, **_ignored):
    """loss.py:355-408 (GMPO): token-level clipping of the log-ratio in the direction of the advantage,
    geometric-mean ratio per sequence, mean over sequences that have tokens."""
    lo = clip_ratio if clip_ratio_low is None else clip_ratio_low
    hi = clip_ratio if clip_ratio_high is None else clip_ratio_high
    nak = log_prob - old_log_prob
    sgn = torch.sign(advantages)
    nak_c = torch.clamp(nak, -lo, hi)
    nak_min = sgn * torch.min(sgn * nak, sgn * nak_c)
    cnt = response_mask.sum(dim=-1)
    ratio = torch.exp((nak_min * response_mask).sum(dim=-1) / (cnt + 1e-8))
    adv = (advantages * response_mask).sum(dim=-1) / (cnt + 1e-8)
    per_row = -adv * ratio
    if sampler_is_weights is not None:
        per_row = per_row * torch.exp((torch.log(sampler_is_weights + 1e-10) * response_mask).sum(dim=-1) / (cnt + 1e-8))
    valid = cnt > 0
    loss = per_row[valid].mean() if valid.any() else per_row.mean()
    clipped = torch.ne(nak, nak_c)
    return loss, {"pg_clipfrac": masked_mean((clipped * (advantages > 0)).float(), response_mask).item(),
                  "ppo_kl": masked_mean(-nak, response_mask).item(),
                  "pg_clipfrac_lower": masked_mean((clipped * (advantages < 0)).float(), response_mask).item()}


def kl_cov_loss(log_prob, old_log_prob, advantages, response_mask, *, kl_cov_ratio=0.0002, ppo_kl_coef=1.0,
                sampler_is_weights=None, token_reduce="sum", batch_reduce="token-mean", **agg_kwargs):
    """loss.py:283-352.  ``(loss, metrics, selected)``; selected = flat indices that carry the KL term."""
    nak = torch.clamp(log_prob - old_log_prob, -20.0, 20.0)
    abs_kl = nak.abs()
    ratio = torch.exp(nak)
    pg1 = -advantages * ratio
    pg_kl = -advantages * ratio + ppo_kl_coef * abs_kl
    losses = pg1.clone()
    valid = response_mask > 0
    valid_idx = torch.nonzero(valid.reshape(-1), as_tuple=True)[0]
    v_adv = advantages[valid].detach().reshape(-1)
    v_lp = log_prob[valid].detach().reshape(-1)
    picked = torch.empty(0, dtype=torch.long)
    if min(kl_cov_ratio, len(v_adv)) != 0 and len(v_adv) > 0:
        cov = (v_adv - v_adv.mean()) * (v_lp - v_lp.mean())
        k = max(1, int(len(cov) * kl_cov_ratio))
        picked = valid_idx[torch.topk(cov, k, largest=True).indices]
        t = advantages.shape[1]
        losses[picked // t, picked % t] = pg_kl[picked // t, picked % t]
    if sampler_is_weights is not None:
        losses = losses * sampler_is_weights
    loss = agg_loss(losses, response_mask, token_reduce=token_reduce, batch_reduce=batch_reduce, **agg_kwargs)
    return loss, {"ppo_kl": float(masked_mean(abs_kl, response_mask).detach())}, picked


def clip_cov_candidates(log_prob, old_log_prob, advantages, response_mask, *, clip_ratio=0.2, clip_ratio_low=None,
                        clip_ratio_high=None, clip_cov_ratio=0.0002, clip_cov_lb=1.0, clip_cov_ub=5.0):
    """loss.py:226-252: ``(candidate mask, clip_num)``: the tokens the random pick draws from and how many it may
    take."""
    lo = clip_ratio if clip_ratio_low is None else clip_ratio_low
    hi = clip_ratio if clip_ratio_high is None else clip_ratio_high
    ratio = torch.exp(torch.clamp(log_prob - old_log_prob, -20.0, 20.0)).detach()
    pg1 = -advantages * ratio
    pg2 = -advantages * torch.clamp(ratio, 1 - lo, 1 + hi)
    clip_by_origin = (pg2 > pg1) & (response_mask > 0)
    cov = (advantages - masked_mean(advantages, response_mask)) * (
        log_prob.detach() - masked_mean(log_prob.detach(), response_mask))
    cov = cov.clone()
    cov[response_mask == 0] = -torch.inf
    cov[clip_by_origin] = -torch.inf
    clip_num = max(int(clip_cov_ratio * response_mask.sum().item()), 1)
    return (cov < clip_cov_ub) & (cov > clip_cov_lb) & (response_mask > 0), clip_num


def clip_cov_loss(log_prob, old_log_prob, advantages, response_mask, *, selected=None, clip_ratio=0.2,
                  clip_ratio_low=None, clip_ratio_high=None, clip_cov_ratio=0.0002, clip_cov_lb=1.0, clip_cov_ub=5.0,
                  sampler_is_weights=None, token_reduce="mean", batch_reduce="token-mean", **agg_kwargs):
    """loss.py:198-280.  The reference draws the zeroed tokens with ``torch.randperm``; ``selected`` (a boolean
    mask of the drawn tokens) replaces that draw so that two implementations can be compared on one draw."""
    lo = clip_ratio if clip_ratio_low is None else clip_ratio_low
    hi = clip_ratio if clip_ratio_high is None else clip_ratio_high
    nak = torch.clamp(log_prob - old_log_prob, -20.0, 20.0)
    ratio = torch.exp(nak)
    pg1 = -advantages * ratio
    pg2 = -advantages * torch.clamp(ratio, 1 - lo, 1 + hi)
    if selected is None:
        cand, clip_num = clip_cov_candidates(log_prob, old_log_prob, advantages, response_mask, clip_ratio=clip_ratio,
                                             clip_ratio_low=clip_ratio_low, clip_ratio_high=clip_ratio_high,
                                             clip_cov_ratio=clip_cov_ratio, clip_cov_lb=clip_cov_lb,
                                             clip_cov_ub=clip_cov_ub)
        idx = torch.nonzero(cand.reshape(-1)).flatten()
        idx = idx[torch.randperm(len(idx))[: min(clip_num, len(idx))]]
        selected = torch.zeros(cand.numel(), dtype=torch.bool)
        selected[idx] = True
        selected = selected.view_as(cand)
    corr = torch.ones_like(advantages)
    corr[selected] = 0
    losses = torch.maximum(pg1, pg2) * corr
    if sampler_is_weights is not None:
        losses = losses * sampler_is_weights
    loss = agg_loss(losses, response_mask, token_reduce=token_reduce, batch_reduce=batch_reduce, **agg_kwargs)
    metrics = {"pg_clipfrac": float(masked_mean((corr == 0).float(), response_mask)),
               "ppo_kl": float(masked_mean(-nak, response_mask).detach())}
    return loss, metrics


def apply_kl_penalty(token_level_scores, old_log_probs, ref_log_prob, response_mask, beta, kl_penalty_type="kl"):
    """axon/utils/rl/kl.py:276-322 without the controller: ``(token_level_rewards, current_kl)``."""
    kld = kl_penalty(old_log_probs, ref_log_prob, kl_penalty_type) * response_mask
    rewards = token_level_scores - beta * kld
    lengths = response_mask.sum(dim=-1).clamp(min=1)
    return rewards, float((kld.sum(dim=-1) / lengths).mean())
