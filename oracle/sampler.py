"""Oracle: sampler–trainer correction in plain torch (CPU).

Restates axon/utils/rl/sampler.py:35-103 (rejection mask), :181-256 (truncated IS
weights), :334-446 (unified interface incl. the per-token veto) and the two masked
reductions of axon/utils/torch/ops.py:123-145 it relies on.  Returns tensors instead of
a DataProto.  ``weight_metrics`` restates the diagnostics of :106-173 / :259-326,
``offpolicy_metrics`` those of :454-518, ``mismatch_stats`` / ``aggregate_mismatch`` the
sufficient statistics of axon/utils/metrics/trainer_sampler_mismatch_metrics.py:36-146.
"""

from __future__ import annotations

import torch

SAFETY_BOUND = 20.0


def masked_sum(values, mask, axis=None):
    """ops.py:123-128: values outside the mask are zeroed before the multiply."""
    return (torch.where(mask.bool(), values, 0.0) * mask).sum(axis=axis)


def masked_mean(values, mask, axis=None):
    """ops.py:131-145: denominator is mask.sum + 1e-8."""
    return masked_sum(values, mask, axis) / (mask.sum(axis=axis) + 1e-8)


def _level_ratio(log_ratio, mask, level):
    if level == "token":
        lr = log_ratio
    elif level == "sequence":
        lr = masked_sum(log_ratio, mask, axis=-1).unsqueeze(-1)
    elif level == "geometric":
        lr = masked_mean(log_ratio, mask, axis=-1).unsqueeze(-1)
    else:
        raise ValueError(level)
    return torch.exp(torch.clamp(lr, min=-SAFETY_BOUND, max=SAFETY_BOUND)).expand_as(log_ratio)


def is_weights(log_ratio, mask, level="token", threshold=2.0):
    """sampler.py:206-231: exp(clamp) * mask, then clamp(max=threshold).  Returns (weights, untruncated)."""
    if level not in ("token", "sequence"):
        raise ValueError(f"Invalid sampler_is: {level}")
    if threshold <= 0:
        raise ValueError("sampler_is_threshold must be positive")
    raw = _level_ratio(log_ratio, mask, level) * mask
    return raw.clamp(max=threshold), raw


def rejection_mask(log_ratio, mask, level="token", upper=None, lower=None):
    """sampler.py:63-83,102: keep iff lower <= ratio <= upper; lower defaults to 1/upper."""
    if level not in ("token", "sequence", "geometric"):
        raise ValueError(f"Invalid sampler_rs: {level}")
    if upper is None:
        raise ValueError("sampler_rs_threshold must be provided")
    lower = 1.0 / upper if lower is None else lower
    w = _level_ratio(log_ratio, mask, level)
    return ((w >= lower) & (w <= upper)).float()


def weight_metrics(prefix, weights, level_log_ratio, mask, level, upper, lower):
    """Diagnostics of untruncated weights (sampler.py:106-173 with prefix "sampler_rs", :259-326 with
    "sampler_is").  ``level_log_ratio`` is the log-ratio at the aggregation level ([B,T] or [B,1])."""
    m = {}
    log_up, log_lo = torch.log(torch.tensor(upper)), torch.log(torch.tensor(lower))
    if level in ("sequence", "geometric"):
        m["max"] = torch.exp(torch.clamp(level_log_ratio.max(), max=SAFETY_BOUND)).item()
        m["min"] = torch.exp(level_log_ratio.min()).item()
        m["mean"] = masked_mean(weights, mask).item()
        m["ratio_fraction_high"] = (level_log_ratio > log_up).float().mean().item()
        m["ratio_fraction_low"] = (level_log_ratio < log_lo).float().mean().item()
    else:
        m["mean"] = masked_mean(weights, mask).item()
        m["ratio_fraction_high"] = masked_mean((weights > upper).float(), mask).item()
        m["ratio_fraction_low"] = masked_mean((weights < lower).float(), mask).item()
        mb = mask.bool()
        m["max"] = weights.masked_fill(~mb, float("-inf")).max().item()
        m["min"] = weights.masked_fill(~mb, float("inf")).min().item()
    clamped = weights.clamp(min=lower, max=upper)
    mean_c = masked_mean(clamped, mask)
    if mask.sum() > 1:
        var = masked_mean(clamped.square(), mask) - mean_c.square()
        m["std"] = torch.sqrt(torch.clamp(var, min=0.0)).item()
    else:
        m["std"] = 0.0
    m["eff_sample_size"] = 1.0 / masked_mean((clamped / (mean_c + 1e-8)).square(), mask).item()
    if weights.dim() > 1:
        seq = masked_mean(weights, mask, axis=-1)
        m["seq_mean"] = seq.mean().item()
        m["seq_std"] = seq.std().item() if seq.numel() > 1 else 0.0
        m["seq_max"], m["seq_min"] = seq.max().item(), seq.min().item()
        m["seq_max_deviation"] = (seq - 1.0).abs().max().item()
        m["seq_fraction_high"] = (seq > upper).float().mean().item()
        m["seq_fraction_low"] = (seq < lower).float().mean().item()
    return {f"{prefix}_{k}": v for k, v in m.items()}


def _level_log_ratio(log_ratio, mask, level):
    if level == "token":
        return log_ratio
    if level == "sequence":
        return masked_sum(log_ratio, mask, axis=-1).unsqueeze(-1)
    return masked_mean(log_ratio, mask, axis=-1).unsqueeze(-1)


def full_metrics(old_log_prob, sampler_log_prob, response_mask, *, sampler_is=None, sampler_is_threshold=2.0,
                 sampler_rs=None, sampler_rs_threshold=2.0, sampler_rs_threshold_lower=None):
    """Every sampler_is_* / sampler_rs_* diagnostic of the unified interface (without the veto pair and
    without the "sampler_corr/" prefix)."""
    lr = old_log_prob - sampler_log_prob
    out = {}
    if sampler_is is not None and sampler_is_threshold is not None:
        raw = _level_ratio(lr, response_mask, sampler_is) * response_mask
        out.update(weight_metrics("sampler_is", raw, _level_log_ratio(lr, response_mask, sampler_is), response_mask,
                                  sampler_is, sampler_is_threshold, 1.0 / sampler_is_threshold))
    if sampler_rs is not None:
        lower = 1.0 / sampler_rs_threshold if sampler_rs_threshold_lower is None else sampler_rs_threshold_lower
        w = _level_ratio(lr, response_mask, sampler_rs)
        out.update(weight_metrics("sampler_rs", w, _level_log_ratio(lr, response_mask, sampler_rs), response_mask,
                                  sampler_rs, sampler_rs_threshold, lower))
        keep = ((w >= lower) & (w <= sampler_rs_threshold)).float()
        out["sampler_rs_masked_fraction"] = masked_mean(1 - keep, response_mask).item()
        if sampler_rs == "token":
            out["sampler_rs_seq_masked_fraction"] = (masked_sum(1 - keep, response_mask, axis=-1) > 0).float().mean().item()
        else:
            out["sampler_rs_seq_masked_fraction"] = (1 - keep[:, 0]).mean().item()
    return out


def offpolicy_metrics(old_log_prob, sampler_log_prob, response_mask):
    """sampler.py:454-518: perplexities, KL / K3 estimators, chi-squared divergences."""
    if not response_mask.any():
        return {}
    m = {}
    a = masked_mean(old_log_prob, response_mask, axis=-1)
    m["training_ppl"] = torch.exp(-a).mean().item()
    m["training_log_ppl"] = (-a).mean().item()
    if sampler_log_prob is None:
        return m
    lr = old_log_prob - sampler_log_prob
    m["kl"] = masked_mean(sampler_log_prob - old_log_prob, response_mask).item()
    m["k3_kl"] = masked_mean(torch.exp(lr) - lr - 1, response_mask).item()
    b = masked_mean(sampler_log_prob, response_mask, axis=-1)
    m["sampler_ppl"] = torch.exp(-b).mean().item()
    m["sampler_log_ppl"] = (-b).mean().item()
    d = b - a
    m["log_ppl_diff"], m["log_ppl_abs_diff"] = d.mean().item(), d.abs().mean().item()
    m["log_ppl_diff_max"], m["log_ppl_diff_min"] = d.max().item(), d.min().item()
    m["ppl_ratio"] = torch.exp(d).mean().item()
    rho = torch.exp(torch.clamp(lr, min=-SAFETY_BOUND, max=SAFETY_BOUND))
    m["chi2_token"] = (masked_mean(rho.square(), response_mask) - 1.0).item()
    lsum = torch.clamp(masked_sum(lr, response_mask, axis=-1), min=-SAFETY_BOUND, max=SAFETY_BOUND)
    m["chi2_seq"] = (torch.exp(2.0 * lsum).mean() - 1.0).item()
    return m


def mismatch_stats(old_log_prob, sampler_log_prob, response_mask):
    """trainer_sampler_mismatch_metrics.py:36-80: extremes and sufficient statistics over valid tokens."""
    mask = response_mask.bool()
    pa, ps = old_log_prob.exp(), sampler_log_prob.exp()
    dp, dl = (pa - ps).abs()[mask], (old_log_prob - sampler_log_prob).abs()[mask]
    am, sm = pa[mask], ps[mask]
    any_ = bool(mask.any())
    f = (lambda t: t.item()) if any_ else (lambda t: 0.0)
    return {
        "batch/sampler_probs_diff_max": f(dp.max()) if any_ else 0.0,
        "batch/sampler_probs_diff_min": f(dp.min()) if any_ else 0.0,
        "batch/sampler_logprobs_diff_max": f(dl.max()) if any_ else 0.0,
        "batch/sampler_logprobs_diff_min": f(dl.min()) if any_ else 0.0,
        "_valid_count": mask.sum().item(),
        "_sum": f(dp.sum()), "_sum_squares": f((dp ** 2).sum()),
        "_logprobs_sum": f(dl.sum()), "_logprobs_sum_squares": f((dl ** 2).sum()),
        "_actor_sum": f(am.sum()), "_sampler_sum": f(sm.sum()),
        "_actor_sum_squares": f((am ** 2).sum()), "_sampler_sum_squares": f((sm ** 2).sum()),
        "_product_sum": f((am * sm).sum()),
    }


def correction(old_log_prob, sampler_log_prob, response_mask, *, sampler_is=None, sampler_is_threshold=2.0,
               sampler_rs=None, sampler_rs_threshold=2.0, sampler_rs_threshold_lower=None,
               sampler_token_veto_threshold=None):
    """sampler.py:334-446.  Returns (weights | None, modified_mask, metrics without prefix).

    All-zero mask -> (None, response_mask, {}) (:368-370).
    """
    if not response_mask.any():
        return None, response_mask, {}
    lr = old_log_prob - sampler_log_prob
    metrics = {}
    weights = None
    if sampler_is is not None and sampler_is_threshold is not None:
        weights, raw = is_weights(lr, response_mask, sampler_is, sampler_is_threshold)
        metrics["sampler_is_mean"] = masked_mean(raw, response_mask).item()
    new_mask = response_mask.clone()
    if sampler_rs is not None:
        keep = rejection_mask(lr, response_mask, sampler_rs, sampler_rs_threshold, sampler_rs_threshold_lower)
        metrics["sampler_rs_masked_fraction"] = masked_mean(1 - keep, response_mask).item()
        new_mask = response_mask * keep
    if sampler_token_veto_threshold is not None:
        if sampler_token_veto_threshold <= 0:
            raise ValueError("sampler_token_veto_threshold must be positive")
        log_thr = torch.log(torch.tensor(sampler_token_veto_threshold))
        bad = (lr < log_thr) & response_mask.bool()
        row_bad = bad.any(dim=-1, keepdim=True)
        metrics["sampler_is_veto_fraction"] = row_bad.float().mean().item()
        metrics["sampler_is_catastrophic_token_fraction"] = masked_mean(bad.float(), response_mask).item()
        new_mask = new_mask * (~row_bad).float()
    else:
        metrics["sampler_is_veto_fraction"] = 0.0
        metrics["sampler_is_catastrophic_token_fraction"] = 0.0
    return weights, new_mask, metrics
