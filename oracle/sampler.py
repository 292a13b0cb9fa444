"""Oracle: sampler–trainer correction in plain torch (CPU).

Restates axon/utils/rl/sampler.py:35-103 (rejection mask), :181-256 (truncated IS
weights), :334-446 (unified interface incl. the per-token veto) and the two masked
reductions of axon/utils/torch/ops.py:123-145 it relies on.  Returns tensors instead of
a DataProto; only the metrics the HIP path also reports are computed.
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
