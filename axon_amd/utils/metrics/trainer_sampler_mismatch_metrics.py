"""Sampler / actor log-prob mismatch statistics on the HIP path.

Same two functions, keys and aggregation rule as
axon/utils/metrics/trainer_sampler_mismatch_metrics.py:36-146.  The per-shard sufficient
statistics come out of the same token pass as the other sampler diagnostics
(``axon_sampler_diag``) in one readback, instead of fourteen reductions with an ``.item()`` each.
"""

from __future__ import annotations

from axon_amd.utils.rl.sampler import _diag_plain

_MEAN_KEYS = ("probs", "logprobs")


def compute_trainer_sampler_mismatch_metrics(batch) -> dict:
    """Per-shard extremes plus sums that add across workers (keys starting with ``_``)."""
    b = batch.batch
    cu = batch.meta_info.get("cu_seqlens", None) if batch.meta_info else None
    d, _ = _diag_plain(b["old_log_probs"], b["sampler_log_probs"], b["response_mask"], cu)
    n = d[0]
    some = n > 0
    pick = (lambda i: d[i]) if some else (lambda i: 0.0)
    return {
        "batch/sampler_probs_diff_max": pick(51),
        "batch/sampler_probs_diff_min": pick(61),
        "batch/sampler_logprobs_diff_max": pick(52),
        "batch/sampler_logprobs_diff_min": pick(62),
        "_valid_count": int(n),
        "_sum": pick(13),
        "_sum_squares": pick(14),
        "_logprobs_sum": pick(15),
        "_logprobs_sum_squares": pick(16),
        "_actor_sum": pick(17),
        "_sampler_sum": pick(18),
        "_actor_sum_squares": pick(19),
        "_sampler_sum_squares": pick(20),
        "_product_sum": pick(21),
    }


def _zero_metrics() -> dict:
    out = {}
    for kind in _MEAN_KEYS:
        for stat in ("max", "mean", "min", "std"):
            out[f"batch/sampler_{kind}_diff_{stat}"] = 0.0
    out["batch/sampler_actor_probs_pearson_corr"] = 0.0
    return out


def aggregate_trainer_sampler_metrics(metrics_list: list[dict]) -> dict:
    """Mean / std / min / max / Pearson correlation from one or more shards' statistics."""
    if not metrics_list:
        return {}
    tot = lambda key: sum(m.get(key, 0.0) for m in metrics_list)  # noqa: E731
    n = tot("_valid_count")
    if n == 0:
        return _zero_metrics()

    def mean_std(s_key, sq_key):
        mean = tot(s_key) / n
        var = tot(sq_key) / n - mean ** 2
        return mean, (var ** 0.5 if var > 0 else 0.0)

    p_mean, p_std = mean_std("_sum", "_sum_squares")
    l_mean, l_std = mean_std("_logprobs_sum", "_logprobs_sum_squares")
    a_mean, s_mean = tot("_actor_sum") / n, tot("_sampler_sum") / n
    cov = tot("_product_sum") / n - a_mean * s_mean
    a_std = max(0, tot("_actor_sum_squares") / n - a_mean ** 2) ** 0.5
    s_std = max(0, tot("_sampler_sum_squares") / n - s_mean ** 2) ** 0.5
    denom = a_std * s_std
    ext = lambda key, fn: fn(m[key] for m in metrics_list)  # noqa: E731
    return {
        "batch/sampler_probs_diff_max": ext("batch/sampler_probs_diff_max", max),
        "batch/sampler_probs_diff_mean": p_mean,
        "batch/sampler_probs_diff_min": ext("batch/sampler_probs_diff_min", min),
        "batch/sampler_probs_diff_std": p_std,
        "batch/sampler_logprobs_diff_max": ext("batch/sampler_logprobs_diff_max", max),
        "batch/sampler_logprobs_diff_mean": l_mean,
        "batch/sampler_logprobs_diff_min": ext("batch/sampler_logprobs_diff_min", min),
        "batch/sampler_logprobs_diff_std": l_std,
        "batch/sampler_actor_probs_pearson_corr": cov / denom if denom > 0 else 0.0,
    }
