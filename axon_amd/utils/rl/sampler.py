"""Sampler–trainer correction on the HIP path.

Public names and semantics follow axon/utils/rl/sampler.py:
``compute_sampler_correction_and_rejection_mask`` (:334-446) with its two halves
``compute_sampler_correction_weights`` (:181-256) and
``compute_sampler_rejection_mask`` (:35-103), and the batch helper
``compute_sampler_correction_and_add_to_batch`` (:526-563).

  log_ratio = old_log_prob - sampler_log_prob
  IS  token:     w = exp(clamp(lr, +-20)) * mask, then min(w, threshold), detached
      sequence:  w = exp(clamp(sum_mask lr, +-20)) broadcast
  RS  token:     keep iff lower <= exp(clamp(lr)) <= upper (lower defaults to 1/upper)
      sequence / geometric: same test on the masked row sum / masked row mean
  veto: a row with any masked token whose lr < log(threshold) is zeroed
  new mask = response_mask * rs * veto

One elementwise launch, or, when a row-level quantity is needed (veto, sequence or geometric level),
one launch in which a workgroup owns whole rows (batches of short rows: a row pass, then an elementwise
pass).  The rejection test runs in log space against fp32 interval ends computed here on the host, so
the 0/1 masks do not depend on the last bit of the device's ``exp``.

Metrics: every ``sampler_corr/*`` key of the reference (importance-weight and rejection statistics,
veto and catastrophic-token fractions, the batch-normalisation factor) from one diagnostics launch
and ONE readback for everything.
"""

from __future__ import annotations

import functools
import math
import struct
from typing import Any

import numpy as np
import torch

from axon_amd import _ops
from axon_amd.protocol import DataProto

SAFETY_BOUND = 20.0

_VALID_IS = {"token", "sequence"}
_VALID_RS = {"token", "sequence", "geometric"}


# --- fp32 interval ends for the rejection test --------------------------------------------

def _f32(x: float) -> float:
    return struct.unpack("f", struct.pack("f", x))[0]


def _ordered(x: float) -> int:
    """Map an fp32 value to an integer that sorts like the float."""
    (u,) = struct.unpack("I", struct.pack("f", x))
    return u ^ 0x80000000 if u < 0x80000000 else 0xFFFFFFFF - u


def _from_ordered(i: int) -> float:
    u = i ^ 0x80000000 if i >= 0x80000000 else 0xFFFFFFFF - i
    return struct.unpack("f", struct.pack("I", u))[0]


def _exp32(x: float) -> float:
    """torch's CPU fp32 exp of one value, taken from the vectorised path."""
    return float(torch.exp(torch.full((64,), x, dtype=torch.float32))[0])


@functools.lru_cache(maxsize=256)
def log_interval_for_ratio_bounds(lower: float, upper: float) -> tuple[float, float]:
    """fp32 ``[lo, hi]`` such that for fp32 ``x``:

        lower <= exp(clamp(x, -20, 20)) <= upper   <=>   lo <= x <= hi

    with the comparison made in fp32 as torch does for a float32 tensor against a Python
    scalar.  Found by bisection over the fp32 number line with torch's CPU ``exp`` as the
    arbiter (``exp`` is monotone there).  An empty set is returned as ``(inf, -inf)``.
    """
    lower32, upper32 = _f32(lower), _f32(upper)
    lo_i, hi_i = _ordered(-SAFETY_BOUND), _ordered(SAFETY_BOUND)

    # hi: largest x in [-20, 20] with exp(x) <= upper
    if _exp32(SAFETY_BOUND) <= upper32:
        hi = math.inf  # every clamped value passes
    elif not (_exp32(-SAFETY_BOUND) <= upper32):
        hi = -math.inf
    else:
        a, b = lo_i, hi_i  # exp(a) <= upper < exp(b)
        while b - a > 1:
            mid = (a + b) // 2
            if _exp32(_from_ordered(mid)) <= upper32:
                a = mid
            else:
                b = mid
        hi = _from_ordered(a)
    # lo: smallest x with exp(x) >= lower
    if _exp32(-SAFETY_BOUND) >= lower32:
        lo = -math.inf
    elif not (_exp32(SAFETY_BOUND) >= lower32):
        lo = math.inf
    else:
        a, b = lo_i, hi_i  # exp(a) < lower <= exp(b)
        while b - a > 1:
            mid = (a + b) // 2
            if _exp32(_from_ordered(mid)) >= lower32:
                b = mid
            else:
                a = mid
        lo = _from_ordered(b)
    if lo > hi:
        return math.inf, -math.inf
    return lo, hi


@functools.lru_cache(maxsize=256)
def _log32(x: float) -> float:
    """``torch.log(torch.tensor(x))`` in fp32 (sampler.py:418)."""
    return float(torch.log(torch.tensor(x, dtype=torch.float32)))


# --- argument checks (same messages as the reference raises) --------------------------------

def _check_is(sampler_is, threshold):
    if sampler_is not in _VALID_IS:
        raise ValueError(f"Invalid sampler_is: {sampler_is}. Must be one of {_VALID_IS}.")
    if threshold <= 0:
        raise ValueError(f"sampler_is_threshold must be positive, got {threshold}.")


def _check_rs(sampler_rs, threshold):
    if sampler_rs not in _VALID_RS:
        raise ValueError(f"Invalid sampler_rs: {sampler_rs}. Must be one of {_VALID_RS}.")
    if threshold is None:
        raise ValueError("sampler_rs_threshold must be provided for rejection sampling.")


def _check_shapes(old_log_prob, sampler_log_prob, response_mask):
    if old_log_prob.shape != sampler_log_prob.shape:
        raise ValueError(
            f"old_log_prob shape {old_log_prob.shape} does not match sampler_log_prob shape {sampler_log_prob.shape}."
        )
    if old_log_prob.shape != response_mask.shape:
        raise ValueError(f"log_prob shape {old_log_prob.shape} does not match response_mask shape {response_mask.shape}.")


# --- metrics from the raw sums of axon_sampler_diag ------------------------------------------------

def _soft(n: float) -> float:
    """``mask.sum() + 1e-8`` as fp32 arithmetic gives it (axon/utils/torch/ops.py:131-145)."""
    return float(np.float32(n) + np.float32(1e-8))


def _weight_metrics(prefix, d, n_rows, level, s_e, s_hi, s_lo, s_c, s_c2, row, lvl, mm_x, mm_dev, mm_l):
    """The diagnostics of untruncated weights (sampler.py:106-173 / :259-326) from raw sums.

    ``d``: the 72 values; token-level slots s_*; row-statistics slots ``row`` (sum x, sum x^2, #hi, #lo);
    row-level-mode slots ``lvl`` (#L>hi, #L<lo, sum w*cnt, sum clamp*cnt, sum clamp^2*cnt); extrema slots.
    """
    n = d[0]
    soft = _soft(n)
    m = {}
    if level == "token":
        m["mean"] = d[s_e] / soft
        m["ratio_fraction_high"] = d[s_hi] / soft
        m["ratio_fraction_low"] = d[s_lo] / soft
        m["max"], m["min"] = d[50], d[60]
        c1, c2 = d[s_c] / soft, d[s_c2] / soft
    else:
        m["max"] = math.exp(min(d[50 + mm_l], SAFETY_BOUND))
        m["min"] = math.exp(d[60 + mm_l])
        m["mean"] = d[lvl + 2] / soft
        m["ratio_fraction_high"] = d[lvl] / n_rows
        m["ratio_fraction_low"] = d[lvl + 1] / n_rows
        c1, c2 = d[lvl + 3] / soft, d[lvl + 4] / soft
    m["std"] = math.sqrt(max(c2 - c1 * c1, 0.0)) if n > 1 else 0.0
    m["eff_sample_size"] = (c1 + 1e-8) ** 2 / c2 if c2 > 0 else float("inf")
    sx, sx2 = d[row], d[row + 1]
    m["seq_mean"] = sx / n_rows
    m["seq_std"] = math.sqrt(max((sx2 - sx * sx / n_rows) / (n_rows - 1), 0.0)) if n_rows > 1 else 0.0
    m["seq_max"], m["seq_min"] = d[50 + mm_x], d[60 + mm_x]
    m["seq_max_deviation"] = d[50 + mm_dev]
    m["seq_fraction_high"] = d[row + 2] / n_rows
    m["seq_fraction_low"] = d[row + 3] / n_rows
    return {f"{prefix}_{k}": v for k, v in m.items()}


def _offpolicy_from_diag(d, n_rows) -> dict[str, float]:
    soft = _soft(d[0])
    return {
        "training_ppl": d[42] / n_rows, "training_log_ppl": d[43] / n_rows,
        "kl": -d[3] / soft, "k3_kl": d[4] / soft,
        "sampler_ppl": d[44] / n_rows, "sampler_log_ppl": d[45] / n_rows,
        "log_ppl_diff": d[46] / n_rows, "log_ppl_abs_diff": d[47] / n_rows,
        "log_ppl_diff_max": d[59], "log_ppl_diff_min": d[69],
        "ppl_ratio": d[48] / n_rows,
        "chi2_token": d[2] / soft - 1.0, "chi2_seq": d[49] / n_rows - 1.0,
    }


# --- public API -------------------------------------------------------------------------------

def compute_sampler_correction_and_rejection_mask(
    old_log_prob: torch.Tensor,
    sampler_log_prob: torch.Tensor,
    response_mask: torch.Tensor,
    sampler_is: str | None = None,
    sampler_is_threshold: float | None = 2.0,
    sampler_rs: str | None = None,
    sampler_rs_threshold: float | None = 2.0,
    sampler_rs_threshold_lower: float | None = None,
    sampler_token_veto_threshold: float | None = None,
    sampler_is_batch_normalize: bool = False,
    cu_seqlens: torch.Tensor | None = None,
) -> tuple[DataProto | None, torch.Tensor, dict[str, float]]:
    """Returns ``(DataProto{"sampler_is_weights"} | None, modified_response_mask, metrics)``.

    An all-zero ``response_mask`` is a no-op: ``(None, response_mask, {})``.
    """
    use_is = sampler_is is not None and sampler_is_threshold is not None
    rs_lo = rs_hi = 0.0
    log_veto = None
    try:
        _check_shapes(old_log_prob, sampler_log_prob, response_mask)
        if use_is:
            _check_is(sampler_is, sampler_is_threshold)
        if sampler_rs is not None:
            if sampler_rs_threshold is None:
                raise ValueError(
                    "sampler_rs_threshold must be explicitly provided when sampler_rs is enabled. "
                    "Set sampler_rs_threshold to the desired threshold value."
                )
            _check_rs(sampler_rs, sampler_rs_threshold)
            upper = sampler_rs_threshold
            lower = sampler_rs_threshold_lower if sampler_rs_threshold_lower is not None else 1.0 / upper
            rs_lo, rs_hi = log_interval_for_ratio_bounds(lower, upper)
        if sampler_token_veto_threshold is not None:
            if sampler_token_veto_threshold <= 0:
                raise ValueError(f"sampler_token_veto_threshold must be positive, got {sampler_token_veto_threshold}.")
            log_veto = _log32(sampler_token_veto_threshold)
    except ValueError:
        # The reference returns the no-op for an all-padding micro-batch before it validates anything
        # (sampler.py:368-370): a bad argument only raises when there is a token to correct.  The valid path keeps
        # its single readback; this one costs an extra one.
        if not bool(response_mask.any()):
            return None, response_mask, {}
        raise

    _ops.require_device(old_log_prob, "compute_sampler_correction_and_rejection_mask")
    rows = _ops.rows_of(old_log_prob, cu_seqlens)
    weights, new_mask, acc = _ops.sampler_correction(
        old_log_prob, sampler_log_prob, response_mask, rows,
        is_mode=_ops.IS_MODES[sampler_is] if use_is else 0,
        is_threshold=sampler_is_threshold if use_is else 1.0,
        rs_mode=_ops.RS_MODES[sampler_rs], rs_lr_lo=rs_lo, rs_lr_hi=rs_hi, log_veto=log_veto,
    )
    is_hi = float(sampler_is_threshold) if use_is else 1.0
    is_lo = 1.0 / is_hi
    rs_hi_t = float(sampler_rs_threshold) if sampler_rs is not None else 1.0
    rs_lo_t = (float(sampler_rs_threshold_lower) if sampler_rs_threshold_lower is not None else 1.0 / rs_hi_t) \
        if sampler_rs is not None else 1.0
    tok_lo, tok_hi = (rs_lo, rs_hi) if sampler_rs == "token" else (-math.inf, math.inf)
    diag = _ops.sampler_diag(
        old_log_prob, sampler_log_prob, response_mask, rows,
        is_mode=_ops.IS_MODES[sampler_is] if use_is else 0, is_lo=is_lo, is_hi=is_hi,
        rs_mode=_ops.RS_MODES[sampler_rs], rs_lo=rs_lo_t, rs_hi=rs_hi_t, rs_lr_lo=tok_lo, rs_lr_hi=tok_hi,
        log_is_lo=_log32(is_lo), log_is_hi=_log32(is_hi), log_rs_lo=_log32(rs_lo_t), log_rs_hi=_log32(rs_hi_t),
    )
    both = torch.cat([acc.double(), diag]).tolist()  # single readback: empty-mask test and every metric
    sums, d = both[:8], both[8:]
    n_valid = sums[0]
    if n_valid == 0:
        return None, response_mask, {}

    metrics: dict[str, float] = {}
    soft = _soft(n_valid)
    if use_is:
        metrics.update(_weight_metrics("sampler_is", d, rows.n_rows, sampler_is, 1, 5, 6, 7, 8, 23, 31, 3, 4, 7))
        if sampler_is_batch_normalize:
            mean_w = sums[5] / soft
            if sampler_is == "sequence":
                # mean over rows that have tokens of the row's (constant) weight
                cnt, per_row, _ = _ops.row_stats(weights, None, response_mask, rows)
                has = (cnt > 0).to(torch.float32)
                mean_w = float(((per_row / (cnt + 1e-8)) * has).sum() / has.sum().clamp_min(1e-8))
            if mean_w > 1e-8:
                weights = weights / mean_w
                metrics["sampler_is_batch_norm_factor"] = mean_w
            else:
                metrics["sampler_is_batch_norm_factor"] = 1.0
    if sampler_rs is not None:
        metrics.update(_weight_metrics("sampler_rs", d, rows.n_rows, sampler_rs, 1, 9, 10, 11, 12, 27, 36, 5, 6, 8))
        metrics["sampler_rs_masked_fraction"] = sums[2] / soft
        metrics["sampler_rs_seq_masked_fraction"] = d[41] / rows.n_rows
    if log_veto is not None:
        metrics["sampler_is_veto_fraction"] = sums[4] / max(rows.n_rows, 1)
        metrics["sampler_is_catastrophic_token_fraction"] = sums[3] / soft
    else:
        metrics["sampler_is_veto_fraction"] = 0.0
        metrics["sampler_is_catastrophic_token_fraction"] = 0.0

    proto = DataProto.from_dict(tensors={"sampler_is_weights": weights}) if weights is not None else None
    return proto, new_mask, {f"sampler_corr/{k}": v for k, v in metrics.items()}


def compute_sampler_correction_weights(
    log_ratio: torch.Tensor,
    response_mask: torch.Tensor,
    sampler_is: str = "token",
    sampler_is_threshold: float = 2.0,
    sampler_is_batch_normalize: bool = False,
    cu_seqlens: torch.Tensor | None = None,
) -> tuple[torch.Tensor, dict[str, float]]:
    """Truncated importance weights from a precomputed log-ratio (sampler.py:181-256)."""
    _check_is(sampler_is, sampler_is_threshold)
    proto, _, metrics = compute_sampler_correction_and_rejection_mask(
        log_ratio, torch.zeros_like(log_ratio), response_mask, sampler_is=sampler_is,
        sampler_is_threshold=sampler_is_threshold, sampler_is_batch_normalize=sampler_is_batch_normalize,
        cu_seqlens=cu_seqlens,
    )
    if proto is None:
        raise ValueError("response_mask must contain at least one valid token (1).")
    short = {k[len("sampler_corr/"):]: v for k, v in metrics.items() if "veto" not in k and "catastrophic" not in k}
    return proto.batch["sampler_is_weights"], short


def compute_sampler_rejection_mask(
    log_ratio: torch.Tensor,
    response_mask: torch.Tensor,
    sampler_rs: str = "token",
    sampler_rs_threshold: float | None = None,
    sampler_rs_threshold_lower: float | None = None,
    cu_seqlens: torch.Tensor | None = None,
) -> tuple[torch.Tensor, dict[str, float]]:
    """Rejection mask from a precomputed log-ratio (sampler.py:35-103)."""
    _check_rs(sampler_rs, sampler_rs_threshold)
    _, new_mask, metrics = compute_sampler_correction_and_rejection_mask(
        log_ratio, torch.zeros_like(log_ratio), response_mask, sampler_rs=sampler_rs,
        sampler_rs_threshold=sampler_rs_threshold, sampler_rs_threshold_lower=sampler_rs_threshold_lower,
        cu_seqlens=cu_seqlens,
    )
    if not metrics:
        raise ValueError("response_mask must contain at least one valid token (1).")
    short = {k[len("sampler_corr/"):]: v for k, v in metrics.items() if "veto" not in k and "catastrophic" not in k}
    return new_mask, short


def _diag_plain(old_log_prob, sampler_log_prob, response_mask, cu_seqlens):
    d = sampler_gap_sums(old_log_prob, sampler_log_prob, response_mask, cu_seqlens)
    return d.tolist(), _ops.rows_of(old_log_prob, cu_seqlens).n_rows


def compute_offpolicy_metrics(old_log_prob, sampler_log_prob, response_mask,
                              cu_seqlens: torch.Tensor | None = None) -> dict[str, Any]:
    """Off-policy diagnostics (sampler.py:454-518): perplexities, KL / K3, chi-squared; no prefix.
    One token pass, one row pass, one readback."""
    _ops.require_device(old_log_prob, "compute_offpolicy_metrics")
    if sampler_log_prob is None:
        rows = _ops.rows_of(old_log_prob, cu_seqlens)
        cnt, ssum, _ = _ops.row_stats(old_log_prob, None, response_mask, rows)
        a = ssum / (cnt + 1e-8)
        vals = torch.stack([cnt.sum(), torch.exp(-a).mean(), (-a).mean()]).tolist()
        if vals[0] == 0:
            return {}
        return {"training_ppl": vals[1], "training_log_ppl": vals[2]}
    d, n_rows = _diag_plain(old_log_prob, sampler_log_prob, response_mask, cu_seqlens)
    if d[0] == 0:
        return {}
    return _offpolicy_from_diag(d, n_rows)


def sampler_gap_sums(log_prob, sampler_log_prob, response_mask, cu_seqlens=None):
    """The device half of ``compute_sampler_corr_metrics_from_logprobs``: the raw sums as a float64 device tensor
    (no readback), for a caller that collects them with other scalars; ``sampler_gap_metrics`` is the host half."""
    rows = _ops.rows_of(log_prob, cu_seqlens)
    return _ops.sampler_diag(log_prob.detach(), sampler_log_prob, response_mask, rows, is_mode=0, is_lo=1.0, is_hi=1.0,
                             rs_mode=0, rs_lo=1.0, rs_hi=1.0, rs_lr_lo=-math.inf, rs_lr_hi=math.inf, log_is_lo=0.0,
                             log_is_hi=0.0, log_rs_lo=0.0, log_rs_hi=0.0)


def sampler_gap_metrics(sums: list, n_rows: int) -> dict[str, float]:
    """``sampler_corr/``-prefixed off-policy metrics from ``sampler_gap_sums`` read back as a list."""
    if sums[0] == 0:
        return {}
    return {f"sampler_corr/{k}": v for k, v in _offpolicy_from_diag(sums, n_rows).items()}


def compute_sampler_corr_metrics_from_logprobs(log_prob, sampler_log_prob, response_mask,
                                               cu_seqlens: torch.Tensor | None = None) -> dict[str, float]:
    """Off-policy gap of the CURRENT policy against the sampler, "sampler_corr/"-prefixed
    (sampler.py:566-597); called inside the actor update as the policy moves."""
    m = compute_offpolicy_metrics(log_prob.detach(), sampler_log_prob, response_mask, cu_seqlens=cu_seqlens)
    return {f"sampler_corr/{k}": v for k, v in m.items()}


def compute_sampler_correction_and_add_to_batch(batch: DataProto, config: dict[str, Any]) -> tuple[DataProto, dict]:
    """Overwrite ``batch.batch["response_mask"]`` and union ``sampler_is_weights`` into the batch
    (sampler.py:526-563); ``config`` is the loss_args dict."""
    with torch.no_grad():
        weights, new_mask, metrics = compute_sampler_correction_and_rejection_mask(
            old_log_prob=batch.batch["old_log_probs"],
            sampler_log_prob=batch.batch["sampler_log_probs"],
            response_mask=batch.batch["response_mask"],
            sampler_is=config.get("sampler_is", None),
            sampler_is_threshold=config.get("sampler_is_threshold", 2.0),
            sampler_rs=config.get("sampler_rs", None),
            sampler_rs_threshold=config.get("sampler_rs_threshold", None),
            sampler_rs_threshold_lower=config.get("sampler_rs_threshold_lower", None),
            sampler_token_veto_threshold=config.get("sampler_token_veto_threshold", None),
            sampler_is_batch_normalize=config.get("sampler_is_batch_normalize", False),
            cu_seqlens=batch.meta_info.get("cu_seqlens", None) if batch.meta_info else None,
        )
    batch.batch["response_mask"] = new_mask
    if weights is not None:
        batch = batch.union(weights)
    return batch, metrics
