"""PPO / DAPO and GSPO clipped policy losses on the HIP path.

Same registry names, batch keys, config keys and metric names as
axon/trainer/algos/loss/loss.py (``ppo_loss_fn`` :47-111, ``gspo_loss_fn``
:114-180).  DAPO's clip-higher is ``clip_ratio_low`` / ``clip_ratio_high`` of the
PPO loss.  One fused kernel evaluates ratio, clip, dual clip, importance
weights, mask, the two-axis aggregation of ``agg_loss`` and the gradient with
respect to ``log_probs``; the metric sums come back in a single readback.

Layouts: the reference's padded ``[B, T]`` tensors, or packed ``[N]`` tensors with
``data.meta_info["cu_seqlens"]`` (int32 ``[S+1]``).
"""

from __future__ import annotations

from typing import Any

import torch

from axon_amd import _lib, _ops
from axon_amd.trainer.algos.constants import VALID_BATCH_REDUCE, VALID_TOKEN_REDUCE
from axon_amd.trainer.algos.loss.registry import LossFn, register_loss

_KIND_PPO, _KIND_GSPO, _KIND_REINFORCE, _KIND_CISPO, _KIND_VALUE = 0, 1, 2, 3, 4


class _ClippedPolicyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_probs, kind, batch, rows, hp):
        acc, grad = _ops.policy_loss(
            kind, log_probs, batch["old_log_probs"], batch["advantages"], batch["response_mask"],
            batch["sampler_is_weights"], rows, **hp,
        )
        ctx.save_for_backward(grad, acc)
        ctx.in_dtype = log_probs.dtype
        ctx.mark_non_differentiable(acc)
        return acc[0].clone(), acc

    @staticmethod
    def backward(ctx, g_loss, _g_acc):
        grad, acc = ctx.saved_tensors
        # acc[5]: the 1/denominator a one-pass token-mean leaves to this multiply
        return _ops.scale_f32(grad, g_loss, acc[5]).to(ctx.in_dtype), None, None, None, None


def _aggregation(b, config, default_token_reduce: str) -> dict:
    """The ``agg_loss`` arguments of a loss call (loss/utils.py:120-251), validated as the reference does."""
    token_reduce = config.get("token_reduce", default_token_reduce)
    batch_reduce = config.get("batch_reduce", "token-mean")
    if token_reduce not in VALID_TOKEN_REDUCE:
        raise ValueError(f"Invalid token_reduce: {token_reduce!r}. Choose from: {sorted(VALID_TOKEN_REDUCE)}")
    if batch_reduce not in VALID_BATCH_REDUCE:
        raise ValueError(f"Invalid batch_reduce: {batch_reduce!r}. Choose from: {sorted(VALID_BATCH_REDUCE)}")
    valid = {
        "token-mean": b.get("valid_token_count", None),
        "step-mean": b.get("valid_batch_size", None),
        "program-mean": b.get("valid_program_count", None),
    }[batch_reduce]
    npt = b.get("num_program_tokens", None)
    nps = b.get("num_program_steps", None)
    if token_reduce == "mean-program":
        assert npt is not None, "num_program_tokens required for token_reduce='mean-program'"
    if batch_reduce == "program-mean":
        assert nps is not None, f"num_program_steps required for batch_reduce='{batch_reduce}'"
        assert valid is not None, "valid_program_count required for batch_reduce='program-mean'"
    return dict(token_reduce=token_reduce, batch_reduce=batch_reduce,
                per_row_token_count=b.get("per_row_token_count", None), num_program_tokens=npt,
                num_program_steps=nps, valid_count=valid)


def policy_loss_spec(kind: int, data, config, default_token_reduce: str, with_log_probs: bool = True):
    """The operands and hyper-parameters of one clipped-policy-loss call, validated as the reference does:
    ``(log_probs, rows, tensors, hp)`` for ``_ops.policy_loss(kind, log_probs, **tensors, rows, **hp)``.
    Without ``with_log_probs`` (a caller that produces them block by block) the first two are None."""
    b = data.batch
    log_probs = b["log_probs"] if with_log_probs else None
    clip = config.get("clip_ratio", 0.2)
    lo = config.get("clip_ratio_low", None)
    hi = config.get("clip_ratio_high", None)
    # CISPO leaves the lower side effectively unclipped unless asked to (loss.py:435-436)
    lo = (1e10 if kind == _KIND_CISPO else clip) if lo is None else lo
    hi = clip if hi is None else hi
    clip_c = config.get("clip_ratio_c", 3.0)
    if kind == _KIND_PPO:
        assert clip_c > 1.0, f"clip_ratio_c must be > 1.0, got {clip_c}"
    if kind == _KIND_CISPO:  # the slot carries the token_level_mask switch instead
        clip_c = 1.0 if config.get("token_level_mask", False) else 0.0
    agg = _aggregation(b, config, default_token_reduce)

    rows = None
    if with_log_probs:
        _lib.require_device(log_probs, "policy loss")
        rows = _ops.rows_of(log_probs, data.meta_info.get("cu_seqlens", None) if data.meta_info else None)
    tensors = {
        "old_log_probs": b["old_log_probs"],
        "advantages": b["advantages"],
        "response_mask": b["response_mask"],
        # CISPO does not read the sampler weights (loss.py:421-468)
        "sampler_is_weights": None if kind == _KIND_CISPO else b.get("sampler_is_weights", None),
    }
    # bounds evaluated in double and rounded once, as torch.clamp does with Python scalars
    hp = dict(ratio_lo=1 - lo, ratio_hi=1 + hi, clip_c=clip_c, **agg)
    return log_probs, rows, tensors, hp


def policy_loss_metrics(kind: int, sums) -> dict[str, Any]:
    """The metrics of a clipped policy loss from the kernel's sums (``acc[1:5]`` as a list)."""
    denom = max(sums[4], 1.0)
    metrics: dict[str, Any] = {"ppo_kl": sums[2] / denom}
    if kind != _KIND_REINFORCE:
        metrics["pg_clipfrac"] = sums[1] / denom
    if kind in (_KIND_PPO, _KIND_GSPO):
        metrics["pg_clipfrac_lower"] = (sums[3] / denom) if kind == _KIND_PPO else 0.0
    return metrics


# registry name -> (kernel kind, default token_reduce) of the losses that run on ``_ops.policy_loss``
POLICY_LOSS_KINDS = {"ppo": (_KIND_PPO, "sum"), "gspo": (_KIND_GSPO, "mean"), "reinforce": (_KIND_REINFORCE, "sum"),
                     "gpg": (_KIND_REINFORCE, "sum"), "cispo": (_KIND_CISPO, "sum")}


def _run(kind: int, data, config, default_token_reduce: str):
    log_probs, rows, tensors, hp = policy_loss_spec(kind, data, config, default_token_reduce)
    loss, acc = _ClippedPolicyLoss.apply(log_probs, kind, tensors, rows, hp)
    sums = acc.tolist()  # the only host sync of the loss
    return loss, policy_loss_metrics(kind, sums)


@register_loss(LossFn.PPO)
def ppo_loss_fn(data, config) -> tuple[torch.Tensor, dict[str, Any]]:
    """Clipped PPO surrogate with dual clip (loss.py:47-111); defaults sum / token-mean."""
    return _run(_KIND_PPO, data, config, "sum")


@register_loss(LossFn.GSPO)
def gspo_loss_fn(data, config) -> tuple[torch.Tensor, dict[str, Any]]:
    """GSPO sequence-level ratio loss (loss.py:114-180); code defaults mean / token-mean (:165-166)."""
    return _run(_KIND_GSPO, data, config, "mean")


@register_loss(LossFn.REINFORCE)
def reinforce_loss_fn(data, config) -> tuple[torch.Tensor, dict[str, Any]]:
    """``-log_prob * A`` (times the sampler weights when present), loss.py:471-512; sum / token-mean."""
    return _run(_KIND_REINFORCE, data, config, "sum")


@register_loss(LossFn.GPG)
def gpg_loss_fn(data, config) -> tuple[torch.Tensor, dict[str, Any]]:
    """Same objective as REINFORCE; pairs with the GPG advantage (loss.py:183-197)."""
    return reinforce_loss_fn(data, config)


@register_loss(LossFn.CISPO)
def cispo_loss_fn(data, config) -> tuple[torch.Tensor, dict[str, Any]]:
    """Clipped, stop-gradient importance weight times ``A * log_prob`` (loss.py:411-468)."""
    return _run(_KIND_CISPO, data, config, "sum")


class _GmpoLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_probs, batch, rows, clip_low, clip_high):
        acc, grad = _ops.gmpo_loss(log_probs, batch["old_log_probs"], batch["advantages"], batch["response_mask"],
                                   batch["sampler_is_weights"], rows, clip_low=clip_low, clip_high=clip_high)
        ctx.save_for_backward(grad)
        ctx.in_dtype = log_probs.dtype
        ctx.mark_non_differentiable(acc)
        return acc[0].clone(), acc

    @staticmethod
    def backward(ctx, g_loss, _g_acc):
        (grad,) = ctx.saved_tensors
        return _ops.scale_f32(grad, g_loss).to(ctx.in_dtype), None, None, None, None


@register_loss(LossFn.GEO_MEAN)
def geo_mean_loss_fn(data, config) -> tuple[torch.Tensor, dict[str, Any]]:
    """GMPO: sequence-level geometric-mean ratio with token-level clipping of the log-ratio
    (loss.py:355-408).  Ignores token_reduce / batch_reduce like the reference."""
    b = data.batch
    clip = config.get("clip_ratio", 0.2)
    lo = config.get("clip_ratio_low", None)
    hi = config.get("clip_ratio_high", None)
    lo = clip if lo is None else lo
    hi = clip if hi is None else hi
    log_probs = b["log_probs"]
    _lib.require_device(log_probs, "policy loss")
    rows = _ops.rows_of(log_probs, data.meta_info.get("cu_seqlens", None) if data.meta_info else None)
    tensors = {"old_log_probs": b["old_log_probs"], "advantages": b["advantages"], "response_mask": b["response_mask"],
               "sampler_is_weights": b.get("sampler_is_weights", None)}
    loss, acc = _GmpoLoss.apply(log_probs, tensors, rows, lo, hi)
    sums = acc.tolist()
    denom = max(sums[4], 1.0)
    return loss, {"pg_clipfrac": sums[1] / denom, "ppo_kl": sums[2] / denom, "pg_clipfrac_lower": sums[3] / denom}


@register_loss(LossFn.VALUE)
def value_loss_fn(data, config) -> tuple[torch.Tensor, dict[str, Any]]:
    """Clipped value-function loss (loss.py:547-591): ``0.5 * agg_loss(max((vpreds - returns)^2,
    (clip(vpreds, values -+ cliprange_value) - returns)^2))``, defaults sum / token-mean; the gradient flows to
    ``vpreds``.  Metrics ``vf_loss``, ``vf_clipfrac``, ``vpred_mean``."""
    b = data.batch
    vpreds = b["vpreds"]
    agg = _aggregation(b, config, "sum")
    _lib.require_device(vpreds, "value loss")
    rows = _ops.rows_of(vpreds, data.meta_info.get("cu_seqlens", None) if data.meta_info else None)
    tensors = {"old_log_probs": b["values"], "advantages": b["returns"], "response_mask": b["response_mask"],
               "sampler_is_weights": None}
    hp = dict(ratio_lo=config.get("cliprange_value", 0.5), ratio_hi=0.0, clip_c=0.0, **agg)
    raw, acc = _ClippedPolicyLoss.apply(vpreds, _KIND_VALUE, tensors, rows, hp)
    loss = 0.5 * raw
    sums = acc.tolist()
    denom = max(sums[4], 1.0)
    return loss, {"vf_loss": 0.5 * sums[0], "vf_clipfrac": sums[1] / denom, "vpred_mean": sums[2] / denom}


class _CovPolicyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, log_probs, kind, batch, rows, hp):
        acc, grad, _, _ = _ops.cov_policy_loss(
            kind, log_probs, batch["old_log_probs"], batch["advantages"], batch["response_mask"],
            batch["sampler_is_weights"], rows, **hp,
        )
        ctx.save_for_backward(grad, acc)
        ctx.in_dtype = log_probs.dtype
        ctx.mark_non_differentiable(acc)
        return acc[0].clone(), acc

    @staticmethod
    def backward(ctx, g_loss, _g_acc):
        grad, acc = ctx.saved_tensors
        return _ops.scale_f32(grad, g_loss, acc[5]).to(ctx.in_dtype), None, None, None, None


def _run_cov(kind: int, data, config, hp: dict, default_token_reduce: str):
    b = data.batch
    log_probs = b["log_probs"]
    agg = _aggregation(b, config, default_token_reduce)
    _lib.require_device(log_probs, "policy loss")
    rows = _ops.rows_of(log_probs, data.meta_info.get("cu_seqlens", None) if data.meta_info else None)
    tensors = {"old_log_probs": b["old_log_probs"], "advantages": b["advantages"],
               "response_mask": b["response_mask"], "sampler_is_weights": b.get("sampler_is_weights", None)}
    loss, acc = _CovPolicyLoss.apply(log_probs, kind, tensors, rows, dict(**hp, **agg))
    sums = acc.tolist()
    return loss, sums, max(sums[4], 1.0)


@register_loss(LossFn.KL_COV)
def kl_cov_loss_fn(data, config) -> tuple[torch.Tensor, dict[str, Any]]:
    """KL-Cov (loss.py:283-352): ``-A * ratio`` everywhere, plus ``ppo_kl_coef * |log ratio|`` on the
    ``kl_cov_ratio`` share of response tokens with the largest advantage / log-prob covariance.  The reference
    takes that top-k on the host; here a radix select finds it on the device.  Defaults sum / token-mean."""
    ratio = config.get("kl_cov_ratio", 0.0002)
    assert ratio > 0, "kl_cov_ratio must be > 0"
    loss, sums, denom = _run_cov(0, data, config, dict(select_ratio=ratio, kl_coef=config.get("ppo_kl_coef", 1.0)),
                                 "sum")
    return loss, {"ppo_kl": sums[2] / denom}


@register_loss(LossFn.CLIP_COV)
def clip_cov_loss_fn(data, config) -> tuple[torch.Tensor, dict[str, Any]]:
    """Clip-Cov (loss.py:198-280): the PPO clipped surrogate with a random ``clip_cov_ratio`` share of the
    unclipped tokens whose covariance lies in ``(clip_cov_lb, clip_cov_ub)`` dropped from the loss.  The draw
    takes its seed from torch's CPU generator, so ``torch.manual_seed`` makes it repeatable, as it does the
    reference's ``randperm``.  Code defaults mean / token-mean (:265)."""
    clip = config.get("clip_ratio", 0.2)
    lo = config.get("clip_ratio_low", None)
    hi = config.get("clip_ratio_high", None)
    lo = clip if lo is None else lo
    hi = clip if hi is None else hi
    ratio = config.get("clip_cov_ratio", 0.0002)
    assert ratio > 0, "clip_cov_ratio must be > 0"
    seed = int(torch.randint(0, 2**31 - 1, (1,)).item())
    hp = dict(select_ratio=ratio, ratio_lo=1 - lo, ratio_hi=1 + hi, cov_lb=config.get("clip_cov_lb", 1.0),
              cov_ub=config.get("clip_cov_ub", 5.0), seed=seed)
    loss, sums, denom = _run_cov(1, data, config, hp, "mean")
    return loss, {"pg_clipfrac": sums[1] / denom, "ppo_kl": sums[2] / denom}
