"""KL penalty estimators, the KL controllers and the KL penalty inside the reward, on the HIP path.

``kl_penalty`` / ``kl_penalty_forward`` keep the signatures and type strings of
axon/utils/rl/kl.py:154-245 ("kl"/"k1", "abs", "mse"/"k2", "low_var_kl"/"k3", the
straight-through variants "k1+"/"k3+"; "full" raises).  One elementwise kernel produces the
estimate and its derivative; the autograd function multiplies the latter by the upstream gradient.
``AdaptiveKLController`` / ``FixedKLController`` / ``get_kl_controller`` (:53-151) are host arithmetic;
``compute_rewards_with_kl`` (:248-273) and ``apply_kl_penalty`` (:276-322) run as one pass over the tokens
(``axon_kl_reward``) and one readback of the scalar the controller needs.
"""

from __future__ import annotations

import numpy as np
import torch

from axon_amd import _ops

__all__ = ["AdaptiveKLController", "FixedKLController", "get_kl_controller", "kl_penalty", "kl_penalty_forward",
           "compute_rewards_with_kl", "apply_kl_penalty"]


class AdaptiveKLController:
    """Proportional controller of the KL coefficient (kl.py:53-97, arXiv 1909.08593): the error
    ``current_kl / target - 1`` is clipped to +-0.2 and scaled by ``n_steps / horizon``."""

    def __init__(self, init_kl_coef: float, target_kl: float, horizon: int):
        self.value = init_kl_coef
        self.target = target_kl
        self.horizon = horizon

    def update(self, current_kl: float, n_steps: int) -> None:
        if self.target == 0:  # any non-zero KL counts as the largest error of its sign
            error = float(np.clip(np.sign(current_kl) * 0.2, -0.2, 0.2)) if current_kl != 0 else 0.0
        else:
            error = float(np.clip(current_kl / self.target - 1, -0.2, 0.2))
        self.value *= 1 + error * n_steps / self.horizon


class FixedKLController:
    """Constant coefficient (kl.py:100-125)."""

    def __init__(self, kl_coef: float):
        self.value = kl_coef

    def update(self, current_kl: float, n_steps: int) -> None:
        pass


def get_kl_controller(kl_ctrl):
    """Controller from a config with ``type`` ("fixed" / "adaptive"), ``kl_coef``, ``target_kl``, ``horizon``
    (kl.py:128-151)."""
    if kl_ctrl.type == "fixed":
        return FixedKLController(kl_coef=kl_ctrl.kl_coef)
    if kl_ctrl.type == "adaptive":
        assert kl_ctrl.horizon > 0, f"horizon must be larger than 0. Got {kl_ctrl.horizon}"
        return AdaptiveKLController(init_kl_coef=kl_ctrl.kl_coef, target_kl=kl_ctrl.target_kl,
                                    horizon=kl_ctrl.horizon)
    raise NotImplementedError


class _KlPenalty(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logprob, ref_logprob, kl_type, kl_plus):
        out, grad = _ops.kl_penalty(logprob, ref_logprob, kl_type, kl_plus)
        ctx.save_for_backward(grad)
        ctx.in_dtype = logprob.dtype
        return out.to(logprob.dtype)

    @staticmethod
    def backward(ctx, g):
        (grad,) = ctx.saved_tensors
        return (grad * g).to(ctx.in_dtype), None, None, None


def kl_penalty(logprob: torch.Tensor, ref_logprob: torch.Tensor, kl_penalty_type: str = "low_var_kl") -> torch.Tensor:
    """KL estimate per token, differentiable w.r.t. ``logprob`` (kl.py:154-190)."""
    kl_type, plus = _ops.kl_type_of(kl_penalty_type)
    return _KlPenalty.apply(logprob, ref_logprob, kl_type, plus)


def kl_penalty_forward(logprob: torch.Tensor, ref_logprob: torch.Tensor,
                       kl_penalty_type: str = "low_var_kl") -> torch.Tensor:
    """Forward value only (kl.py:193-245): the "+" suffix is ignored."""
    kl_type, _ = _ops.kl_type_of(kl_penalty_type.rstrip("+"))
    return _ops.kl_penalty(logprob, ref_logprob, kl_type, 0)[0].to(logprob.dtype)


def _stage(t):
    if t.is_cuda:
        return t, None
    if not torch.cuda.is_available():
        _ops.require_device(t, "apply_kl_penalty")
    return t.cuda(), t.device


@torch.no_grad()
def compute_rewards_with_kl(token_level_scores, old_log_prob, ref_log_prob, kl_coef: float) -> torch.Tensor:
    """``score - kl_coef * (old_log_prob - ref_log_prob)`` (kl.py:248-273)."""
    scores, home = _stage(token_level_scores)
    old, _ = _stage(old_log_prob)
    ref, _ = _stage(ref_log_prob)
    rows = _ops.rows_of(scores if scores.dim() == 2 else scores.reshape(1, -1))
    ones = torch.ones(rows.shape, device=scores.device)
    rewards, _, _ = _ops.kl_reward(scores, old, ref, ones, rows, kl_type=1, beta=kl_coef)
    rewards = rewards.view(token_level_scores.shape)
    return rewards if home is None else rewards.to(home)


@torch.no_grad()
def apply_kl_penalty(token_level_scores, old_log_probs, ref_log_prob, response_mask, kl_ctrl,
                     kl_penalty_type: str = "kl", cu_seqlens=None):
    """``(token_level_rewards, metrics)`` of kl.py:276-322: ``rewards = scores - beta * kld * mask``; the mean
    over sequences of the per-sequence mean KL updates the controller (``n_steps`` = number of sequences).
    Packed tensors are accepted with ``cu_seqlens``."""
    kl_type, _ = _ops.kl_type_of(kl_penalty_type.rstrip("+"))
    scores, home = _stage(token_level_scores)
    old, _ = _stage(old_log_probs)
    ref, _ = _stage(ref_log_prob)
    mask, _ = _stage(response_mask)
    rows = _ops.rows_of(scores, cu_seqlens)
    beta = kl_ctrl.value
    rewards, cnt, ksum = _ops.kl_reward(scores, old, ref, mask, rows, kl_type=kl_type, beta=beta)
    current_kl = (ksum / cnt.clamp(min=1)).mean().item()
    kl_ctrl.update(current_kl=current_kl, n_steps=rows.n_rows)
    if home is not None:
        rewards = rewards.to(home)
    return rewards, {"actor/reward_kl_penalty": current_kl, "actor/reward_kl_penalty_coeff": beta}
