"""Group-normalised GRPO advantage on the HIP path.

``grpo_advantage_fn`` follows axon/trainer/algos/advantages/advantage.py:78-109:
score = sum_t token_level_rewards, per-uid mean/std (Bessel, std floored at
sqrt(eps), then +eps again in the divide), singleton groups -> 0, broadcast over
``response_mask``.  Three launches: ragged row sum, one-workgroup group
statistics, masked broadcast.
"""

from __future__ import annotations

import torch

from axon_amd import _ops
from axon_amd.trainer.algos.advantages.registry import AdvantageFn, register_advantage
from axon_amd.utils.rl.advantage import as_torch_index


def _stage(t: torch.Tensor):
    """Tensors produced on the driver live on the CPU; the kernels need them in HBM."""
    if t.is_cuda:
        return t, None
    if not torch.cuda.is_available():
        _ops.require_device(t, "grpo_advantage_fn")
    return t.cuda(), t.device


def _group_advantage(data, mode: int, eps: float, clamp_abs: float):
    """score = sum of token rewards per row -> per-row scalar by group (mode: axon_group_stats) ->
    broadcast over the response mask."""
    rewards, home = _stage(data.batch["token_level_rewards"])
    mask, _ = _stage(data.batch["response_mask"])
    uid = data.non_tensor_batch["uid"]
    norm = mode

    cu = data.meta_info.get("cu_seqlens", None) if data.meta_info else None
    rows = _ops.rows_of(rewards, cu)
    # group ids are ranked on the host (labels are strings); the group count is read there as well, so
    # that nothing here waits for the GPU
    gidx_host = as_torch_index(uid, device="cpu")
    if gidx_host.numel() != rows.n_rows:
        raise ValueError(f"uid has {gidx_host.numel()} entries, batch has {rows.n_rows} rows")
    n_groups = int(gidx_host.max()) + 1 if gidx_host.numel() else 0
    gidx = gidx_host.to(rewards.device, non_blocking=True)
    _, scores, _ = _ops.row_stats(rewards, None, None, rows, want_cnt=False)
    _, _, _, scalar = _ops.group_stats(scores, gidx, n_groups, eps, norm)
    adv = _ops.row_broadcast_mask(scalar, mask, rows, clamp_abs=clamp_abs)
    if home is not None:
        adv = adv.to(home)
    return adv, adv


@register_advantage(AdvantageFn.GRPO)
def grpo_advantage_fn(data, config, clamp_abs: float = 0.0) -> tuple[torch.Tensor, torch.Tensor]:
    """Group-normalised outcome advantage (advantage.py:78-109)."""
    mode = 1 if config.get("norm_adv_by_std", True) else 0
    return _group_advantage(data, mode, config.get("epsilon", 1e-6), clamp_abs)


@register_advantage(AdvantageFn.RLOO)
@register_advantage(AdvantageFn.LOOP)
def rloo_advantage_fn(data, config, clamp_abs: float = 0.0) -> tuple[torch.Tensor, torch.Tensor]:
    """Leave-one-out advantage ``(n*s_i - S_g)/(n-1)``, 0 for singleton groups (advantage.py:112-146)."""
    return _group_advantage(data, 2, 1e-6, clamp_abs)


@register_advantage(AdvantageFn.GPG)
def gpg_advantage_fn(data, config, clamp_abs: float = 0.0) -> tuple[torch.Tensor, torch.Tensor]:
    """``alpha * (score - group_mean) / f_norm`` with ``alpha = rows / count_nonzero(scores)``
    (advantage.py:336-371)."""
    return _group_advantage(data, 3, float(config.get("f_norm", 1.0)), clamp_abs)
