"""The advantage estimators of axon/trainer/algos/advantages/advantage.py on the HIP path.

``grpo_advantage_fn`` follows advantage.py:78-109: score = sum_t token_level_rewards, per-uid mean/std
(Bessel, std floored at sqrt(eps), then +eps again in the divide), singleton groups -> 0, broadcast over
``response_mask``.  Three launches: ragged row sum, one-workgroup group statistics, masked broadcast.  The
other group-based estimators differ in the per-row scalar only.  The return-based estimators (GAE,
REINFORCE++, ReMax) run their time recurrence as a wavefront scan per row, then the global masked
whitening where the reference has one.  Group labels are ranked on the host (they are strings); nothing
here waits for the GPU.
"""

from __future__ import annotations

import collections

import numpy as np
import torch

from axon_amd import _ops
from axon_amd.trainer.algos.advantages.registry import AdvantageFn, register_advantage
from axon_amd.utils.rl.advantage import as_torch_index


def _rows(data, like):
    cu = data.meta_info.get("cu_seqlens", None) if getattr(data, "meta_info", None) else None
    return _ops.rows_of(like, cu)


def _home(t, home):
    return t if home is None else t.to(home)


# Ranking the group labels (strings: a sort on the host) costs more than the kernels of a small batch, and a
# trainer asks for the same labels again on every pass over a batch: the ranking is kept per label sequence.
_RANKED: "collections.OrderedDict" = collections.OrderedDict()
_RANKED_MAX = 16


def _ranked_groups(uid, device=None):
    """``(gidx on the host, n_groups, gidx on `device` or None)`` for the group labels ``uid``; remembered for
    label arrays (the key is the label sequence itself, so equal labels always give the same answer)."""
    key = None
    if isinstance(uid, np.ndarray) and uid.ndim == 1:
        key = (uid.dtype.str, tuple(uid.tolist()) if uid.dtype == object else uid.tobytes())
        hit = _RANKED.get(key)
        if hit is not None:
            _RANKED.move_to_end(key)
    else:
        hit = None
    if hit is None:
        gidx = as_torch_index(uid, device="cpu")
        n_groups = int(gidx.max()) + 1 if gidx.numel() else 0
        hit = [gidx, n_groups, {}]
        if key is not None:
            _RANKED[key] = hit
            while len(_RANKED) > _RANKED_MAX:
                _RANKED.popitem(last=False)
    on_dev = None
    if device is not None:
        on_dev = hit[2].get(device)
        if on_dev is None:
            on_dev = hit[0].to(device)
            hit[2][device] = on_dev
    return hit[0], hit[1], on_dev


def _host_groups(data, n_rows: int):
    """``(gidx on the host, n_groups, members, offsets)``: members lists the rows group by group (row order
    kept inside a group), offsets[g] .. offsets[g+1] is group g's range in it."""
    gidx, n_groups, _ = _ranked_groups(data.non_tensor_batch["uid"])
    if gidx.numel() != n_rows:
        raise ValueError(f"uid has {gidx.numel()} entries, batch has {n_rows} rows")
    if gidx.numel() and int(gidx.min()) < 0:
        raise ValueError("group labels must be non-negative")
    members = torch.argsort(gidx, stable=True)
    offsets = torch.zeros(n_groups + 1, dtype=torch.int64)
    if n_groups:
        offsets[1:] = torch.cumsum(torch.bincount(gidx, minlength=n_groups), 0)
    return gidx, n_groups, members, offsets


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
    gidx_host, n_groups, gidx = _ranked_groups(uid, rewards.device)
    if gidx_host.numel() != rows.n_rows:
        raise ValueError(f"uid has {gidx_host.numel()} entries, batch has {rows.n_rows} rows")
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


def _group_scalar_advantage(data, mode: int, *, want_lens: bool, eps=1e-6, normalize=True, coef=0.0, threshold=1.0,
                            check_groups=None):
    rewards, home = _stage(data.batch["token_level_rewards"])
    mask, _ = _stage(data.batch["response_mask"])
    rows = _rows(data, rewards)
    gidx, n_groups, members, offsets = _host_groups(data, rows.n_rows)
    if check_groups is not None:
        check_groups(gidx, offsets)
    _, scores, _ = _ops.row_stats(rewards, None, None, rows, want_cnt=False)
    lens = None
    if want_lens:
        lens, _, _ = _ops.row_stats(rewards, None, mask, rows, want_sum=False)
    scalar = _ops.group_scalar(mode, scores, lens, members, offsets, n_groups, eps=eps, normalize=normalize, coef=coef,
                               threshold=threshold)
    return _ops.row_broadcast_mask(scalar, mask, rows), mask, home


@register_advantage(AdvantageFn.GAE)
def gae_advantage_fn(data, config) -> tuple[torch.Tensor, torch.Tensor]:
    """Generalised advantage estimation (advantage.py:40-75): the time loop as a scan per row, returns =
    raw advantages + values, advantages whitened over the response mask."""
    rewards, home = _stage(data.batch["token_level_rewards"])
    values, _ = _stage(data.batch["values"])
    mask, _ = _stage(data.batch["response_mask"])
    adv, ret = _ops.reverse_scan(_ops.SCAN_GAE, rewards, values, mask, _rows(data, rewards),
                                 gamma=config.get("gamma", 0.99), lam=config.get("lam", 0.95))
    adv, _ = _ops.masked_whiten(adv, mask, inplace=True)
    return _home(adv, home), _home(ret, home)


@register_advantage(AdvantageFn.CHUNKED_GAE)
def chunked_gae_advantage_fn(data, config) -> tuple[torch.Tensor, torch.Tensor]:
    """GAE over the response tokens only, zero elsewhere, then whitened (advantage.py:480-540).  The reference
    splits the recurrence into ``chunk_size`` blocks to shorten its Python loop; the scan here has no such
    loop, so ``chunk_size`` is accepted and not used."""
    rewards, home = _stage(data.batch["token_level_rewards"])
    values, _ = _stage(data.batch["values"])
    mask, _ = _stage(data.batch["response_mask"])
    adv, ret = _ops.reverse_scan(_ops.SCAN_GAE_RESPONSE_ONLY, rewards, values, mask, _rows(data, rewards),
                                 gamma=config.get("gamma", 0.99), lam=config.get("lam", 0.95))
    adv, _ = _ops.masked_whiten(adv, mask, inplace=True)
    return _home(adv, home), _home(ret, home)


@register_advantage(AdvantageFn.REINFORCE_PLUS_PLUS)
def reinforce_plus_plus_advantage_fn(data, config) -> tuple[torch.Tensor, torch.Tensor]:
    """Discounted returns that restart after the response ends, whitened and masked (advantage.py:149-176)."""
    rewards, home = _stage(data.batch["token_level_rewards"])
    mask, _ = _stage(data.batch["response_mask"])
    _, ret = _ops.reverse_scan(_ops.SCAN_DISCOUNTED, rewards, None, mask, _rows(data, rewards),
                               gamma=config.get("gamma", 1.0))
    adv, _ = _ops.masked_whiten(ret, mask, remask=True)
    return _home(adv, home), _home(ret, home)


@register_advantage(AdvantageFn.REINFORCE_PLUS_PLUS_BASELINE)
def reinforce_plus_plus_baseline_advantage_fn(data, config) -> tuple[torch.Tensor, torch.Tensor]:
    """Score minus the group mean (0 for a group of one), broadcast, then whitened over the whole batch and
    masked (advantage.py:179-217)."""
    spread, mask, home = _group_scalar_advantage(data, _ops.GROUP_MEAN_BASELINE, want_lens=False)
    adv, _ = _ops.masked_whiten(spread, mask, remask=True, inplace=True)
    adv = _home(adv, home)
    return adv, adv


@register_advantage(AdvantageFn.REMAX)
def remax_advantage_fn(data, config) -> tuple[torch.Tensor, torch.Tensor]:
    """Reward-to-go of the masked rewards minus the greedy-decoding baseline (advantage.py:220-240)."""
    rewards, home = _stage(data.batch["token_level_rewards"])
    mask, _ = _stage(data.batch["response_mask"])
    base, _ = _stage(data.batch["reward_baselines"])
    adv, ret = _ops.reverse_scan(_ops.SCAN_SUFFIX_SUM, rewards, None, mask, _rows(data, rewards), row_baseline=base)
    return _home(adv, home), _home(ret, home)


@register_advantage(AdvantageFn.OPO)
def opo_advantage_fn(data, config) -> tuple[torch.Tensor, torch.Tensor]:
    """Score minus the length-weighted group baseline, 0 baseline for a group of one (advantage.py:243-280)."""
    adv, _, home = _group_scalar_advantage(data, _ops.GROUP_OPO, want_lens=True)
    adv = _home(adv, home)
    return adv, adv


@register_advantage(AdvantageFn.GRPO_PASSK)
def grpo_passk_advantage_fn(data, config) -> tuple[torch.Tensor, torch.Tensor]:
    """Only the best response of a group gets ``r_max - r_second_max`` (over std + eps when
    ``norm_adv_by_std``); a group of one sample raises (advantage.py:283-333)."""
    uid = data.non_tensor_batch["uid"]

    def check_groups(gidx, offsets):
        sizes = offsets[1:] - offsets[:-1]
        small = torch.nonzero((sizes > 0) & (sizes < 2)).flatten()
        if small.numel():
            row = int(torch.nonzero(gidx == int(small[0])).flatten()[0])
            raise ValueError(f"Pass@k requires at least 2 samples per group. Got 1 for group {uid[row]}.")

    adv, _, home = _group_scalar_advantage(data, _ops.GROUP_PASSK, want_lens=False, eps=config.get("epsilon", 1e-6),
                                           normalize=config.get("norm_adv_by_std", True), check_groups=check_groups)
    adv = _home(adv, home)
    return adv, adv


@register_advantage(AdvantageFn.KIMI_K1_5)
def kimi_k1_5_advantage_fn(data, config) -> tuple[torch.Tensor, torch.Tensor]:
    """GRPO on scores shaped by the Kimi k1.5 length reward (advantage.py:543-626): ``length_coef`` follows the
    warm-up / ramp schedule on ``data.meta_info["global_steps"]``; the length term is
    ``coef * (0.5 - (len - min)/(max - min))`` over the whole group, capped at 0 for scores below
    ``correct_threshold``, off when all lengths agree."""
    target = float(config.get("length_coef", 0.0))
    warmup = int(config.get("length_coef_warmup_steps", 0))
    ramp = int(config.get("length_coef_ramp_steps", 0))
    step = 0
    if getattr(data, "meta_info", None):
        step = int(data.meta_info.get("global_steps", 0) or 0)
    if step < warmup:
        coef = 0.0
    elif ramp > 0 and step < warmup + ramp:
        coef = target * (step - warmup) / ramp
    else:
        coef = target
    adv, _, home = _group_scalar_advantage(
        data, _ops.GROUP_KIMI, want_lens=True, eps=config.get("epsilon", 1e-6),
        normalize=config.get("norm_adv_by_std", True), coef=coef,
        threshold=float(config.get("correct_threshold", 1.0)))
    adv = _home(adv, home)
    return adv, adv


@register_advantage(AdvantageFn.IDENTITY)
def identity_advantage_fn(data, config) -> tuple[torch.Tensor, torch.Tensor]:
    """``token_level_rewards * response_mask`` (advantage.py:629-645): the program computed the advantages
    already.  One elementwise multiply; torch's own kernel does it."""
    rewards, home = _stage(data.batch["token_level_rewards"])
    mask, _ = _stage(data.batch["response_mask"])
    _ops.require_device(rewards, "identity_advantage_fn")
    adv = _home(rewards * mask, home)
    return adv, adv
