"""Advantage estimation (axon/trainer/algos/advantages/__init__.py:38-79)."""

from __future__ import annotations

from enum import Enum

import torch

from axon_amd.trainer.algos.advantages import advantage as _advantage  # noqa: F401  (registers grpo)
from axon_amd.trainer.algos.advantages.registry import (
    AdvantageFn,
    AdvantageRegistryEntry,
    _advantage_registry,
    get_advantage_entry,
    get_advantage_fn,
    register_advantage,
)


def _cfg_get(config, key, default=None):
    if isinstance(config, dict):
        return config.get(key, default)
    return getattr(config, key, default)


def compute_advantage(data, config=None):
    """Look up ``config.advantage`` in the registry, pass ``config.advantage_args`` as the
    estimator's config, optionally clamp to [-1, 1], and write ``advantages`` / ``returns``."""
    name = _cfg_get(config, "advantage")
    if name is None:
        raise ValueError("Config must have 'advantage' field specifying the estimator name")
    if isinstance(name, Enum):
        name = name.value
    adv_cfg = _cfg_get(config, "advantage_args", {}) or {}
    advantages, returns = _advantage_registry.compute(name, data, adv_cfg)
    if adv_cfg.get("clip_advantages", False):
        advantages = torch.clamp(advantages, -1, 1)
    data.batch["advantages"] = advantages
    data.batch["returns"] = returns
    return data


__all__ = [
    "AdvantageFn", "AdvantageRegistryEntry", "register_advantage", "get_advantage_entry", "get_advantage_fn",
    "compute_advantage",
]
