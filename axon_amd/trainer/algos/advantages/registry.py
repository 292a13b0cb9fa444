"""Advantage-estimator registry (axon/trainer/algos/advantages/registry.py:44-88)."""

from __future__ import annotations

from enum import Enum

from axon_amd.utils.registry import FunctionRegistry, FunctionRegistryEntry

AdvantageRegistryEntry = FunctionRegistryEntry


class AdvantageFn(str, Enum):
    """The reference's estimator names (registry.py:44-59)."""

    GAE = "gae"
    GRPO = "grpo"
    RLOO = "rloo"
    LOOP = "loop"  # alias of RLOO
    REINFORCE_PLUS_PLUS = "reinforce_plus_plus"
    REINFORCE_PLUS_PLUS_BASELINE = "reinforce_plus_plus_baseline"
    REMAX = "remax"
    OPO = "opo"
    GRPO_PASSK = "grpo_passk"
    GPG = "gpg"
    CHUNKED_GAE = "chunked_gae"
    IDENTITY = "identity"
    KIMI_K1_5 = "kimi_k1_5"


_advantage_registry: FunctionRegistry = FunctionRegistry(name="advantage estimator")
ADV_REGISTRY = _advantage_registry._registry


def register_advantage(name_or_enum):
    """Decorator: ``fn(data: DataProto, config: dict-like) -> (advantages, returns)``."""
    return _advantage_registry.register(name_or_enum)


def get_advantage_entry(name_or_enum) -> AdvantageRegistryEntry:
    return _advantage_registry.get_entry(name_or_enum)


def get_advantage_fn(name_or_enum):
    return _advantage_registry.get_fn(name_or_enum)
