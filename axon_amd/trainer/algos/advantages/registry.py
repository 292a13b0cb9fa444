"""Advantage-estimator registry (axon/trainer/algos/advantages/registry.py:44-88)."""

from __future__ import annotations

from enum import Enum

from axon_amd.utils.registry import FunctionRegistry, FunctionRegistryEntry

AdvantageRegistryEntry = FunctionRegistryEntry


class AdvantageFn(str, Enum):
    """Estimators this path provides (the outcome-reward, group-baseline family; the reference also
    lists GAE and other value- or return-based estimators)."""

    GRPO = "grpo"
    RLOO = "rloo"
    LOOP = "loop"  # alias of RLOO
    GPG = "gpg"


_advantage_registry: FunctionRegistry = FunctionRegistry(name="advantage estimator")
ADV_REGISTRY = _advantage_registry._registry


def register_advantage(name_or_enum):
    """Decorator: ``fn(data: DataProto, config: dict-like) -> (advantages, returns)``."""
    return _advantage_registry.register(name_or_enum)


def get_advantage_entry(name_or_enum) -> AdvantageRegistryEntry:
    return _advantage_registry.get_entry(name_or_enum)


def get_advantage_fn(name_or_enum):
    return _advantage_registry.get_fn(name_or_enum)
