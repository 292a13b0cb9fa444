"""Policy-loss registry and dispatcher.

Mirrors axon/trainer/algos/loss/registry.py:36-111: ``register_loss`` /
``get_loss_fn`` / ``compute_loss_fn``.  ``compute_loss_fn`` first applies the
sampler–trainer correction when any of ``sampler_is`` / ``sampler_rs`` /
``sampler_token_veto_threshold`` is set and the batch carries
``sampler_log_probs`` (:97-106), then calls the registered loss with
``loss_fn_args`` as its config (:108).
"""

from __future__ import annotations

from enum import Enum
from typing import Any

from axon_amd.utils.registry import FunctionRegistry, FunctionRegistryEntry

LossRegistryEntry = FunctionRegistryEntry


class LossFn(str, Enum):
    """Losses this path provides (the reference enum also lists clip_cov, kl_cov and value, which are
    not on it)."""

    PPO = "ppo"
    GSPO = "gspo"
    GPG = "gpg"
    CLIP_COV = "clip_cov"
    KL_COV = "kl_cov"
    CISPO = "cispo"
    REINFORCE = "reinforce"
    GEO_MEAN = "geo_mean"
    VALUE = "value"


_loss_registry: FunctionRegistry = FunctionRegistry(name="policy loss")


def register_loss(name_or_enum):
    """Decorator: ``fn(data: DataProto, config: dict-like) -> (loss, metrics)``."""
    return _loss_registry.register(name_or_enum)


def get_loss_entry(name_or_enum) -> LossRegistryEntry:
    return _loss_registry.get_entry(name_or_enum)


def get_loss_fn(name_or_enum):
    return _loss_registry.get_fn(name_or_enum)


_SAMPLER_SWITCHES = ("sampler_is", "sampler_rs", "sampler_token_veto_threshold")


def compute_loss_fn(data, loss_fn: str, loss_fn_args: dict | None = None) -> tuple[Any, dict[str, Any]]:
    args = {} if loss_fn_args is None else loss_fn_args
    fn = _loss_registry.get_fn(loss_fn)

    corr_metrics: dict[str, Any] = {}
    wants_correction = any(args.get(k, None) is not None for k in _SAMPLER_SWITCHES)
    if wants_correction and "sampler_log_probs" in data.batch:
        from axon_amd.utils.rl.sampler import compute_sampler_correction_and_add_to_batch

        data, corr_metrics = compute_sampler_correction_and_add_to_batch(data, args)

    loss, metrics = fn(data, args)
    metrics.update(corr_metrics)
    return loss, metrics
