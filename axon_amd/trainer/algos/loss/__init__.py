"""Policy losses (axon/trainer/algos/loss)."""

from axon_amd.trainer.algos.loss import loss as _loss  # noqa: F401  (registers the functions)
from axon_amd.trainer.algos.loss.registry import (
    LossFn,
    LossRegistryEntry,
    compute_loss_fn,
    get_loss_entry,
    get_loss_fn,
    register_loss,
)
from axon_amd.trainer.algos.loss.utils import agg_loss, masked_mean

__all__ = [
    "LossFn", "LossRegistryEntry", "compute_loss_fn", "get_loss_entry", "get_loss_fn", "register_loss",
    "agg_loss", "masked_mean",
]
