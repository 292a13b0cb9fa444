from .trainer_sampler_mismatch_metrics import (  # noqa: F401
    aggregate_trainer_sampler_metrics,
    compute_trainer_sampler_mismatch_metrics,
)
