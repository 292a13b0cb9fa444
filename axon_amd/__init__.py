"""axon_amd — MI355X-native trainer-side per-token hot path.

LM-head log-prob/entropy (fused, logits never materialised), sampler–trainer
correction, GRPO advantage and the PPO/DAPO/GSPO clipped loss, behind the same
plugin points modelcorp/axon exposes (``linear_cross_entropy``,
``@register_loss``, ``@register_advantage``).  Module paths mirror the
reference's (``axon.X`` -> ``axon_amd.X``) for the parts that exist here.
All computation runs in hand-written HIP kernels in ``libaxon_amd.so``.
"""

from . import _lib  # noqa: F401

__version__ = "0.1.0"
