"""Group helpers ``as_torch_index`` and ``group_mean_std``, and the masked moments ``masked_mean``,
``masked_var``, ``masked_whiten``.

Same behaviour as axon/utils/rl/advantage.py:46-190.  ``as_torch_index`` is host logic (``np.unique`` over
arbitrary labels); ``group_mean_std`` runs in libaxon_amd.so (``axon_group_stats``), the masked moments in
``axon_masked_whiten`` (sums in a fixed order, statistics left on the device).
"""

from __future__ import annotations

from typing import Any

import numpy as np
import torch

from axon_amd import _lib, _ops

__all__ = ["as_torch_index", "group_mean_std", "masked_mean", "masked_var", "masked_whiten"]

_INT_DTYPES = (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8, torch.bool)
_FLOAT_DTYPES = (torch.float16, torch.float32, torch.float64, torch.bfloat16)


def _inverse_index(labels: np.ndarray) -> np.ndarray:
    try:
        inv = np.unique(labels, return_inverse=True)[1]
    except Exception:  # labels of mixed, unorderable types: compare their str()
        inv = np.unique(np.array([str(x) for x in labels], dtype=object), return_inverse=True)[1]
    return inv.reshape(-1).astype(np.int64, copy=False)


def as_torch_index(index: Any, device=None) -> torch.Tensor:
    """Group labels -> 1-D int64 tensor.

    Integer (and bool) labels pass through unchanged, floats that are whole numbers are
    rounded, everything else is ranked with ``np.unique`` so equal labels share an id.
    """
    target = device if device is not None else ("cuda" if torch.cuda.is_available() else "cpu")

    if isinstance(index, torch.Tensor):
        flat = index.reshape(-1)
        if flat.dtype in _INT_DTYPES:
            return flat.to(device=target, dtype=torch.long)
        if flat.dtype in _FLOAT_DTYPES:
            wide = flat.to(torch.float64)
            whole = torch.round(wide)
            if torch.allclose(wide, whole, rtol=0.0, atol=1e-6):
                return whole.to(device=target, dtype=torch.long)
        labels = np.array([str(x.item()) for x in flat], dtype=object)
        return torch.from_numpy(_inverse_index(labels)).to(target)

    try:
        arr = np.asarray(index)
    except Exception:
        arr = np.array(list(index), dtype=object)
    arr = arr.reshape(-1)
    if arr.dtype != object:
        if np.issubdtype(arr.dtype, np.integer):
            return torch.from_numpy(arr.astype(np.int64, copy=False)).to(target)
        if np.issubdtype(arr.dtype, np.floating):
            whole = np.rint(arr.astype(np.float64))
            if np.allclose(arr.astype(np.float64), whole, rtol=0.0, atol=1e-6):
                return torch.from_numpy(whole.astype(np.int64)).to(target)
    try:  # numeric strings, bools, ints stored as objects
        return torch.from_numpy(arr.astype(np.int64)).to(target)
    except Exception:
        pass
    return torch.from_numpy(_inverse_index(arr.astype(object))).to(target)


@torch.no_grad()
def group_mean_std(scores: torch.Tensor, gidx: torch.Tensor, eps: float = 1e-6, device=None):
    """Per-group (mean, std, count) with Bessel correction; groups of one get mean 0, std 1."""
    target = device if device is not None else scores.device
    scores = scores.reshape(-1).to(device=target, dtype=torch.float32)
    gidx = gidx.reshape(-1).to(device=target, dtype=torch.long)
    if scores.numel() != gidx.numel():
        raise ValueError(f"scores and gidx length mismatch: {scores.numel()} vs {gidx.numel()}")
    if gidx.numel() == 0:
        empty = torch.empty(0, device=target, dtype=torch.float32)
        return empty, empty, empty
    _lib.require_device(scores, "group_mean_std")
    n_groups = int(gidx.max().item()) + 1
    mean, std, count, _ = _ops.group_stats(scores, gidx, n_groups, eps, want_scalar=False)
    return mean, std, count


@torch.no_grad()
def masked_mean(values: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """``sum(values * mask) / max(sum(mask), 1)`` as a 0-d device tensor (advantage.py:153-157)."""
    _, stats = _ops.masked_whiten(values, mask, stats_only=True)
    return stats[0]


@torch.no_grad()
def masked_var(values: torch.Tensor, mask: torch.Tensor, bessel_correction: bool = True) -> torch.Tensor:
    """Masked variance about the masked mean, times n/(n-1) when n > 1 (advantage.py:160-170)."""
    _, stats = _ops.masked_whiten(values, mask, stats_only=True)
    if bessel_correction:
        return stats[2]
    n = stats[1]
    return torch.where(n > 1, stats[2] * (n - 1) / n.clamp_min(1.0), stats[2])


@torch.no_grad()
def masked_whiten(values: torch.Tensor, mask: torch.Tensor, shift_mean: bool = True) -> torch.Tensor:
    """``(values - mean) * rsqrt(var + 1e-8)`` with the moments taken over the mask; the mean is added back when
    ``shift_mean`` is False (advantage.py:173-190)."""
    out, stats = _ops.masked_whiten(values, mask)
    out = out.view(values.shape)
    return out if shift_mean else out + stats[0]
