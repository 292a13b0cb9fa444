"""Minimal DataProto: the subset of axon/protocol.py:362-378 the hot path touches.

The reference type wraps a ``tensordict.TensorDict``; the loss, advantage and
sampler-correction functions only use ``data.batch[k]``, ``data.batch.get``,
``k in data.batch``, ``data.batch[k] = v``, ``data.non_tensor_batch[...]``,
``data.meta_info``, ``len(data)``, ``from_dict`` (protocol.py:518-563),
``union`` (:757-772), ``select`` (:611-640) and ``select_idxs`` (:642-668).
This shim provides exactly those on a plain dict so that neither ``tensordict``
nor ``ray`` is needed.  A real TensorDict also satisfies every access made by
the functions in this package.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass, field

import numpy as np
import torch

__all__ = ["DataProto", "TensorBatch"]


class TensorBatch(dict):
    """dict of tensors sharing dim 0 — the slice of the TensorDict API used here."""

    def __init__(self, tensors=None, batch_size=None):
        super().__init__(tensors or {})
        if batch_size is None:
            batch_size = next(iter(self.values())).shape[:1] if len(self) else (0,)
        self.batch_size = torch.Size(tuple(batch_size))

    def __setitem__(self, key, value):
        if isinstance(value, torch.Tensor) and len(self.batch_size) and value.dim() > 0:
            if value.shape[0] != self.batch_size[0]:
                raise RuntimeError(
                    f"batch dimension mismatch for '{key}': got {tuple(value.shape)}, expected dim 0 = {self.batch_size[0]}"
                )
        super().__setitem__(key, value)

    def select(self, *keys) -> "TensorBatch":
        return TensorBatch({k: self[k] for k in keys}, self.batch_size)

    def to(self, device) -> "TensorBatch":
        return TensorBatch({k: v.to(device) for k, v in self.items()}, self.batch_size)

    @property
    def device(self):
        return next(iter(self.values())).device if len(self) else None


def _same(a, b) -> bool:
    if isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor):
        return a.shape == b.shape and bool(torch.equal(a, b))
    if isinstance(a, np.ndarray) or isinstance(b, np.ndarray):
        return np.array_equal(np.asarray(a), np.asarray(b))
    return a == b


def _merge(dst: dict, src: dict, what: str) -> dict:
    for key, val in src.items():
        if key in dst:
            assert _same(dst[key], val), f"Conflicting values for {what} key '{key}'"
        else:
            dst[key] = val
    return dst


@dataclass
class DataProto:
    batch: TensorBatch | None = None
    non_tensor_batch: dict = field(default_factory=dict)
    meta_info: dict = field(default_factory=dict)

    def __post_init__(self):
        if self.batch is not None and not hasattr(self.batch, "batch_size"):
            self.batch = TensorBatch(dict(self.batch))
        n = len(self)
        for key, val in self.non_tensor_batch.items():
            assert isinstance(val, np.ndarray), f"non_tensor_batch['{key}'] must be a numpy array"
            assert val.shape[0] == n, f"non_tensor_batch['{key}'] has {val.shape[0]} rows, batch has {n}"

    def __len__(self) -> int:
        if self.batch is not None:
            return int(self.batch.batch_size[0])
        if self.non_tensor_batch:
            return int(next(iter(self.non_tensor_batch.values())).shape[0])
        return 0

    @classmethod
    def from_dict(cls, tensors=None, non_tensors=None, meta_info=None) -> "DataProto":
        tensors = dict(tensors) if tensors else {}
        rows = None
        first = None
        for key, t in tensors.items():
            if rows is None:
                rows, first = t.shape[0], key
            assert t.shape[0] == rows, f"Batch size mismatch: '{first}' has {rows}, '{key}' has {t.shape[0]}"
        nt = {
            k: (v if isinstance(v, np.ndarray) else np.array(v, dtype=object))
            for k, v in (non_tensors or {}).items()
        }
        batch = TensorBatch(tensors, (rows,)) if tensors else None
        return cls(batch=batch, non_tensor_batch=nt, meta_info=dict(meta_info or {}))

    def to(self, device) -> "DataProto":
        if self.batch is not None:
            self.batch = self.batch.to(device)
        return self

    def select(self, batch_keys=None, non_tensor_batch_keys=None, meta_info_keys=None, deepcopy=False):
        batch = self.batch.select(*batch_keys) if batch_keys else self.batch
        nt = (
            {k: v for k, v in self.non_tensor_batch.items() if k in non_tensor_batch_keys}
            if non_tensor_batch_keys
            else self.non_tensor_batch
        )
        meta = {k: v for k, v in self.meta_info.items() if k in meta_info_keys} if meta_info_keys else self.meta_info
        if deepcopy:
            nt, meta = copy.deepcopy(nt), copy.deepcopy(meta)
        return type(self)(batch=batch, non_tensor_batch=nt, meta_info=meta)

    def select_idxs(self, idxs) -> "DataProto":
        if isinstance(idxs, list):
            is_bool = any(isinstance(i, bool) for i in idxs)
            idxs = torch.tensor(idxs, dtype=torch.bool if is_bool else torch.int64)
        idx_t = torch.from_numpy(idxs) if isinstance(idxs, np.ndarray) else idxs
        idx_np = idxs if isinstance(idxs, np.ndarray) else idx_t.detach().cpu().numpy()
        rows = int(idx_np.sum()) if idx_np.dtype == bool else int(idx_np.shape[0])
        batch = None
        if self.batch is not None:
            batch = TensorBatch({k: v[idx_t.to(v.device)] for k, v in self.batch.items()}, (rows,))
        return type(self)(
            batch=batch,
            non_tensor_batch={k: v[idx_np] for k, v in self.non_tensor_batch.items()},
            meta_info=self.meta_info,
        )

    def union(self, other: "DataProto") -> "DataProto":
        if other.batch is not None:
            if self.batch is None:
                self.batch = TensorBatch(dict(other.batch), other.batch.batch_size)
            else:
                assert self.batch.batch_size == other.batch.batch_size, (
                    f"Batch sizes must match: {self.batch.batch_size} vs {other.batch.batch_size}"
                )
                _merge(self.batch, other.batch, "batch")
        _merge(self.non_tensor_batch, other.non_tensor_batch, "non_tensor_batch")
        _merge(self.meta_info, other.meta_info, "meta_info")
        return self
