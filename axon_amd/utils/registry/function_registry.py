"""Name -> function registry with the reference's re-registration rule.

Same surface as axon/utils/registry/function_registry.py:62-158: ``register``
is a decorator factory taking a str or Enum; registering a *different*
function under a taken name raises ``ValueError`` (:112-113); the same function
may be registered again.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum
from typing import Callable, Generic, TypeVar

T = TypeVar("T")

__all__ = ["FunctionRegistry", "FunctionRegistryEntry"]


@dataclass
class FunctionRegistryEntry:
    fn: Callable


def _key(name_or_enum) -> str:
    return name_or_enum.value if isinstance(name_or_enum, Enum) else name_or_enum


class FunctionRegistry(Generic[T]):
    def __init__(self, name: str):
        self.name = name
        self._registry: dict[str, FunctionRegistryEntry] = {}

    def register(self, name_or_enum):
        key = _key(name_or_enum)

        def bind(fn):
            taken = self._registry.get(key)
            if taken is not None and taken.fn != fn:
                raise ValueError(f"{self.name.title()} '{key}' already registered with different function")
            self._registry[key] = FunctionRegistryEntry(fn=fn)
            return fn

        return bind

    def get_entry(self, name_or_enum) -> FunctionRegistryEntry:
        key = _key(name_or_enum)
        try:
            return self._registry[key]
        except KeyError:
            raise ValueError(f"Unknown {self.name}: '{key}'. Available: {list(self._registry)}") from None

    def get_fn(self, name_or_enum) -> Callable[..., T]:
        return self.get_entry(name_or_enum).fn

    def compute(self, name_or_enum, data, config) -> T:
        return self.get_entry(name_or_enum).fn(data, config)

    def keys(self) -> list[str]:
        return list(self._registry)

    def __contains__(self, name_or_enum) -> bool:
        return _key(name_or_enum) in self._registry
