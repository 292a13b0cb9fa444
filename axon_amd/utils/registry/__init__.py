from .function_registry import FunctionRegistry, FunctionRegistryEntry

__all__ = ["FunctionRegistry", "FunctionRegistryEntry"]
