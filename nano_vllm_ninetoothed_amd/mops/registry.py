"""String-keyed operator registry with the API of the reference's mops/registry.py:1-39.

Same three functions, same error behaviour: `set_current_backend` raises ValueError for an unknown
backend (registry.py:13-18), `register_op(backend)` keys the function by its `__name__` and raises
RuntimeError on a duplicate (registry.py:21-29), `get_op` prints a message and returns None when the op
is missing (registry.py:32-39).  The closed set of backend names gains one key, "hip".
"""
from typing import Callable, Dict, Optional

_BACKEND_REGISTRY: Dict[str, Dict[str, Callable]] = {
    "triton": {},
    "ninetoothed": {},
    "torch": {},
    "hip": {},
}

_CURRENT_BACKEND: Optional[str] = None


def set_current_backend(backend: str) -> None:
    global _CURRENT_BACKEND
    if backend not in _BACKEND_REGISTRY:
        raise ValueError(f"Backend {backend} not supported")
    _CURRENT_BACKEND = backend


def get_current_backend() -> Optional[str]:
    return _CURRENT_BACKEND


def register_op(backend: str):
    def decorator(func: Callable) -> Callable:
        op_name = func.__name__
        if op_name in _BACKEND_REGISTRY[backend]:
            raise RuntimeError(f"Operator {op_name} already registered for {backend}")
        _BACKEND_REGISTRY[backend][op_name] = func
        return func

    return decorator


def has_op(op_name: str, backend: str = None) -> bool:
    """True if `backend` (default: the current one) registered `op_name`; unlike get_op it prints nothing."""
    return op_name in _BACKEND_REGISTRY.get(backend if backend is not None else _CURRENT_BACKEND, {})


def get_op(op_name: str, backend: str = None) -> Callable:
    if backend is None:
        backend = _CURRENT_BACKEND
    op = _BACKEND_REGISTRY[backend].get(op_name)
    if op is None:
        print(f"Operator [{op_name}] not found in {backend} backend")
    return op
