"""Facade with the surface of the reference's mops/__init__.py:1-26.

The backend is read once from the BACKEND environment variable (here defaulting to "hip"), the `hip`
backend is imported, and the eleven op handles are bound as module attributes so that layer code can
keep writing `from mops import store_kvcache, flash_attn_varlen_func, ...`.
Only the `hip` backend ships in this package; other backend names stay valid registry keys so that a
test harness (or the reference's own backends) can register into them and be fetched side by side with
`get_op(name, backend=...)`.
"""
import os

from .registry import get_current_backend, get_op, has_op, register_op, set_current_backend

_BACKEND = os.environ.get("BACKEND", "hip").lower()
set_current_backend(_BACKEND)

from . import hip  # noqa: E402  (registers the hip ops)

OP_NAMES = (
    "linear",
    "rms_forward",
    "add_rms_forward",
    "softmax",
    "siluAndMul",
    "sampler_forward",
    "apply_rotary_emb",
    "embedding",
    "store_kvcache",
    "flash_attn_varlen_func",
    "flash_attn_with_kvcache",
)

# Operators this backend adds to the reference's eleven; a backend need not provide them.
EXTENSION_OP_NAMES = ("qk_norm_rope_store",)


def rebind(backend: str = None) -> None:
    """(Re)binds the module-level op handles to `backend` (default: the current one)."""
    if backend is not None:
        set_current_backend(backend)
    g = globals()
    for name in OP_NAMES:
        g[name] = get_op(name)
    for name in EXTENSION_OP_NAMES:
        g[name] = get_op(name) if has_op(name) else None


rebind()
