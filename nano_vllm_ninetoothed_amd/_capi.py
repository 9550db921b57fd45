"""ctypes binding of libmops_hip.so — the only way the Python host code reaches the HIP kernels.

The library is loaded lazily on first use and the load fails loudly: there is no CPU or torch
fallback behind these functions.  Signatures mirror include/mops_hip.h one to one.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

# MOPS_HIP_LIB points at another build of the same ABI (kernel tuning experiments)
LIB_PATH = Path(os.environ.get("MOPS_HIP_LIB") or Path(__file__).resolve().parent / "lib" / "libmops_hip.so")

# name -> (restype, argtypes); the exported surface declared in include/mops_hip.h
SIGNATURES = {
    "mops_hip_abi_version": (c_int, []),
    "mops_hip_status_string": (c_char_p, [c_int]),
    "mops_hip_last_hip_error": (c_int, []),
    "mops_hip_store_kvcache": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
                                       c_int64, c_int64, c_int64, c_void_p]),
    "mops_hip_embedding": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64,
                                   c_void_p]),
    "mops_hip_rms_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                     c_float, c_void_p]),
    "mops_hip_add_rms_forward": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
                                         c_int64, c_int64, c_float, c_void_p]),
    "mops_hip_paged_decode_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_int64]),
    "mops_hip_attn_paged_decode_bf16": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                                c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                c_int64, c_int64, c_int64, c_float, c_void_p, c_int64,
                                                c_void_p]),
    "mops_hip_attn_paged_decode_planned_bf16": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                                c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                c_int64, c_int64, c_int64, c_float, c_void_p, c_int64,
                                                c_int, c_void_p]),
    "mops_hip_attn_paged_decode_noalloc_bf16": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                                        c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                                        c_int64, c_int64, c_int64, c_float, c_void_p]),
    "mops_hip_attn_varlen_causal_bf16": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                                 c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64,
                                                 c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                                 c_int64, c_int64, c_int64, c_float, c_void_p]),
    "mops_hip_silu_and_mul": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p]),
    "mops_hip_apply_rotary_emb": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p,
                                          c_int64, c_int64, c_int64, c_void_p]),
    "mops_hip_sampler_argmax": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p]),
    "mops_hip_launch_floor": (c_int, [c_void_p]),
    "mops_hip_qk_norm_rope_store": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64,
                                            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                            c_int64, c_int64, c_float, c_void_p]),
    "mops_hip_linear_bf16": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                     c_int64, c_void_p, c_int64, c_void_p]),
    "mops_hip_linear_pin_solution": (c_int, [c_int64, c_int64, c_int64, c_int]),
    "mops_hip_linear_tune": (c_int, [c_int64, c_int64, c_int64, c_int64, c_int, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
}

ABI_VERSION = 9

_lib = None


class MopsHipError(RuntimeError):
    """A launcher of libmops_hip.so returned a negative status."""

    def __init__(self, func: str, status: int, text: str):
        super().__init__(f"{func} failed with status {status}: {text}")
        self.func = func
        self.status = status


def load() -> ctypes.CDLL:
    """Loads the library (once) and fixes the prototypes.  Raises if it is missing or stale."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: the hip backend has no fallback. Build it with "
            "`python -m nano_vllm_ninetoothed_amd.build` (needs hipcc, no GPU required)."
        )
    try:
        # torch wheels carry their own HIP runtime and hipBLASLt under the sonames this library links
        # against; importing torch first keeps one copy of each in the process, whichever order the caller
        # imports things in (and the GEMM solution table was measured against that copy)
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.mops_hip_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI {lib.mops_hip_abi_version()}, binding expects {ABI_VERSION}; rebuild")
    _lib = lib
    return lib


def check(func: str, status: int) -> None:
    if status != 0:
        lib = load()
        text = lib.mops_hip_status_string(status).decode()
        if status == -5:  # MOPS_HIP_ELAUNCH
            text += f" (hipError {lib.mops_hip_last_hip_error()})"
        raise MopsHipError(func, status, text)
