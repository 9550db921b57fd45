"""Builds libmops_hip.so (the C-ABI library of hand-written gfx950 kernels) in-tree with hipcc.

Usage: ``python -m nano_vllm_ninetoothed_amd.build [--force]``.  The library lands next to this file
under ``lib/`` so that it travels with the source tree; nothing is written outside the package.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
OBJ_DIR = PKG_DIR / "build"
LIB_PATH = LIB_DIR / "libmops_hip.so"

ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # the direct-to-LDS loads are inline assembly that writes M0 and says so in its clobber list; the compiler warns
    # that M0 is a reserved register (it never keeps a value there across statements, which is what the loads rely on)
    "-Wno-inline-asm",
    # packed fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def sources() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


def build(force: bool = True, verbose: bool = False) -> Path:
    """Compiles every csrc/*.hip for gfx950 and links lib/libmops_hip.so.  Returns its path."""
    hipcc = _hipcc()
    LIB_DIR.mkdir(exist_ok=True)
    OBJ_DIR.mkdir(exist_ok=True)
    srcs = sources()
    headers = list(CSRC_DIR.glob("*.h")) + [PKG_DIR.parent / "include" / "mops_hip.h"]
    newest_header = max(h.stat().st_mtime for h in headers)

    def compile_one(src: Path) -> Path:
        obj = OBJ_DIR / (src.stem + ".o")
        stale = force or not obj.exists() or obj.stat().st_mtime < max(src.stat().st_mtime, newest_header)
        if stale:
            cmd = [hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)]
            if verbose:
                print(" ".join(cmd), file=sys.stderr)
            _run(cmd)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    # hipBLASLt is the one library dependency: the `linear` entry point is a library GEMM
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs), "-lhipblaslt"])
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build(force="--force" in sys.argv, verbose=True)
    print(path)
