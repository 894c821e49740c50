"""Locate, build and load libpccl_hip.so.

Keeps the name and call convention of the reference's JIT step
(`from pccl.build_kernels import build`, benchmark_raw_collectives/reduce_scatter.py:10,45-51;
pccl/build_kernels.py:22-116) but there is nothing torch- or MPI-specific to
compile: one `hipcc --offload-arch=gfx950` command produces a torch-free
shared library with a C ABI (include/pccl_hip.h), loaded through ctypes.
"""
from __future__ import annotations

import os
import shutil
import subprocess

from . import _native

BUILT = False

CSRC_DIR = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc"))


def compile_library(force: bool = False, verbose: bool = False) -> str:
    """Run the Makefile in csrc/ (hipcc cross-compiles gfx950 without a GPU)."""
    if shutil.which("make") is None:
        raise RuntimeError("cannot build libpccl_hip.so: `make` not found")
    cmd = ["make", "-C", CSRC_DIR] + (["-B"] if force else [])
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or proc.returncode:
        print(proc.stdout)
        print(proc.stderr)
    if proc.returncode:
        raise RuntimeError(f"building libpccl_hip.so failed (exit {proc.returncode}):\n{proc.stderr[-2000:]}")
    return _native.LIB_PATH


def build(force: bool = False, verbose: bool = False):
    """Make the native library available in this process.

    Loads the in-tree build; compiles it first only if it is missing (or
    `force`).  Raises if it can be neither found nor built: there is no
    pure-Python fallback."""
    global BUILT
    if BUILT and not force:
        return _native.load()
    if force or not _native.is_built():
        compile_library(force=force, verbose=verbose)
    lib = _native.load()
    BUILT = True
    return lib
