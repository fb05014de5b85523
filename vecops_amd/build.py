"""Builds the native libraries in-tree (hipcc cross-compiles gfx950 without a GPU)."""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def _make(directory: str, *targets: str, force: bool) -> None:
    cmd = ["make", "-C", directory, "-j8"] + (["-B"] if force else []) + list(targets)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)} failed:\n{proc.stdout[-4000:]}\n{proc.stderr[-4000:]}")


def build_kernels(force: bool = True) -> str:
    """vecops_amd/lib/libvecops_hip.so: the gfx950 kernels and their C ABI."""
    _make(os.path.join(HERE, "csrc"), force=force)
    return os.path.join(HERE, "lib", "libvecops_hip.so")


def build_host(force: bool = True) -> None:
    """The C++ host layer (runtime surface, HIP provider, artifact DSOs), when present."""
    host = os.path.join(HERE, "host")
    if os.path.exists(os.path.join(host, "Makefile")):
        _make(host, force=force)


def build_all(force: bool = True) -> None:
    build_kernels(force)
    build_host(force)
