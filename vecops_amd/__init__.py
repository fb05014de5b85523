"""MI355X-native matmul path behind the vecops Operator API.

The product is native code: ``vecops_amd/lib/libvecops_hip.so`` (hand-written
gfx950 kernels behind a C ABI, ``include/vecops_hip.h``) and the C++ host layer
under ``vecops_amd/host`` that plugs it into the vecops runtime surface.  The
Python modules here only bind that C ABI for the test-suite and the benchmark
(device memory and streams come from PyTorch-ROCm) and build the libraries.
"""
from . import capi, synth  # noqa: F401

__all__ = ["capi", "synth"]
