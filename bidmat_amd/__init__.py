"""bidmat_amd — MI355X (gfx950) native implementation of BIDMat's sparse-dense product path.

The product is the shared library libbidmathip.so (hand-written HIP kernels behind the C ABI
of include/bidmat_hip.h). This package holds its sources (csrc/), the ctypes binding used by
the tests and the benchmark (hip_abi, device), the host-side mirror of BIDMat's GMat / GSMat
operator interface (host/, mats) and the seeded input generators (gen/).
"""
__all__ = ["hip_abi", "device"]
