"""bnk_amd: MI355X-native batched WireGuard transport AEAD and packet filter.

The compute lives in ``libbnkhip.so`` (hand-written HIP for gfx950 behind a C
ABI, see ``include/bnkhip.h``).  This package holds the HIP/C++ sources
(``csrc/``), the C++ host-side mirror of the reference's filter interface
(``host/``), a ctypes binding used by the tests and the benchmark, and the
seeded workload generators.
"""
__all__ = ["lib", "workloads"]
