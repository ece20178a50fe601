"""ctypes binding of libbnkprobe.so: the benchmark's measurement probes
(instruction-rate and copy-bandwidth ceilings).  Not part of the product path."""
from __future__ import annotations

import ctypes as C
import os

SO_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libbnkprobe.so")

PROBE_OPS = {"v_add_u32": 0, "v_xor_b32": 1, "v_alignbit_b32": 2, "v_mad_u64_u32": 3,
             "v_fma_f64": 4, "v_mul_lo_u32": 5, "v_add_f64": 6}

_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            raise FileNotFoundError(f"{SO_PATH} is missing: build it with `make -C bnk_amd/csrc`")
        _lib = C.CDLL(SO_PATH)
    return _lib


def valu(op: str | int, iters: int = 2000, device: int = 0) -> float:
    """Lane-ops per second of a dependency-free stream of one instruction kind."""
    code = PROBE_OPS[op] if isinstance(op, str) else op
    r = C.c_double()
    rc = load().bnkp_valu(C.c_int(device), C.c_int(code), C.c_uint32(iters), C.byref(r))
    if rc != 0:
        raise RuntimeError(f"bnkp_valu failed: {rc}")
    return float(r.value)


def copy(nbytes: int, iters: int, device: int = 0) -> float:
    """Bytes read plus bytes written per second of a plain device-to-device copy."""
    r = C.c_double()
    rc = load().bnkp_copy(C.c_int(device), C.c_size_t(nbytes), C.c_uint32(iters), C.byref(r))
    if rc != 0:
        raise RuntimeError(f"bnkp_copy failed: {rc}")
    return float(r.value)
