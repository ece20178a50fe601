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


PAIR_KINDS = {"v_add_u32": 0, "v_xor_b32": 1, "v_alignbit_b32": 2, "v_mad_u64_u32": 3,
              "v_addc_co_u32": 4, "v_lshlrev_b32": 5, "v_lshrrev_b32": 6, "v_mov_b32": 7}


def pair(kind_a: str, kind_b: str | None, iters: int = 20000, device: int = 0) -> tuple[float, float]:
    """Nanoseconds per instruction of two streams that share each SIMD (waves 0-3 of a
    workgroup run kind_a, waves 4-7 kind_b; None: the first four run alone)."""
    a, b = C.c_double(), C.c_double()
    rc = load().bnkp_pair(C.c_int(device), C.c_int(PAIR_KINDS[kind_a]),
                          C.c_int(-1 if kind_b is None else PAIR_KINDS[kind_b]), C.c_uint32(iters),
                          C.byref(a), C.byref(b))
    if rc != 0:
        raise RuntimeError(f"bnkp_pair failed: {rc}")
    return float(a.value), float(b.value)


def mix(raised_priority: bool, waves_per_simd: int, iters: int = 500, device: int = 0) -> float:
    """VALU lane-ops per second of the ChaCha20 quarter-round stream."""
    r = C.c_double()
    rc = load().bnkp_mix(C.c_int(device), C.c_int(1 if raised_priority else 0), C.c_int(waves_per_simd),
                         C.c_uint32(iters), C.byref(r))
    if rc != 0:
        raise RuntimeError(f"bnkp_mix failed: {rc}")
    return float(r.value)


def aead_compute(paired: bool, waves_per_simd: int, data_blocks: int = 48, device: int = 0) -> float:
    """64-byte blocks per second of the AEAD arithmetic with no packet movement."""
    r = C.c_double()
    rc = load().bnkp_aead_compute(C.c_int(device), C.c_int(1 if paired else 0), C.c_int(waves_per_simd),
                                  C.c_uint32(data_blocks), C.byref(r))
    if rc != 0:
        raise RuntimeError(f"bnkp_aead_compute failed: {rc}")
    return float(r.value)


def line_copy(packets: int = 1 << 20, stride: int = 1440, length: int = 1420, waves_per_simd: int = 2,
              depth: int = 1, spin: int = 0, iters: int = 20, device: int = 0) -> float:
    """Milliseconds per launch of the AEAD kernel's packet movement alone (see bnkprobe.h)."""
    r = C.c_double(0)
    rc = load().bnkp_line_copy(C.c_int(device), C.c_uint32(packets), C.c_uint32(stride), C.c_uint32(length),
                               C.c_int(waves_per_simd), C.c_int(depth), C.c_uint32(spin), C.c_uint32(iters),
                               C.byref(r))
    if rc:
        raise RuntimeError(f"bnkp_line_copy failed: {rc}")
    return r.value
