"""ctypes binding of libgranite_hip_calibration.so (include/granite_hip_calibration.h): the
matrix-core rate kernel that bench.py's mfma_calibration workload runs.  A measurement aid
beside the attention library, not part of it."""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libgranite_hip_calibration.so"
_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m granite_amd.build`")
        lib = C.CDLL(str(LIB_PATH))
        lib.granite_hip_cal_mfma_rate.restype = C.c_int
        lib.granite_hip_cal_mfma_rate.argtypes = [C.c_int, C.c_void_p, C.c_uint64, C.c_uint32, C.c_int, C.c_int,
                                                  C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double),
                                                  C.POINTER(C.c_float)]
        lib.granite_hip_cal_mfma_mix.restype = C.c_int
        lib.granite_hip_cal_mfma_mix.argtypes = [C.c_int, C.c_void_p, C.c_uint64, C.c_uint32, C.c_int, C.c_int,
                                                 C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_double),
                                                 C.POINTER(C.c_float)]
        _lib = lib
    return _lib


def mfma_rate(operands, n_halves: int, iterations: int, shape: int = 32, waves_per_simd: int = 2,
              mix=(0, 0, 0), device: int = 0):
    """One timed launch (after three untimed ones); returns (MFMA flops, milliseconds).
    mix = (float FMAs, exponentials, 16-byte LDS reads) issued after every MFMA."""
    flops, ms = C.c_double(0.0), C.c_float(0.0)
    ptr = operands.ptr if hasattr(operands, "ptr") else int(operands)
    rc = load().granite_hip_cal_mfma_rate(device, ptr, n_halves, iterations, shape, waves_per_simd, mix[0], mix[1],
                                          mix[2], C.byref(flops), C.byref(ms))
    if rc != 0:
        raise RuntimeError(f"granite_hip_cal_mfma_rate failed with {rc}")
    return flops.value, ms.value


def mfma_mix(operands, n_halves: int, iterations: int, shape: int = 32, waves_per_simd: int = 2,
             per_pair=(0, 0, 0, 0), device: int = 0):
    """One timed launch (after three untimed ones); returns (MFMA flops, milliseconds).
    per_pair = (float FMAs, exponentials, 16-byte LDS reads, scalar additions) issued per pair of MFMAs."""
    flops, ms = C.c_double(0.0), C.c_float(0.0)
    ptr = operands.ptr if hasattr(operands, "ptr") else int(operands)
    rc = load().granite_hip_cal_mfma_mix(device, ptr, n_halves, iterations, shape, waves_per_simd, *per_pair,
                                         C.byref(flops), C.byref(ms))
    if rc != 0:
        raise RuntimeError(f"granite_hip_cal_mfma_mix failed with {rc}")
    return flops.value, ms.value
