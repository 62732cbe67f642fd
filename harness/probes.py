"""ctypes face of libshrikeprobe.so: the benchmark's measurement aids (an empty launch, a kernel that only reads
a byte range of listed pool cells, a chain of dependent loads, matrix and vector instructions side by side). Not part of the product's ABI: nothing in libshrikehip or in the
operator mirror depends on it."""
from __future__ import annotations

import ctypes as C
import os

from shrike_amd.capi import PoolBases, ShrikeError

_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "libshrikeprobe.so")
        if not os.path.exists(path):
            raise ShrikeError(f"{path} is not built (make -C harness)")
        _lib = C.CDLL(path)
        _lib.shrike_probe_last_error.restype = C.c_char_p
        _lib.shrike_probe_empty_launch.restype = C.c_int
        _lib.shrike_probe_empty_launch.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p]
        _lib.shrike_probe_read.restype = C.c_int
        _lib.shrike_probe_read.argtypes = [C.c_void_p, C.POINTER(PoolBases), C.c_uint64, C.c_void_p, C.c_uint32,
                                           C.c_uint64, C.c_uint64, C.c_void_p]
        _lib.shrike_probe_dependent_loads.restype = C.c_int
        _lib.shrike_probe_dependent_loads.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p]
        _lib.shrike_probe_timestamp.restype = C.c_int
        _lib.shrike_probe_timestamp.argtypes = [C.c_void_p, C.c_void_p]
        _lib.shrike_probe_issue.restype = C.c_int
        _lib.shrike_probe_issue.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        _lib.shrike_probe_wall_clock_khz.restype = C.c_int
        _lib.shrike_probe_wall_clock_khz.argtypes = []
    return _lib


def last_error() -> str:
    return load().shrike_probe_last_error().decode()


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise ShrikeError(f"{what} failed with {rc}: {last_error()}")
