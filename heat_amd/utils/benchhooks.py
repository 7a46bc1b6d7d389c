"""
ctypes binding of include/hkm_bench.h: the measuring hooks of libhkm (event pairs around the dominant kernel,
the query for the launch geometry of the resident matrix-core kernels) and the microbenchmarks of
libhkm_bench.so.  Used by bench.py and the tests; nothing on the clustering path imports this module, and the
product library never loads libhkm_bench.so.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int32, c_size_t, c_void_p
from typing import Optional

from .. import _native

_BENCH_LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc", "libhkm_bench.so")
_bench_lib: Optional[ctypes.CDLL] = None

# name -> (library, restype, argtypes); every symbol declared in include/hkm_bench.h
SIGNATURES = {
    "hkm_profile_enable": ("hkm", ctypes.c_int, [c_int32]),
    "hkm_profile_collect": ("hkm", ctypes.c_int, [c_void_p, c_int32, c_void_p]),
    "hkm_point_blocks": ("hkm", ctypes.c_int, [c_int32, c_void_p]),
    "hkm_point_blocks_trial": ("hkm", ctypes.c_int, [c_void_p, c_void_p]),
    "hkm_bench_last_error": ("bench", c_char_p, []),
    "hkm_probe_mfma_f32": ("bench", ctypes.c_int, [c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
    "hkm_probe_stream": ("bench", ctypes.c_int, [c_void_p, c_void_p, c_size_t, c_int32, c_void_p, c_void_p]),
}


def _bind(lib: ctypes.CDLL, which: str) -> None:
    for name, (home, res, args) in SIGNATURES.items():
        if home == which:
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args


def hkm() -> ctypes.CDLL:
    """libhkm with the hooks of hkm_bench.h bound."""
    lib = _native.load()
    _bind(lib, "hkm")
    return lib


def bench_lib_path() -> str:
    return _BENCH_LIB_PATH


def bench() -> ctypes.CDLL:
    """libhkm_bench.so (the microbenchmarks), loaded on first use."""
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(_BENCH_LIB_PATH):
            raise ImportError(f"{_BENCH_LIB_PATH} is missing: build it with `make -C heat_amd/csrc`")
        lib = ctypes.CDLL(_BENCH_LIB_PATH)
        _bind(lib, "bench")
        _bench_lib = lib
    return _bench_lib


def check_probe(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(f"libhkm_bench error {rc}: {bench().hkm_bench_last_error().decode()}")


def profile_enable(on: bool) -> None:
    """Record an event pair around the distance kernel of every assign / lloyd_step call of this thread."""
    _native.check(hkm().hkm_profile_enable(1 if on else 0))


def profile_collect() -> list:
    """Durations (ms) of the distance kernels launched since the last collect, in call order.  Waits."""
    buf = (ctypes.c_float * 512)()
    cnt = c_int32(0)
    _native.check(hkm().hkm_profile_collect(ctypes.cast(buf, c_void_p), 512, ctypes.cast(ctypes.pointer(cnt), c_void_p)))
    return [float(buf[i]) for i in range(min(cnt.value, 512))]


def point_blocks(d: int):
    """(point blocks per wave a resident matrix-core kernel would use for d features now -- 0 if d has no
    such kernel --, whether that is the verdict of a trial on the current device)."""
    tuned = ctypes.c_int32(0)
    pb = hkm().hkm_point_blocks(d, ctypes.cast(ctypes.pointer(tuned), c_void_p))
    return int(pb), bool(tuned.value)


def point_blocks_trial():
    """(verdict of the trial on the current device: 0 while there is none, else 1 or 2; ms per step of its
    last window with two point blocks; ms per step of its window with one)."""
    two, one = ctypes.c_float(0.0), ctypes.c_float(0.0)
    v = hkm().hkm_point_blocks_trial(ctypes.cast(ctypes.pointer(two), c_void_p), ctypes.cast(ctypes.pointer(one), c_void_p))
    return int(v), float(two.value), float(one.value)
