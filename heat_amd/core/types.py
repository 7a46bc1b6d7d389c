"""
The handful of Heat datatypes the k-means path touches, with Heat's "intuitive" promotion rule.

Mirrors the public names of heat/core/types.py (``ht.float32`` ... are classes with a
``torch_type()`` static method, ``heat_type_of``, ``canonical_heat_type``, ``promote_types``,
``iinfo``/``finfo``); only what ``cdist`` and ``KMeans`` need is here.
"""

from __future__ import annotations

import numpy as np
import torch


class datatype:
    """Base class of the Heat-style dtypes; calling one casts (``ht.float32(arr)``)."""

    _torch = None
    _bits = 0
    _kind = "?"

    def __new__(cls, *value, device=None, comm=None):
        from . import factories

        if len(value) != 1:
            raise TypeError(f"{cls.__name__}() takes exactly one argument")
        return factories.array(value[0], dtype=cls, device=device, comm=comm)

    @classmethod
    def torch_type(cls) -> torch.dtype:
        return cls._torch

    @classmethod
    def char(cls) -> str:
        return f"{cls._kind}{cls._bits // 8}"


def _make(name, tdt, bits, kind):
    return type(name, (datatype,), {"_torch": tdt, "_bits": bits, "_kind": kind})


bool = _make("bool", torch.bool, 1, "b")  # noqa: A001
uint8 = _make("uint8", torch.uint8, 8, "u")
int8 = _make("int8", torch.int8, 8, "i")
int16 = _make("int16", torch.int16, 16, "i")
int32 = _make("int32", torch.int32, 32, "i")
int64 = _make("int64", torch.int64, 64, "i")
float32 = _make("float32", torch.float32, 32, "f")
float64 = _make("float64", torch.float64, 64, "f")
bool_ = bool
int = int32  # noqa: A001
long = int64
float = float32  # noqa: A001
double = float64

_ALL = [bool, uint8, int8, int16, int32, int64, float32, float64]
_FROM_TORCH = {t._torch: t for t in _ALL}
_FROM_STR = {t.__name__: t for t in _ALL}
_FROM_STR.update({"f4": float32, "f8": float64, "i4": int32, "i8": int64, "i2": int16, "i1": int8, "u1": uint8})


def canonical_heat_type(a_type):
    """Heat dtype for a Heat dtype, torch dtype, numpy dtype, python type or string (types.py:611-650)."""
    import builtins

    if isinstance(a_type, type) and issubclass(a_type, datatype):
        return a_type
    if isinstance(a_type, torch.dtype):
        if a_type in _FROM_TORCH:
            return _FROM_TORCH[a_type]
        raise TypeError(f"data type {a_type} is not supported")
    if a_type is builtins.bool:
        return bool
    if a_type is builtins.int:
        return int32
    if a_type is builtins.float:
        return float32
    if isinstance(a_type, str) and a_type in _FROM_STR:
        return _FROM_STR[a_type]
    try:
        return _FROM_STR[np.dtype(a_type).name]
    except Exception:
        raise TypeError(f"data type {a_type} is not understood")


def heat_type_of(obj):
    """Heat dtype of a DNDarray, tensor, ndarray or scalar (types.py:735-790)."""
    if hasattr(obj, "dtype"):
        return canonical_heat_type(obj.dtype)
    return canonical_heat_type(type(obj))


def promote_types(type1, type2):
    """
    Smallest type both operands cast to "intuitively", i.e. keeping the bit length where possible:
    int32 + float32 -> float32, int64 + float32 -> float64, int8 + uint8 -> int16
    (heat/core/types.py:915-959).
    """
    a, b = canonical_heat_type(type1), canonical_heat_type(type2)
    if a is b:
        return a
    if a._kind == "f" or b._kind == "f":
        return float64 if max(a._bits, b._bits) > 32 else float32
    return _FROM_TORCH[torch.promote_types(a._torch, b._torch)]


class iinfo:
    """Integer type limits (types.py:1120)."""

    def __init__(self, dtype):
        t = canonical_heat_type(dtype)
        info = torch.iinfo(t._torch)
        self.bits, self.max, self.min = info.bits, info.max, info.min


class finfo:
    """Floating type limits."""

    def __init__(self, dtype):
        t = canonical_heat_type(dtype)
        info = torch.finfo(t._torch)
        self.bits, self.max, self.min, self.eps, self.tiny = info.bits, info.max, info.min, info.eps, info.tiny


__all__ = [
    "datatype", "bool", "bool_", "uint8", "int8", "int16", "int32", "int64", "int", "long",
    "float32", "float64", "float", "double", "canonical_heat_type", "heat_type_of",
    "promote_types", "iinfo", "finfo",
]
