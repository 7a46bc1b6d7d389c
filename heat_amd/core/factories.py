"""
Array construction the way callers of the k-means path do it (heat/core/factories.py:150-430,1545):
``array`` wraps a torch tensor without copying where torch.as_tensor would not copy, ``zeros``/``ones``/
``empty`` allocate on the chosen device.
"""

from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from . import devices, types
from .communication import sanitize_comm
from .dndarray import DNDarray


def _sanitize_split(split, ndim):
    if split is None:
        return None
    if not isinstance(split, int):
        raise TypeError(f"split must be None or int, was {type(split)}")
    if not (-ndim <= split < max(ndim, 1)):
        raise ValueError(f"split axis {split} out of range for {ndim}-dimensional array")
    return split % ndim if ndim else None


def array(obj, dtype=None, copy=None, ndmin: int = 0, order: str = "C", split: Optional[int] = None,
          is_split: Optional[int] = None, device=None, comm=None) -> DNDarray:
    """
    Create a DNDarray.  A torch tensor already on the target device with the target dtype is shared,
    not copied (factories.py:371-378), unless ``copy=True``.  ``is_split`` means "this is my local
    chunk"; at one rank it is the same as ``split``.
    """
    if split is not None and is_split is not None:
        raise ValueError("split and is_split are mutually exclusive parameters")
    if isinstance(obj, DNDarray):
        dev = obj.device if device is None else devices.sanitize_device(device)
        t = obj.larray
        sp = obj.split if split is None and is_split is None else (split if split is not None else is_split)
    else:
        sp = split if split is not None else is_split
        if isinstance(obj, torch.Tensor) and device is None:
            # a tensor keeps its own device (the reference would move it to the default device;
            # here that would silently pull GPU data back to the host)
            dev = devices.sanitize_device(obj.device.type)
        else:
            dev = devices.sanitize_device(device)
        if isinstance(obj, torch.Tensor):
            t = obj
        else:
            try:
                t = torch.as_tensor(np.asarray(obj) if not np.isscalar(obj) else obj)
            except (RuntimeError, TypeError, ValueError):
                raise TypeError(f"invalid data of type {type(obj)}")
            if t.dtype == torch.float64 and dtype is None and not isinstance(obj, np.ndarray):
                t = t.to(torch.float32)  # python floats default to float32 in Heat
            if t.dtype == torch.int64 and dtype is None and not isinstance(obj, np.ndarray):
                t = t.to(torch.int64)
    if dtype is not None:
        dtype = types.canonical_heat_type(dtype)
        t2 = t.to(dtype.torch_type())
    else:
        dtype = types.canonical_heat_type(t.dtype)
        t2 = t
    t2 = t2.to(dev.torch_device)
    if copy is True and t2.data_ptr() == t.data_ptr():
        t2 = t2.clone()
    while t2.dim() < ndmin:
        t2 = t2.unsqueeze(0)
    sp = _sanitize_split(sp, t2.dim())
    return DNDarray(t2, tuple(t2.shape), dtype, sp, dev, sanitize_comm(comm), True)


def _filled(fn, shape, dtype, split, device, comm):
    dtype = types.canonical_heat_type(dtype)
    dev = devices.sanitize_device(device)
    if isinstance(shape, int):
        shape = (shape,)
    t = fn(tuple(shape), dtype=dtype.torch_type(), device=dev.torch_device)
    return DNDarray(t, tuple(t.shape), dtype, _sanitize_split(split, t.dim()), dev, sanitize_comm(comm), True)


def zeros(shape, dtype=types.float32, split=None, device=None, comm=None, order="C") -> DNDarray:
    return _filled(torch.zeros, shape, dtype, split, device, comm)


def ones(shape, dtype=types.float32, split=None, device=None, comm=None, order="C") -> DNDarray:
    return _filled(torch.ones, shape, dtype, split, device, comm)


def empty(shape, dtype=types.float32, split=None, device=None, comm=None, order="C") -> DNDarray:
    return _filled(torch.empty, shape, dtype, split, device, comm)


__all__ = ["array", "zeros", "ones", "empty"]
