"""
DNDarray: the metadata carrier the k-means path is called with (heat/core/dndarray.py:40-145).

At one rank the process-local tensor IS the array, so only the attributes and the few methods the
path and its callers touch are provided: ``larray``, ``gshape``/``shape``/``lshape``, ``dtype``,
``split``, ``device``, ``comm``, ``balanced``, ``astype``, ``copy``, ``resplit``, ``item``,
``numpy``, comparison with scalars, ``__bool__``.  General distributed indexing and redistribution
are outside this package.
"""

from __future__ import annotations

from typing import Optional, Tuple

import numpy as np
import torch

from . import types
from .communication import Communication
from .devices import Device


class DNDarray:
    def __init__(
        self,
        array: torch.Tensor,
        gshape: Tuple[int, ...],
        dtype,
        split: Optional[int],
        device: Device,
        comm: Communication,
        balanced: Optional[bool],
    ):
        self.__array = array
        self.__gshape = tuple(gshape)
        self.__dtype = dtype
        self.__split = split
        self.__device = device
        self.__comm = comm
        self.__balanced = balanced
        # same consistency check as heat/core/dndarray.py:89, tolerant of "cuda" vs "cuda:0"
        dev = str(array.device)
        assert dev == device.torch_device or dev.split(":")[0] == device.torch_device.split(":")[0]

    # ---- metadata --------------------------------------------------------------------------
    @property
    def larray(self) -> torch.Tensor:
        return self.__array

    @larray.setter
    def larray(self, array: torch.Tensor):
        if not isinstance(array, torch.Tensor):
            raise TypeError(f"Expected a torch.Tensor, got {type(array)}")
        self.__array = array

    @property
    def balanced(self):
        return self.__balanced

    @property
    def comm(self) -> Communication:
        return self.__comm

    @property
    def device(self) -> Device:
        return self.__device

    @property
    def dtype(self):
        return self.__dtype

    @property
    def gshape(self) -> Tuple[int, ...]:
        return self.__gshape

    @property
    def shape(self) -> Tuple[int, ...]:
        return self.__gshape

    @property
    def lshape(self) -> Tuple[int, ...]:
        return tuple(self.__array.shape)

    @property
    def ndim(self) -> int:
        return len(self.__gshape)

    @property
    def size(self) -> int:
        return int(np.prod(self.__gshape)) if self.__gshape else 1

    @property
    def split(self) -> Optional[int]:
        return self.__split

    @property
    def T(self):
        return DNDarray(self.__array.T, self.__gshape[::-1], self.__dtype,
                        None if self.__split is None else self.ndim - 1 - self.__split,
                        self.__device, self.__comm, self.__balanced)

    def is_distributed(self) -> bool:
        return self.__split is not None and self.__comm.is_distributed()

    def is_balanced(self, force_check: bool = False) -> bool:
        return True

    # ---- conversions -----------------------------------------------------------------------
    def astype(self, dtype, copy: bool = True) -> "DNDarray":
        """Cast; with copy=False and an unchanged dtype no new tensor is made (dndarray.py:523-563)."""
        dtype = types.canonical_heat_type(dtype)
        casted = self.__array.type(dtype.torch_type())
        if copy:
            if casted is self.__array:
                casted = casted.clone()
            return DNDarray(casted, self.__gshape, dtype, self.__split, self.__device, self.__comm, self.__balanced)
        self.__array = casted
        self.__dtype = dtype
        return self

    def copy(self) -> "DNDarray":
        """heat/core/memory.py:13-43."""
        return DNDarray(self.__array.clone(), self.__gshape, self.__dtype, self.__split,
                        self.__device, self.__comm, self.__balanced)

    def resplit(self, axis: Optional[int] = None) -> "DNDarray":
        """Out-of-place resplit; at one rank every layout holds the same data, so this is a copy with
        the new split recorded (heat/core/manipulations.py:3897-3901)."""
        if axis is not None and not (-self.ndim <= axis < self.ndim):
            raise ValueError(f"axis {axis} out of range for {self.ndim}-dimensional array")
        return DNDarray(self.__array.clone(), self.__gshape, self.__dtype, axis,
                        self.__device, self.__comm, self.__balanced)

    def cpu(self) -> "DNDarray":
        from . import devices

        return DNDarray(self.__array.cpu(), self.__gshape, self.__dtype, self.__split, devices.cpu,
                        self.__comm, self.__balanced)

    def numpy(self) -> np.ndarray:
        return self.__array.cpu().numpy()

    def item(self):
        if self.size > 1:
            raise ValueError("only one-element DNDarrays can be converted to Python scalars")
        return self.__array.item()

    def tolist(self):
        return self.__array.tolist()

    def __cast(self, cast_function):
        # dndarray.py:605-635: only one-element arrays cast to python scalars
        if np.prod(self.shape) == 1:
            return cast_function(self.__array.item())
        raise TypeError("only size-1 arrays can be converted to Python scalars")

    def __bool__(self) -> bool:
        return self.__cast(bool)

    def __float__(self) -> float:
        return self.__cast(float)

    def __int__(self) -> int:
        return self.__cast(int)

    def __len__(self) -> int:
        try:
            return self.__gshape[0]
        except IndexError:
            raise TypeError("len() of unsized DNDarray")

    # ---- the few operators callers of the path use ---------------------------------------------
    def __wrap(self, t: torch.Tensor, split) -> "DNDarray":
        return DNDarray(t, tuple(t.shape), types.canonical_heat_type(t.dtype), split, self.__device,
                        self.__comm, self.__balanced)

    def __compare(self, other, op):
        if isinstance(other, DNDarray):
            other = other.larray
        elif not np.isscalar(other) and not isinstance(other, torch.Tensor):
            raise TypeError(f"Only DNDarrays and numeric scalars are supported, but input was {type(other)}")
        elif isinstance(other, str):
            raise TypeError("Data type not supported, input was a string")
        return self.__wrap(op(self.__array, other), self.__split)

    def __eq__(self, other):
        # heat/core/relational.py:65-81: a non-numeric operand compares unequal instead of raising,
        # which is what lets ``init == "kmeans++"`` work when init is a DNDarray
        try:
            return self.__compare(other, torch.eq)
        except (TypeError, ValueError, RuntimeError):
            return False

    def __ne__(self, other):
        try:
            return self.__compare(other, torch.ne)
        except (TypeError, ValueError, RuntimeError):
            return True

    def __le__(self, other):
        return self.__compare(other, torch.le)

    def __lt__(self, other):
        return self.__compare(other, torch.lt)

    def __ge__(self, other):
        return self.__compare(other, torch.ge)

    def __gt__(self, other):
        return self.__compare(other, torch.gt)

    __hash__ = None

    def __getitem__(self, key):
        """Local indexing; valid because one rank holds the whole array."""
        if isinstance(key, DNDarray):
            key = key.larray
        elif isinstance(key, tuple):
            key = tuple(k.larray if isinstance(k, DNDarray) else k for k in key)
        t = self.__array[key]
        split = self.__split if (self.__split is not None and t.dim() > self.__split and t.dim() == self.ndim) else None
        return self.__wrap(t, split)

    def __repr__(self) -> str:
        return (f"DNDarray({self.__array.cpu().tolist() if self.size <= 64 else '...'}, "
                f"dtype=ht.{self.__dtype.__name__}, device={self.__device}, split={self.__split})")


__all__ = ["DNDarray"]
