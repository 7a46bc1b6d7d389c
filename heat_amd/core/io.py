"""
Loading a data matrix straight onto the device: ``load_csv`` / ``load`` with the signatures of
heat/core/io.py:895-1115 (CSV only; the HDF5 / NetCDF / Zarr readers of the reference are not part
of the k-means path).  One rank: the file is parsed once on the host and copied to the device in a
single transfer; ``split`` only sets the metadata.
"""

from __future__ import annotations

import os
from typing import Optional

import numpy as np
import torch

from . import devices, types
from .communication import sanitize_comm
from .dndarray import DNDarray

__all__ = ["load", "load_csv"]


def load_csv(path: str, header_lines: int = 0, sep: str = ",", dtype=types.float32, encoding: str = "utf-8",
             split: Optional[int] = None, device=None, comm=None) -> DNDarray:
    """Load a numeric CSV file as a 2-D DNDarray (heat/core/io.py:968-1115 at one rank)."""
    if not isinstance(path, str):
        raise TypeError(f"path must be str, not {type(path)}")
    if not isinstance(sep, str):
        raise TypeError(f"separator must be str, not {type(sep)}")
    if not isinstance(header_lines, int):
        raise TypeError(f"header_lines must int, not {type(header_lines)}")
    if split not in (None, 0, 1):
        if not isinstance(split, int):
            raise TypeError(f"split must be None or int, not {type(split)}")
        raise ValueError(f"split must be in [None, 0, 1], but is {split}")
    htype = types.canonical_heat_type(dtype)
    dev = devices.sanitize_device(device)
    comm = sanitize_comm(comm)
    with open(path, "r", encoding=encoding) as f:
        rows = [line for i, line in enumerate(f) if i >= header_lines and line.strip()]
    data = np.array([[float(v) for v in line.strip().split(sep)] for line in rows], dtype=np.float64)
    if data.ndim == 1:
        data = data.reshape(len(rows), -1)
    t = torch.from_numpy(data).to(htype.torch_type()).to(dev.torch_device)
    return DNDarray(t, tuple(t.shape), htype, split, dev, comm, True)


def load(path: str, *args, **kwargs) -> DNDarray:
    """Dispatch on the file extension (heat/core/io.py:895-966); only ``.csv`` is built."""
    if not isinstance(path, str):
        raise TypeError(f"Expected path to be str, but was {type(path)}")
    extension = os.path.splitext(path)[-1].strip().lower()
    if extension == ".csv":
        return load_csv(path, *args, **kwargs)
    if extension in (".h5", ".hdf5", ".nc", ".nc4", ".netcdf", ".npy", ".zarr"):
        raise RuntimeError(f"loading {extension} files is not part of this build")
    raise ValueError(f"Unsupported file extension {extension}")
