"""
Pairwise distances with the interface of heat/spatial/distance.py:136-156 (``cdist``), backed by
the hkm_cdist_f32 kernel.  Only the quadratic-expansion metric on float32 is computed here; that
is the branch KMeans uses (heat/cluster/kmeans.py:67).
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _native
from ..core import types
from ..core.dndarray import DNDarray

__all__ = ["cdist"]


def _check_inputs(X: DNDarray, Y: Optional[DNDarray]):
    """Shape/split validation in the order of heat/spatial/distance.py:234-235,362-390."""
    if not isinstance(X, DNDarray):
        raise TypeError(f"X needs to be a ht.DNDarray, but was {type(X)}")
    if len(X.shape) > 2:
        raise NotImplementedError("Only 2D data matrices are currently supported")
    if Y is None:
        if X.split is not None and X.split != 0:
            raise NotImplementedError(
                f"Input split was X.split = {X.split}. Splittings other than 0 or None currently not supported."
            )
        return X.split
    if not isinstance(Y, DNDarray):
        raise TypeError(f"Y needs to be a ht.DNDarray, but was {type(Y)}")
    if len(Y.shape) > 2:
        raise NotImplementedError(
            f"Only 2D data matrices are supported, but input shapes were X: {X.shape}, Y: {Y.shape}"
        )
    if X.comm != Y.comm:
        raise NotImplementedError("Differing communicators not supported")
    if X.split is None:
        if Y.split is None:
            return None
        if Y.split == 0:
            return 1
    elif X.split == 0:
        if Y.split is None or Y.split == 0:
            return 0
    raise NotImplementedError(
        f"Input splits were X.split = {X.split}, Y.split = {Y.split}. Splittings other than 0 or None currently not supported."
    )


def _as_f32_matrix(a: DNDarray, promoted) -> torch.Tensor:
    t = a.larray
    if t.dim() != 2:
        raise NotImplementedError("Only 2D data matrices are currently supported")
    if promoted is not types.float32:
        raise NotImplementedError(
            f"the gfx950 kernels compute in float32; inputs promote to {promoted.__name__}"
        )
    if t.dtype != torch.float32:
        t = t.to(torch.float32)
    if t.stride(-1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
        t = t.contiguous()
    return t


def cdist(X: DNDarray, Y: Optional[DNDarray] = None, quadratic_expansion: bool = False) -> DNDarray:
    """
    Euclidean distance between all rows of ``X`` (m x f) and ``Y`` (n x f): an (m, n) DNDarray of
    square-rooted distances in promote(X, Y, float32), ``split = X.split`` (1 when only ``Y`` is
    split).  ``Y=None`` means ``Y = X``.

    Only ``quadratic_expansion=True`` is built: |x-y|^2 = |x|^2 + |y|^2 - 2xy clamped at 0, in
    float32.  The other metric of the reference (``torch.cdist``) is not part of this package.
    """
    split = _check_inputs(X, Y)
    if not quadratic_expansion:
        raise NotImplementedError(
            "cdist(quadratic_expansion=False) is not built in heat_amd; use quadratic_expansion=True"
        )
    promoted = types.promote_types(X.dtype, types.float32)
    if Y is not None:
        promoted = types.promote_types(types.promote_types(X.dtype, Y.dtype), types.float32)
    x = _as_f32_matrix(X, promoted)
    y = x if Y is None else _as_f32_matrix(Y, promoted)
    if x.shape[1] != y.shape[1]:
        raise ValueError("Inputs must have same shape[1]")
    out = torch.empty((x.shape[0], y.shape[0]), dtype=torch.float32, device=x.device)
    _native.cdist(x, y, out, sqrt=True)
    return DNDarray(out, tuple(out.shape), types.float32, split, X.device, X.comm, True)
