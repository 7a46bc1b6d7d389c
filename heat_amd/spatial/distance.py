"""
Pairwise distances with the interface of heat/spatial/distance.py:136-206 (``cdist``, ``rbf``,
``manhattan``), backed by the hkm_pairwise_f32 / hkm_pairwise_f64 kernels on one rank, in the
dtype the reference's promote(X, Y, float32) gives.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _native
from ..core import types
from ..core.dndarray import DNDarray

__all__ = ["cdist", "manhattan", "rbf"]


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
    """The local matrix in the promoted dtype (float32 or float64), row-major."""
    t = a.larray
    if t.dim() != 2:
        raise NotImplementedError("Only 2D data matrices are currently supported")
    if promoted not in (types.float32, types.float64):
        raise NotImplementedError(f"inputs promote to {promoted.__name__}, which the kernels do not cover")
    want = torch.float64 if promoted is types.float64 else torch.float32
    if t.dtype != want:
        t = t.to(want)
    if t.stride(-1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
        t = t.contiguous()
    return t


def _pairwise(X: DNDarray, Y: Optional[DNDarray], metric: int, sigma: float = 1.0) -> DNDarray:
    """Shared driver of cdist / rbf / manhattan: the checks and promotion of ``_dist``
    (heat/spatial/distance.py:209-414) at one rank, then one kernel launch."""
    split = _check_inputs(X, Y)
    promoted = types.promote_types(X.dtype, types.float32)
    if Y is not None:
        promoted = types.promote_types(types.promote_types(X.dtype, Y.dtype), types.float32)
    x = _as_f32_matrix(X, promoted)
    y = x if Y is None else _as_f32_matrix(Y, promoted)
    if x.shape[1] != y.shape[1]:
        raise ValueError("Inputs must have same shape[1]")
    out = torch.empty((x.shape[0], y.shape[0]), dtype=x.dtype, device=x.device)
    _native.pairwise(x, y, out, metric, sigma)
    return DNDarray(out, tuple(out.shape), promoted, split, X.device, X.comm, True)


def cdist(X: DNDarray, Y: Optional[DNDarray] = None, quadratic_expansion: bool = False) -> DNDarray:
    """
    Euclidean distance between all rows of ``X`` (m x f) and ``Y`` (n x f): an (m, n) DNDarray of
    square-rooted distances in promote(X, Y, float32), ``split = X.split`` (1 when only ``Y`` is
    split).  ``Y=None`` means ``Y = X``.

    ``quadratic_expansion=True``: |x-y|^2 = |x|^2 + |y|^2 - 2xy clamped at 0 (the metric KMeans
    uses); ``False``: sum((x-y)^2) directly (heat/spatial/distance.py:136-156).
    """
    return _pairwise(X, Y, _native.METRIC_EUCLID_QE if quadratic_expansion else _native.METRIC_EUCLID)


def rbf(X: DNDarray, Y: Optional[DNDarray] = None, sigma: float = 1.0,
        quadratic_expansion: bool = False) -> DNDarray:
    """Gaussian kernel exp(-|x-y|^2 / (2 sigma^2)) between all rows (heat/spatial/distance.py:159-183)."""
    return _pairwise(X, Y, _native.METRIC_GAUSS_QE if quadratic_expansion else _native.METRIC_GAUSS, sigma)


def manhattan(X: DNDarray, Y: Optional[DNDarray] = None, expand: bool = False) -> DNDarray:
    """Manhattan distance sum|x_i - y_i| between all rows; ``expand`` selects between two evaluation
    strategies in the reference and has no effect here (heat/spatial/distance.py:186-206)."""
    return _pairwise(X, Y, _native.METRIC_MANHATTAN)
