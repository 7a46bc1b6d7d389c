"""
Graph Laplacian with the interface of heat/graph/laplacian.py.

``construct`` calls the similarity function (``ht.spatial.cdist`` / ``rbf`` ..., whose full-matrix kernels
produce S) and hands S to ``hkm_laplacian_f32``: one read for the degrees, one read and one write for L,
in place of the reference's chain of whole-matrix operations (:119-142).
"""

from __future__ import annotations

from typing import Callable

import torch

from .. import _native
from ..core import types
from ..core.dndarray import DNDarray


class Laplacian:
    def __init__(self, similarity: Callable, weighted: bool = True, definition: str = "norm_sym",
                 mode: str = "fully_connected", threshold_key: str = "upper", threshold_value: float = 1.0,
                 neighbours: int = 10):  # noqa: D107
        self.similarity_metric = similarity
        self.weighted = weighted
        if definition not in ["simple", "norm_sym"]:
            raise NotImplementedError("Currently only simple and normalized symmetric graph laplacians are supported")
        self.definition = definition
        if mode not in ["eNeighbour", "fully_connected"]:
            raise NotImplementedError("Only eNeighborhood and fully-connected graphs supported at the moment.")
        self.mode = mode
        if threshold_key not in ["upper", "lower"]:
            raise ValueError("Only 'upper' and 'lower' threshold types supported for eNeighbouhood graph construction")
        self.epsilon = (threshold_key, threshold_value)
        self.neighbours = neighbours

    def construct(self, X: DNDarray) -> DNDarray:
        """heat/graph/laplacian.py:100-142.  float32 and float64 similarities keep their type; of an unweighted
        eNeighbour graph the simple Laplacian is an int64 matrix and the normalised one float32, as in the
        reference (an int32 adjacency matrix, :129-133, minus the int64 diagonal of its row sums, :110-112,
        resp. divided by the float32 square roots of those sums, :96-97)."""
        S = self.similarity_metric(X)
        if not isinstance(S, DNDarray) or len(S.shape) != 2 or S.shape[0] != S.shape[1]:
            raise ValueError("the similarity function must return a square DNDarray")
        # the reference zeroes the diagonal of what the similarity call returned, in place (:123): a caller that
        # keeps that matrix sees the same change here
        S.larray.fill_diagonal_(0)
        s = S.larray
        if s.dtype not in (torch.float32, torch.float64):
            s = s.to(torch.float32)
        if s.stride(-1) != 1:
            s = s.contiguous()
        n = s.shape[0]
        mode = 0 if self.mode == "fully_connected" else (1 if self.epsilon[0] == "upper" else 2)
        degree = torch.empty((n,), dtype=s.dtype, device=s.device)
        # L gets storage of its own: the similarity callable may have returned a matrix it keeps (a cached
        # or precomputed one), which the reference leaves intact apart from the diagonal zeroed above
        out = torch.empty((n, n), dtype=s.dtype, device=s.device)
        _native.laplacian(s, out, 0 if self.definition == "simple" else 1, mode, bool(self.weighted),
                          float(self.epsilon[1]), degree)
        if self.mode == "eNeighbour" and not self.weighted:
            # the reference's unweighted adjacency is an int32 matrix: D - A comes out as int64, and the
            # normalised form divides it by float32 square roots of the integer degrees
            out = out.to(torch.int64 if self.definition == "simple" else torch.float32)
        return DNDarray(out, (n, n), types.canonical_heat_type(out.dtype), S.split, S.device, S.comm, True)
