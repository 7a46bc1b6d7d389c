"""
K-Medians with the interface of heat/cluster/kmedians.py: Manhattan assignment, per-cluster
coordinate-wise median.

The reference loops over the clusters in Python and sorts every cluster's rows for ``ht.median``;
here one iteration is a fused Manhattan distance+argmin kernel and one radix-selection update for all
clusters and coordinates at once (``hkm_assign_l1_f32``, ``hkm_update_median_f32``).
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from .. import _native
from ..core import types
from ..core.dndarray import DNDarray
from ..spatial import distance
from ._kcluster import _KCluster
from ._sampling import draw_rows


class KMedians(_KCluster):
    def __init__(self, n_clusters: int = 8, init: Union[str, DNDarray] = "random", max_iter: int = 300,
                 tol: float = 1e-4, random_state: Optional[int] = None):  # noqa: D107
        if isinstance(init, str) and init == "kmedians++":
            init = "probability_based"
        super().__init__(
            metric=lambda x, y: distance.manhattan(x, y, expand=True),
            n_clusters=n_clusters,
            init=init,
            max_iter=max_iter,
            tol=tol,
            random_state=random_state,
        )
        self._p = 1
        self._l1_metric = True

    def _median_step(self, xt: torch.Tensor, lab32: torch.Tensor, centers: torch.Tensor, sampler) -> torch.Tensor:
        """
        New centres from int32 labels (heat/cluster/kmedians.py:76-118): the median of every coordinate
        over the cluster's rows, rows that are entirely zero left out as the reference's
        ``x * selection`` bookkeeping does; a cluster without rows restarts at a random data row.
        """
        k, dev = self.n_clusters, xt.device
        # the reference draws a row only for clusters that turn out empty; drawing one per cluster up
        # front keeps the update free of a host round trip (its random stream is not reproducible anyway)
        fallback = draw_rows(sampler, xt.shape[0], k, dev)
        c_new = torch.empty_like(centers)
        _native.update_median(xt, lab32, c_new, self._workspace(dev), fallback_rows=fallback, skip_zero_rows=True)
        return c_new

    def _update_centroids(self, x: DNDarray, matching_centroids: DNDarray) -> DNDarray:
        xt = self._local_l1(x)
        lab = matching_centroids.larray.reshape(-1).to(torch.int32)
        c_new = self._median_step(xt, lab, self._local_f32(self._cluster_centers, like=xt), self._make_sampler(xt.device))
        return DNDarray(c_new, tuple(c_new.shape), types.canonical_heat_type(c_new.dtype), None, x.device, x.comm, True)

    def fit(self, x: DNDarray, oversampling: float = 2, iter_multiplier: float = 1) -> "KMedians":
        """Loop of heat/cluster/kmedians.py:120-147: assign, medians, squared centre movement <= tol."""
        if not isinstance(x, DNDarray):
            raise ValueError(f"input needs to be a ht.DNDarray, but was {type(x)}")
        self._initialize_cluster_centers(x, oversampling, iter_multiplier)
        self._n_iter = 0
        self._check_split(x)
        xt = self._local_l1(x)
        dev = xt.device
        n, d = xt.shape
        sampler = self._make_sampler(dev)
        centers = self._local_f32(self._cluster_centers, like=xt).clone()
        lab32 = torch.empty((n,), dtype=torch.int32, device=dev)
        shift = torch.zeros((), dtype=xt.dtype, device=dev)
        if self.max_iter <= 0:
            raise ValueError(f"max_iter must be positive, but was {self.max_iter}")
        for _ in range(self.max_iter):
            self._n_iter += 1
            _native.assign_l1(xt, centers, lab32, None)
            c_new = self._median_step(xt, lab32, centers, sampler)
            _native.shift(centers, c_new, shift)
            centers = c_new
            if self.tol is not None and shift.item() <= self.tol:
                break
        lab64 = torch.empty((n, 1), dtype=torch.int64, device=dev)
        _native.widen_labels(lab32, lab64)
        self._cluster_centers = DNDarray(centers, (self.n_clusters, d), types.canonical_heat_type(centers.dtype), None, x.device, x.comm, True)
        self._inertia = DNDarray(shift.clone(), (), types.canonical_heat_type(shift.dtype), None, x.device, x.comm, True)
        self._labels = DNDarray(lab64, (n, 1), types.int64, x.split, x.device, x.comm, True)
        return self
