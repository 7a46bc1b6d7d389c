"""
K-Medoids with the interface of heat/cluster/kmedoids.py: Manhattan assignment, and every centre is
the data row closest (Manhattan) to its cluster's coordinate-wise median.
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


class KMedoids(_KCluster):
    def __init__(self, n_clusters: int = 8, init: Union[str, DNDarray] = "random", max_iter: int = 300,
                 random_state: Optional[int] = None):  # noqa: D107
        if isinstance(init, str) and init == "kmedoids++":
            init = "probability_based"
        super().__init__(
            metric=lambda x, y: distance.manhattan(x, y, expand=True),
            n_clusters=n_clusters,
            init=init,
            max_iter=max_iter,
            tol=0.0,
            random_state=random_state,
        )
        self._l1_metric = True

    def _medoid_step(self, xt: torch.Tensor, lab32: torch.Tensor, centers: torch.Tensor, sampler) -> torch.Tensor:
        """
        heat/cluster/kmedoids.py:57-115: median of the cluster's non-zero rows, then the row of the
        WHOLE data set closest to it (first index on ties); an empty cluster restarts at a random row.
        The reference measures that distance in float64 against the float64 median, and so does the
        snap here (``hkm_update_median_q64_f32`` hands over the medians before their rounding to float32,
        ``hkm_closest_rows_l1_q64_f32`` sums in float64): two rows at exactly the same distance -- the two
        members of a cluster on either side of their midpoint -- come out equal and the first one wins.
        """
        k, dev = self.n_clusters, xt.device
        ws = self._workspace(dev)
        fallback = draw_rows(sampler, xt.shape[0], k, dev)
        med = torch.empty_like(centers)
        med64 = torch.empty(centers.shape, dtype=torch.float64, device=dev)
        counts = torch.empty((k,), dtype=torch.int64, device=dev)
        _native.update_median(xt, lab32, med, ws, fallback_rows=fallback, counts=counts, skip_zero_rows=True,
                              median64=med64)
        idx = torch.empty((k,), dtype=torch.int64, device=dev)
        _native.closest_rows_l1_q64(xt, med64, idx, None, ws)
        # an empty cluster already holds its restart row, which is its own closest row
        return xt[idx]

    def _update_centroids(self, x: DNDarray, matching_centroids: DNDarray) -> DNDarray:
        xt = self._local_l1(x)
        lab = matching_centroids.larray.reshape(-1).to(torch.int32)
        c_new = self._medoid_step(xt, lab, self._local_f32(self._cluster_centers, like=xt), self._make_sampler(xt.device))
        return DNDarray(c_new, tuple(c_new.shape), types.canonical_heat_type(c_new.dtype), None, x.device, x.comm, True)

    def fit(self, x: DNDarray, oversampling: float = 2, iter_multiplier: float = 1) -> "KMedoids":
        """Loop of heat/cluster/kmedoids.py:117-156: stops when no centre changes."""
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
        if self.max_iter <= 0:
            raise ValueError(f"max_iter must be positive, but was {self.max_iter}")
        for _ in range(self.max_iter):
            self._n_iter += 1
            _native.assign_l1(xt, centers, lab32, None)
            c_new = self._medoid_step(xt, lab32, centers, sampler)
            if torch.equal(centers, c_new):
                break
            centers = c_new
        lab64 = torch.empty((n, 1), dtype=torch.int64, device=dev)
        _native.widen_labels(lab32, lab64)
        self._cluster_centers = DNDarray(centers, (self.n_clusters, d), types.canonical_heat_type(centers.dtype), None, x.device, x.comm, True)
        self._labels = DNDarray(lab64, (n, 1), types.int64, x.split, x.device, x.comm, True)
        return self
