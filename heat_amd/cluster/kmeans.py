"""
KMeans with the interface of heat/cluster/kmeans.py:14-148, running Lloyd's iteration as fused
gfx950 kernels: one call per iteration computes labels, the per-cluster means and the centroid
shift on the device; the host only reads the 4-byte shift to decide convergence.
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from .. import _native
from ._lloyd import LloydLoop
from ..core import types
from ..core.dndarray import DNDarray
from ..spatial import distance
from ._kcluster import _KCluster


class KMeans(_KCluster):
    """
    K-Means clustering (Lloyd's algorithm).

    Parameters
    ----------
    n_clusters : int
        Number of clusters / centroids.
    init : str or DNDarray
        ``"random"`` (K rows of the data), a (n_clusters, n_features) DNDarray of initial centers;
        ``"kmeans++"`` is accepted as an alias of ``"probability_based"`` like in the reference.
    max_iter : int
        Maximum number of Lloyd iterations.
    tol : float
        The loop stops once the squared centroid movement of an iteration is <= tol
        (``None`` disables the check).
    random_state : int
        Seed for ``init="random"``.
    """

    def __init__(self, n_clusters: int = 8, init: Union[str, DNDarray] = "random", max_iter: int = 300,
                 tol: float = 1e-4, random_state: Optional[int] = None):
        if isinstance(init, str) and init == "kmeans++":
            init = "probability_based"
        super().__init__(
            metric=lambda x, y: distance.cdist(x, y, quadratic_expansion=True),
            n_clusters=n_clusters, init=init, max_iter=max_iter, tol=tol, random_state=random_state,
        )
        self._p = 2

    def _update_centroids(self, x: DNDarray, matching_centroids: DNDarray) -> DNDarray:
        """
        Mean of the points assigned to each centroid; an empty cluster becomes a zero row
        (heat/cluster/kmeans.py:76-103).  Deterministic two-pass reduction on the device.
        """
        xt = self._local_f32(x)
        lab = matching_centroids.larray.reshape(-1).to(torch.int32)
        k = self.n_clusters
        c_new = torch.empty((k, xt.shape[1]), dtype=xt.dtype, device=xt.device)
        _native.update(xt, lab, c_new, None, self._workspace(xt.device))
        return DNDarray(c_new, tuple(c_new.shape), types.canonical_heat_type(xt.dtype), None, x.device, x.comm, True)

    def fit(self, x: DNDarray, oversampling: float = 2, iter_multiplier: float = 1) -> "KMeans":
        """
        Compute the centroids (heat/cluster/kmeans.py:105-148).  After the call ``labels_`` holds the
        assignment of the LAST iteration (against the centroids before their final update),
        ``inertia_`` the last squared centroid movement and ``n_iter_`` the iterations run.
        """
        if not isinstance(x, DNDarray):
            raise TypeError(f"Input needs to be a ht.DNDarray, but was {type(x)}")

        self._initialize_cluster_centers(x, oversampling, iter_multiplier)
        self._n_iter = 0
        self._check_split(x)

        xt = self._local_f32(x)
        dev = xt.device
        n, d = xt.shape
        k = self.n_clusters
        # the reference evaluates ``inertia <= tol`` on the host every iteration (kmeans.py:143); the
        # loop keeps the next step enqueued while the host looks at the shift of the current one
        loop = LloydLoop(xt, self._local_f32(self._cluster_centers, like=xt), self._workspace(dev))
        self._n_iter = loop.run(self.max_iter, self.tol)
        if self._n_iter == 0:
            raise ValueError(f"max_iter must be positive, but was {self.max_iter}")
        c_cur, lab32, shift = loop.centers, loop.labels, loop.last_shift

        lab64 = torch.empty((n, 1), dtype=torch.int64, device=dev)
        _native.widen_labels(lab32, lab64)
        ftype = types.canonical_heat_type(xt.dtype)
        self._cluster_centers = DNDarray(c_cur, (k, d), ftype, None, x.device, x.comm, True)
        self._inertia = DNDarray(shift.clone(), (), ftype, None, x.device, x.comm, True)
        self._labels = DNDarray(lab64, (n, 1), types.int64, x.split, x.device, x.comm, True)
        return self
