"""
KMeans with the interface of heat/cluster/kmeans.py:14-148, running Lloyd's iteration as fused
gfx950 kernels: one call per iteration computes labels, the per-cluster means and the centroid
shift on the device; the host only reads the 4-byte shift to decide convergence.
"""

from __future__ import annotations

import os
import threading
import warnings
from typing import Optional, Union

import torch

from .. import _native
from ._lloyd import LloydLoop
from ..core import types
from ..core.dndarray import DNDarray
from ..spatial import distance
from ._kcluster import _KCluster


# pinned status words of the one-launch fit (iterations run or a negative status, bits of the last shift): one pair
# per device and host thread, allocated once -- a pinned allocation costs more than the fit it would serve
_FIT_INFO = {}


def _fit_info(device: torch.device):
    key = (device.index, threading.get_ident())
    pair = _FIT_INFO.get(key)
    if pair is None:
        t = torch.zeros((2,), dtype=torch.int32, pin_memory=True)
        pair = (t, t.numpy())
        _FIT_INFO[key] = pair
    return pair


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
        if self.max_iter >= 1 and xt.dtype == torch.float32 and os.environ.get("HKM_FIT") != "steps" \
                and _native.lloyd_fit_supported(n, d, k):
            # a few hundred thousand narrow rows: the whole loop is one launch (the rows stay in registers, the
            # stop decision is taken on the device); on a negative status the loop below runs instead
            if self._fit_one_launch(x, xt):
                return self
        # the reference evaluates ``inertia <= tol`` on the host every iteration (kmeans.py:143); the
        # loop keeps the next step enqueued while the host looks at the shift of the current one
        loop = LloydLoop(xt, self._local_f32(self._cluster_centers, like=xt), self._workspace(dev))
        # the (N, 1) int64 labels the reference returns: for the narrow shapes the step known to be the last writes
        # them itself
        lab64 = torch.empty((n, 1), dtype=torch.int64, device=dev)
        loop.final_labels64(lab64.view(-1))
        self._n_iter = loop.run(self.max_iter, self.tol)
        if self._n_iter == 0:
            raise ValueError(f"max_iter must be positive, but was {self.max_iter}")
        loop.labels64_into(lab64)
        c_cur, shift = loop.centers, loop.last_shift
        ftype = types.canonical_heat_type(xt.dtype)
        self._cluster_centers = DNDarray(c_cur, (k, d), ftype, None, x.device, x.comm, True)
        self._inertia = DNDarray(shift.clone(), (), ftype, None, x.device, x.comm, True)
        self._labels = DNDarray(lab64, (n, 1), types.int64, x.split, x.device, x.comm, True)
        return self

    def _fit_one_launch(self, x: DNDarray, xt: torch.Tensor) -> bool:
        """The loop of heat/cluster/kmeans.py:131-146 as one launch of hkm_lloyd_fit_f32.  True if it delivered;
        False if the kernel reported that it could not (a wait between its workgroups ran out, or the data hold a
        non-finite value), in which case nothing has been set and the caller runs the loop step by step."""
        dev = xt.device
        n, d = xt.shape
        k = self.n_clusters
        c0 = self._local_f32(self._cluster_centers, like=xt)
        _native._require_gpu(xt, c0)
        c_out = torch.empty((k, d), dtype=torch.float32, device=dev)
        lab64 = torch.empty((n, 1), dtype=torch.int64, device=dev)
        shift = torch.empty((), dtype=torch.float32, device=dev)
        info, info_np = _fit_info(dev)
        info_np[0] = 0
        _native.lloyd_fit(xt, c0.contiguous(), self.max_iter, self.tol, c_out, lab64.view(-1), shift, info,
                          self._workspace(dev))
        torch.cuda.current_stream().synchronize()
        n_iter = int(info_np[0])
        if n_iter < 1:
            if n_iter == -1:
                warnings.warn("the one-launch k-means fit gave up waiting for its workgroups (is the GPU shared?); "
                              "running the loop step by step instead")
            return False
        ftype = types.canonical_heat_type(xt.dtype)
        self._n_iter = n_iter
        self._cluster_centers = DNDarray(c_out, (k, d), ftype, None, x.device, x.comm, True)
        self._inertia = DNDarray(shift, (), ftype, None, x.device, x.comm, True)
        self._labels = DNDarray(lab64, (n, 1), types.int64, x.split, x.device, x.comm, True)
        return True
