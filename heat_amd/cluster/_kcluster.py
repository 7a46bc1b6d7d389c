"""
Base of the k-clustering estimators, with the interface of heat/cluster/_kcluster.py:13-415.

The reference composes assignment from generic array ops (cdist -> argmin); here
``_assign_to_cluster`` is one call into the fused distance+argmin kernel, so the N x K matrix is
never built.
"""

from __future__ import annotations

import math
import warnings
from typing import Optional, Union

import torch

from .. import _native
from ..core import types
from ..core.base import BaseEstimator, ClusteringMixin
from ..core.dndarray import DNDarray
from ._sampling import DeviceSampler


class _KCluster(ClusteringMixin, BaseEstimator):
    def __init__(self, metric, n_clusters: int, init: Union[str, DNDarray], max_iter: int, tol: float,
                 random_state: Optional[int]):  # noqa: D107
        self.n_clusters = n_clusters
        self.init = init
        self.max_iter = max_iter
        self.tol = tol
        self.random_state = random_state

        self._metric = metric
        self._cluster_centers = None
        self._functional_value = None
        self._labels = None
        self._inertia = None
        self._n_iter = None
        self._p = None
        self._l1_metric = False
        self._ws = None

    # ---- read-only results (heat/cluster/_kcluster.py:63-98) -----------------------------------
    @property
    def cluster_centers_(self) -> DNDarray:
        return self._cluster_centers

    @property
    def labels_(self) -> DNDarray:
        return self._labels

    @property
    def inertia_(self):
        """Squared centroid movement of the last iteration (what the reference stores, kmeans.py:141)."""
        return self._inertia

    @property
    def n_iter_(self) -> int:
        return self._n_iter

    @property
    def functional_value_(self) -> DNDarray:
        return self._functional_value

    # ---- helpers ---------------------------------------------------------------------------
    def _workspace(self, device: torch.device) -> _native.Workspace:
        if self._ws is None or self._ws.device != device:
            self._ws = _native.Workspace(device)
        return self._ws

    @staticmethod
    def _local_f32(x: DNDarray, like: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The local tensor as a row-major matrix in the compute dtype: float32, or float64 where the
        reference's promote(X, C, float32) gives float64 (float64 and int64 data).  ``like`` forces the
        dtype of another operand (centroids follow the data)."""
        t = x.larray
        if t.dim() != 2:
            raise NotImplementedError("Only 2D data matrices are currently supported")
        want = torch.float64 if types.promote_types(x.dtype, types.float32) is types.float64 else torch.float32
        if like is not None:
            want = like.dtype
        if t.dtype != want:
            t = t.to(want)
        if t.stride(1) != 1 or (t.shape[0] > 1 and t.stride(0) < t.shape[1]):
            t = t.contiguous()
        return t

    def _local_l1(self, x: DNDarray) -> torch.Tensor:
        """The local matrix for the Manhattan-metric estimators: float32 runs on the fused kernels, float64
        (float64 and int64 data, which the reference keeps in float64) on the composed float64 steps."""
        return self._local_f32(x)

    def _manhattan_metric(self) -> bool:
        """True for the estimators constructed with the Manhattan metric (KMedians, KMedoids set it)."""
        return self._l1_metric

    @staticmethod
    def _check_split(x: DNDarray) -> None:
        # the reference raises this from cdist (heat/spatial/distance.py:386-390)
        if x.split is not None and x.split != 0:
            raise NotImplementedError(
                f"Input splits were X.split = {x.split}, Y.split = None. Splittings other than 0 or None currently not supported."
            )

    def _initialize_cluster_centers(self, x: DNDarray, oversampling: float, iter_multiplier: float):
        """
        Initial centroids; checks in the order of heat/cluster/_kcluster.py:116-143,276-281.
        ``"random"`` (K rows drawn with a generator seeded by ``random_state``), an explicit (K, D)
        DNDarray, which is copied so later changes by the caller do not leak in,
        ``"probability_based"`` (k-means||) and ``"batchparallel"``.
        """
        if not isinstance(x, DNDarray):
            raise ValueError(f"Input x needs to be a ht.DNDarray, but was {type(x)}")
        if oversampling < 2:
            raise ValueError(f"Oversampling factor should be at least 2, but was {oversampling}")
        if iter_multiplier < 1:
            raise ValueError(f"Iteration multiplier should be at least 1, but was {iter_multiplier}")

        if isinstance(self.init, str) and self.init == "random":
            gen = torch.Generator(device="cpu")
            if self.random_state is not None:
                gen.manual_seed(int(self.random_state))
            else:
                gen.seed()
            # same index range as the reference: randint(0, n - 1) excludes the last row
            hi = max(x.shape[0] - 1, 1)
            idx = torch.randint(0, hi, (self.n_clusters,), generator=gen).to(x.larray.device)
            cent = x.larray[idx, :].clone()
            self._cluster_centers = DNDarray(cent, tuple(cent.shape), x.dtype, None, x.device, x.comm, True)
        elif isinstance(self.init, DNDarray):
            if len(self.init.shape) != 2:
                raise ValueError(f"passed centroids need to be two-dimensional, but are {len(self.init)}")
            if self.init.shape[0] != self.n_clusters or self.init.shape[1] != x.shape[1]:
                raise ValueError("passed centroids do not match cluster count or data shape")
            self._cluster_centers = self.init.resplit(None)
        elif isinstance(self.init, str) and self.init == "probability_based":
            if x.split is None or x.split == 0:
                cent = self._kmeans_parallel(x, oversampling, iter_multiplier)
                self._cluster_centers = DNDarray(cent, tuple(cent.shape), types.canonical_heat_type(cent.dtype), None,
                                                 x.device, x.comm, True)
            else:
                raise NotImplementedError("Not implemented for other splitting-axes")
        elif isinstance(self.init, str) and self.init == "batchparallel":
            if x.split == 0:
                if self._p == 2:
                    from .batchparallelclustering import BatchParallelKMeans

                    clusterer = BatchParallelKMeans(n_clusters=self.n_clusters, init="k-means++", max_iter=100,
                                                    random_state=self.random_state)
                elif self._p == 1:
                    from .batchparallelclustering import BatchParallelKMedians

                    clusterer = BatchParallelKMedians(n_clusters=self.n_clusters, init="k-medians++", max_iter=100,
                                                      random_state=self.random_state)
                else:
                    raise ValueError("Batch parallel initialization only implemented for KMeans and KMedians")
                clusterer.fit(x)
                self._cluster_centers = clusterer.cluster_centers_
            else:
                raise NotImplementedError(
                    f"Batch parallel initalization only implemented for split = 0, but split was {x.split}"
                )
        else:
            raise ValueError(
                'init needs to be one of "random", ht.DNDarray, "kmeans++", or "batchparallel", but was {}'.format(
                    self.init
                )
            )

    # ---- k-means|| (heat/cluster/_kcluster.py:146-247, 283-350) --------------------------------
    def _make_sampler(self, device: torch.device):
        """Source of the initialiser's random draws; replaced in tests to feed fixed numbers."""
        return DeviceSampler(device, self.random_state)

    def _centroid_sampling_helper(self, xt: torch.Tensor, centroids: torch.Tensor, oversampling: float,
                                  num_iters: int, sampler, ws, dmin: Optional[torch.Tensor] = None) -> torch.Tensor:
        """
        ``num_iters`` rounds of: distance of every row to its closest current candidate, then every
        row joins the candidates with probability ``oversampling * distance / sum(distance)``
        (heat/cluster/_kcluster.py:283-350).  ``dmin``, if given, holds the squared distances to the
        closest of the candidates passed in (it is overwritten).  The reference recomputes the distances to ALL
        candidates in every round; the minimum over a grown set is the minimum of the old minimum and
        the distances to the new members, so a round here costs one fused distance+argmin launch
        against the handful of NEW candidates, one pass that merges the minimum and sums the next
        round's cost, and one ordered selection; only the number of new candidates comes back to the
        host.
        """
        n = xt.shape[0]
        dev = xt.device
        lab = torch.empty((n,), dtype=torch.int32, device=dev)
        if dmin is None:
            dmin = torch.empty((n,), dtype=xt.dtype, device=dev)
            _native.assign(xt, centroids, lab, dmin, ws)
        dnew = torch.empty_like(dmin)
        cost = torch.empty((), dtype=torch.float32, device=dev)
        count = torch.zeros((), dtype=torch.int64, device=dev)
        idx = torch.empty((max(1024, int(16 * oversampling)),), dtype=torch.int64, device=dev)
        f32 = dmin.dtype == torch.float32
        _native.min_dist_sum(dmin if f32 else dmin.float(), cost, ws)
        for it in range(num_iters):
            d2 = dmin if f32 else dmin.float()  # the draw itself runs in float32
            u = sampler.uniform(n)
            _native.sample_select(d2, u, cost, oversampling, idx, count, ws)
            c = int(count.item())
            if c > idx.numel():
                idx = torch.empty((c,), dtype=torch.int64, device=dev)
                _native.sample_select(d2, u, cost, oversampling, idx, count, ws)
            if c == 0:
                continue
            fresh = xt[idx[:c]]
            centroids = torch.cat((centroids, fresh), dim=0)
            if it + 1 < num_iters:
                _native.assign(xt, fresh, lab, dnew, ws)
                if f32:
                    _native.min_merge_sum(dmin, dnew, cost, ws)  # running minimum and the next round's cost
                else:
                    torch.minimum(dmin, dnew, out=dmin)
                    _native.min_dist_sum(dmin.float(), cost, ws)
        return centroids

    def _kmeans_parallel(self, x: DNDarray, oversampling: float, iter_multiplier: float) -> torch.Tensor:
        """(K, D) initial centroids by k-means|| and a weighted k-means++ reclustering of the candidates."""
        from .batchparallelclustering import _kmex

        xt = self._local_f32(x)
        n = xt.shape[0]
        dev = xt.device
        ws = self._workspace(dev)
        sampler = self._make_sampler(dev)
        # randint(0, n - 1) of the reference excludes the last row
        first = sampler.randint(max(n - 1, 1))
        init_centroids = xt[first : first + 1].clone()
        lab = torch.empty((n,), dtype=torch.int32, device=dev)
        dmin = torch.empty((n,), dtype=xt.dtype, device=dev)
        cost = torch.empty((), dtype=torch.float32, device=dev)
        _native.assign(xt, init_centroids, lab, dmin, ws)
        _native.min_dist_sum(dmin if dmin.dtype == torch.float32 else dmin.float(), cost, ws)
        init_cost = float(cost.item())
        # the order of magnitude of the initial cost sets the number of rounds (_kcluster.py:172-175);
        # all rows equal gives cost 0, where the reference fails in int(-inf): one round instead
        num_iters = max(1, int(iter_multiplier * math.log(init_cost))) if init_cost > 0.0 else 1
        self._init_rounds = num_iters
        centroids = self._centroid_sampling_helper(xt, init_centroids, oversampling, num_iters, sampler, ws,
                                                   dmin.clone())
        if centroids.shape[0] <= self.n_clusters:
            warnings.warn(
                f"Oversampling={oversampling} is too low for data set."
                "Increasing it by factor 10 automatically. And restarting centroid initialization.",
                UserWarning,
            )
            oversampling = 10 * oversampling
            centroids = self._centroid_sampling_helper(xt, init_centroids, oversampling, num_iters, sampler, ws, dmin)
        if centroids.shape[0] <= self.n_clusters:
            raise ValueError(
                f"The parameter oversampling={oversampling} and/or iter_multiplier={iter_multiplier} "
                "are chosen too small for the initialization of cluster centers."
            )
        # weight of a candidate = number of rows closest to it (_kcluster.py:198-208)
        m = centroids.shape[0]
        _native.assign(xt, centroids, lab, None, ws)
        counts = torch.empty((m,), dtype=torch.int64, device=dev)
        _native.label_counts(lab, m, counts)
        weights = counts.to(torch.float32)
        centers, _ = _kmex(centroids, 2, self.n_clusters, "++", self.max_iter, self.tol, sampler, weights, ws)
        return centers

    def _assign_to_cluster(self, x: DNDarray, eval_functional_value: bool = False) -> DNDarray:
        """
        (N, 1) int64 labels of the closest centroid, ``split = x.split``; optionally sets
        ``functional_value_`` = ||min_k dist||_2 ** 2 (heat/cluster/_kcluster.py:352-370).
        """
        self._check_split(x)
        xt = self._local_f32(x)
        if self._manhattan_metric() and xt.dtype != torch.float32:
            raise NotImplementedError("the Manhattan-metric kernels cover float32 data only")
        ct = self._local_f32(self._cluster_centers, like=xt)
        if xt.shape[1] != ct.shape[1]:
            raise ValueError("Inputs must have same shape[1]")
        dev = xt.device
        n = xt.shape[0]
        ws = self._workspace(dev)
        lab32 = torch.empty((n,), dtype=torch.int32, device=dev)
        min_d2 = torch.empty((n,), dtype=xt.dtype, device=dev) if eval_functional_value else None
        if self._manhattan_metric():
            # k-medians / k-medoids: fused sum|x - c| + argmin; the functional is the squared 2-norm of
            # the minimum distances, so they are squared before the same reduction
            _native.assign_l1(xt, ct, lab32, min_d2)
            if min_d2 is not None:
                min_d2.mul_(min_d2)
        else:
            _native.assign(xt, ct, lab32, min_d2, ws)
        lab64 = torch.empty((n, 1), dtype=torch.int64, device=dev)
        _native.widen_labels(lab32, lab64)
        if eval_functional_value:
            fv = torch.empty((), dtype=xt.dtype, device=dev)
            _native.functional_value(min_d2, fv, ws)
            self._functional_value = DNDarray(fv, (), types.canonical_heat_type(xt.dtype), None, x.device, x.comm,
                                              True)
        return DNDarray(lab64, (n, 1), types.int64, x.split, x.device, x.comm, True)

    def _update_centroids(self, x: DNDarray, matching_centroids: DNDarray):
        raise NotImplementedError()

    def fit(self, x: DNDarray):
        raise NotImplementedError()

    def predict(self, x: DNDarray) -> DNDarray:
        """Index of the closest centroid for every row of ``x`` (heat/cluster/_kcluster.py:398-415)."""
        if not isinstance(x, DNDarray):
            raise ValueError(f"input needs to be a ht.DNDarray, but was  {type(x)}")
        return self._assign_to_cluster(x, eval_functional_value=True)
