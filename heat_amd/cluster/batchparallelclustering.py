"""
Single-device k-means++ seeding and Lloyd iteration on a local matrix, and the batch-parallel
estimator built from them; interface of heat/cluster/batchparallelclustering.py.

The reference runs these helpers with ``torch.cdist`` / ``torch.argmin`` / ``torch.mean``; here every
distance + argmin is one call of the fused kernel (``hkm_assign_f32``) and every mean one call of the
deterministic update (``hkm_update_f32``), torch only supplies memory, the random draws and a few
elementwise operations on K x D or N-element vectors.
"""

from __future__ import annotations

from typing import Optional, Tuple, Union
from warnings import warn

import torch

from .. import _native
from ..core import types
from ..core.base import BaseEstimator, ClusteringMixin
from ..core.dndarray import DNDarray
from ._sampling import DeviceSampler, draw_rows


def _dist_to_row(x: torch.Tensor, row: torch.Tensor, p: int) -> torch.Tensor:
    """Distance of every row of x to one row: sqrt(sum((x_i - row)^2)) for p = 2 (direct form: exactly
    zero for the row itself, which a quadratic expansion does not guarantee), sum|x_i - row| for p = 1."""
    out = torch.empty((x.shape[0], 1), dtype=x.dtype, device=x.device)
    _native.pairwise(x, row.reshape(1, -1).contiguous(), out,
                     _native.METRIC_MANHATTAN if p == 1 else _native.METRIC_EUCLID)
    return out.view(-1)


def _initialize_plus_plus(x: torch.Tensor, n_clusters: int, p: int, sampler, weights=1.0,
                          max_samples: int = 2**24 - 1, ws: Optional[_native.Workspace] = None) -> torch.Tensor:
    """
    k-means++ seeding as heat/cluster/batchparallelclustering.py:22-46 does it: the first centre
    uniformly, every further one with probability proportional to ``weights * distance`` (the plain
    p-norm distance to the closest centre chosen so far, not its square).  More than ``max_samples`` rows
    are subsampled first because a categorical draw is limited to 2**24 categories.  Up to
    ``_native.SEED_MAX_ROWS`` float32 rows with a sampler that allows it (``fused_seeding``) are seeded by
    one kernel launch that draws by inverse CDF from one uniform number per centre.  The reference
    recomputes the distances to all chosen centres in every step; the running minimum kept here is
    the same number and needs one N x 1 distance column per step.
    """
    if x.shape[0] > max_samples:
        x = x[draw_rows(sampler, x.shape[0], max_samples, x.device)].contiguous()
    if (getattr(sampler, "fused_seeding", False) and x.dtype == torch.float32 and x.shape[0] <= _native.SEED_ROWS_MAX
            and p in (1, 2)):
        # every draw by inverse CDF from one uniform number, none of them waiting for the host: a small
        # row set (the candidates of k-means||) in ONE launch, a large one in two launches per centre
        w = None
        if isinstance(weights, torch.Tensor):
            w = weights.to(device=x.device, dtype=torch.float32).contiguous()
        elif float(weights) != 1.0:
            w = torch.full((x.shape[0],), float(weights), dtype=torch.float32, device=x.device)
        first = sampler.randint(x.shape[0])
        u = sampler.uniform(max(n_clusters - 1, 1))
        idx = torch.empty((n_clusters,), dtype=torch.int64, device=x.device)
        xc = x.contiguous() if x.stride(1) != 1 else x
        if x.shape[0] <= _native.SEED_MAX_ROWS:
            _native.seed_plus_plus(xc, w, first, u, n_clusters, p, idx)
        else:
            _native.seed_plus_plus_rows(xc, w, first, u, n_clusters, p, idx, ws or _native.Workspace(x.device))
        if bool((idx < 0).any()):
            raise RuntimeError("invalid multinomial distribution (sum of probabilities <= 0)")
        return x[idx]
    # the drawn indices stay on the device where the sampler can leave them there: a draw only feeds
    # the gather of the next centre, and reading each one back would stall the queue n_clusters times
    draw = getattr(sampler, "multinomial_on_device", None) or sampler.multinomial
    idxs = [sampler.randint(x.shape[0])]
    dist = _dist_to_row(x, x[idxs[0]], p)
    for i in range(1, n_clusters):
        idxs.append(draw(weights * dist))
        if i + 1 < n_clusters:
            dist = torch.minimum(dist, _dist_to_row(x, x[idxs[-1]].reshape(-1), p))
    return x[torch.stack([torch.as_tensor(i, device=x.device).reshape(()) for i in idxs])]


def _kmex(x: torch.Tensor, p: int, n_clusters: int, init: Union[str, torch.Tensor], max_iter: int, tol: float,
          sampler=None, weights=1.0, ws: Optional[_native.Workspace] = None) -> Tuple[torch.Tensor, int]:
    """
    Lloyd iteration on a local matrix (heat/cluster/batchparallelclustering.py:49-88): an empty
    cluster KEEPS its centre (unlike KMeans._update_centroids), the loop stops when
    ``allclose(centers, previous, atol=tol)`` (rtol 1e-5).  p = 1 is k-medians: Manhattan assignment
    and ``torch.median``, i.e. the LOWER middle value of every coordinate.  Any other p runs as p = 2,
    like the reference.  Returns (centers, iterations run).
    """
    _native._require_gpu(x)
    ws = ws or _native.Workspace(x.device)
    sampler = sampler or DeviceSampler(x.device)
    if isinstance(init, torch.Tensor):
        if init.shape != (n_clusters, x.shape[1]):
            raise ValueError("if a torch tensor, init must have shape (n_clusters, n_features).")
        centers = init.to(x.dtype).contiguous()
    elif init == "++":
        centers = _initialize_plus_plus(x, n_clusters, p, sampler, weights, ws=ws)
    elif init == "random":
        centers = x[draw_rows(sampler, x.shape[0], n_clusters, x.device)]
    else:
        raise ValueError("init must be a torch tensor with initial centers, string '++', or 'random'.")
    n = x.shape[0]
    lab = torch.empty((n,), dtype=torch.int32, device=x.device)
    counts = torch.empty((n_clusters,), dtype=torch.int64, device=x.device)
    means = torch.empty_like(centers)
    it = 0
    for it in range(max_iter):
        if p == 1:
            _native.assign_l1(x, centers, lab, None)
            new = torch.empty_like(centers)
            _native.update_median(x, lab, new, ws, c_old=centers.contiguous(), lower=True)
        else:
            _native.assign(x, centers, lab, None, ws)
            _native.update(x, lab, means, counts, ws)
            new = torch.where(counts.unsqueeze(1) > 0, means, centers)
        done = bool(torch.allclose(new, centers, atol=tol))
        centers = new
        if done:
            break
    return centers, it + 1


class _BatchParallelKCluster(ClusteringMixin, BaseEstimator):
    """Checks and result attributes of heat/cluster/batchparallelclustering.py:99-331 at one rank."""

    def __init__(self, p: int, n_clusters: int, init: str, max_iter: int, tol: float,
                 random_state: Optional[int], n_procs_to_merge: Optional[int]):  # noqa: D107
        if not isinstance(n_clusters, int):
            raise TypeError(f"n_clusters must be int, but was {type(n_clusters)}")
        if n_clusters <= 0:
            raise ValueError(f"n_clusters must be positive, but was {n_clusters}")
        if not isinstance(max_iter, int):
            raise TypeError(f"max_iter must be int, but was {type(max_iter)}")
        if max_iter <= 0:
            raise ValueError(f"max_iter must be positive, but was {max_iter}")
        if not isinstance(tol, float):
            raise TypeError(f"tol must be float, but was {type(tol)}")
        if tol <= 0:
            raise ValueError(f"tol must be positive, but was {tol}")
        if not isinstance(random_state, int) and random_state is not None:
            raise TypeError(f"random_state must be int or None, but was {type(random_state)}")
        if not isinstance(n_procs_to_merge, int) and n_procs_to_merge is not None:
            raise TypeError(f"procs_to_merge must be int or None, but was {type(n_procs_to_merge)}")
        if n_procs_to_merge is not None and n_procs_to_merge <= 1:
            raise ValueError(f"If an integer, procs_to_merge must be > 1, but was {n_procs_to_merge}.")

        self.n_clusters = n_clusters
        self._init = init
        self.max_iter = max_iter
        self.tol = tol
        self.random_state = random_state
        self.n_procs_to_merge = n_procs_to_merge
        if not (p == 1 or p == 2):
            warn(
                "p should be 1 (k-Medians) or 2 (k-Means). For other choice of p, we proceed as for p=2 and hope for the best.",
                UserWarning,
            )
        self._p = p
        self._cluster_centers = None
        self._n_iter = None
        self._functional_value = None
        self._ws = None

    @property
    def cluster_centers_(self) -> DNDarray:
        return self._cluster_centers

    @property
    def n_iter_(self):
        return self._n_iter

    @property
    def functional_value_(self):
        return self._functional_value

    def _make_sampler(self, device: torch.device, rank: int = 0):
        seed = None if self.random_state is None else self.random_state + rank
        return DeviceSampler(device, seed)

    def _local_f32(self, x: DNDarray) -> torch.Tensor:
        """Local rows in the compute dtype: float64 stays float64, everything else becomes float32."""
        t = x.larray
        if t.dtype == torch.float64:
            return t.contiguous()
        if t.dtype != torch.float32:
            t = t.to(torch.float32)
        return t.contiguous()

    def fit(self, x: DNDarray):
        """One rank: the local clustering is the global one (batchparallelclustering.py:177-269)."""
        if not isinstance(x, DNDarray):
            raise TypeError(f"input needs to be a ht.DNDarray, but was {type(x)}")
        if not x.ndim == 2:
            raise ValueError(f"input needs to be 2D, but was {x.ndim}D")
        if x.split != 0:
            raise ValueError(f"input needs to be split along the sample axis, but was split along {x.split}")
        xt = self._local_f32(x)
        if self._ws is None or self._ws.device != xt.device:
            self._ws = _native.Workspace(xt.device)
        centers, n_iter = _kmex(xt, self._p, self.n_clusters, self._init, self.max_iter, self.tol,
                                self._make_sampler(xt.device, x.comm.rank), ws=self._ws)
        self._cluster_centers = DNDarray(centers, (self.n_clusters, x.shape[1]),
                                         types.canonical_heat_type(centers.dtype), None, x.device, x.comm, True)
        self._n_iter = n_iter
        return self

    def predict(self, x: DNDarray) -> DNDarray:
        """(N, 1) int32 labels; sets ``functional_value_`` (batchparallelclustering.py:271-331)."""
        if not isinstance(x, DNDarray):
            raise TypeError(f"input needs to be a ht.DNDarray, but was {type(x)}")
        if not x.ndim == 2:
            raise ValueError(f"input needs to be 2D, but was {x.ndim}D")
        if x.split != 0:
            raise ValueError(f"input needs to be split along the sample axis, but was split along {x.split}")
        if self._cluster_centers is None:
            raise RuntimeError("fit needs to be called before predict")
        if x.shape[1] != self._cluster_centers.shape[1]:
            raise ValueError(
                f"input needs to have {self._cluster_centers.shape[1]} features, but has {x.shape[1]}"
            )
        xt = self._local_f32(x)
        if self._ws is None or self._ws.device != xt.device:
            self._ws = _native.Workspace(xt.device)
        n = xt.shape[0]
        lab = torch.empty((n, 1), dtype=torch.int32, device=xt.device)
        d2 = torch.empty((n,), dtype=xt.dtype, device=xt.device)
        fv = torch.empty((), dtype=xt.dtype, device=xt.device)
        if self._p == 1:
            # sum of the Manhattan distances to the closest centre: min_dist_sum adds sqrt(v), so it is
            # fed the squared distances
            _native.assign_l1(xt, self._cluster_centers.larray.to(xt.dtype), lab.view(-1), d2)
            if xt.dtype == torch.float64:
                fv = d2.sum()
            else:
                _native.min_dist_sum(d2.mul_(d2), fv, self._ws)
        else:
            # ||x - C[labels]||_F ** 2 = sum of the squared distances to the closest centre
            _native.assign(xt, self._cluster_centers.larray.to(xt.dtype), lab.view(-1), d2, self._ws)
            _native.functional_value(d2, fv, self._ws)
        self._functional_value = fv.item()
        return DNDarray(lab, (n, 1), types.int32, x.split, x.device, x.comm, x.balanced)


class BatchParallelKMeans(_BatchParallelKCluster):
    """Batch-parallel k-means (heat/cluster/batchparallelclustering.py:339-397)."""

    def __init__(self, n_clusters: int = 8, init: str = "k-means++", max_iter: int = 300, tol: float = 1e-4,
                 random_state: Optional[int] = None, n_procs_to_merge: Optional[int] = None):  # noqa: D107
        if not isinstance(init, str):
            raise TypeError(f"init must be str, but was {type(init)}")
        if init == "k-means++":
            _init = "++"
        elif init == "random":
            raise NotImplementedError(
                "random initialization for batch parallel k-means is currently not supported due to instable behaviour of the algorithm. Use init='k-means++' instead."
            )
        else:
            raise ValueError(f"init must be 'k-means++' or 'random', but was {init}")
        super().__init__(p=2, n_clusters=n_clusters, init=_init, max_iter=max_iter, tol=tol,
                         random_state=random_state, n_procs_to_merge=n_procs_to_merge)
        self.init = init


class BatchParallelKMedians(_BatchParallelKCluster):
    """Batch-parallel k-medians (heat/cluster/batchparallelclustering.py:400-458)."""

    def __init__(self, n_clusters: int = 8, init: str = "k-medians++", max_iter: int = 300, tol: float = 1e-4,
                 random_state: Optional[int] = None, n_procs_to_merge: Optional[int] = None):  # noqa: D107
        if not isinstance(init, str):
            raise TypeError(f"init must be str, but was {type(init)}")
        if init == "k-medians++":
            _init = "++"
        elif init == "random":
            raise NotImplementedError(
                "random initialization for batch parallel k-medians is currently not supported due to instable behaviour of the algorithm. Use init='k-medians++' instead."
            )
        else:
            raise ValueError(f"init must be 'k-medians++' or 'random', but was {init}")
        super().__init__(p=1, n_clusters=n_clusters, init=_init, max_iter=max_iter, tol=tol,
                         random_state=random_state, n_procs_to_merge=n_procs_to_merge)
        self.init = init
