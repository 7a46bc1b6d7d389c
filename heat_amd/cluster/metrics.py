"""
Silhouette coefficient with the interface of heat/cluster/metrics.py (``silhouette_samples``,
``silhouette_score``) in float32 on one rank.

The reference forms the full distance matrix ``cdist(X, X)`` and multiplies it with the one-hot label mask
(:130-151).  Here ``hkm_cluster_distance_sums_f32`` produces those per-sample, per-cluster sums directly
from the rows grouped by cluster, and ``hkm_silhouette_finish_f32`` turns them into coefficients.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _native
from ..core import types
from ..core.dndarray import DNDarray
from ..spatial import distance

__all__ = ["silhouette_samples", "silhouette_score"]


def _validate_input(X, labels, metric: str = "euclidean"):
    """Checks of heat/cluster/metrics.py:9-84 that apply to one rank."""
    if not isinstance(X, DNDarray) or not isinstance(labels, DNDarray):
        raise TypeError(f"Input must be a DNDarray, is {type(X)} and {type(labels)}")
    if metric == "precomputed":
        if len(X.shape) != 2 or X.shape[-1] != X.shape[-2]:
            raise ValueError(f"Precomputed distance matrix needs to be 2D and square but has shape {X.shape}")
        diag = torch.diagonal(X.larray)
        eps = torch.finfo(X.larray.dtype).eps if X.larray.dtype.is_floating_point else 0.0
        if bool((diag.abs() > eps * 100).any()):
            raise ValueError("The precomputed distance matrix contains non-zero elements on the diagonal")
    lab = labels.larray
    if lab.dim() > 1:
        if lab.numel() == X.shape[0]:
            lab = lab.reshape(-1)
        else:
            raise ValueError(f"labels should be a 1D array or a column vector but has shape {labels.shape}.")
    if X.shape[0] != lab.shape[0]:
        raise ValueError(
            "Found input variables with inconsistent number of samples and labels! "
            f"Got: {X.shape[0]} samples and {lab.shape[0]} labels"
        )
    return X, lab


def silhouette_samples(X: DNDarray, labels: DNDarray, *, metric: str = "euclidean") -> DNDarray:
    """
    heat/cluster/metrics.py:87-177.  ``metric="euclidean"`` never forms the distance matrix;
    ``metric="precomputed"`` takes it as given and multiplies it with the label mask.
    """
    X, lab = _validate_input(X, labels, metric=metric)
    if metric not in ("precomputed", "euclidean"):
        raise NotImplementedError(f"{metric=} not implemented, choose from 'precomputed' and 'euclidean'.")
    promoted = types.promote_types(X.dtype, types.float32)
    if promoted is types.float64:
        return _silhouette_samples_f64(X, lab, metric)
    xt = distance._as_f32_matrix(X, promoted)
    dev = xt.device
    n = xt.shape[0]
    lab = lab.to(dev)
    _, enc = torch.unique(lab, sorted=True, return_inverse=True)
    enc = enc.to(torch.int64).contiguous()
    k = int(enc.max().item()) + 1 if n else 1
    counts = torch.bincount(enc, minlength=k)
    sums = torch.empty((n, k), dtype=torch.float32, device=dev)
    if metric == "precomputed":
        mask = torch.zeros((n, k), dtype=torch.float32, device=dev)
        mask.scatter_(1, enc.view(-1, 1), 1.0)
        torch.matmul(xt, mask, out=sums)
    else:
        perm = torch.sort(enc, stable=True).indices.contiguous()
        offsets = torch.zeros((k + 1,), dtype=torch.int64, device=dev)
        offsets[1:] = torch.cumsum(counts, 0)
        _native.cluster_distance_sums(xt, perm, offsets, sums)
    out = torch.empty((n,), dtype=torch.float32, device=dev)
    _native.silhouette_finish(sums, enc, counts, out)
    return DNDarray(out, (n,), types.float32, X.split, X.device, X.comm, True)


def _silhouette_samples_f64(X: DNDarray, lab: torch.Tensor, metric: str) -> DNDarray:
    """float64 and int64 data, which the reference keeps in float64: the per-cluster sums come from the
    library's float64 pairwise kernel in row chunks times the one-hot labels (metrics.py:135-151), the
    coefficients (:153-176) from a few torch operations on the (samples x clusters) sums."""
    from .. import _f64_paths

    xt = X.larray.to(torch.float64)
    if xt.stride(-1) != 1:
        xt = xt.contiguous()
    dev = xt.device
    n = xt.shape[0]
    _, enc = torch.unique(lab.to(dev), sorted=True, return_inverse=True)
    enc = enc.to(torch.int64).contiguous()
    k = int(enc.max().item()) + 1 if n else 1
    counts = torch.bincount(enc, minlength=k)
    if metric == "precomputed":
        mask = torch.zeros((n, k), dtype=torch.float64, device=dev)
        mask.scatter_(1, enc.view(-1, 1), 1.0)
        sums = xt @ mask
    else:
        sums = _f64_paths.cluster_distance_sums(xt, enc, k)
    own = counts[enc]
    a = sums.gather(1, enc.view(-1, 1)).view(-1) / (own - 1).clamp_min(1).to(torch.float64)
    mean_other = sums / counts.to(torch.float64).view(1, -1)
    mean_other.scatter_(1, enc.view(-1, 1), float("inf"))
    b = mean_other.min(dim=1).values
    out = (b - a) / torch.maximum(a, b)
    out = torch.where(own == 1, torch.zeros_like(out), out)
    out = torch.nan_to_num(out, nan=0.0)
    return DNDarray(out, (n,), types.float64, X.split, X.device, X.comm, True)


def silhouette_score(X: DNDarray, labels: DNDarray, *, metric: str = "euclidean", sample_size: Optional[int] = None,
                     random_state: Optional[int] = None, **kwargs) -> float:
    """heat/cluster/metrics.py:193-269: the mean coefficient, optionally over a random subset of the samples
    (drawn here with a seeded torch generator; the reference draws it from its own counter-based one)."""
    if sample_size is not None:
        X, lab = _validate_input(X, labels)
        if metric == "precomputed":
            raise NotImplementedError(
                "Random sampling in silhouette with precomputed distance matrix is not currently supported."
            )
        g = torch.Generator()
        if random_state is not None:
            g.manual_seed(int(random_state))
        indices = torch.randperm(X.shape[0], generator=g)[:sample_size].to(X.larray.device)
        xs = X.larray[indices]
        ls = lab.to(X.larray.device)[indices]
        X = DNDarray(xs, tuple(xs.shape), X.dtype, X.split, X.device, X.comm, True)
        labels = DNDarray(ls, tuple(ls.shape), types.int64, X.split, X.device, X.comm, True)
    return float(silhouette_samples(X, labels, metric=metric, **kwargs).larray.mean().item())
