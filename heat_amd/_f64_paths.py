"""
float64 forms of the Manhattan-metric steps (assignment, per-cluster medians, closest row) and of the
k-nearest-rows / distance-sum steps, for float64 and int64 data, which the reference keeps in float64
(promote(X, Y, float32), heat/spatial/distance.py:392-403).

These are correctness paths, not tuned ones: every distance comes from the library's float64 pairwise kernel
(``hkm_pairwise_f64``) in row chunks, the selections on top of it -- argmin, the order statistics of the
medians -- are torch's device routines.  All tensors stay on the GPU; nothing here runs on the host.
"""

from __future__ import annotations

from typing import Optional

import torch

_CHUNK_BYTES = 1 << 30  # distance-matrix bytes per chunk of rows


def _pairwise(x: torch.Tensor, y: torch.Tensor, metric: int) -> torch.Tensor:
    from . import _native

    out = torch.empty((x.shape[0], y.shape[0]), dtype=torch.float64, device=x.device)
    _native.pairwise(x, y, out, metric)
    return out


def _row_chunks(n: int, cols: int):
    step = max(1, _CHUNK_BYTES // (8 * max(cols, 1)))
    for s in range(0, n, step):
        yield s, min(n, s + step)


def assign_l1(x: torch.Tensor, c: torch.Tensor, labels: torch.Tensor, min_dist: Optional[torch.Tensor]) -> None:
    """labels[i] = argmin_k sum |x_i - c_k| (first index on ties), optional minimum distance."""
    from . import _native

    for s, e in _row_chunks(x.shape[0], c.shape[0]):
        dist = _pairwise(x[s:e], c, _native.METRIC_MANHATTAN)
        m, i = torch.min(dist, dim=1)
        labels[s:e] = i.to(labels.dtype)
        if min_dist is not None:
            min_dist[s:e] = m


def closest_rows_l1(x: torch.Tensor, q: torch.Tensor, idx: torch.Tensor, dist: Optional[torch.Tensor]) -> None:
    """idx[m] = row of x closest to q[m] in the Manhattan metric (first index on ties)."""
    from . import _native

    best = torch.full((q.shape[0],), float("inf"), dtype=torch.float64, device=x.device)
    idx.fill_(0)
    for s, e in _row_chunks(x.shape[0], q.shape[0]):
        d = _pairwise(q, x[s:e], _native.METRIC_MANHATTAN)  # (M, rows)
        m, i = torch.min(d, dim=1)
        better = m < best  # strict: an earlier chunk keeps exact ties
        best = torch.where(better, m, best)
        idx.copy_(torch.where(better, i + s, idx))
    if dist is not None:
        dist.copy_(best.to(dist.dtype))


def update_median(x: torch.Tensor, labels: torch.Tensor, c_new: torch.Tensor,
                  fallback_rows: Optional[torch.Tensor], c_old: Optional[torch.Tensor],
                  counts: Optional[torch.Tensor], lower: bool, skip_zero_rows: bool,
                  median64: Optional[torch.Tensor]) -> None:
    """
    c_new[k][d] = median over the rows of cluster k of x[:, d] (see hkm_update_median_f32 in include/hkm.h for
    the two modes, the rows left out and what an empty cluster becomes), by two stable sorts per column:
    by value, then by cluster.
    """
    n, d = x.shape
    k = c_new.shape[0]
    dev = x.device
    lab = labels.to(torch.int64).clone()
    lab[(lab < 0) | (lab >= k)] = k  # ignored rows go to a bin of their own
    if skip_zero_rows:
        lab[(x != 0).sum(dim=1) == 0] = k
    cnt = torch.bincount(lab, minlength=k + 1)[:k]
    offs = torch.cumsum(cnt, 0) - cnt
    vals, order = torch.sort(x, dim=0, stable=True)              # every column ascending
    lab_cols = lab[order]                                        # cluster of every sorted entry
    by_cluster = torch.argsort(lab_cols, dim=0, stable=True)     # grouped by cluster, values still ascending
    grouped = torch.gather(vals, 0, by_cluster)
    nonempty = cnt > 0
    safe = torch.where(nonempty, cnt, torch.ones_like(cnt))
    lo_i = (offs + (safe - 1) // 2).clamp_(0, max(n - 1, 0))
    hi_i = (offs + safe // 2).clamp_(0, max(n - 1, 0))
    if n == 0:
        med = torch.zeros((k, d), dtype=x.dtype, device=dev)
    else:
        lo = grouped[lo_i]
        hi = grouped[hi_i]
        med = lo if lower else lo + (hi - lo) * 0.5
    if fallback_rows is not None:
        empty_val = x[fallback_rows.clamp(0, max(n - 1, 0))] if n else torch.zeros((k, d), dtype=x.dtype, device=dev)
    elif c_old is not None:
        empty_val = c_old.to(x.dtype)
    else:
        empty_val = torch.zeros((k, d), dtype=x.dtype, device=dev)
    med = torch.where(nonempty.view(-1, 1), med, empty_val)
    c_new.copy_(med.to(c_new.dtype))
    if median64 is not None:
        median64.copy_(med.to(torch.float64))
    if counts is not None:
        counts.copy_(cnt)


def knn(q: torch.Tensor, x: torch.Tensor, k: int, idx: torch.Tensor, dist: Optional[torch.Tensor]) -> None:
    """The k rows of x closest to every row of q in the Euclidean metric (direct form), ascending."""
    from . import _native

    best_d = torch.full((q.shape[0], k), float("inf"), dtype=torch.float64, device=q.device)
    best_i = torch.full((q.shape[0], k), -1, dtype=torch.int64, device=q.device)
    for s, e in _row_chunks(x.shape[0], q.shape[0]):
        d = _pairwise(q, x[s:e], _native.METRIC_EUCLID)
        ids = torch.arange(s, e, device=q.device).expand(q.shape[0], -1)
        alld = torch.cat([best_d, d], dim=1)
        alli = torch.cat([best_i, ids], dim=1)
        order = torch.argsort(alld, dim=1, stable=True)[:, :k]  # earlier rows first among equal distances
        best_d = torch.gather(alld, 1, order)
        best_i = torch.gather(alli, 1, order)
    idx.copy_(best_i)
    if dist is not None:
        dist.copy_(best_d.to(dist.dtype))


def cluster_distance_sums(x: torch.Tensor, enc: torch.Tensor, k: int) -> torch.Tensor:
    """S[i][c] = sum over the rows j with enc[j] == c of |x_i - x_j| (Euclidean, direct form): the product of
    the distance matrix with the one-hot labels of heat/cluster/metrics.py:135-151, in row chunks."""
    from . import _native

    n = x.shape[0]
    onehot = torch.zeros((n, k), dtype=torch.float64, device=x.device)
    onehot.scatter_(1, enc.view(-1, 1), 1.0)
    out = torch.empty((n, k), dtype=torch.float64, device=x.device)
    for s, e in _row_chunks(n, n):
        out[s:e] = _pairwise(x[s:e], x, _native.METRIC_EUCLID) @ onehot
    return out
