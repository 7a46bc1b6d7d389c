"""
CPU oracle for the k-means Lloyd path of Heat (cdist -> argmin -> per-cluster mean).

THIS IS TEST INFRASTRUCTURE, NOT THE PRODUCT.  Only the test-suite, the smoke check and the
``cpu_baseline`` leg of the benchmark may import it.  The shipped path (``heat_amd``) never calls
anything in this file and has no CPU fallback.

The reference is pure Python whose arithmetic is delegated to PyTorch's CPU backend; it cannot be
imported in this environment (it needs ``mpi4py`` at import time, ``heat/core/communication.py:12``).
This file restates the reference's op sequence with the *same* torch routines in the *same* order,
at one MPI rank, so every collective of the reference is a no-op (``heat/core/_operations.py:509``).

Two flavours are provided:

``*_literal``  op-for-op restatement, including the full N x K matrix, the float64 promotion of
               ``x * selection`` and the divide-before-sum of ``KMeans._update_centroids``.  Memory
               and time grow as the reference's do, so it is for small and medium inputs and for
               the timed CPU baseline.
``*_fast``     the same mathematics in row chunks (distances) and with an fp64 ``index_add_``
               (update).  Used where the literal form does not fit; cross-checked against the literal
               form in the tests.

Pins (what each function is checked against, see tests/test_oracle_pins.py):

* quadratic_expand / euclidian_fast / cdist : the known-answer vectors of the reference's
  ``tests/spatial/test_distances.py:16-58,207-222`` (ones vs zeros, D=4 -> 2.0; X vs X -> 0;
  row-scaled ones vs ``torch.cdist``), fp64 brute force ``sum((x-c)**2)`` on small inputs,
  invariants (>= 0, symmetric, zero diagonal).
* assign_to_cluster : ``torch.argmin(keepdim=True)`` as in ``tests/core/test_statistics.py:136-143``;
  first-index tie-break; brute-force python loop.
* update_centroids_* : python-loop per-cluster mean in fp64, ``sum_k cnt_k == N``,
  ``sum_k cnt_k * C_k == sum_i x_i``, empty cluster -> zero row; structurally identical
  sum-then-divide baselines of ``benchmarks/2020/kmeans/torch-cpu.py:36-50``.
* kmeans_fit : closed-form special cases (init at optimum -> n_iter 1 and shift 0; K=1 -> global
  mean; K=N distinct points -> fixed point), translated-copies invariant of
  ``doc/source/tutorials/tutorial_clustering.rst:22-80``, scikit-learn Lloyd with identical init.
  End-to-end KMeans numerics are not pinned by any value stored in the reference
  (``tests/cluster/test_kmeans.py`` asserts types and shapes only): for the composed loop the parity
  statement rests on the per-function pins above plus these closed forms.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

INT64_MAX = 9223372036854775807


# --------------------------------------------------------------------------------------------------
# distances
# --------------------------------------------------------------------------------------------------
def quadratic_expand(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """|x-y|^2 = |x|^2 + |y|^2 - 2xy, clamped at 0.  Follows heat/spatial/distance.py:47-64."""
    x_norm = (x**2).sum(1).view(-1, 1)
    y_t = torch.transpose(y, 0, 1)
    y_norm = (y**2).sum(1).view(1, -1)
    dist = x_norm + y_norm - 2.0 * torch.mm(x, y_t)
    return torch.clamp(dist, 0.0, np.inf)


def euclidian_fast(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """sqrt of the quadratic expansion.  Follows heat/spatial/distance.py:32-44."""
    return torch.sqrt(quadratic_expand(x, y))


def _promote_for_dist(x: torch.Tensor, y: Optional[torch.Tensor]) -> torch.dtype:
    """
    Result dtype of ``_dist``: promote(X, Y, float32) with Heat's "intuitive" promotion
    (same bit length where possible: int32+float32 -> float32, int64+float32 -> float64).
    Follows heat/spatial/distance.py:237-253,392-403 and heat/core/types.py:915-959.
    """

    def bits(t: torch.Tensor) -> int:
        if t.dtype == torch.bool:
            return 1
        return torch.finfo(t.dtype).bits if t.dtype.is_floating_point else torch.iinfo(t.dtype).bits

    need = max(32, bits(x), bits(y) if y is not None else 0)
    return torch.float64 if need > 32 else torch.float32


def cdist(
    X: torch.Tensor, Y: Optional[torch.Tensor] = None, quadratic_expansion: bool = True
) -> torch.Tensor:
    """
    ht.spatial.cdist at one rank: (m, n) matrix of square-rooted distances in promote(X, Y, float32).
    Follows heat/spatial/distance.py:136-156 (entry), :209-277 (Y is None -> metric(X, X)),
    :392-414 (dtype promotion, the N x K zeros allocation, metric on the local tensors).
    """
    if X.dim() > 2 or (Y is not None and Y.dim() > 2):
        raise NotImplementedError("Only 2D data matrices are currently supported")
    dt = _promote_for_dist(X, Y)
    x = X.to(dt)
    y = x if Y is None else Y.to(dt)
    _ = torch.zeros((x.shape[0], y.shape[0]), dtype=dt)  # distance.py:405-407, discarded at :414
    if quadratic_expansion:
        return euclidian_fast(x, y)
    return torch.cdist(x, y)  # distance.py:17-29


# --------------------------------------------------------------------------------------------------
# assignment
# --------------------------------------------------------------------------------------------------
def assign_to_cluster_literal(
    x: torch.Tensor, centers: torch.Tensor, eval_functional_value: bool = False
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """
    labels (N, 1) int64 = argmin_k sqrt(d2[i, k]) with first-index ties, optionally the functional
    value ||min_k d||_2 ** 2.  Follows heat/cluster/_kcluster.py:352-370; the argmin goes through
    torch.min(dim=1, keepdim=True) and a float64 value|index packing (heat/core/statistics.py:162-190,
    heat/core/_operations.py:516-522); the norm is sqrt(dot(m, m)) (heat/core/linalg/basics.py:1245-1255).
    """
    distances = cdist(x, centers, quadratic_expansion=True)
    minima, indices = torch.min(distances, dim=1, keepdim=True)
    packed = torch.cat([minima.double(), indices.double()])
    labels = packed.chunk(2)[-1].type(torch.int64)
    fval = None
    if eval_functional_value:
        m = torch.min(distances, dim=1).values
        fval = torch.sqrt(torch.dot(m, m)) ** 2
    return labels, fval


def assign_to_cluster_fast(
    x: torch.Tensor, centers: torch.Tensor, chunk: int = 1 << 16, want_min: bool = False
):
    """
    Row-chunked version of :func:`assign_to_cluster_literal` that never holds the whole N x K matrix.
    Returns (labels (N,1) int64, min_d2 (N,) of the clamped pre-sqrt values or None).
    A chunked sgemm is not guaranteed bit-identical to one big call; differences are ulp-level.
    """
    n = x.shape[0]
    labels = torch.empty((n, 1), dtype=torch.int64)
    min_d2 = torch.empty((n,), dtype=x.dtype) if want_min else None
    for s in range(0, n, chunk):
        q = quadratic_expand(x[s : s + chunk], centers)
        idx = torch.min(torch.sqrt(q), dim=1, keepdim=True).indices
        labels[s : s + chunk] = idx
        if want_min:
            min_d2[s : s + chunk] = q.gather(1, idx).view(-1)
    return labels, min_d2


# --------------------------------------------------------------------------------------------------
# update
# --------------------------------------------------------------------------------------------------
def update_centroids_literal(
    x: torch.Tensor, labels: torch.Tensor, centers: torch.Tensor
) -> torch.Tensor:
    """
    Per-cluster mean exactly as heat/cluster/kmeans.py:76-103 evaluates it for float32 ``x``:

    * ``selection = (labels == i).astype(int64)``                       (relational.py:37-81)
    * ``x * selection`` is promoted to float64                           (types.py:945-959, _operations.py:85,204)
    * ``selection.sum(0, keepdims).clip(1.0, int64max)`` comes back as a float32 *tensor* (torch's
      clamp of an int64 tensor with a float bound) inside a DNDarray still declared int64
      (rounding.py:156-164), so the count is rounded to fp32 and then widened to float64 by the
      division's cast (_operations.py:204)
    * the division happens before the sum, in float64; the (1, D) result is cast to the centroid
      dtype by ``__setitem__``                                           (dndarray.py:1778-1779)
    * an empty cluster yields a row of zeros (count clipped to 1, sum 0).
    """
    k = centers.shape[0]
    new_centers = centers.clone()
    prom = torch.promote_types(x.dtype, torch.float64) if x.dtype.is_floating_point else torch.float64
    for i in range(k):
        selection = (labels == i).to(torch.int64)
        assigned = x.to(prom) * selection.to(prom)
        cnt = selection.sum(dim=0, keepdim=True).clamp(1.0, INT64_MAX)
        new_centers[i : i + 1, :] = (assigned / cnt.to(prom)).sum(dim=0, keepdim=True).to(
            new_centers.dtype
        )
    return new_centers


def update_centroids_fast(
    x: torch.Tensor, labels: torch.Tensor, k: int, out_dtype: torch.dtype = torch.float32
) -> Tuple[torch.Tensor, torch.Tensor]:
    """
    Same mean via fp64 ``index_add_`` (sum, then divide by double(float(count))).  Returns
    (centers (K, D) out_dtype, counts (K,) int64).  Differs from the literal form only by the
    order of fp64 roundings (<= a few 1e-16 relative before the final cast).
    """
    d = x.shape[1]
    lab = labels.view(-1)
    sums = torch.zeros((k, d), dtype=torch.float64)
    step = 1 << 20
    for s in range(0, x.shape[0], step):
        sums.index_add_(0, lab[s : s + step], x[s : s + step].to(torch.float64))
    counts = torch.bincount(lab, minlength=k)[:k]
    cnt = counts.clamp(1.0, INT64_MAX).to(torch.float64)  # fp32 rounding of the count, as above
    return (sums / cnt.view(-1, 1)).to(out_dtype), counts


# --------------------------------------------------------------------------------------------------
# the fit loop
# --------------------------------------------------------------------------------------------------
def centroid_shift(c_old: torch.Tensor, c_new: torch.Tensor) -> torch.Tensor:
    """((C - C_new) ** 2).sum() in the centroid dtype.  Follows heat/cluster/kmeans.py:141."""
    return ((c_old - c_new) ** 2).sum()


def kmeans_fit(
    x: torch.Tensor,
    init_centers: torch.Tensor,
    max_iter: int,
    tol: Optional[float],
    literal: bool = True,
    chunk: int = 1 << 16,
):
    """
    KMeans.fit with explicit initial centroids.  Follows heat/cluster/kmeans.py:105-148 and the
    explicit-init branch of heat/cluster/_kcluster.py:136-143 (shape checks, ``resplit(None)`` = copy).

    Returns dict(cluster_centers (K,D), labels (N,1) int64 -- those of the LAST assignment, i.e.
    against the centroids *before* the last update (kmeans.py:146), inertia = last centroid shift
    (kmeans.py:141), n_iter, shifts = per-iteration list).
    The loop stops when ``tol is not None and shift <= tol`` (kmeans.py:143): with tol = 0 it still
    stops early on an exactly-zero shift.
    """
    if init_centers.dim() != 2:
        raise ValueError("passed centroids need to be two-dimensional")
    k = init_centers.shape[0]
    if init_centers.shape[1] != x.shape[1]:
        raise ValueError("passed centroids do not match cluster count or data shape")
    centers = init_centers.clone()
    n_iter = 0
    shifts = []
    labels = None
    inertia = None
    for _ in range(max_iter):
        n_iter += 1
        if literal:
            labels, _ = assign_to_cluster_literal(x, centers)
            new_centers = update_centroids_literal(x, labels, centers)
        else:
            labels, _ = assign_to_cluster_fast(x, centers, chunk=chunk)
            new_centers, _ = update_centroids_fast(x, labels, k, out_dtype=centers.dtype)
        inertia = centroid_shift(centers, new_centers)
        shifts.append(float(inertia))
        centers = new_centers.clone()
        if tol is not None and bool(inertia <= tol):
            break
    return {
        "cluster_centers": centers,
        "labels": labels,
        "inertia": inertia,
        "n_iter": n_iter,
        "shifts": shifts,
    }


def predict(x: torch.Tensor, centers: torch.Tensor, literal: bool = True, chunk: int = 1 << 16):
    """
    _KCluster.predict: labels (N,1) int64 and functional_value_ (fp32 scalar).
    Follows heat/cluster/_kcluster.py:398-415.
    """
    if literal:
        return assign_to_cluster_literal(x, centers, eval_functional_value=True)
    labels, min_d2 = assign_to_cluster_fast(x, centers, chunk=chunk, want_min=True)
    m = torch.sqrt(min_d2)
    return labels, torch.sqrt(torch.dot(m, m)) ** 2


# --------------------------------------------------------------------------------------------------
# parity checker (gap-aware label comparison)
# --------------------------------------------------------------------------------------------------
def label_agreement(
    x: torch.Tensor,
    centers: torch.Tensor,
    labels_a: torch.Tensor,
    labels_b: torch.Tensor,
    rel_gap: float = 1e-5,
    chunk: int = 1 << 16,
):
    """
    Compare two labelings of ``x`` against ``centers``.  For every row where they differ, the fp64
    squared distances (direct ``sum((x-c)**2)``) of both chosen centroids are compared with the best
    one; a disagreement is *excused* (a numerical tie) when both lie within

        rel_gap * d2_best  +  max(2, sqrt(D)/4) * eps32 * (|x|^2 + |c|^2)

    of the best.  The first term is the stated gap rule.  The second is the resolution of the
    reference's own arithmetic: in fp32, ``(|x|^2 + |c|^2) - 2 x.c`` is a difference of two numbers of
    that magnitude, so its value is a multiple of their ulp and carries the rounding of a D-term dot
    product; squared distances closer than that are not ordered reliably by the reference either.

    Returns dict(n, n_diff, n_unexcused, agreement).
    """
    a = labels_a.view(-1).to(torch.int64).cpu()
    b = labels_b.view(-1).to(torch.int64).cpu()
    n = a.numel()
    diff = torch.nonzero(a != b).view(-1)
    n_unexcused = 0
    c64 = centers.to(torch.float64).cpu()
    cn = (c64**2).sum(1)
    dfac = max(2.0, math.sqrt(x.shape[1]) / 4.0) * float(torch.finfo(torch.float32).eps)
    for s in range(0, diff.numel(), chunk):
        rows = diff[s : s + chunk]
        xr = x[rows].to(torch.float64).cpu()
        d2 = ((xr[:, None, :] - c64[None, :, :]) ** 2).sum(-1)
        best = d2.min(dim=1).values
        da = d2.gather(1, a[rows].view(-1, 1)).view(-1)
        db = d2.gather(1, b[rows].view(-1, 1)).view(-1)
        mag = (xr**2).sum(1) + torch.maximum(cn[a[rows]], cn[b[rows]])
        lim = best * (1.0 + rel_gap) + dfac * mag + 1e-300
        ok = (da <= lim) & (db <= lim)
        n_unexcused += int((~ok).sum())
    return {
        "n": n,
        "n_diff": int(diff.numel()),
        "n_unexcused": n_unexcused,
        "agreement": 1.0 - diff.numel() / max(n, 1),
    }


def rel_err_centers(c_a: torch.Tensor, c_b: torch.Tensor) -> float:
    """||dC||_inf / max|C| in fp64."""
    a = c_a.to(torch.float64).cpu()
    b = c_b.to(torch.float64).cpu()
    denom = max(float(b.abs().max()), 1e-300)
    return float((a - b).abs().max()) / denom


def rel_err_scalar(a: float, b: float, floor: float = 0.0) -> float:
    """|a-b| / max(|b|, floor)."""
    return abs(float(a) - float(b)) / max(abs(float(b)), floor, 1e-300)


def brute_force_d2(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """fp64 sum((x_i - y_k)**2): the mathematical definition, used to pin the expansion."""
    a = x.to(torch.float64)
    b = y.to(torch.float64)
    return ((a[:, None, :] - b[None, :, :]) ** 2).sum(-1)


def sse(x: torch.Tensor, centers: torch.Tensor, labels: torch.Tensor, chunk: int = 1 << 18) -> float:
    """fp64 sum_i |x_i - c_label(i)|^2."""
    tot = 0.0
    lab = labels.view(-1)
    c64 = centers.to(torch.float64)
    for s in range(0, x.shape[0], chunk):
        d = x[s : s + chunk].to(torch.float64) - c64[lab[s : s + chunk]]
        tot += float((d * d).sum())
    return tot


__all__ = [
    "quadratic_expand",
    "euclidian_fast",
    "cdist",
    "assign_to_cluster_literal",
    "assign_to_cluster_fast",
    "update_centroids_literal",
    "update_centroids_fast",
    "centroid_shift",
    "kmeans_fit",
    "predict",
    "label_agreement",
    "rel_err_centers",
    "rel_err_scalar",
    "brute_force_d2",
    "sse",
]
