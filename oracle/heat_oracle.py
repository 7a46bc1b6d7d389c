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
* centroid_sampling_helper / kmeans_parallel_init / initialize_plus_plus / kmex (k-means||
  initialisation and its k-means++ reclustering): closed forms (probabilities sum to the
  oversampling factor, so the expected number of new candidates per round equals it; a row at
  distance 0 is never drawn; with a huge oversampling factor every row at non-zero distance is
  drawn), the D-sampling law of k-means++ on a hand-made case, the empty-cluster-keeps-its-centre
  rule and the allclose stop of ``_kmex``, and recovery of well-separated blobs.  **Parity unpinned**
  for the random draws themselves: the reference takes them from Heat's counter-based generator and
  from torch's unseeded global generator, and stores no seeded result anywhere.
* InverseCdfSampler (categorical draw of the one-launch k-means++ seeding as the inverse CDF of a
  given uniform number): a hand-made case (weights 1, 0, 2, 1 and u on both sides of every boundary),
  zero-weight entries are never drawn, and the frequencies of 20 000 draws against the weights.
* manhattan / assign_l1 / heat_median_axis0 / update_medians / kmedians_fit / kmedoids_fit: the
  known answers of ``tests/spatial/test_distances.py:20-23,42-48,67-73`` (ones vs zeros, D=4 -> 4.0;
  X vs X -> 0), scipy's cityblock distances, ``numpy.median`` and a python sort, hand-made cases for
  the dropped all-zero rows and the empty-cluster restart, brute force for the medoid (a data row, at
  minimal Manhattan distance from the median), K = 1 closed form (the coordinate-wise median after
  one iteration), and the reference's own assertion that every medoid is a data point
  (``tests/cluster/test_kmedoids.py:44-48``).  End-to-end numbers: parity unpinned, as for KMeans.
* knn_one_hot / knn_predict (k-nearest-neighbours classifier): the one-hot known answer of
  ``tests/classification/test_knn.py:69-76``; scikit-learn's brute-force ``KNeighborsClassifier`` and
  ``NearestNeighbors`` (neighbour sets and classes on the iris data and on random blobs); a python
  sort of float64 distances on a tiny input; k = 1 on the training rows returns every row itself.
  The reference stores no predicted class anywhere (``test_knn.py`` asserts types and shapes).
* silhouette_samples / silhouette_score: the known answers of ``tests/cluster/test_metrics.py:92-122``
  (sample 0 of the four-point example = 0.9, score 0.76439) and of the docstring
  (``heat/cluster/metrics.py:121-126``: 0.7452, 0.7836, 0.7452, 0.7836), the special cases of
  ``test_metrics.py:45-88`` (all samples alone, one cluster, perfect and worst clustering), and
  scikit-learn's ``silhouette_samples`` to 1e-6 as in the reference's own test (``:16-42``).
* laplacian (graph Laplacian from a similarity matrix): ``scipy.sparse.csgraph.laplacian`` (plain and
  normalised) on fully connected weighted graphs, closed forms (rows of D - A sum to zero, unit diagonal
  and symmetry of the normalised form, an isolated vertex keeps degree 1 in the normalisation), a
  hand-made 3-vertex case for both thresholds, and the ones on the diagonal of the unweighted "upper"
  graph that follow from thresholding after the diagonal is zeroed.  The reference's test
  (``tests/graph/test_laplacian.py``) asserts types and shapes only.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

INT64_MAX = 9223372036854775807


class CpuSampler:
    """
    Random draws for the initialisers from one seeded torch CPU generator, with the interface the
    product's sampler has (randint / uniform / multinomial).  ``device`` only says where ``uniform``
    puts its result, the numbers are always generated on the CPU, so two implementations constructed
    with the same seed see the same draws.  The categorical draw is an inverse-CDF lookup in fp64 so
    that it depends on the weights only through their cumulative sums.
    """

    def __init__(self, seed: int, device="cpu"):
        self._gen = torch.Generator(device="cpu")
        self._gen.manual_seed(int(seed))
        self.device = torch.device(device)

    def randint(self, high: int) -> int:
        return int(torch.randint(0, int(high), (1,), generator=self._gen).item())

    def uniform(self, n: int) -> torch.Tensor:
        return torch.rand((int(n),), generator=self._gen, dtype=torch.float32).to(self.device)

    def multinomial(self, weights: torch.Tensor) -> int:
        w = weights.detach().to("cpu", torch.float64)
        cdf = torch.cumsum(w, 0)
        r = torch.rand((1,), generator=self._gen, dtype=torch.float64) * cdf[-1]
        i = int(torch.searchsorted(cdf, r, right=True).item())
        return min(i, w.numel() - 1)


class RecordingSampler(CpuSampler):
    """A CpuSampler that keeps every draw (and the weights of every categorical draw) in ``tape``."""

    def __init__(self, seed: int):
        super().__init__(seed, "cpu")
        self.tape = []

    def randint(self, high: int) -> int:
        r = super().randint(high)
        self.tape.append(("randint", int(high), r))
        return r

    def uniform(self, n: int) -> torch.Tensor:
        u = super().uniform(n)
        self.tape.append(("uniform", int(n), u))
        return u

    def multinomial(self, weights: torch.Tensor) -> int:
        i = super().multinomial(weights)
        self.tape.append(("multinomial", weights.detach().clone(), i))
        return i


class ReplaySampler:
    """
    Replays the tape of a RecordingSampler to a second implementation, so both walk the same random
    path even where a draw sits close to a decision boundary.  Each call must be the same kind of draw
    with the same argument; for a categorical draw the weights must agree with the recorded ones to
    ``rtol`` relative plus ``atol_frac`` of the largest weight.  The absolute part is there for the
    rows already chosen as centres: their distance is exactly 0 in a direct evaluation, while
    ``torch.cdist`` switches to a quadratic expansion above 25 rows and returns about
    sqrt(eps) * |x| instead, which is then multiplied by a weight of up to thousands.
    """

    def __init__(self, tape, device="cpu", rtol: float = 1e-3, atol_frac: float = 1e-2):
        self.tape = list(tape)
        self.pos = 0
        self.device = torch.device(device)
        self.rtol, self.atol_frac = rtol, atol_frac

    def _next(self, kind: str):
        assert self.pos < len(self.tape), f"more draws than recorded (next would be {kind})"
        rec = self.tape[self.pos]
        self.pos += 1
        assert rec[0] == kind, f"draw {self.pos - 1}: recorded {rec[0]}, asked for {kind}"
        return rec

    def randint(self, high: int) -> int:
        rec = self._next("randint")
        assert rec[1] == int(high), (rec[1], high)
        return rec[2]

    def uniform(self, n: int) -> torch.Tensor:
        rec = self._next("uniform")
        assert rec[1] == int(n), (rec[1], n)
        return rec[2].to(self.device)

    def multinomial(self, weights: torch.Tensor) -> int:
        rec = self._next("multinomial")
        w = weights.detach().to("cpu", torch.float32)
        ref = rec[1].to(torch.float32)
        assert w.shape == ref.shape, (w.shape, ref.shape)
        tol = self.rtol * ref.abs() + self.atol_frac * float(ref.abs().max())
        bad = (w - ref).abs() > tol
        assert not bool(bad.any()), f"categorical weights differ at {int(bad.sum())} of {w.numel()} entries"
        return rec[2]

    def exhausted(self) -> bool:
        return self.pos == len(self.tape)


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

    Next to that, the rule is also evaluated WITHOUT the second term, exactly as it is stated: a
    differing row is *strict* when its fp64 best and second-best squared distances (over all centroids)
    are further apart than ``rel_gap`` relative, ``(d2_second - d2_best) / d2_best > rel_gap`` -- such a
    row has one clear nearest centroid and the two labelings should not differ on it.  ``n_strict`` counts
    them, ``max_strict_gap`` is the largest such relative gap over all differing rows (0 if none differ)
    and ``max_strict_abs`` the largest absolute gap in units of eps32 * (|x|^2 + |c|^2), i.e. in units of
    the resolution of the fp32 expansion at that row.  On a strict row one of the two labelings is not the
    fp64 nearest centroid: ``n_strict_a_wrong`` counts the strict rows where that is ``labels_a``,
    ``n_strict_b_wrong`` those where it is ``labels_b`` (with ``labels_b`` the reference's labels these are
    the rows its own fp32 rounding misorders: an evaluation in exact arithmetic differs from it there too).

    Which side an unexcused row is due to: ``n_unexcused_a`` counts the differing rows where the centroid
    ``labels_a`` chose lies outside that limit, ``n_unexcused_b`` the same for ``labels_b``; ``worst_a_ulp`` and
    ``worst_b_ulp`` are the largest excess of a side's chosen distance over ``(1 + rel_gap) * d2_best``, in units
    of eps32 * (|x|^2 + |c|^2) (the limit allows max(2, sqrt(D)/4) of them).

    Returns dict(n, n_diff, n_unexcused, n_unexcused_a, n_unexcused_b, worst_a_ulp, worst_b_ulp, agreement,
    n_strict, n_strict_a_wrong, n_strict_b_wrong, max_strict_gap, max_strict_abs).
    """
    a = labels_a.view(-1).to(torch.int64).cpu()
    b = labels_b.view(-1).to(torch.int64).cpu()
    n = a.numel()
    diff = torch.nonzero(a != b).view(-1)
    n_unexcused = n_unexcused_a = n_unexcused_b = 0
    worst_a = worst_b = 0.0
    n_strict = n_strict_a = n_strict_b = 0
    max_strict_gap = 0.0
    max_strict_abs = 0.0
    eps32 = float(torch.finfo(torch.float32).eps)
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
        n_unexcused_a += int((da > lim).sum())
        n_unexcused_b += int((db > lim).sum())
        res = (eps32 * mag).clamp_min(1e-300)
        worst_a = max(worst_a, float(((da - best * (1.0 + rel_gap)) / res).max()))
        worst_b = max(worst_b, float(((db - best * (1.0 + rel_gap)) / res).max()))
        if d2.shape[1] > 1:
            two = torch.topk(d2, 2, dim=1, largest=False).values
            gap_abs = two[:, 1] - two[:, 0]
            gap = gap_abs / two[:, 0].clamp_min(1e-300)
            strict = gap > rel_gap
            n_strict += int(strict.sum())
            true_lab = d2.argmin(dim=1)
            n_strict_a += int((strict & (a[rows] != true_lab)).sum())
            n_strict_b += int((strict & (b[rows] != true_lab)).sum())
            max_strict_gap = max(max_strict_gap, float(gap.max()))
            max_strict_abs = max(max_strict_abs, float((gap_abs / (eps32 * mag).clamp_min(1e-300)).max()))
    return {
        "n": n,
        "n_diff": int(diff.numel()),
        "n_unexcused": n_unexcused,
        "n_unexcused_a": n_unexcused_a,
        "n_unexcused_b": n_unexcused_b,
        "worst_a_ulp": worst_a,
        "worst_b_ulp": worst_b,
        "agreement": 1.0 - diff.numel() / max(n, 1),
        "n_strict": n_strict,
        "n_strict_a_wrong": n_strict_a,
        "n_strict_b_wrong": n_strict_b,
        "max_strict_gap": max_strict_gap,
        "max_strict_abs": max_strict_abs,
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


# --------------------------------------------------------------------------------------------------
# k-means|| initialisation and its k-means++ reclustering
# --------------------------------------------------------------------------------------------------
def _min_distance(x: torch.Tensor, centroids: torch.Tensor, chunk: int = 1 << 15) -> Tuple[torch.Tensor, torch.Tensor]:
    """``cdist(x, centroids, quadratic_expansion=True)`` then min / argmin over axis 1, in row chunks."""
    vals, idxs = [], []
    for i0 in range(0, x.shape[0], chunk):
        v, i = torch.min(euclidian_fast(x[i0 : i0 + chunk], centroids), dim=1)
        vals.append(v)
        idxs.append(i)
    return torch.cat(vals), torch.cat(idxs)


def centroid_sampling_helper(x: torch.Tensor, centroids: torch.Tensor, oversampling: float, num_iters: int,
                             sampler) -> torch.Tensor:
    """Follows heat/cluster/_kcluster.py:283-350 at one rank."""
    for _ in range(num_iters):
        min_distance, _i = _min_distance(x, centroids)
        min_dist_sum = torch.maximum(min_distance.sum(), torch.tensor(1e-12))
        prob = oversampling * min_distance / min_dist_sum
        sample = sampler.uniform(x.shape[0])
        idx = torch.where(sample <= prob)[0]
        centroids = torch.cat((centroids, x[idx].reshape(-1, x.shape[1])), dim=0)
    return centroids


class InverseCdfSampler:
    """Sampler for :func:`initialize_plus_plus` whose categorical draw is the inverse CDF of one given
    uniform number per draw: the first index whose inclusive prefix sum (float64) of the weights
    exceeds u * total.  ``picks`` records the drawn indices, ``prefixes`` (prefix sums, u * total) of
    every draw so a test can tell a rounding tie from a wrong pick."""

    def __init__(self, first: int, u: torch.Tensor):
        self.first, self.u, self.k = int(first), u.double().cpu(), 0
        self.picks, self.prefixes = [], []

    def randint(self, high: int) -> int:
        return self.first

    def multinomial(self, weights: torch.Tensor) -> int:
        cum = torch.cumsum(weights.double(), 0)
        target = float(self.u[self.k]) * float(cum[-1])
        self.k += 1
        hit = torch.nonzero((cum > target) & (weights > 0))
        i = int(hit[0]) if hit.numel() else int(torch.nonzero(weights > 0)[-1])
        self.picks.append(i)
        self.prefixes.append((cum, target))
        return i


def initialize_plus_plus(x: torch.Tensor, n_clusters: int, sampler, weights=1.0, p: int = 2) -> torch.Tensor:
    """Follows heat/cluster/batchparallelclustering.py:22-46 (no subsampling)."""
    idxs = torch.zeros(n_clusters, dtype=torch.long)
    idxs[0] = sampler.randint(x.shape[0])
    for i in range(1, n_clusters):
        dist = torch.cdist(x, x[idxs[:i]], p=p)
        dist = torch.min(dist, dim=1)[0]
        idxs[i] = sampler.multinomial(weights * dist)
    return x[idxs]


def kmex(x: torch.Tensor, n_clusters: int, init, max_iter: int, tol: float, sampler=None,
         weights=1.0, p: int = 2) -> Tuple[torch.Tensor, int]:
    """Follows heat/cluster/batchparallelclustering.py:49-88 (p = 2: means, p = 1: torch.median)."""
    if isinstance(init, torch.Tensor):
        if init.shape != (n_clusters, x.shape[1]):
            raise ValueError("if a torch tensor, init must have shape (n_clusters, n_features).")
        centers = init.clone()
    elif init == "++":
        centers = initialize_plus_plus(x, n_clusters, sampler, weights, p)
    elif init == "random":
        centers = x[torch.tensor([sampler.randint(x.shape[0]) for _ in range(n_clusters)])]
    else:
        raise ValueError("init must be a torch tensor with initial centers, string '++', or 'random'.")
    it = 0
    for it in range(max_iter):
        dist = torch.cdist(x, centers, p=p)
        labels = torch.argmin(dist, dim=1)
        centers_old = centers.clone()
        for i in range(n_clusters):
            if (labels == i).any():
                if p == 1:
                    centers[i] = torch.median(x[labels == i], dim=0)[0]
                else:
                    centers[i] = torch.mean(x[labels == i], dim=0)
        if torch.allclose(centers, centers_old, atol=tol):
            break
    return centers, it + 1


def kmeans_parallel_init(x: torch.Tensor, n_clusters: int, oversampling: float, iter_multiplier: float,
                         max_iter: int, tol: float, sampler) -> Tuple[torch.Tensor, dict]:
    """
    ``init="probability_based"`` of heat/cluster/_kcluster.py:146-247 at one rank.  Returns the
    (K, D) centres and a dict with the intermediate quantities (number of rounds, candidates,
    weights) for step-wise comparisons.
    """
    n = x.shape[0]
    init_idx = sampler.randint(max(n - 1, 1))
    init_centroids = x[init_idx : init_idx + 1].clone()
    init_min_distance, _i = _min_distance(x, init_centroids)
    init_cost = init_min_distance.sum()
    num_iters = max(1, int(iter_multiplier * torch.log(init_cost))) if float(init_cost) > 0 else 1
    centroids = centroid_sampling_helper(x, init_centroids, oversampling, num_iters, sampler)
    if centroids.shape[0] <= n_clusters:
        oversampling = 10 * oversampling
        centroids = centroid_sampling_helper(x, init_centroids, oversampling, num_iters, sampler)
    if centroids.shape[0] <= n_clusters:
        raise ValueError(
            f"The parameter oversampling={oversampling} and/or iter_multiplier={iter_multiplier} "
            "are chosen too small for the initialization of cluster centers."
        )
    _d, final_idx = _min_distance(x, centroids)
    weights = torch.zeros(centroids.shape[0])
    for i in range(centroids.shape[0]):
        weights[i] = torch.sum(final_idx == i)
    centers, n_it = kmex(centroids, n_clusters, "++", max_iter, tol, sampler, weights)
    info = {"init_idx": init_idx, "init_cost": float(init_cost), "num_iters": num_iters,
            "candidates": centroids, "weights": weights, "kmex_iters": n_it, "oversampling": oversampling}
    return centers, info


# --------------------------------------------------------------------------------------------------
# k-medians / k-medoids (Manhattan metric)
# --------------------------------------------------------------------------------------------------
def manhattan(x: torch.Tensor, y: torch.Tensor, expand: bool = False) -> torch.Tensor:
    """heat/spatial/distance.py:106-133: torch.cdist(p=1), or the broadcast form with ``expand``."""
    if expand:
        return torch.sum(torch.abs(x.unsqueeze(1) - y.unsqueeze(0)), dim=2)
    return torch.cdist(x, y, p=1)


def assign_l1(x: torch.Tensor, centers: torch.Tensor, chunk: int = 1 << 12) -> Tuple[torch.Tensor, torch.Tensor]:
    """_KCluster._assign_to_cluster with the metric of KMedians / KMedoids (manhattan, expand=True);
    returns labels (N, 1) int64 and the minimum distances (N,)."""
    labs, mins = [], []
    for i0 in range(0, x.shape[0], chunk):
        v, i = torch.min(manhattan(x[i0 : i0 + chunk], centers, expand=True), dim=1, keepdim=True)
        labs.append(i)
        mins.append(v.view(-1))
    return torch.cat(labs), torch.cat(mins)


def heat_median_axis0(a: torch.Tensor) -> torch.Tensor:
    """
    ht.median(a, axis=0) = percentile 50 with linear interpolation, heat/core/statistics.py:1460-1718:
    sort, index q/100 * (n - 1) as a float32 tensor, floors + (ceils - floors) * fraction in the
    (float64, see update_medians) dtype of the data.
    """
    n = a.shape[0]
    sorted_a, _ = torch.sort(a, dim=0)
    perc = torch.tensor(50) / 100 * (n - 1)
    lo, hi = sorted_a[perc.floor().type(torch.int)], sorted_a[perc.ceil().type(torch.int)]
    return lo + (hi - lo) * (perc - perc.floor())


def update_medians(x: torch.Tensor, labels: torch.Tensor, centers: torch.Tensor, sampler,
                   snap_to_sample: bool = False) -> torch.Tensor:
    """
    KMedians._update_centroids (heat/cluster/kmedians.py:60-118) and, with ``snap_to_sample``,
    KMedoids._update_centroids (heat/cluster/kmedoids.py:57-115).  ``x * selection`` is float64
    (heat/core/types.py promotes float32 * int64), rows whose absolute sum is zero are dropped, an
    empty cluster restarts at a random row, the result is stored into the float32 centres.
    """
    new_centers = centers.clone()
    k = centers.shape[0]
    for i in range(k):
        selection = (labels == i).to(torch.int64)
        assigned = x.to(torch.float64) * selection
        rows = assigned.abs().sum(dim=1) != 0
        clean = assigned[rows]
        if clean.shape[0] == 0:
            new_centers[i, :] = x[sampler.randint(x.shape[0])]
        else:
            median = heat_median_axis0(clean).reshape(1, -1)
            if snap_to_sample:
                dist = manhattan(x.to(torch.float64), median, expand=True)
                idx = int(torch.argmin(dist, dim=0))
                new_centers[i, :] = x[idx]
            else:
                new_centers[i : i + 1, :] = median.to(centers.dtype)
    return new_centers


def kmedians_fit(x: torch.Tensor, init_centers: torch.Tensor, max_iter: int, tol: Optional[float], sampler):
    """KMedians.fit with explicit initial centroids (heat/cluster/kmedians.py:120-147)."""
    centers = init_centers.clone()
    n_iter, labels, inertia = 0, None, None
    for _ in range(max_iter):
        n_iter += 1
        labels, _d = assign_l1(x, centers)
        new_centers = update_medians(x, labels, centers, sampler)
        inertia = ((centers - new_centers) ** 2).sum()
        centers = new_centers.clone()
        if tol is not None and bool(inertia <= tol):
            break
    return {"cluster_centers": centers, "labels": labels, "inertia": inertia, "n_iter": n_iter}


def kmedoids_fit(x: torch.Tensor, init_centers: torch.Tensor, max_iter: int, sampler):
    """KMedoids.fit with explicit initial centroids (heat/cluster/kmedoids.py:117-156)."""
    centers = init_centers.clone()
    n_iter, labels = 0, None
    for _ in range(max_iter):
        n_iter += 1
        labels, _d = assign_l1(x, centers)
        new_centers = update_medians(x, labels, centers, sampler, snap_to_sample=True)
        if torch.equal(centers, new_centers):
            break
        centers = new_centers.clone()
    return {"cluster_centers": centers, "labels": labels, "n_iter": n_iter}


def label_agreement_l1(x: torch.Tensor, centers: torch.Tensor, lab_a: torch.Tensor, lab_b: torch.Tensor,
                       rel_gap: float = 1e-5) -> dict:
    """Like label_agreement for the Manhattan metric: a difference is excused when both chosen
    centres lie within rel_gap * best + D * eps32 * (|x|_1 + |c|_1) of the best fp64 distance."""
    a, b = lab_a.view(-1).long(), lab_b.view(-1).long()
    diff = torch.nonzero(a != b).view(-1)
    out = {"n": int(a.numel()), "n_diff": int(diff.numel()), "n_unexcused": 0,
           "agreement": 1.0 - diff.numel() / max(1, a.numel())}
    if diff.numel():
        xd = x[diff].double()
        d = (xd.unsqueeze(1) - centers.double().unsqueeze(0)).abs().sum(2)
        best = d.min(1).values
        mag = xd.abs().sum(1) + centers.double().abs().sum(1).max()
        tol = rel_gap * best + x.shape[1] * 1.2e-7 * mag
        da, db = d.gather(1, a[diff].view(-1, 1)).view(-1), d.gather(1, b[diff].view(-1, 1)).view(-1)
        out["n_unexcused"] = int(((da - best > tol) | (db - best > tol)).sum())
    return out


# --------------------------------------------------------------------------------------------------
# k-nearest-neighbours classifier
# --------------------------------------------------------------------------------------------------
def knn_one_hot(labels: torch.Tensor) -> torch.Tensor:
    """heat/classification/kneighborsclassifier.py:44-61: float32 (n, max + 1), one 1 per row."""
    lab = labels.reshape(-1).long()
    n_features = int(lab.max().item()) + 1
    one_hot = torch.zeros((lab.shape[0], n_features), dtype=torch.float32)
    one_hot[range(lab.shape[0]), lab] = 1
    return one_hot


def knn_predict(x_train: torch.Tensor, y: torch.Tensor, x_test: torch.Tensor, n_neighbors: int):
    """
    heat/classification/kneighborsclassifier.py:114-132 at one rank: ``cdist`` with its default
    ``quadratic_expansion=False`` is ``torch.cdist`` (heat/spatial/distance.py:17-29), ``ht.topk`` is
    ``torch.topk(..., largest=False, sorted=True)`` on the local matrix, the label rows of the neighbours
    are summed over the neighbour axis and the first largest entry is the class.
    Returns (classes, indices, distances).
    """
    y2 = knn_one_hot(y) if y.dim() == 1 else y
    distances = torch.cdist(x_test, x_train)
    values, indices = torch.topk(distances, n_neighbors, dim=-1, largest=False, sorted=True)
    predictions = y2[indices.flatten()]
    predictions = predictions.reshape(tuple(indices.shape) + (y2.shape[1],))
    predictions = torch.sum(predictions, dim=1)
    return torch.argmax(predictions, dim=1), indices, values


def knn_neighbours_f64(x_train: torch.Tensor, x_test: torch.Tensor, n_neighbors: int, chunk: int = 2048):
    """The k + 1 smallest float64 distances of every test row and their rows, ascending in distance (rows
    at exactly the same distance in no particular order): what a neighbour list is judged against.
    Candidates are chosen with the float64 expansion |q|^2 + |x|^2 - 2 q.x (a plain matrix product, safe
    at any size), their distances are then recomputed directly as sqrt(sum (q - x)^2).
    Returns (distances (m, k + 1), rows)."""
    xt, xq = x_train.double(), x_test.double()
    kk = min(n_neighbors + 1, xt.shape[0])
    wide = min(kk + 2, xt.shape[0])
    xn = (xt * xt).sum(1)
    out_d, out_i = [], []
    for a in range(0, xq.shape[0], chunk):
        qa = xq[a:a + chunk]
        d2 = (qa * qa).sum(1, keepdim=True) + xn[None, :] - 2.0 * (qa @ xt.T)
        _, cand = torch.topk(d2, wide, dim=1, largest=False, sorted=True)
        direct = (qa[:, None, :] - xt[cand]).pow(2).sum(-1).sqrt()
        vals, pos = torch.sort(direct, dim=1, stable=True)
        out_d.append(vals[:, :kk])
        out_i.append(torch.gather(cand, 1, pos)[:, :kk])
    return torch.cat(out_d), torch.cat(out_i)


# --------------------------------------------------------------------------------------------------
# silhouette coefficient
# --------------------------------------------------------------------------------------------------
def silhouette_samples(x: torch.Tensor, labels: torch.Tensor, metric: str = "euclidean") -> torch.Tensor:
    """heat/cluster/metrics.py:128-177 at one rank, op for op: the full distance matrix (``torch.cdist``,
    heat/spatial/distance.py:17-29), its product with the label mask, a, b and the quotient."""
    labels = labels.reshape(-1)
    unique_labels, labels_encoded = torch.unique(labels, sorted=True, return_inverse=True)
    labels_freqs = torch.bincount(labels_encoded)
    dist = x if metric == "precomputed" else torch.cdist(x, x)
    full_mask = labels.reshape(-1, 1) == unique_labels.reshape(1, -1)
    clust_dists = torch.matmul(dist, full_mask.to(dist.dtype))
    a_clust_dists = torch.sum(clust_dists * full_mask, dim=1)
    denominator_a = labels_freqs[labels_encoded] - 1
    denominator_a = torch.where(denominator_a > 0, denominator_a, torch.ones_like(denominator_a))
    a = a_clust_dists / denominator_a
    b_clust_means = clust_dists / labels_freqs
    b_clust_means[full_mask] = float("inf")
    b = torch.min(b_clust_means, dim=1).values
    sil = (b - a) / torch.maximum(a, b)
    sil = torch.where(labels_freqs[labels_encoded] > 1, sil, torch.zeros_like(sil))
    return torch.nan_to_num(sil)


def silhouette_score(x: torch.Tensor, labels: torch.Tensor, metric: str = "euclidean") -> float:
    """heat/cluster/metrics.py:269: the mean of the per-sample coefficients."""
    return float(torch.mean(silhouette_samples(x, labels, metric=metric)))


# --------------------------------------------------------------------------------------------------
# graph Laplacian
# --------------------------------------------------------------------------------------------------
def laplacian(sim: torch.Tensor, definition: str = "norm_sym", mode: str = "fully_connected", weighted: bool = True,
              threshold_key: str = "upper", threshold_value: float = 1.0) -> torch.Tensor:
    """heat/graph/laplacian.py:63-98,119-142 on a given similarity matrix, op for op (the unweighted
    adjacency is the reference's ``ht.int(S < eps)``, an int32 matrix)."""
    s = sim.clone()
    s.fill_diagonal_(0.0)
    if mode == "eNeighbour":
        keep = s < threshold_value if threshold_key == "upper" else s > threshold_value
        s = torch.where(keep, s, torch.zeros_like(s)) if weighted else keep.to(torch.int32)
    if definition == "simple":
        degree = torch.sum(s, dim=1)
        return torch.diag(degree) - s
    degree = torch.sum(s, dim=1)
    degree = torch.where(degree == 0, torch.ones_like(degree), degree)
    lap = s / torch.sqrt(degree.unsqueeze(1))
    lap = lap / torch.sqrt(degree.unsqueeze(0))
    lap = lap * (-1.0)
    lap.fill_diagonal_(1.0)
    return lap
