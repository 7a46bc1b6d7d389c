"""
GPU parity of the Manhattan-metric path: fused L1 distance+argmin, closest data row, per-cluster
medians by radix selection, and the estimators built on them (KMedians, KMedoids,
BatchParallelKMedians) against the CPU oracle.

Bars: labels equal except where the two best fp64 Manhattan distances are within 1e-5 relative (plus
the fp32 resolution of the sums); minimum distances within 1e-5 * (|x|_1 + |c|_1); medians BIT-EXACT
(order statistics are integer work, the even-count interpolation follows the reference's float64
formula); medoids exact rows of the data.
"""
import os

import numpy as np
import pytest
import torch

import heat_amd as ht
from heat_amd import _native
from heat_amd.cluster import batchparallelclustering as bpc
from heat_amd.utils import synthetic
from oracle import heat_oracle as orc

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _data(n, d, k, seed, spread=3.0):
    g = torch.Generator().manual_seed(seed)
    c = torch.randn((k, d), generator=g) * spread
    x = c[torch.randint(0, k, (n,), generator=g)] + torch.randn((n, d), generator=g)
    return x.contiguous(), c.contiguous()


class _Fixed:
    """Sampler whose integer draws are all the same row (restart row of empty clusters)."""

    def __init__(self, row):
        self.row = row

    def randint(self, high):
        return self.row


@pytest.mark.parametrize("n,d,k", [(1, 3, 8), (1000, 3, 8), (5000, 8, 16), (4096, 32, 256), (999, 17, 1),
                                   (1300, 50, 37), (700, 130, 70), (65, 16, 65)])
def test_assign_l1_matches_oracle(cuda, n, d, k):
    print(f"assign_l1 n={n} d={d} k={k}", flush=True)
    x, c = _data(n, d, k, seed=n + d + k)
    lab = torch.full((n,), -7, dtype=torch.int32, device=cuda)
    md = torch.full((n,), -1.0, device=cuda)
    _native.assign_l1(x.to(cuda), c.to(cuda), lab, md)
    ref_lab, ref_min = orc.assign_l1(x, c)
    rep = orc.label_agreement_l1(x, c, lab.cpu(), ref_lab)
    assert rep["n_unexcused"] == 0 and rep["agreement"] >= 0.999, rep
    scale = x.abs().sum(1) + c.abs().sum(1).max()
    best = (x.double().unsqueeze(1) - c.double().unsqueeze(0)).abs().sum(2).min(1).values
    assert torch.all((md.cpu().double() - best).abs() <= 1e-5 * scale + 1e-6)
    # without the distance output, and deterministic
    lab2 = torch.empty_like(lab)
    _native.assign_l1(x.to(cuda), c.to(cuda), lab2, None)
    assert torch.equal(lab, lab2)


def test_assign_l1_ties_strides_and_functional_value(cuda):
    x, c = _data(3000, 6, 5, seed=1)
    cc = torch.cat([c, c, c[:2]])  # duplicates: the first copy must win
    lab = torch.empty((3000,), dtype=torch.int32, device=cuda)
    _native.assign_l1(x.to(cuda), cc.to(cuda), lab, None)
    assert int(lab.max()) < 5
    wide = torch.randn((3000, 10), generator=torch.Generator().manual_seed(2)).to(cuda)
    wide[:, :6] = x.to(cuda)
    lab_s = torch.empty_like(lab)
    _native.assign_l1(wide[:, :6], c.to(cuda), lab_s, None)  # leading dimension 10
    lab_c = torch.empty_like(lab)
    _native.assign_l1(x.to(cuda), c.to(cuda), lab_c, None)
    assert torch.equal(lab_s, lab_c)
    # predict() of the Manhattan estimators: labels + functional value = |min dist|_2 ** 2
    km = ht.cluster.KMedians(n_clusters=5, init=ht.array(c.to(cuda)))
    km._cluster_centers = ht.array(c.to(cuda))
    pred = km.predict(ht.array(x.to(cuda), split=0))
    ref_lab, ref_min = orc.assign_l1(x, c)
    assert pred.shape == (3000, 1) and pred.dtype is ht.int64 and torch.equal(pred.larray.cpu(), ref_lab)
    fv = float((ref_min.double() ** 2).sum())
    assert abs(float(km.functional_value_.larray) - fv) <= 1e-4 * fv


def test_closest_rows_l1(cuda):
    g = torch.Generator().manual_seed(5)
    x = torch.randn((70001, 9), generator=g)
    x[60000] = x[123]  # duplicate rows: the first index wins
    q = torch.cat([x[[123, 5, 69999]] + 1e-3, torch.randn((70, 9), generator=g)])
    idx = torch.empty((q.shape[0],), dtype=torch.int64, device=cuda)
    dist = torch.empty((q.shape[0],), device=cuda)
    _native.closest_rows_l1(x.to(cuda), q.to(cuda), idx, dist, _native.Workspace(cuda))
    d = (x.double().unsqueeze(0) - q.double().unsqueeze(1)).abs().sum(2)  # (M, N)
    ref = d.argmin(1)
    got = idx.cpu()
    assert int(got[0]) == 123
    for m in range(q.shape[0]):  # same row, or a numerical tie
        assert got[m] == ref[m] or abs(float(d[m, got[m]] - d[m, ref[m]])) <= 1e-5 * float(d[m, ref[m]]) + 1e-6
    assert torch.allclose(dist.cpu().double(), d.min(1).values, rtol=1e-5, atol=1e-6)
    # tiny inputs
    one = torch.randn((1, 4)).to(cuda)
    idx1 = torch.empty((1,), dtype=torch.int64, device=cuda)
    _native.closest_rows_l1(one, one.clone(), idx1, None, _native.Workspace(cuda))
    assert int(idx1) == 0


@pytest.mark.parametrize("n,d,k,ints", [(5000, 3, 8, False), (20000, 32, 50, False), (3001, 33, 7, True),
                                        (40000, 8, 300, True), (9000, 70, 5000, False), (64, 2, 3, False),
                                        (100000, 4, 2, False)])
def test_update_median_is_bit_exact(cuda, n, d, k, ints):
    print(f"median n={n} d={d} k={k} ints={ints}", flush=True)
    g = torch.Generator().manual_seed(n + k)
    x = torch.randn((n, d), generator=g) * 5
    if ints:
        x = x.round()  # many equal values, many exact zeros, whole zero rows
        x[::13] = 0.0
    x[1] = -x[1].abs()
    lab = torch.randint(0, k, (n,), generator=g)
    lab[lab == k - 1] = 0  # the last cluster is empty
    c_old = torch.randn((k, d), generator=g)
    ws = _native.Workspace(cuda)
    xg, lg = x.to(cuda), lab.to(torch.int32).to(cuda)
    # the reference's median: zero rows dropped, mean of the middles in float64, restart row for empties
    fb = torch.full((k,), 17 % n, dtype=torch.int64, device=cuda)
    out = torch.empty((k, d), device=cuda)
    cnt = torch.empty((k,), dtype=torch.int64, device=cuda)
    _native.update_median(xg, lg, out, ws, fallback_rows=fb, counts=cnt, skip_zero_rows=True)
    ref = orc.update_medians(x, lab.view(-1, 1), c_old, _Fixed(17 % n))
    assert torch.equal(out.cpu(), ref), float((out.cpu() - ref).abs().max())
    nz = x.abs().sum(1) != 0
    assert torch.equal(cnt.cpu(), torch.bincount(lab[nz], minlength=k))
    # torch.median flavour: lower middle, nothing dropped, an empty cluster keeps its centre
    out2 = torch.empty((k, d), device=cuda)
    _native.update_median(xg, lg, out2, ws, c_old=c_old.to(cuda), lower=True)
    for i in range(min(k, 40)):
        sel = x[lab == i]
        want = torch.median(sel, dim=0)[0] if sel.shape[0] else c_old[i]
        assert torch.equal(out2[i].cpu(), want), i
    # neither restart rows nor old centres: zero row; and a second run is identical
    out3 = torch.full((k, d), 9.0, device=cuda)
    _native.update_median(xg, lg, out3, ws, skip_zero_rows=True)
    filled = (cnt > 0)
    assert torch.equal(out3[~filled], torch.zeros_like(out3[~filled])) and int((~filled).sum()) >= 1
    assert torch.equal(out3[filled], out[filled])


@pytest.mark.parametrize("n,d,k", [(3000, 4, 5), (20000, 16, 12)])
def test_kmedians_and_kmedoids_fit_match_oracle(cuda, n, d, k):
    x, _ = _data(n, d, k, seed=40 + n, spread=6.0)
    init = x[torch.randperm(n, generator=torch.Generator().manual_seed(1))[:k]].contiguous()
    xg = ht.array(x.to(cuda), split=0)
    ref = orc.kmedians_fit(x, init, 30, 1e-4, _Fixed(3))
    km = ht.cluster.KMedians(n_clusters=k, init=ht.array(init.to(cuda)), max_iter=30, tol=1e-4)
    km._make_sampler = lambda dev: _Fixed(3)
    km.fit(xg)
    rep = orc.label_agreement_l1(x, ref["cluster_centers"], km.labels_.larray.cpu(), ref["labels"])
    assert km.n_iter_ == ref["n_iter"] and rep["n_unexcused"] == 0
    assert orc.rel_err_centers(km.cluster_centers_.larray.cpu(), ref["cluster_centers"]) <= 1e-6
    assert abs(float(km.inertia_.larray) - float(ref["inertia"])) <= 1e-5 * max(1.0, float(ref["inertia"]))
    assert km.labels_.shape == (n, 1) and km.labels_.dtype is ht.int64 and km.cluster_centers_.split is None
    # _update_centroids on its own, as the reference exposes it
    upd = km._update_centroids(xg, km.labels_)
    assert upd.shape == (k, d)

    refm = orc.kmedoids_fit(x, init, 30, _Fixed(3))
    kd = ht.cluster.KMedoids(n_clusters=k, init=ht.array(init.to(cuda)), max_iter=30)
    kd._make_sampler = lambda dev: _Fixed(3)
    kd.fit(xg)
    c = kd.cluster_centers_.larray.cpu()
    assert kd.n_iter_ == refm["n_iter"]
    assert torch.equal(c, refm["cluster_centers"])
    for i in range(k):  # every medoid is a data row (tests/cluster/test_kmedoids.py:44-48)
        assert bool((x == c[i]).all(1).any())


def test_reference_style_checks_of_the_manhattan_estimators(cuda):
    iris = torch.from_numpy(np.loadtxt(os.path.join(GOLD, "iris.csv"), delimiter=";", dtype=np.float32))
    x = ht.array(iris.to(cuda), split=0)
    for est, pp in ((ht.cluster.KMedians, "kmedians++"), (ht.cluster.KMedoids, "kmedoids++")):
        for init in ("random", pp):
            m = est(n_clusters=3, init=init, random_state=1).fit(x)
            assert isinstance(m.cluster_centers_, ht.DNDarray) and m.cluster_centers_.shape == (3, 4)
            if est is ht.cluster.KMedoids:
                c = m.cluster_centers_.larray.cpu()
                assert all(bool((iris == c[i]).all(1).any()) for i in range(3))
        with pytest.raises(NotImplementedError):
            est(n_clusters=3).fit(ht.array(iris.to(cuda), split=1))
        with pytest.raises(ValueError):
            est(n_clusters=3).set_params(foo="bar")
        with pytest.raises(ValueError):
            est(n_clusters=3, init="random_number").fit(x)
        with pytest.raises(ValueError):
            est(n_clusters=3).fit(iris)
    with pytest.raises(ValueError):  # tests/cluster/test_kmedoids.py:66-69
        ht.cluster.KMedoids(n_clusters=3, init="batchparallel").fit(x)
    for n, dtype, radius, offset in ((20, torch.float32, 1.0, 4.0), (100, torch.float32, 1.0, 4.0),
                                     (20, torch.int32, 10.0, 40.0)):
        data = synthetic.spherical_dataset(n, radius, offset, dtype, seed=1)
        xs = ht.array(data.to(cuda), split=0)
        m = ht.cluster.KMedians(n_clusters=4, init="kmedians++", random_state=2).fit(xs)
        assert m.cluster_centers_.shape == (4, 3)
        m = ht.cluster.KMedians(n_clusters=4, init="batchparallel", random_state=2).fit(xs)
        assert m.cluster_centers_.shape == (4, 3)
        m = ht.cluster.KMedoids(n_clusters=4, init="kmedoids++", random_state=2).fit(xs)
        c = m.cluster_centers_.larray.cpu()
        assert all(bool((data.float() == c[i]).all(1).any()) for i in range(4))
        for seed in (1, None):
            bp = ht.cluster.BatchParallelKMedians(n_clusters=4, init="k-medians++", random_state=seed).fit(xs)
            assert bp.cluster_centers_.shape == (4, 3) and isinstance(bp.n_iter_, int)
            labels = bp.predict(xs)
            assert labels.shape == (4 * n, 1) and labels.dtype is ht.int32 and isinstance(bp.functional_value_, float)
            cc = bp.cluster_centers_.larray.cpu().double()
            fv = float((data.double() - cc[labels.larray.view(-1).cpu().long()]).abs().sum())
            assert abs(bp.functional_value_ - fv) <= 1e-4 * fv + 1e-6


def test_batchparallel_kmedians_matches_oracle(cuda):
    x, _ = _data(20000, 6, 7, seed=9, spread=8.0)
    rec = orc.RecordingSampler(13)
    ref, n_it = orc.kmex(x, 7, "++", 60, 1e-4, rec, p=1)
    bp = ht.cluster.BatchParallelKMedians(n_clusters=7, max_iter=60, tol=1e-4)
    bp._make_sampler = lambda dev, rank=0: orc.ReplaySampler(rec.tape, dev)
    bp.fit(ht.array(x.to(cuda), split=0))
    assert bp.n_iter_ == n_it
    assert orc.rel_err_centers(bp.cluster_centers_.larray.cpu(), ref) <= 1e-6


def test_closest_rows_in_float64_resolves_exact_ties_like_the_reference(cuda):
    """hkm_update_median_q64_f32 + hkm_closest_rows_l1_q64_f32: the medians before their rounding to
    float32, and the snap in float64.  Clusters of two rows have their median at the midpoint, where
    both rows are at exactly the same float64 distance: the first row must win (the reference's argmin),
    whichever way float32 rounding would have tipped it."""
    g = torch.Generator().manual_seed(9)
    n_pairs, d = 300, 7
    a = torch.randn((n_pairs, d), generator=g) * 5
    b = a + torch.randn((n_pairs, d), generator=g)
    x = torch.empty((2 * n_pairs, d))
    x[0::2], x[1::2] = a, b                       # rows 2k and 2k + 1 form cluster k
    lab = torch.arange(n_pairs).repeat_interleave(2).to(torch.int32)
    ws = _native.Workspace(cuda)
    xg = x.to(cuda)
    med = torch.empty((n_pairs, d), device=cuda)
    med64 = torch.empty((n_pairs, d), dtype=torch.float64, device=cuda)
    _native.update_median(xg, lab.to(cuda), med, ws, skip_zero_rows=True, median64=med64)
    want64 = a.double() + (b.double() - a.double()) * 0.5
    lo, hi = torch.minimum(a, b).double(), torch.maximum(a, b).double()
    assert torch.equal(med64.cpu(), lo + (hi - lo) * 0.5) and torch.allclose(med64.cpu(), want64, rtol=0, atol=1e-12)
    assert torch.equal(med.cpu(), med64.cpu().float())
    idx = torch.empty((n_pairs,), dtype=torch.int64, device=cuda)
    dist = torch.empty((n_pairs,), dtype=torch.float64, device=cuda)
    _native.closest_rows_l1_q64(xg, med64, idx, dist, ws)
    ref = (x.double()[None, :, :] - med64.cpu()[:, None, :]).abs().sum(-1)   # (pairs, rows) in float64
    assert torch.equal(idx.cpu(), ref.argmin(dim=1))
    # the two members are equidistant, so the argmin is the even row unless a third row is closer
    own = ref[torch.arange(n_pairs), 2 * torch.arange(n_pairs)]
    mine = idx.cpu() // 2 == torch.arange(n_pairs)
    assert int(mine.sum()) > n_pairs // 2 and bool((idx.cpu()[mine] % 2 == 0).all())
    assert torch.allclose(dist.cpu(), ref.min(dim=1).values, rtol=1e-14, atol=0) and bool((dist.cpu() <= own).all())
    # general case against a float64 evaluation: many rows, several splits of the data
    x2 = torch.randn((50_000, 19), generator=g)
    q = torch.randn((70, 19), generator=g, dtype=torch.float64)
    idx2 = torch.empty((70,), dtype=torch.int64, device=cuda)
    _native.closest_rows_l1_q64(x2.to(cuda), q.to(cuda), idx2, None, ws)
    ref2 = torch.cdist(q, x2.double(), p=1.0)
    assert torch.equal(idx2.cpu(), ref2.argmin(dim=1))
