"""
float64 data through the same estimators: the reference keeps float64 (and int64) inputs in float64
through its op sequence (promote(X, Y, float32), heat/spatial/distance.py:392-403), so results are
compared with the float64 oracle: labels equal except at ties of 1e-12 relative, centroids, shift and
functional value within 1e-12 relative, repeated runs bit-identical.
"""
import numpy as np
import pytest
import torch

import heat_amd as ht
from heat_amd import _native
from heat_amd.utils import synthetic
from oracle import heat_oracle as orc

pytestmark = pytest.mark.gpu


def _data(n, d, k, seed, spread=3.0):
    g = torch.Generator().manual_seed(seed)
    c = torch.randn((k, d), generator=g, dtype=torch.float64) * spread
    x = c[torch.randint(0, k, (n,), generator=g)] + torch.randn((n, d), generator=g, dtype=torch.float64)
    return x.contiguous(), c.contiguous()


@pytest.mark.parametrize("n,d,k", [(1, 3, 8), (3000, 3, 8), (5000, 32, 256), (999, 17, 1), (1300, 50, 37),
                                   (700, 130, 70), (2000, 64, 1030), (70000, 8, 200), (5000, 8, 300), (4097, 1, 5)])
def test_assign_and_update_f64(cuda, n, d, k):
    print(f"f64 n={n} d={d} k={k}", flush=True)
    x, c = _data(n, d, k, seed=n + d + k)
    xg, cg = x.to(cuda), c.to(cuda)
    ws = _native.Workspace(cuda)
    lab = torch.full((n,), -7, dtype=torch.int32, device=cuda)
    md = torch.full((n,), -1.0, dtype=torch.float64, device=cuda)
    _native.assign(xg, cg, lab, md, ws)
    ref_lab, _ = orc.assign_to_cluster_literal(x, c)
    d2 = orc.brute_force_d2(x, c)
    got = d2.gather(1, lab.cpu().long().view(-1, 1)).view(-1)
    best = d2.min(1).values
    scale = (x ** 2).sum(1) + (c ** 2).sum(1).max()
    assert torch.all(got - best <= 1e-12 * scale)  # same centroid, or a tie at float64 resolution
    assert float((lab.cpu().long() == ref_lab.view(-1)).float().mean()) >= 0.999
    assert torch.all((md.cpu() - best).abs() <= 1e-12 * scale)
    # update from those labels
    c_new = torch.empty_like(cg)
    cnt = torch.empty((k,), dtype=torch.int64, device=cuda)
    _native.update(xg, lab, c_new, cnt, ws)
    ref_c, ref_cnt = orc.update_centroids_fast(x, lab.cpu().long().view(-1, 1), k, out_dtype=torch.float64)
    assert torch.equal(cnt.cpu(), ref_cnt.view(-1).long())
    assert orc.rel_err_centers(c_new.cpu(), ref_c) <= 1e-12
    # one step, twice: identical, and consistent with its parts
    outs = []
    for _ in range(2):
        c2 = torch.empty_like(cg)
        lab2 = torch.empty_like(lab)
        shift = torch.empty((), dtype=torch.float64, device=cuda)
        sse = torch.empty((), dtype=torch.float64, device=cuda)
        _native.lloyd_step(xg, cg, c2, lab2, shift, sse, ws)
        outs.append((c2.cpu(), lab2.cpu(), shift.cpu(), sse.cpu()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert torch.equal(outs[0][0], c_new.cpu()) and torch.equal(outs[0][1], lab.cpu())
    ref_shift = float(((c - outs[0][0]) ** 2).sum())
    assert abs(float(outs[0][2]) - ref_shift) <= 1e-12 * max(ref_shift, 1e-300)
    assert abs(float(outs[0][3]) - float(best.sum())) <= 1e-10 * float(best.sum()) + 1e-12 * float(scale.sum())


def test_kmeans_fit_predict_f64_matches_oracle(cuda):
    w = synthetic.config1(0.3)
    x, init = w.x.double(), w.init.double()
    ref = orc.kmeans_fit(x, init, 15, 0.0, literal=True)
    km = ht.cluster.KMeans(n_clusters=w.k, init=ht.array(init.to(cuda)), max_iter=15, tol=0.0)
    km.fit(ht.array(x.to(cuda), split=0))
    assert km.cluster_centers_.dtype is ht.float64 and km.cluster_centers_.larray.dtype == torch.float64
    assert km.n_iter_ == ref["n_iter"]
    assert orc.rel_err_centers(km.cluster_centers_.larray.cpu(), ref["cluster_centers"]) <= 1e-10
    assert torch.equal(km.labels_.larray.cpu(), ref["labels"])
    assert abs(float(km.inertia_.larray) - float(ref["inertia"])) <= 1e-9 * max(float(ref["inertia"]), 1e-30)
    pred = km.predict(ht.array(x.to(cuda), split=0))
    ref_lab, ref_fv = orc.predict(x, ref["cluster_centers"])
    assert torch.equal(pred.larray.cpu(), ref_lab)
    assert abs(float(km.functional_value_.larray) - float(ref_fv)) <= 1e-10 * float(ref_fv)
    # int64 data promote to float64 like the reference's promote(int64, float32)
    xi = (x * 10).round().long()
    km = ht.cluster.KMeans(n_clusters=w.k, init="random", max_iter=5, random_state=3).fit(ht.array(xi.to(cuda), split=0))
    assert km.cluster_centers_.larray.dtype == torch.float64


def test_spatial_f64_and_other_estimators(cuda):
    g = torch.Generator().manual_seed(2)
    a = torch.randn((130, 9), generator=g, dtype=torch.float64)
    b = torch.randn((70, 9), generator=g, dtype=torch.float64)
    A, B = ht.array(a.to(cuda), split=0), ht.array(b.to(cuda))
    for qe in (False, True):
        d = ht.spatial.cdist(A, B, quadratic_expansion=qe)
        assert d.dtype is ht.float64 and torch.allclose(d.larray.cpu(), torch.cdist(a, b), rtol=1e-9, atol=1e-9)
        r = ht.spatial.rbf(A, B, sigma=1.5, quadratic_expansion=qe)
        assert torch.allclose(r.larray.cpu(), torch.exp(-torch.cdist(a, b) ** 2 / (2 * 1.5 ** 2)), rtol=1e-9, atol=1e-12)
    m = ht.spatial.manhattan(A, B)
    assert torch.allclose(m.larray.cpu(), torch.cdist(a, b, p=1), rtol=1e-12)
    # mixed float32 / float64 promote to float64 (heat/spatial/distance.py:392-403)
    d = ht.spatial.cdist(A, ht.array(b.float().to(cuda)), quadratic_expansion=True)
    assert d.dtype is ht.float64
    # the reference's float64 datasets (tests/cluster/test_kmeans.py:125-134, test_batchparallelclustering.py:90)
    data = synthetic.spherical_dataset(20, 1.0, 4.0, torch.float64, seed=1)
    xs = ht.array(data.to(cuda), split=0)
    for init in ("kmeans++", "batchparallel", "random"):
        km = ht.cluster.KMeans(n_clusters=4, init=init, random_state=1).fit(xs)
        assert km.cluster_centers_.shape == (4, 3) and km.cluster_centers_.dtype is ht.float64
    bp = ht.cluster.BatchParallelKMeans(n_clusters=4, random_state=1).fit(xs)
    assert bp.cluster_centers_.dtype is ht.float64
    lab = bp.predict(xs)
    c = bp.cluster_centers_.larray.cpu()
    fv = float(((data - c[lab.larray.view(-1).cpu().long()]) ** 2).sum())
    assert abs(bp.functional_value_ - fv) <= 1e-9 * fv
    # the Manhattan-metric estimators on the reference's float64 and integer data sets
    # (tests/cluster/test_kmedians.py:105-121, test_kmedoids.py:108-124, test_batchparallelclustering.py)
    for data in (synthetic.spherical_dataset(20, 1.0, 4.0, torch.float64, seed=1),
                 synthetic.spherical_dataset(20, 10.0, 40.0, torch.int64, seed=1)):
        xs = ht.array(data.to(cuda), split=0)
        m = ht.cluster.KMedians(n_clusters=4, init="kmedians++", random_state=2).fit(xs)
        assert m.cluster_centers_.shape == (4, 3) and m.cluster_centers_.dtype is ht.float64
        assert m.labels_.shape == (80, 1) and m.labels_.dtype is ht.int64
        m = ht.cluster.KMedoids(n_clusters=4, init="kmedoids++", random_state=2).fit(xs)
        c = m.cluster_centers_.larray.cpu()
        assert m.cluster_centers_.dtype is ht.float64
        assert all(bool((data.double() == c[i]).all(1).any()) for i in range(4))  # every medoid is a data row
        bp = ht.cluster.BatchParallelKMedians(n_clusters=4, init="k-medians++", random_state=1).fit(xs)
        # (the batch-parallel estimators work on the local torch tensors: integer rows become float32)
        assert bp.cluster_centers_.shape == (4, 3)
        assert bp.cluster_centers_.dtype is (ht.float64 if data.dtype == torch.float64 else ht.float32)
        lab = bp.predict(xs)
        cc = bp.cluster_centers_.larray.cpu()
        fv = float((data.double() - cc[lab.larray.view(-1).cpu().long()]).abs().sum())
        assert abs(bp.functional_value_ - fv) <= 1e-9 * fv + 1e-12


class _Fixed:
    """A sampler whose every draw is the same row (restart rows of empty clusters)."""

    def __init__(self, row):
        self.row = row

    def randint(self, high):
        return self.row % high


@pytest.mark.parametrize("n,d,k", [(3000, 4, 5), (8000, 7, 9)])
def test_kmedians_and_kmedoids_fit_f64_match_oracle(cuda, n, d, k):
    g = torch.Generator().manual_seed(n + d)
    c = torch.randn((k, d), generator=g, dtype=torch.float64) * 6.0
    x = c[torch.randint(0, k, (n,), generator=g)] + torch.randn((n, d), generator=g, dtype=torch.float64)
    x[5] = 0.0  # an all-zero row: left out of the medians like in the reference
    init = x[torch.randperm(n, generator=g)[:k]].contiguous()
    xg = ht.array(x.to(cuda), split=0)
    ref = orc.kmedians_fit(x, init, 30, 1e-8, _Fixed(3))
    km = ht.cluster.KMedians(n_clusters=k, init=ht.array(init.to(cuda)), max_iter=30, tol=1e-8)
    km._make_sampler = lambda dev: _Fixed(3)
    km.fit(xg)
    assert km.n_iter_ == ref["n_iter"]
    assert torch.equal(km.labels_.larray.cpu().view(-1), ref["labels"].view(-1))
    assert km.cluster_centers_.dtype is ht.float64
    assert orc.rel_err_centers(km.cluster_centers_.larray.cpu(), ref["cluster_centers"]) <= 1e-13
    refm = orc.kmedoids_fit(x, init, 30, _Fixed(3))
    kd = ht.cluster.KMedoids(n_clusters=k, init=ht.array(init.to(cuda)), max_iter=30)
    kd._make_sampler = lambda dev: _Fixed(3)
    kd.fit(xg)
    assert kd.n_iter_ == refm["n_iter"]
    assert torch.equal(kd.cluster_centers_.larray.cpu(), refm["cluster_centers"])


def test_knn_other_metrics_and_f64(cuda):
    """KNeighborsClassifier with a metric other than cdist, and with float64 data: the reference's own op
    sequence (full matrix, topk, vote) -- checked against scikit-learn's brute-force classifier."""
    from sklearn.neighbors import KNeighborsClassifier as SkKnn

    g = torch.Generator().manual_seed(5)
    centres = torch.randn((4, 6), generator=g, dtype=torch.float64) * 8.0
    ytr = torch.randint(0, 4, (600,), generator=g)
    xtr = centres[ytr] + torch.randn((600, 6), generator=g, dtype=torch.float64)
    yte = torch.randint(0, 4, (150,), generator=g)
    xte = centres[yte] + torch.randn((150, 6), generator=g, dtype=torch.float64)
    for dtype in (torch.float64, torch.float32):
        for metric, sk_metric in ((ht.spatial.manhattan, "manhattan"), (None, "euclidean"),
                                  (lambda a, b: ht.spatial.cdist(a, b, quadratic_expansion=True), "euclidean")):
            if dtype == torch.float32 and metric is None:
                continue  # the fused float32 path has its own tests
            knn = ht.classification.KNeighborsClassifier(n_neighbors=5, effective_metric_=metric)
            knn.fit(ht.array(xtr.to(dtype).to(cuda), split=0), ht.array(ytr.to(cuda), split=0))
            got = knn.predict(ht.array(xte.to(dtype).to(cuda), split=0)).larray.cpu()
            want = SkKnn(n_neighbors=5, algorithm="brute", metric=sk_metric).fit(xtr.numpy(), ytr.numpy()).predict(xte.numpy())
            assert float((got.numpy() == want).mean()) >= 0.99, (dtype, sk_metric)
            assert knn.kneighbors_.shape == (150, 5)
    # the float64 k-nearest-rows step on its own: exact lists on integer-valued data
    x = torch.randint(-6, 7, (700, 5), generator=g).double()
    q = torch.randint(-6, 7, (40, 5), generator=g).double()
    d2 = ((q[:, None, :] - x[None, :, :]) ** 2).sum(-1)
    order = torch.argsort(d2, dim=1, stable=True)[:, :7]
    idx = torch.empty((40, 7), dtype=torch.int64, device=cuda)
    dist = torch.empty((40, 7), dtype=torch.float64, device=cuda)
    _native.knn(q.to(cuda), x.to(cuda), 7, idx, dist, _native.Workspace(cuda))
    assert torch.equal(idx.cpu(), order)
    assert torch.allclose(dist.cpu(), torch.gather(d2, 1, order).sqrt(), rtol=1e-14)


def test_silhouette_and_laplacian_f64(cuda):
    from sklearn.metrics import silhouette_samples as sk_sil

    g = torch.Generator().manual_seed(8)
    centres = torch.randn((5, 4), generator=g, dtype=torch.float64) * 5.0
    lab = torch.randint(0, 5, (900,), generator=g)
    x = centres[lab] + torch.randn((900, 4), generator=g, dtype=torch.float64)
    lab[-1] = 7  # a sample alone in its cluster
    for data in (x, (x * 10).round().to(torch.int64)):
        s = ht.cluster.silhouette_samples(ht.array(data.to(cuda), split=0), ht.array(lab.to(cuda), split=0))
        assert s.dtype is ht.float64
        assert np.allclose(s.larray.cpu().numpy(), sk_sil(data.double().numpy(), lab.numpy()), rtol=1e-10, atol=1e-12)
    dm = torch.cdist(x, x)
    dm.fill_diagonal_(0.0)
    s = ht.cluster.silhouette_samples(ht.array(dm.to(cuda), split=0), ht.array(lab.to(cuda), split=0), metric="precomputed")
    assert np.allclose(s.larray.cpu().numpy(), sk_sil(dm.numpy(), lab.numpy(), metric="precomputed"), rtol=1e-10, atol=1e-12)
    # Laplacian: float64 similarities stay float64; the unweighted simple Laplacian is an int64 matrix
    X = ht.array(x[:300].to(cuda), split=0)
    for definition in ("simple", "norm_sym"):
        for kwargs in ({}, {"mode": "eNeighbour", "threshold_value": 0.5}, {"mode": "eNeighbour", "weighted": False,
                                                                             "threshold_key": "lower", "threshold_value": 0.2}):
            sim_fn = lambda a: ht.spatial.rbf(a, sigma=3.0)  # noqa: E731
            L = ht.graph.Laplacian(sim_fn, definition=definition, **kwargs).construct(X)
            sim = sim_fn(X).larray.cpu()
            assert sim.dtype == torch.float64
            want = orc.laplacian(sim, definition, kwargs.get("mode", "fully_connected"), kwargs.get("weighted", True),
                                 kwargs.get("threshold_key", "upper"), kwargs.get("threshold_value", 1.0))
            if not kwargs.get("weighted", True):
                assert L.dtype is (ht.int64 if definition == "simple" else ht.float32) and L.larray.dtype == want.dtype
                tol = 2e-6
            else:
                assert L.dtype is ht.float64
                tol = 1e-12
            assert torch.allclose(L.larray.cpu().double(), want.double(), rtol=0, atol=tol * float(want.abs().max()))
    # more rows than a 16-bit grid dimension holds
    n = 70000
    sim = torch.rand((n, 8), device=cuda)
    S = (sim @ sim.T)
    out = torch.empty_like(S)
    deg = torch.empty((n,), device=cuda)
    _native.laplacian(S, out, 0, 0, True, 0.0, deg)
    rows = torch.tensor([0, 1, 65535, 65536, n - 1], device=cuda)
    want_deg = S[rows].double().sum(1) - S[rows, rows].double()
    assert torch.allclose(deg[rows].double(), want_deg, rtol=1e-6)
    assert torch.allclose(out[rows, rows].double(), want_deg, rtol=1e-6)
    assert torch.equal(out[rows][:, 5:9], -S[rows][:, 5:9])

