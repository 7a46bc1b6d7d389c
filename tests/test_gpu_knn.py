"""
k nearest rows + label vote (hkm_knn_f32, hkm_knn_vote_f32, KNeighborsClassifier) against the oracle's
restatement of heat/classification/kneighborsclassifier.py:114-132 and against float64 evaluations.

Bars: on integer-valued data every squared distance is exact in fp32, so the neighbour lists must equal
a stable sort of the exact distances bit for bit (ties to the smaller row index) and the classes must
equal the oracle's.  On real-valued data the j-th neighbour returned must be at the j-th smallest float64
distance to within 1e-5 relative plus the fp32 resolution of the squared norms (rows closer together than
that may swap), and the distances returned must match float64 to 1e-5; from 16 features on the
squared distance is the clamped expansion |q|^2 + |x|^2 - 2 q.x (matrix cores), so there both bars are on
squared distances with 4e-7 (|q|^2 + max |x|^2) of slack.
"""
import os

import numpy as np
import pytest
import torch

import heat_amd as ht
from heat_amd import _native
from oracle import heat_oracle as orc

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _exact_lists(q, x, k):
    d2 = ((q.double()[:, None, :] - x.double()[None, :, :]) ** 2).sum(-1)
    order = torch.argsort(d2, dim=1, stable=True)[:, :k]
    return order, torch.gather(d2, 1, order)


@pytest.mark.parametrize("m,n,d,k", [
    (1, 1, 1, 1), (3, 5, 2, 5), (64, 64, 16, 4), (65, 63, 17, 5), (200, 1000, 8, 8), (130, 777, 5, 9),
    (7, 20000, 12, 16), (33, 9000, 3, 17), (500, 300, 33, 40), (2, 70000, 6, 3), (4097, 130, 20, 1),
    (40, 5000, 4, 100),
])
def test_integer_data_gives_the_exact_sorted_lists(cuda, m, n, d, k):
    g = torch.Generator().manual_seed(m * 7 + n * 3 + d + k)
    x = torch.randint(-6, 7, (n, d), generator=g).float()
    q = torch.randint(-6, 7, (m, d), generator=g).float()
    want_i, want_d2 = _exact_lists(q, x, k)
    ws = _native.Workspace(cuda)
    idx = torch.full((m, k + 2), -7, dtype=torch.int64, device=cuda)[:, :k]
    dist = torch.full((m, k + 1), -7.0, device=cuda)[:, :k]
    xg = torch.zeros((n, d + 3), device=cuda)[:, :d]
    xg.copy_(x)
    _native.knn(q.to(cuda), xg, k, idx, dist, ws)
    assert torch.equal(idx.cpu(), want_i)
    assert torch.equal(dist.cpu(), torch.from_numpy(np.sqrt(want_d2.numpy()).astype(np.float32)))
    assert bool((idx._base[:, k:] == -7).all()) and bool((dist._base[:, k:] == -7.0).all())
    # twice on the same workspace, and without the distances
    idx2 = torch.empty((m, k), dtype=torch.int64, device=cuda)
    _native.knn(q.to(cuda), xg, k, idx2, None, ws)
    assert torch.equal(idx2, idx)


@pytest.mark.parametrize("seed", [1, 2])
def test_random_shapes_give_the_exact_sorted_lists(cuda, seed):
    """Seeded sweep on both sides of every tile and dispatch boundary (feature counts around 16, 32, 64, 128,
    rows around 32, 64, 128), dense and padded rows (the padded ones take the kernels without vector
    loads), integer-valued data so that the expected lists are exact."""
    import random

    rng = random.Random(seed)
    ws = _native.Workspace(cuda)
    for case in range(40):
        m = rng.choice([1, 2, 31, 32, 33, 127, 128, 129, 500])
        n = rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 257, 1000, 5000])
        d = rng.choice([1, 3, 4, 8, 15, 16, 17, 20, 31, 32, 33, 36, 48, 63, 64, 65, 100, 128, 129, 200])
        k = min(n, rng.choice([1, 2, 5, 8, 9, 16, 17, 33]))
        padq, padx = rng.choice([0, 0, 1, 4]), rng.choice([0, 0, 1, 4])
        what = f"seed={seed} case={case} m={m} n={n} d={d} k={k} padq={padq} padx={padx}"
        print(what, flush=True)
        g = torch.Generator().manual_seed(seed * 7919 + case)
        x = torch.randint(-5, 6, (n, d), generator=g).float()
        q = torch.randint(-5, 6, (m, d), generator=g).float()
        want_i, want_d2 = _exact_lists(q, x, k)
        xg = torch.zeros((n, d + padx), device=cuda)[:, :d]
        xg.copy_(x)
        qg = torch.zeros((m, d + padq), device=cuda)[:, :d]
        qg.copy_(q)
        idx = torch.full((m, k), -7, dtype=torch.int64, device=cuda)
        dist = torch.full((m, k), -7.0, device=cuda)
        _native.knn(qg, xg, k, idx, dist, ws)
        assert torch.equal(idx.cpu(), want_i), what
        assert torch.equal(dist.cpu(), torch.from_numpy(np.sqrt(want_d2.numpy()).astype(np.float32))), what


def test_training_rows_beyond_4gib(cuda):
    """A training matrix whose byte offsets do not fit 32 bits: the neighbours of a few test rows placed next
    to known training rows on both sides of the 4 GiB offset and at the very end."""
    n, d, k = 40_000_000, 32, 5
    g = torch.Generator(device=cuda).manual_seed(3)
    x = torch.empty((n, d), device=cuda)
    step = 1 << 23
    for a in range(0, n, step):
        b = min(n, a + step)
        x[a:b] = torch.randn((b - a, d), device=cuda, generator=g) * 4
    assert x.numel() * 4 > 1 << 32
    r4 = (1 << 32) // (4 * d)
    rows = torch.tensor([0, 77, r4 - 1, r4, r4 + 1, n // 2 + 5, n - 2, n - 1], device=cuda)
    q = torch.cat([x[rows] + 1e-3, torch.randn((120, d), device=cuda, generator=g) * 4])
    idx = torch.empty((q.shape[0], k), dtype=torch.int64, device=cuda)
    dist = torch.empty((q.shape[0], k), device=cuda)
    _native.knn(q, x, k, idx, dist, _native.Workspace(cuda))
    assert torch.equal(idx[:8, 0], rows)
    # all lists against a float64 evaluation in row chunks
    best_d = torch.full((q.shape[0], k), float("inf"), dtype=torch.float64, device=cuda)
    best_i = torch.zeros((q.shape[0], k), dtype=torch.int64, device=cuda)
    qd = q.double()
    for a in range(0, n, 1 << 22):
        b = min(n, a + (1 << 22))
        xd = x[a:b].double()
        d2 = (qd * qd).sum(1, keepdim=True) + (xd * xd).sum(1)[None] - 2.0 * (qd @ xd.T)
        v, i = torch.topk(d2, k, dim=1, largest=False)
        cat_d, cat_i = torch.cat([best_d, v], 1), torch.cat([best_i, i + a], 1)
        best_d, pos = torch.topk(cat_d, k, dim=1, largest=False)
        best_i = torch.gather(cat_i, 1, pos)
    got_d2 = (qd[:, None, :] - x[idx].double()).pow(2).sum(-1)
    scale2 = (qd * qd).sum(1, keepdim=True) + float((x[:1 << 20].double() ** 2).sum(1).max())
    assert int(((got_d2 - best_d.clamp_min(0)).abs() > 1e-5 * best_d.abs() + 1e-6 * scale2).sum()) == 0
    assert float((idx == best_i).double().mean()) > 0.99


@pytest.mark.parametrize("m,n,d,k,spread", [
    (300, 4000, 32, 5, 3.0), (64, 50000, 64, 10, 0.1), (5000, 700, 7, 8, 100.0), (1000, 1000, 130, 20, 1.0),
    (20000, 100000, 16, 5, 3.0),
])
def test_real_data_against_float64_neighbours(cuda, m, n, d, k, spread):
    g = torch.Generator(device=cuda).manual_seed(n + k)
    c = torch.randn((32, d), device=cuda, generator=g) * spread
    x = c[torch.randint(0, 32, (n,), device=cuda, generator=g)] + torch.randn((n, d), device=cuda, generator=g)
    q = c[torch.randint(0, 32, (m,), device=cuda, generator=g)] + torch.randn((m, d), device=cuda, generator=g)
    x[n // 2] = x[3]                                  # an exact duplicate: the smaller index comes first
    ws = _native.Workspace(cuda)
    idx = torch.empty((m, k), dtype=torch.int64, device=cuda)
    dist = torch.empty((m, k), device=cuda)
    _native.knn(q, x, k, idx, dist, ws)
    assert int(idx.min()) >= 0 and int(idx.max()) < n
    srt = idx.sort(dim=1).values
    assert not bool((srt[:, 1:] == srt[:, :-1]).any()), "a row listed twice"
    want_d, want_i = orc.knn_neighbours_f64(x, q, k)
    got_d = (q.double()[:, None, :] - x.double()[idx]).pow(2).sum(-1).sqrt()
    # squared scale of the operands: from 16 features on the distances are the expanded square, whose
    # rounding error is relative to |q|^2 + |x|^2 and not to the distance
    scale2 = (q.double() ** 2).sum(1, keepdim=True) + float((x.double() ** 2).sum(1).max())
    tol2 = 1e-5 * want_d[:, :k] ** 2 + (4e-7 if d >= 16 else 1e-12) * scale2
    assert int(((got_d ** 2 - want_d[:, :k] ** 2).abs() > tol2).sum()) == 0
    assert int(((dist.double() ** 2 - got_d ** 2).abs() > 1e-5 * got_d ** 2 + 4e-7 * scale2).sum()) == 0
    dup = (want_i[:, :k] == 3) | (want_i[:, :k] == n // 2)   # the float64 lists hold the duplicate pair in either order
    assert float((idx == want_i[:, :k])[~dup].double().mean()) > 0.99
    both = (idx == 3).any(1) & (idx == n // 2).any(1)
    pos3 = (idx == 3).double().argmax(1)
    posd = (idx == n // 2).double().argmax(1)
    assert bool((pos3[both] + 1 == posd[both]).all())


def test_vote_and_classifier_match_the_oracle(cuda):
    g = torch.Generator().manual_seed(11)
    n, m, d, ncls = 3000, 800, 6, 7
    x = torch.randint(-9, 10, (n, d), generator=g).float()
    q = torch.randint(-9, 10, (m, d), generator=g).float()
    y = torch.randint(0, ncls, (n,), generator=g)
    for k in (1, 5, 12):
        want_i, _ = _exact_lists(q, x, k)
        votes = orc.knn_one_hot(y)[want_i.flatten()].reshape(m, k, -1).sum(1)
        want_cls = votes.argmax(1)
        knn = ht.classification.KNeighborsClassifier(n_neighbors=k)
        knn.fit(ht.array(x.to(cuda), split=0), ht.array(y.to(cuda), split=0))
        got = knn.predict(ht.array(q.to(cuda), split=0))
        assert isinstance(got, ht.DNDarray) and got.shape == (m,) and got.dtype is ht.int64
        assert torch.equal(knn.kneighbors_.larray.cpu(), want_i)
        assert torch.equal(got.larray.cpu(), want_cls)
        # where no two training rows are equally far, the oracle's own op sequence gives the same classes
        o_cls, o_idx, _ = orc.knn_predict(x, y, q, k)
        same = (o_idx.sort(1).values == want_i.sort(1).values).all(1)
        assert int(same.sum()) > 0 and torch.equal(o_cls[same], want_cls[same])
    # label rows given as a matrix of weights, padded row stride, -1 entries skipped
    w = torch.randint(0, 5, (n, 4), generator=g).float()
    wg = torch.zeros((n, 6), device=cuda)[:, :4]
    wg.copy_(w)
    want_i, _ = _exact_lists(q, x, 9)
    idx = want_i.clone()
    idx[::3, 4] = -1
    sums = torch.where((idx >= 0)[:, :, None], w[idx.clamp_min(0)], torch.zeros(())).sum(1)
    cls = torch.empty((m,), dtype=torch.int64, device=cuda)
    _native.knn_vote(idx.to(cuda), wg, cls)
    assert torch.equal(cls.cpu(), sums.argmax(1))
    # more classes than lanes in a wave
    y2 = torch.randint(0, 300, (n,), generator=g)
    oh = orc.knn_one_hot(y2)
    _native.knn_vote(want_i.to(cuda), oh.to(cuda), cls)
    assert torch.equal(cls.cpu(), oh[want_i.flatten()].reshape(m, 9, -1).sum(1).argmax(1))


def test_reference_style_checks_on_iris(cuda):
    """tests/classification/test_knn.py:16-100 on the csv copy of the iris data: integral and one-hot labels."""
    iris = torch.from_numpy(np.loadtxt(os.path.join(GOLD, "iris.csv"), delimiter=";", dtype=np.float32))
    x = ht.array(iris.to(cuda), split=0)
    y = torch.zeros(150, dtype=torch.int64)
    y[50:100], y[100:] = 1, 2
    knn = ht.classification.KNeighborsClassifier(n_neighbors=5)
    knn.fit(x, ht.array(y.to(cuda)))
    result = knn.predict(x)
    assert ht.is_estimator(knn) and ht.is_classifier(knn)
    assert isinstance(result, ht.DNDarray) and result.shape == (150,)
    o_cls, o_idx, _ = orc.knn_predict(iris, y, iris, 5)
    d64, _ = orc.knn_neighbours_f64(iris, iris, 5)
    clear = (d64[:, 1:] - d64[:, :-1]).min(dim=1).values > 1e-3
    assert int(clear.sum()) >= 20
    assert torch.equal(result.larray.cpu()[clear], o_cls[clear])
    assert float((result.larray.cpu() == y).double().mean()) > 0.95
    y1h = torch.zeros((150, 3), dtype=torch.int64)
    y1h[range(150), y] = 1
    knn2 = ht.classification.KNeighborsClassifier(n_neighbors=5)
    knn2.fit(x, ht.array(y1h.to(cuda)))
    assert torch.equal(knn2.predict(x).larray, result.larray)
    assert torch.equal(knn.fit_predict(x, ht.array(y.to(cuda))).larray, result.larray)


def test_argument_checks(cuda):
    ws = _native.Workspace(cuda)
    x = torch.zeros((10, 3), device=cuda)
    idx = torch.empty((4, 11), dtype=torch.int64, device=cuda)
    with pytest.raises(_native.HkmError):
        _native.knn(x[:4], x, 11, idx, None, ws)          # more neighbours than rows
    with pytest.raises(ValueError):
        _native.knn(x[:4], x, 2, idx, None, ws)           # idx of the wrong shape
    with pytest.raises(TypeError):
        _native.knn(x[:4].double(), x, 2, idx[:, :2], None, ws)
    knn = ht.classification.KNeighborsClassifier(n_neighbors=11)
    knn.fit(ht.array(x), ht.array(torch.zeros(10, dtype=torch.int64, device=cuda)))
    with pytest.raises(ValueError):
        knn.predict(ht.array(x))
    empty = torch.empty((0, 2), dtype=torch.int64, device=cuda)
    _native.knn(x[:0], x, 2, empty, None, ws)             # no test rows: nothing to do


@pytest.mark.parametrize("m,n,d,k", [
    (40, 300, 8, 5),       # vector-ALU kernel
    (500, 300, 32, 5),     # matrix-core kernel, one split of the training rows
    (7, 20000, 32, 6),     # matrix-core kernel, many splits
    (130, 400, 64, 16),    # matrix-core kernel, wide rows, full lists
    (9, 30000, 64, 20),    # many splits and a second pass (k > 16)
    (33, 200, 100, 3),     # unaligned feature count on the matrix cores
])
def test_non_finite_rows_are_never_neighbours(cuda, m, n, d, k):
    """A NaN training row, a training row whose squared norm overflows, and a NaN query row: the bad training
    rows must never be returned (torch.topk(largest=False) ranks NaN last), every other list must equal the
    exact one over the remaining rows, and the NaN query's slots hold index -1 and distance inf."""
    g = torch.Generator().manual_seed(m + n + d + k)
    x = torch.randint(-6, 7, (n, d), generator=g).float()
    q = torch.randint(-6, 7, (m, d), generator=g).float()
    nan_row, big_row, nan_query = 3, n - 2, m - 1
    x[nan_row, d // 2] = float("nan")
    x[big_row] = 3e19           # |x|^2 = inf in float32
    q[nan_query, 0] = float("nan")
    good = torch.ones(n, dtype=torch.bool)
    good[nan_row] = good[big_row] = False
    rows = torch.nonzero(good).view(-1)
    want_i, want_d2 = _exact_lists(q[:nan_query], x[good], k)
    want_i = rows[want_i]
    idx = torch.full((m, k), -7, dtype=torch.int64, device=cuda)
    dist = torch.full((m, k), -7.0, device=cuda)
    print(f"knn non-finite m={m} n={n} d={d} k={k}", flush=True)
    _native.knn(q.to(cuda), x.to(cuda), k, idx, dist, _native.Workspace(cuda))
    idx, dist = idx.cpu(), dist.cpu()
    assert not bool(((idx == nan_row) | (idx == big_row)).any())
    assert torch.equal(idx[:nan_query], want_i)
    assert torch.equal(dist[:nan_query], torch.from_numpy(np.sqrt(want_d2.numpy()).astype(np.float32)))
    assert bool((idx[nan_query] == -1).all()) and bool(torch.isinf(dist[nan_query]).all())
