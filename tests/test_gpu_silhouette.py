"""
Silhouette coefficient (hkm_cluster_distance_sums_f32, hkm_silhouette_finish_f32, ht.cluster.silhouette_samples /
silhouette_score) against the oracle's op-for-op restatement of heat/cluster/metrics.py, against scikit-learn
(the check the reference's own test makes, tests/cluster/test_metrics.py:16-42, atol 1e-6) and against the
known answers that test file holds.  Bar: 1e-5 absolute on the coefficients against scikit-learn (float32
sums of up to 10^4 distances in a different order) and against the oracle up to 25 rows -- above that the
oracle, like the reference, takes torch.cdist's expanded square and is itself only good to 1e-4 ... 1e-3 -- and
1e-6 relative on the distance sums against float64.
"""
import numpy as np
import pytest
import torch

import heat_amd as ht
from heat_amd import _native
from oracle import heat_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,d,k", [(8, 1, 3), (17, 2, 5), (17, 3, 3), (64, 16, 2), (65, 17, 4), (1000, 33, 7),
                                   (5000, 8, 64), (3000, 64, 300)])
def test_samples_against_oracle_and_scikit_learn(cuda, n, d, k):
    from sklearn.metrics import silhouette_samples as sk_silhouette

    g = torch.Generator().manual_seed(n + d + k)
    x = torch.rand((n, d), generator=g)
    lab = torch.randint(0, k, (n,), generator=g) * 3 + 10        # label values with gaps
    got = ht.cluster.silhouette_samples(ht.array(x.to(cuda), split=0), ht.array(lab.to(cuda), split=0))
    assert isinstance(got, ht.DNDarray) and got.shape == (n,) and got.dtype is ht.float32
    want = orc.silhouette_samples(x, lab)
    # the oracle inherits torch.cdist's expanded square above 25 rows (self-distances of ~3e-4, coefficients
    # off by 1e-5 ... 1e-3 against scikit-learn, growing with the feature count); the kernel sums (x - y)^2 directly
    assert torch.allclose(got.larray.cpu(), want, rtol=0, atol=1e-5 if n <= 25 else 2e-3)
    if len(torch.unique(lab)) > 1:
        sk = sk_silhouette(x.numpy(), lab.numpy(), metric="euclidean")
        assert np.allclose(got.larray.cpu().numpy(), sk, atol=1e-5)
    # a precomputed distance matrix gives the same coefficients
    dist = ht.spatial.cdist(ht.array(x.to(cuda)), ht.array(x.to(cuda)))
    dist.larray.fill_diagonal_(0.0)
    pre = ht.cluster.silhouette_samples(dist, ht.array(lab.to(cuda)), metric="precomputed")
    assert torch.allclose(pre.larray, got.larray, rtol=0, atol=1e-5)
    score = ht.cluster.silhouette_score(ht.array(x.to(cuda)), ht.array(lab.to(cuda)))
    assert score == pytest.approx(float(want.mean()), abs=1e-5 if n <= 25 else 2e-3)


def test_distance_sums_against_float64(cuda):
    g = torch.Generator(device=cuda).manual_seed(2)
    n, d, k = 20_000, 24, 9
    xw = torch.zeros((n, d + 4), device=cuda)
    x = xw[:, :d]
    x.copy_(torch.randn((n, d), device=cuda, generator=g) * 3)
    enc = torch.randint(0, k, (n,), device=cuda, generator=g)
    enc[enc == 4] = 5                                               # an empty cluster in the middle
    counts = torch.bincount(enc, minlength=k)
    perm = torch.sort(enc, stable=True).indices.contiguous()
    offsets = torch.zeros((k + 1,), dtype=torch.int64, device=cuda)
    offsets[1:] = torch.cumsum(counts, 0)
    out = torch.full((n, k + 2), -7.0, device=cuda)[:, :k]
    _native.cluster_distance_sums(x, perm, offsets, out)
    mask = torch.zeros((n, k), dtype=torch.float64, device=cuda)
    mask.scatter_(1, enc.view(-1, 1), 1.0)
    want = torch.zeros((n, k), dtype=torch.float64, device=cuda)
    xd = x.double()
    for a in range(0, n, 200):
        want[a:a + 200] = (xd[a:a + 200, None, :] - xd[None, :, :]).pow(2).sum(-1).sqrt() @ mask
    assert float((out.double() - want).abs().max()) <= 1e-6 * float(want.max())
    assert bool((out[:, 4] == 0).all()) and bool((out._base[:, k:] == -7.0).all())
    with pytest.raises(ValueError):
        _native.cluster_distance_sums(x, perm + 1, offsets, out)
    with pytest.raises(ValueError):
        _native.silhouette_finish(out.contiguous(), enc + 1, counts, torch.empty((n,), device=cuda))


def test_known_answers_and_special_cases_of_the_reference_tests(cuda):
    """tests/cluster/test_metrics.py:45-122 and the docstring of heat/cluster/metrics.py:121-126."""
    def arr(t):
        return ht.array(t.to(cuda), split=0)

    x = torch.tensor([[0.0, 0.0], [10.0, 10.0], [20.0, 20.0], [1.0, 1.0]])
    sil = ht.cluster.silhouette_samples(arr(x), arr(torch.tensor([0, 2, 1, 0], dtype=torch.int32)))
    assert float(sil.larray[0]) == pytest.approx(0.9, abs=1e-6)
    lab = torch.tensor([0, 0, 1, 1])
    # int64 rows are float64 rows in the reference (the docstring example of heat/cluster/metrics.py:121-126)
    s64 = ht.cluster.silhouette_samples(arr(torch.tensor([[1, 2], [1, 1], [4, 4], [4, 5]])), arr(lab))
    assert s64.dtype is ht.float64 and s64.larray.tolist() == pytest.approx([0.7452, 0.7836, 0.7452, 0.7836], abs=5e-5)
    x = torch.tensor([[1.0, 2.0], [1.0, 1.0], [4.0, 4.0], [4.0, 5.0]])
    assert ht.cluster.silhouette_samples(arr(x), arr(lab)).larray.tolist() == pytest.approx(
        [0.7452, 0.7836, 0.7452, 0.7836], abs=5e-5)
    score = ht.cluster.silhouette_score(arr(x), arr(lab))
    assert isinstance(score, float) and score == pytest.approx(0.76439, rel=1e-5)  # numpy.allclose default of the reference test
    n = 16
    g = torch.Generator().manual_seed(4)
    data = torch.rand((n, 3), generator=g)
    assert ht.cluster.silhouette_score(arr(data), arr(torch.arange(n))) == 0.0
    assert ht.cluster.silhouette_score(arr(data), arr(torch.zeros(n, dtype=torch.int64))) == 0.0
    data = torch.zeros((n, 3))
    data[n // 2:, 0] = 1.0
    lab = torch.zeros(n, dtype=torch.int64)
    lab[n // 2:] = 2
    assert ht.cluster.silhouette_score(arr(data), arr(lab)) == pytest.approx(1.0)
    assert ht.cluster.silhouette_score(arr(data), arr(lab.view(-1, 1))) == pytest.approx(1.0)   # column vector
    worst = (n / 4) / (n / 2) / ((n / 4) / (n / 2 - 1)) - 1
    got = ht.cluster.silhouette_score(arr(data), arr(torch.arange(n) % 2))
    assert got == pytest.approx(worst) and got < 0
    # random subset: the score of the same subset taken by hand
    data = torch.rand((64, 3), generator=g)
    lab = torch.randint(0, 4, (64,), generator=g)
    s1 = ht.cluster.silhouette_score(arr(data), arr(lab), sample_size=32, random_state=7)
    s2 = ht.cluster.silhouette_score(arr(data), arr(lab), sample_size=32, random_state=7)
    pick = torch.randperm(64, generator=torch.Generator().manual_seed(7))[:32]
    assert s1 == s2 == pytest.approx(orc.silhouette_score(data[pick], lab[pick]), abs=1e-4)
    # input validation (tests/cluster/test_metrics.py:158-177)
    with pytest.raises(ValueError):
        ht.cluster.silhouette_samples(arr(data), arr(lab[:10]))
    with pytest.raises(ValueError):
        ht.cluster.silhouette_samples(arr(data), arr(lab), metric="precomputed")
    with pytest.raises(NotImplementedError):
        ht.cluster.silhouette_samples(arr(data), arr(lab), metric="manhattan")
    with pytest.raises(TypeError):
        ht.cluster.silhouette_samples(data, arr(lab))
