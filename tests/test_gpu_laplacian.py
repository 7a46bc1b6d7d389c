"""
Graph Laplacian (hkm_laplacian_f32, ht.graph.Laplacian) against the oracle's op-for-op restatement of
heat/graph/laplacian.py on the same similarity matrix: every definition x mode x threshold x weighting.
Bar: entries of the adjacency are selected bit-exactly (same comparisons on the same float32 values);
degrees are float64 sums rounded once, so L agrees to 2e-6 relative to its largest entry.
"""
import itertools

import pytest
import torch

import heat_amd as ht
from heat_amd import _native
from oracle import heat_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 2, 7, 256, 257, 1500])
def test_every_variant_against_the_oracle(cuda, n):
    g = torch.Generator().manual_seed(n)
    x = torch.rand((n, 5), generator=g)
    sim = torch.exp(-torch.cdist(x, x) ** 2)
    sim[n // 2] = 0.0                                       # an isolated vertex in the thresholded graphs
    sim[:, n // 2] = 0.0
    variants = itertools.product(("simple", "norm_sym"), ("fully_connected", "eNeighbour"), (True, False),
                                 ("upper", "lower"))
    for definition, mode, weighted, key in variants:
        want = orc.laplacian(sim, definition, mode, weighted, key, 0.6).float()
        pad = torch.zeros((n, n + 3), device=cuda)
        s = pad[:, :n]
        s.copy_(sim)
        out = torch.full((n, n + 1), -7.0, device=cuda)[:, :n]
        degree = torch.empty((n,), device=cuda)
        m = 0 if mode == "fully_connected" else (1 if key == "upper" else 2)
        _native.laplacian(s, out, 0 if definition == "simple" else 1, m, weighted, 0.6, degree)
        tol = 2e-6 * float(want.abs().max()) + 1e-30
        assert float((out.cpu() - want).abs().max()) <= tol, (definition, mode, weighted, key)
        assert torch.equal((out.cpu() == 0), (want == 0)), (definition, mode, weighted, key)
        assert bool((out._base[:, n:] == -7.0).all())
        _native.laplacian(s, s, 0 if definition == "simple" else 1, m, weighted, 0.6, degree)   # in place
        assert torch.equal(s, out)


def test_reference_style_checks(cuda):
    """tests/graph/test_laplacian.py:10-80: types, shapes, the exception matrix; plus values against the oracle."""
    x = torch.ones((6, 4))
    x[0] *= 0.0
    x[1] *= 0.5
    X = ht.array(x.to(cuda), split=0)
    for kwargs in ({}, {"weighted": False}, {"definition": "simple"}, {"mode": "eNeighbour"},
                   {"mode": "eNeighbour", "threshold_key": "lower", "threshold_value": 3.0}):
        for sim_fn, sim_t in ((lambda a: ht.spatial.cdist(a, quadratic_expansion=True), None),
                              (lambda a: ht.spatial.rbf(a, sigma=1.0, quadratic_expansion=True), None)):
            res = ht.graph.Laplacian(sim_fn, **kwargs).construct(X)
            assert isinstance(res, ht.DNDarray) and res.shape == (6, 6) and res.split == 0
            sim = sim_fn(X).larray.cpu()
            want = orc.laplacian(sim, kwargs.get("definition", "norm_sym"), kwargs.get("mode", "fully_connected"),
                                 kwargs.get("weighted", True), kwargs.get("threshold_key", "upper"),
                                 kwargs.get("threshold_value", 1.0)).float()
            assert torch.allclose(res.larray.cpu(), want, rtol=0, atol=2e-6 * float(want.abs().max()) + 1e-30)
    with pytest.raises(ValueError):
        ht.graph.Laplacian(lambda a: ht.spatial.cdist(a), threshold_key="both")
    with pytest.raises(NotImplementedError):
        ht.graph.Laplacian(lambda a: ht.spatial.cdist(a), mode="kNN")
    with pytest.raises(NotImplementedError):
        ht.graph.Laplacian(lambda a: ht.spatial.cdist(a), definition="norm_rw")
