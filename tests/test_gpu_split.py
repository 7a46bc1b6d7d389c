"""
The opt-in split-bf16 product path (environment HKM_PRODUCTS=bf16x3) of the resident matrix-core
kernels, held to the same bars as the default fp32 path: labels by the gap rule against the oracle,
min_d2 within the resolution of the quadratic expansion, the one-sweep step equal to assign + update,
bit-identical repeats -- plus a direct measurement of its accuracy next to the fp32 path's.
"""
import os

import pytest
import torch

from heat_amd import _native
from oracle import heat_oracle as orc

pytestmark = pytest.mark.gpu


@pytest.fixture()
def split_products(monkeypatch):
    monkeypatch.setenv("HKM_PRODUCTS", "bf16x3")
    yield
    monkeypatch.delenv("HKM_PRODUCTS", raising=False)


def _data(n, d, k, seed, spread=3.0):
    g = torch.Generator().manual_seed(seed)
    c = torch.randn((k, d), generator=g) * spread
    x = c[torch.randint(0, k, (n,), generator=g)] + torch.randn((n, d), generator=g)
    return x.contiguous(), c.contiguous()


# resident shapes with 16 < D <= 32: ragged N, K no multiple of 32, D no multiple of 4 (scalar loads)
@pytest.mark.parametrize("n,d,k", [(4096, 32, 256), (1000, 20, 33), (999, 17, 1), (257, 24, 64), (70001, 32, 129),
                                   (5000, 30, 400)])
def test_split_assign_matches_oracle(cuda, split_products, n, d, k):
    x, c = _data(n, d, k, seed=n + d + k)
    xs, cs = x.to(cuda), c.to(cuda)
    lab = torch.full((n,), -7, dtype=torch.int32, device=cuda)
    md = torch.full((n,), -1.0, device=cuda)
    ws = _native.Workspace(cuda)
    _native.assign(xs, cs, lab, md, ws)
    lab2 = torch.empty_like(lab)
    _native.assign(xs, cs, lab2, None, ws)
    assert torch.equal(lab, lab2)
    lab, md = lab.cpu(), md.cpu()
    ref_lab, _ = orc.assign_to_cluster_literal(x, c)
    assert lab.min() >= 0 and lab.max() < k
    rep = orc.label_agreement(x, c, lab, ref_lab)
    assert rep["n_unexcused"] == 0 and rep["agreement"] >= 0.999, rep
    scale = (x.double() ** 2).sum(1) + (c.double() ** 2).sum(1).max()
    d2 = orc.brute_force_d2(x, c).min(dim=1).values
    assert torch.all((md.double() - d2).abs() <= 2e-5 * scale + 1e-6)


# wide rows (D > 64): the 2-D streaming kernel, whose staging threads split the panels; 16 < D <= 64 with
# more centroids than LDS holds: the tiled kernel, whose staging threads split the centroid tiles
@pytest.mark.parametrize("n,d,k", [(1500, 100, 170), (900, 512, 130), (513, 130, 1030), (300, 130, 3),
                                   (2048, 64, 1024), (3000, 64, 300), (700, 33, 500), (1300, 50, 437), (5000, 20, 900)])
def test_split_streaming_and_tiled_assign_match_oracle(cuda, split_products, n, d, k):
    assert _native.assign_kernel_name(n, d, k) in ("mfma_stream", "mfma_tiled")
    x, c = _data(n, d, k, seed=n + d + k)
    xs, cs = x.to(cuda), c.to(cuda)
    ws = _native.Workspace(cuda)
    out = []
    for _ in range(2):
        lab = torch.full((n,), -7, dtype=torch.int32, device=cuda)
        md = torch.full((n,), -1.0, device=cuda)
        _native.assign(xs, cs, lab, md, ws)
        out.append((lab.cpu(), md.cpu()))
    assert torch.equal(out[0][0], out[1][0]) and torch.equal(out[0][1], out[1][1])
    lab, md = out[0]
    ref_lab, _ = orc.assign_to_cluster_literal(x, c)
    assert lab.min() >= 0 and lab.max() < k
    rep = orc.label_agreement(x, c, lab, ref_lab)
    assert rep["n_unexcused"] == 0 and rep["agreement"] >= 0.999, rep
    scale = (x.double() ** 2).sum(1) + (c.double() ** 2).sum(1).max()
    d2 = orc.brute_force_d2(x, c).min(dim=1).values
    assert torch.all((md.double() - d2).abs() <= 2e-5 * scale + 1e-6)


def test_split_products_are_as_accurate_as_fp32_products(cuda, monkeypatch):
    """min_d2 of both paths against fp64 on data with large norms and small distances (the hard case
    for the quadratic expansion): the split path's error must stay within 1.5x the fp32 path's."""
    g = torch.Generator().manual_seed(3)
    k, d, n = 256, 32, 200_000
    c = (torch.rand((k, d), generator=g) - 0.5) * 10
    x = c[torch.randint(0, k, (n,), generator=g)] + 0.5 * torch.randn((n, d), generator=g)
    best = orc.brute_force_d2(x, c).min(dim=1).values
    err = {}
    for mode in ("fp32", "bf16x3"):
        if mode == "bf16x3":
            monkeypatch.setenv("HKM_PRODUCTS", "bf16x3")
        else:
            monkeypatch.delenv("HKM_PRODUCTS", raising=False)
        lab = torch.empty((n,), dtype=torch.int32, device=cuda)
        md = torch.empty((n,), device=cuda)
        _native.assign(x.to(cuda), c.to(cuda), lab, md, _native.Workspace(cuda))
        e = (md.cpu().double() - best).abs()
        err[mode] = (float(e.max()), float(e.mean()))
    monkeypatch.delenv("HKM_PRODUCTS", raising=False)
    print("min_d2 abs error (max, mean):", err, flush=True)
    assert err["bf16x3"][0] <= 1.5 * err["fp32"][0] + 1e-6
    assert err["bf16x3"][1] <= 1.5 * err["fp32"][1] + 1e-7


@pytest.mark.parametrize("n,d,k", [(100003, 32, 256), (50000, 20, 37), (1537, 24, 3), (40000, 30, 100), (768, 17, 5)])
def test_split_one_sweep_step_equals_assign_plus_update(cuda, split_products, n, d, k):
    # (the name does not look at the environment: with split products the matrix-core kernel runs these shapes all)
    assert _native.lloyd_kernel_name(n, d, k) in ("lloyd_mfma_resident", "lloyd_few")
    x, _ = _data(n, d, k, seed=5 * n + d)
    x[::97] = 0.0
    c0 = x[torch.randperm(n, generator=torch.Generator().manual_seed(4))[:k]].contiguous()
    xs, cs = x.to(cuda), c0.to(cuda)
    ws = _native.Workspace(cuda)
    out = []
    for _ in range(2):
        c_step = torch.empty_like(cs)
        lab_step = torch.empty((n,), dtype=torch.int32, device=cuda)
        shift = torch.empty((), device=cuda)
        sse = torch.empty((), device=cuda)
        _native.lloyd_step(xs, cs, c_step, lab_step, shift, sse, ws)
        out.append((c_step.clone(), lab_step.clone(), float(shift), float(sse)))
    assert torch.equal(out[0][0], out[1][0]) and torch.equal(out[0][1], out[1][1]) and out[0][2:] == out[1][2:]
    c_step, lab_step, shift, sse = out[0]
    lab2 = torch.empty_like(lab_step)
    md = torch.empty((n,), device=cuda)
    _native.assign(xs, cs, lab2, md, ws)
    assert torch.equal(lab_step, lab2)
    cnt = torch.bincount(lab2.cpu().long(), minlength=k)
    ref = torch.zeros((k, d), dtype=torch.float64).index_add_(0, lab2.cpu().long(), x.double())
    ref = (ref / cnt.clamp(min=1).double().unsqueeze(1)).float()
    assert orc.rel_err_centers(c_step.cpu(), ref) <= 1e-6
    ref_shift = float(((c0.double() - ref.double()) ** 2).sum())
    assert orc.rel_err_scalar(shift, ref_shift, floor=1e-12) <= 1e-4
    assert orc.rel_err_scalar(sse, float(md.double().sum()), floor=1e-9) <= 1e-5
    ref_lab, _ = orc.assign_to_cluster_literal(x, c0)
    rep = orc.label_agreement(x, c0, lab2.cpu(), ref_lab)
    assert rep["n_unexcused"] == 0 and rep["agreement"] >= 0.999, rep


def test_split_path_is_off_by_default_and_only_covers_its_shapes(cuda, monkeypatch):
    """Without the environment variable nothing changes; with it, shapes outside 16 < D <= 32 keep the
    fp32 kernels (same bits as without)."""
    monkeypatch.delenv("HKM_PRODUCTS", raising=False)
    for n, d, k in ((3000, 64, 100), (2000, 8, 16), (4096, 32, 256)):  # resident D=64, narrow, resident D=32
        x, c = _data(n, d, k, seed=1)
        xs, cs = x.to(cuda), c.to(cuda)
        ws = _native.Workspace(cuda)
        res = []
        for env in (None, "bf16x3", "fp32"):
            if env is None:
                monkeypatch.delenv("HKM_PRODUCTS", raising=False)
            else:
                monkeypatch.setenv("HKM_PRODUCTS", env)
            lab = torch.empty((n,), dtype=torch.int32, device=cuda)
            md = torch.empty((n,), device=cuda)
            _native.assign(xs, cs, lab, md, ws)
            res.append((lab.cpu(), md.cpu()))
        assert torch.equal(res[0][0], res[2][0]) and torch.equal(res[0][1], res[2][1])
        if d != 32:
            assert torch.equal(res[0][1], res[1][1])  # resident shapes wider than 32 and narrow ones have no split variant
    monkeypatch.delenv("HKM_PRODUCTS", raising=False)
