"""
Seeded sweep over random shapes: the entry points of the library against float64 evaluations on the
GPU, at sizes on both sides of every tile, chunk and dispatch boundary (1, 63, 64, 65, ... rows; feature
counts around 8, 16, 32, 64, 128; centroid counts around 8, 32, 256, 1024), with padded row strides,
duplicated centroids (exact ties take the first index) and spreads from 0.01 to 100.

Bars: a label may differ from the float64 argmin only where the two squared distances differ by less
than 1e-5 relative plus the fp32 resolution of the expansion; means within 1e-6 of the float64 means
of the returned labels; the step equals assignment + update; full matrices within 4e-6 of the squared
scale (quadratic expansion) or 1e-5 relative (direct forms); medians bit-exact; float64 to 1e-12.
"""
import random

import pytest
import torch

from heat_amd import _native

pytestmark = pytest.mark.gpu

DS = [1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 17, 20, 24, 31, 32, 33, 40, 48, 63, 64, 65, 100, 128, 130, 200]
KS = [1, 2, 3, 7, 8, 9, 16, 31, 32, 33, 64, 100, 255, 256, 257, 500, 1000, 1025]
NS = [1, 2, 63, 64, 65, 127, 255, 256, 257, 1000, 4095, 4097, 10000, 33333]


def _d2_f64(x, c):
    xd, cd = x.double(), c.double()
    return ((xd * xd).sum(1, keepdim=True) + (cd * cd).sum(1)[None] - 2 * xd @ cd.T).clamp_min(0), xd, cd


@pytest.mark.parametrize("products", ["fp32", "bf16x3"])
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_kmeans_entry_points_on_random_shapes(cuda, seed, products, monkeypatch):
    # bf16x3: the opt-in split-product kernels (read from the environment on every call), same bars
    if products == "bf16x3":
        monkeypatch.setenv("HKM_PRODUCTS", "bf16x3")
    else:
        monkeypatch.delenv("HKM_PRODUCTS", raising=False)
    rng = random.Random(seed)
    ws = _native.Workspace(cuda)
    for case in range(40):
        d, k, n, pad = rng.choice(DS), rng.choice(KS), rng.choice(NS), rng.choice([0, 0, 1, 3, 4])
        spread, noise, dup = rng.choice([0.1, 3.0, 100.0]), rng.choice([0.0, 0.5, 2.0]), rng.choice([0, 0, 1])
        what = f"seed={seed} case={case} n={n} d={d} k={k} pad={pad} spread={spread} noise={noise} dup={dup}"
        print(what, flush=True)
        g = torch.Generator(device=cuda).manual_seed(seed * 100003 + case * 7919 + 13)
        c = torch.randn((k, d), device=cuda, generator=g) * spread
        xw = torch.zeros((n, d + pad), device=cuda)
        x = xw[:, :d] if pad else xw
        x.copy_(c[torch.randint(0, k, (n,), device=cuda, generator=g)]
                + torch.randn((n, d), device=cuda, generator=g) * noise)
        if dup:
            c[k // 2] = c[0]
        lab = torch.full((n,), -7, dtype=torch.int32, device=cuda)
        md = torch.full((n,), -7.0, device=cuda)
        _native.assign(x, c, lab, md, ws)
        d2, xd, _ = _d2_f64(x, c)
        best = d2.min(1).values
        assert int(((lab < 0) | (lab >= k)).sum()) == 0, what
        got = d2.gather(1, lab.long().view(-1, 1)).view(-1)
        scale = (xd * xd).sum(1) + (c.double() ** 2).sum(1).max()
        # accuracy against the exact distances (no reference labels here): the centroid chosen is the
        # nearest up to 1e-5 relative plus two roundings of the fp32 expansion (eps32 = 1.19e-7)
        tol = 1e-5 * best + 2.4e-7 * max(2.0, d ** 0.5 / 4) * scale
        assert int((got - best > tol).sum()) == 0, what
        assert int(((md.double() - best).abs() > tol + 1e-6 * scale).sum()) == 0, what
        if dup and k // 2 != 0:
            assert int((lab == k // 2).sum()) == 0, what + ": the first of two identical centroids wins"
        c_step = torch.empty_like(c)
        lab_step = torch.empty_like(lab)
        shift = torch.empty((), device=cuda)
        sse = torch.empty((), device=cuda)
        _native.lloyd_step(x, c, c_step, lab_step, shift, sse, ws)
        c_upd = torch.empty_like(c)
        cnt = torch.empty((k,), dtype=torch.int64, device=cuda)
        _native.update(x, lab, c_upd, cnt, ws)
        assert torch.equal(lab_step, lab), what
        ref_cnt = torch.bincount(lab.long(), minlength=k)
        assert torch.equal(cnt, ref_cnt), what
        sums = torch.zeros((k, d), dtype=torch.float64, device=cuda).index_add_(0, lab.long(), xd)
        ref = (sums / ref_cnt.clamp_min(1).view(-1, 1)).float()
        den = float(ref.abs().max()) + 1e-30
        assert float((c_upd - ref).abs().max()) / den <= 1e-6, what
        assert float((c_step - ref).abs().max()) / den <= 1e-6, what
        ref_shift = float(((c.double() - c_step.double()) ** 2).sum())
        assert abs(float(shift) - ref_shift) <= 1e-4 * ref_shift + 1e-6 * float((c.double() ** 2).sum(1).mean()), what
        ref_sse = float(got.sum())
        assert abs(float(sse) - ref_sse) <= 1e-4 * ref_sse + 1e-5 * float(scale.sum()), what


@pytest.mark.parametrize("seed", [1, 2])
def test_matrices_manhattan_and_float64_on_random_shapes(cuda, seed):
    rng = random.Random(seed)
    ws = _native.Workspace(cuda)
    for case in range(40):
        d = rng.choice([1, 2, 3, 4, 5, 8, 9, 15, 16, 17, 31, 32, 33, 48, 64, 65, 100, 130])
        m = rng.choice([1, 2, 63, 64, 65, 127, 128, 129, 300, 1000])
        n = rng.choice([1, 2, 63, 64, 65, 127, 128, 129, 257, 700])
        k = rng.choice([1, 2, 7, 8, 16, 33, 64, 100, 256, 300])
        rows = rng.choice([1, 5, 64, 257, 3000, 20001])
        mag = rng.choice([0.01, 1.0, 30.0])
        what = f"seed={seed} case={case} m={m} n={n} d={d} mag={mag} | rows={rows} k={k}"
        print(what, flush=True)
        g = torch.Generator(device=cuda).manual_seed(seed * 100003 + case * 31 + 7)
        x = torch.randn((m, d), device=cuda, generator=g) * mag
        y = torch.randn((n, d), device=cuda, generator=g)
        if m > 2 and n > 2:
            y[1] = x[2]
        xd, yd = x.double(), y.double()
        scale = float((xd * xd).sum(1).max() + (yd * yd).sum(1).max())
        for metric, p in ((_native.METRIC_EUCLID_QE, 2.0), (_native.METRIC_EUCLID, 2.0), (_native.METRIC_MANHATTAN, 1.0)):
            out = torch.full((m, n + 3), -7.0, device=cuda)[:, :n]
            _native.pairwise(x, y, out, metric)
            ref = torch.cdist(xd, yd, p=p, compute_mode="donot_use_mm_for_euclid_dist")
            if metric == _native.METRIC_EUCLID_QE:
                assert float((out.double() ** 2 - ref ** 2).abs().max()) <= 4e-6 * scale, what
            else:
                assert float((out.double() - ref).abs().max()) <= 1e-5 * float(ref.abs().max()) + 1e-30, what
            assert bool((out._base[:, n:] == -7.0).all()), what + ": stores beyond the last column"
            assert not bool((out < 0).any()), what
        sig = 1.7
        ref = torch.exp(-torch.cdist(xd, yd, compute_mode="donot_use_mm_for_euclid_dist") ** 2 / (2 * sig * sig))
        out = torch.empty((m, n), device=cuda)
        _native.pairwise(x, y, out, _native.METRIC_GAUSS, sig)
        assert float((out.double() - ref).abs().max()) <= 2e-5, what
        _native.pairwise(x, y, out, _native.METRIC_GAUSS_QE, sig)
        assert float((out.double() - ref).abs().max()) <= 2e-5 + 4e-6 * scale / (2 * sig * sig), what
        # Manhattan assignment, lower median, float64 assignment
        c = torch.randn((k, d), device=cuda, generator=g) * 3
        xs = c[torch.randint(0, k, (rows,), device=cuda, generator=g)] + torch.randn((rows, d), device=cuda, generator=g)
        lab = torch.full((rows,), -7, dtype=torch.int32, device=cuda)
        md = torch.empty((rows,), device=cuda)
        _native.assign_l1(xs, c, lab, md)
        d1 = torch.cdist(xs.double(), c.double(), p=1.0)
        best = d1.min(1).values
        assert int(((lab < 0) | (lab >= k)).sum()) == 0, what
        got = d1.gather(1, lab.long().view(-1, 1)).view(-1)
        assert int((got - best > 1e-5 * best + 1e-5).sum()) == 0, what
        med = torch.empty_like(c)
        _native.update_median(xs, lab, med, ws, c_old=c.contiguous(), lower=True)
        for kk in range(min(k, 6)):
            sel = xs[lab == kk]
            want = sel.median(dim=0).values if sel.shape[0] else c[kk]
            assert torch.equal(med[kk], want), what + f" cluster {kk}"
        lab64 = torch.empty((rows,), dtype=torch.int32, device=cuda)
        md64 = torch.empty((rows,), dtype=torch.float64, device=cuda)
        _native.assign(xs.double(), c.double(), lab64, md64, ws)
        d2 = torch.cdist(xs.double(), c.double(), compute_mode="donot_use_mm_for_euclid_dist") ** 2
        b2 = d2.min(1).values
        sc = (xs.double() ** 2).sum(1) + (c.double() ** 2).sum(1).max()
        assert int((d2.gather(1, lab64.long().view(-1, 1)).view(-1) - b2 > 1e-12 * sc).sum()) == 0, what
        assert int(((md64 - b2).abs() > 1e-12 * sc).sum()) == 0, what
