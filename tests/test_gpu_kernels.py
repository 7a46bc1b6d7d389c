"""
GPU parity of the C-ABI entry points against the CPU oracle, kernel by kernel.
Every call goes through libhkm via ctypes (heat_amd._native).

Tolerances (fp32 path): labels must agree except where the fp64 best/second-best squared distances
are within 1e-5 relative; min_d2 within 2e-5 * (|x|^2 + |c|^2) absolute (cancellation in the quadratic
expansion); centroids within 1e-5 relative to max|C|; counts exact; two runs bit-identical.
"""
import numpy as np
import pytest
import torch

from heat_amd import _native
from oracle import heat_oracle as orc

pytestmark = pytest.mark.gpu

# (N, D, K): covers the VALU kernel (D <= 16), the LDS-resident MFMA kernel and the streaming MFMA
# kernel, with ragged sizes, K not a multiple of 32, D not a multiple of 4 (scalar-load path)
ASSIGN_SHAPES = [
    (1, 3, 8), (1000, 3, 8), (5000, 8, 16), (777, 16, 40), (300, 1, 5), (2000, 5, 700),
    (4096, 32, 256), (1000, 20, 33), (999, 17, 1), (3000, 64, 100), (1300, 50, 37), (257, 24, 64),
    (2048, 64, 1024), (1500, 100, 70), (900, 512, 130), (700, 33, 500), (513, 130, 1030),
    # 65 to 128 features with the centroids resident in LDS (beyond, or with more centroids: the streaming kernel)
    (3000, 128, 8), (1111, 65, 3), (2000, 96, 32), (1500, 97, 40), (900, 128, 96), (900, 128, 97), (800, 127, 1),
    (3000, 16, 1100), (2500, 8, 1500), (1800, 6, 2000), (4000, 4, 33), (3000, 13, 32),
    # 9 to 16 features with few centroids: the narrow kernel
    (3001, 16, 8), (2000, 9, 24), (4003, 12, 5), (1000, 15, 15), (2500, 10, 1), (3000, 14, 16), (2222, 11, 20), (1999, 13, 3),
]


def _data(n, d, k, seed, spread=3.0):
    g = torch.Generator().manual_seed(seed)
    c = torch.randn((k, d), generator=g) * spread
    lab = torch.randint(0, k, (n,), generator=g)
    x = c[lab] + torch.randn((n, d), generator=g)
    return x.contiguous(), c.contiguous()


def _assign_gpu(x, c, dev, want_min=True):
    xs, cs = x.to(dev), c.to(dev)
    lab = torch.full((x.shape[0],), -7, dtype=torch.int32, device=dev)
    md = torch.full((x.shape[0],), -1.0, dtype=torch.float32, device=dev) if want_min else None
    _native.assign(xs, cs, lab, md, _native.Workspace(dev))
    torch.cuda.synchronize()
    return lab.cpu(), (md.cpu() if want_min else None)


@pytest.mark.parametrize("n,d,k", [(1, 3, 8), (1001, 3, 8), (5000, 8, 16), (4003, 12, 5), (300, 1, 5), (2222, 11, 20),
                                   (70000, 2, 64), (3001, 16, 8), (999, 5, 31)])
def test_narrow_assign_stores_int64_labels_itself(cuda, n, d, k):
    """hkm_assign_labels64_f32: the labels of hkm_assign_f32, stored as int64 by the kernel itself (no second pass
    that widens them), on rows with and without padding; shapes of other kernels are refused."""
    assert _native.assign_kernel_name(n, d, k) == "valu_fused"
    x, c = _data(n, d, k, seed=n + d)
    xs, cs = x.to(cuda), c.to(cuda)
    pad = torch.zeros((n, d + 3), device=cuda)
    pad[:, :d] = xs
    for rows in (xs, pad[:, :d]):
        lab = torch.empty((n,), dtype=torch.int32, device=cuda)
        md = torch.empty((n,), device=cuda)
        _native.assign(rows, cs, lab, md, _native.Workspace(cuda))
        lab64 = torch.full((n,), -5, dtype=torch.int64, device=cuda)
        md64 = torch.full((n,), -1.0, device=cuda)
        _native.assign_labels64(rows, cs, lab64, md64)
        torch.cuda.synchronize()
        assert torch.equal(lab64, lab.long()) and torch.equal(md64, md)
        only = torch.full((n,), -5, dtype=torch.int64, device=cuda)
        _native.assign_labels64(rows, cs, only, None)
        assert torch.equal(only, lab.long())
    with pytest.raises(_native.HkmError) as e:
        _native.assign_labels64(torch.zeros((10, 32), device=cuda), torch.zeros((4, 32), device=cuda),
                                torch.zeros((10,), dtype=torch.int64, device=cuda), None)
    assert e.value.code == _native.HKM_EUNSUPPORTED


@pytest.mark.parametrize("n,d,k", ASSIGN_SHAPES)
def test_assign_matches_oracle(cuda, n, d, k):
    print(f"assign n={n} d={d} k={k} kernel={_native.assign_kernel_name(n, d, k)}", flush=True)
    x, c = _data(n, d, k, seed=n + d + k)
    lab, md = _assign_gpu(x, c, cuda)
    ref_lab, _ = orc.assign_to_cluster_literal(x, c)
    assert lab.min() >= 0 and lab.max() < k
    rep = orc.label_agreement(x, c, lab, ref_lab)
    assert rep["n_unexcused"] == 0, rep
    assert rep["agreement"] >= 0.999, rep
    ref_q = orc.quadratic_expand(x, c).gather(1, lab.view(-1, 1).long()).view(-1)
    scale = (x.double() ** 2).sum(1) + (c.double() ** 2).sum(1).max()
    assert torch.all((md.double() - ref_q.double()).abs() <= 2e-5 * scale + 1e-6)
    # against the mathematical definition too
    d2 = orc.brute_force_d2(x, c).min(dim=1).values
    assert torch.all((md.double() - d2).abs() <= 2e-5 * scale + 1e-6)


def test_assign_ties_take_first_index(cuda):
    # Duplicated centroids give bit-identical distances in the kernels (same instruction sequence for
    # every centroid), i.e. exact ties; torch.min's rule -- the first index wins -- must then hold.
    # The CPU sgemm does NOT always produce exact ties for duplicated columns (it blocks columns), so
    # the oracle is compared modulo the duplication.
    g = torch.Generator().manual_seed(5)
    for d in (3, 32, 80):
        base = torch.randn((6, d), generator=g)
        c = torch.cat([base, base, base])  # k = 18, centroid j == j+6 == j+12
        x = base[torch.randint(0, 6, (500,), generator=g)] + 0.01 * torch.randn((500, d), generator=g)
        lab, _ = _assign_gpu(x, c, cuda)
        ref, _ = orc.assign_to_cluster_literal(x, c)
        assert int(lab.max()) < 6, d
        assert bool((lab.long() == ref.view(-1) % 6).all()), d


def test_assign_point_equals_centroid_clamps_at_zero(cuda):
    # x_i == c_k: the expansion may go slightly negative and must be clamped to exactly 0
    g = torch.Generator().manual_seed(6)
    for d in (8, 32, 128):
        c = torch.randn((40, d), generator=g) * 50
        x = c[torch.arange(40).repeat(10)].contiguous()
        lab, md = _assign_gpu(x, c, cuda)
        assert torch.equal(lab.long(), torch.arange(40).repeat(10))
        assert md.min() >= 0.0
        assert md.max() <= 2e-6 * float((c.double() ** 2).sum(1).max())


@pytest.mark.parametrize("d,k", [(8, 16), (8, 14), (8, 12), (4, 16), (4, 14)])
def test_narrow_matrix_core_scan_keeps_the_reference_rules(cuda, d, k):
    # 12 to 16 centroids of 4 or 8 coordinates: the narrow kernels take the cross terms from the matrix cores
    # (16 points x 16 centroids per instruction) and find the minimum in registers after a transpose across
    # lanes.  Same rules as everywhere: first index on exact ties, clamp at 0, rows of NaN go to cluster 0.
    g = torch.Generator().manual_seed(40 + d + k)
    n = 3001
    base = torch.randn((k // 2, d), generator=g) * 3
    c = torch.cat([base, base])  # centroid j == j + k/2: exact ties
    x = base[torch.randint(0, k // 2, (n,), generator=g)] + 0.05 * torch.randn((n, d), generator=g)
    x[7] = c[3]            # on a centroid: the expansion may come out below zero
    x[11] = float("nan")
    lab, md = _assign_gpu(x, c, cuda)
    ref, _ = orc.assign_to_cluster_literal(torch.nan_to_num(x, nan=0.0), c)
    ok = torch.ones(n, dtype=torch.bool)
    ok[11] = False
    assert int(lab.max()) < k // 2
    assert bool((lab.long()[ok] == (ref.view(-1) % (k // 2))[ok]).all())
    assert int(lab[11]) == 0
    assert 0.0 <= float(md[7]) <= 2e-6 * float((c[3].double() ** 2).sum()) and float(md[ok].min()) >= 0.0
    # distinct centroids, a leading dimension, an unaligned base, a ragged end: against the oracle, and the
    # step's labels equal to the assignment's
    cw = torch.randn((k, d + 3), generator=g) * 3
    xw = cw[torch.randint(0, k, (n,), generator=g), 2:2 + d] + torch.randn((n, d), generator=g)
    xbuf = torch.zeros((n, d + 5))
    xbuf[:, 1:1 + d] = xw
    xs, cs = xbuf.to(cuda)[:, 1:1 + d], cw.to(cuda)[:, 2:2 + d]
    lab2 = torch.empty((n,), dtype=torch.int32, device=cuda)
    _native.assign(xs, cs, lab2, None, _native.Workspace(cuda))
    ref2, _ = orc.assign_to_cluster_literal(xw.contiguous(), cw[:, 2:2 + d].contiguous())
    rep = orc.label_agreement(xw, cw[:, 2:2 + d], lab2.cpu(), ref2)
    assert rep["n_unexcused"] == 0 and rep["n_strict"] == 0, rep
    c_new = torch.empty((k, d), device=cuda)
    lab3 = torch.empty_like(lab2)
    _native.lloyd_step(xs, cs.contiguous(), c_new, lab3, torch.empty((), device=cuda), None, _native.Workspace(cuda))
    torch.cuda.synchronize()
    assert torch.equal(lab3, lab2)


@pytest.mark.parametrize("d,k", [(2, 64), (2, 13), (3, 40), (3, 57), (2, 80), (3, 14), (1, 100), (1, 30), (1, 13)])
def test_narrow_scan_four_at_a_time_keeps_the_reference_rules(cuda, d, k, monkeypatch):
    # Up to 3 coordinates, a dozen centroids or more: the narrow kernels take the centroids four at a time, keep
    # the block in which the minimum fell and look the position up at the end.  Against the scan one centroid
    # at a time (forced through the environment) on duplicated centroids -- exact ties, the first index must
    # win --, a row on a centroid, NaN and inf rows, K not a multiple of four: same labels, same distances,
    # same step; and against the oracle.
    print(f"narrow blocked scan d={d} k={k}", flush=True)
    assert _native.lloyd_kernel_name(3001, d, k) == "lloyd_small"
    g = torch.Generator().manual_seed(90 + d + k)
    n = 3001
    half = (k + 1) // 2
    base = torch.randn((half, d), generator=g) * 3
    c = torch.cat([base, base])[:k].contiguous()  # centroid j == j + half: exact ties
    x = base[torch.randint(0, half, (n,), generator=g)] + 0.05 * torch.randn((n, d), generator=g)
    x[7] = c[3]
    x[11] = float("nan")
    x[13] = float("inf")
    x[17, 0] = 3e38  # the squared norm and the cross terms overflow
    res = {}
    for name, thr in (("one", "100000"), ("four", "2")):
        monkeypatch.setenv("HKM_SMALL_BLOCKED_MIN_K", thr)
        lab, md = _assign_gpu(x, c, cuda)
        c_new = torch.empty((k, d), device=cuda)
        lab_s = torch.empty((n,), dtype=torch.int32, device=cuda)
        shift = torch.empty((), device=cuda)
        _native.lloyd_step(x.to(cuda), c.to(cuda), c_new, lab_s, shift, None, _native.Workspace(cuda))
        torch.cuda.synchronize()
        res[name] = (lab, md, lab_s.cpu(), c_new.cpu(), shift.cpu())
    one, four = res["one"], res["four"]
    assert torch.equal(one[0], four[0]) and torch.equal(one[2], four[2]) and torch.equal(four[0], four[2])
    assert torch.equal(torch.nan_to_num(one[1], nan=-1.0), torch.nan_to_num(four[1], nan=-1.0))
    assert torch.equal(torch.nan_to_num(one[3], nan=-1.0), torch.nan_to_num(four[3], nan=-1.0))
    lab = four[0]
    bad = torch.zeros(n, dtype=torch.bool)
    bad[[11, 13, 17]] = True
    assert int(lab[~bad].max()) < half and int(lab[11]) == 0
    ref, _ = orc.assign_to_cluster_literal(x[~bad].contiguous(), c)
    assert bool((lab.long()[~bad] == ref.view(-1) % half).all())
    assert 0.0 <= float(four[1][7]) <= 2e-6 * float((c[3].double() ** 2).sum())


def test_assign_strided_rows(cuda):
    # X and C as column slices of wider buffers: ld > D, base pointers not 16-byte aligned
    g = torch.Generator().manual_seed(7)
    for d, k in ((3, 8), (32, 64), (96, 200), (32, 8), (44, 5)):
        xw = torch.randn((1200, d + 5), generator=g)
        cw = torch.randn((k, d + 3), generator=g)
        xs, cs = xw.to(cuda)[:, 1 : 1 + d], cw.to(cuda)[:, 2 : 2 + d]
        lab = torch.empty((1200,), dtype=torch.int32, device=cuda)
        _native.assign(xs, cs, lab, None, _native.Workspace(cuda))
        ref, _ = orc.assign_to_cluster_literal(xw[:, 1 : 1 + d].contiguous(), cw[:, 2 : 2 + d].contiguous())
        rep = orc.label_agreement(xw[:, 1 : 1 + d], cw[:, 2 : 2 + d], lab.cpu(), ref)
        assert rep["n_unexcused"] == 0, (d, k, rep)


UPDATE_SHAPES = [(1000, 3, 8), (5000, 8, 16), (4096, 32, 256), (3000, 64, 100), (70000, 20, 33),
                 (900, 512, 130), (2500, 130, 1030), (100000, 32, 7),
                 # wide rows (D >= 128, D % 4 == 0): 128-column slices, several cluster ranges
                 (30000, 128, 50), (20000, 132, 500), (6000, 512, 1024), (777, 256, 3)]


@pytest.mark.parametrize("path", ["sorted", "lists"])
@pytest.mark.parametrize("n,d,k", UPDATE_SHAPES + [(20000, 5, 5000)])
def test_update_matches_oracle(cuda, n, d, k, path, monkeypatch):
    # two implementations of hkm_update_f32: stable sort + segmented sums (default up to K = 4096) and
    # the list-based kernels (larger K, and the fallback of the one-sweep MFMA step)
    print(f"update n={n} d={d} k={k} path={path}", flush=True)
    if path == "lists":
        monkeypatch.setenv("HKM_UPDATE_LISTS", "1")
    g = torch.Generator().manual_seed(n + k)
    x = torch.randn((n, d), generator=g) * 4 + 1
    lab = torch.randint(0, k, (n,), generator=g)
    lab[lab == k // 2] = 0  # force an empty cluster (k >= 2)
    c_new = torch.full((k, d), 123.0, device=cuda)
    cnt = torch.full((k,), -1, dtype=torch.int64, device=cuda)
    _native.update(x.to(cuda), lab.to(torch.int32).to(cuda), c_new, cnt, _native.Workspace(cuda))
    torch.cuda.synchronize()
    again = torch.empty_like(c_new)
    _native.update(x.to(cuda), lab.to(torch.int32).to(cuda), again, None, _native.Workspace(cuda))
    assert torch.equal(again, c_new), "two runs must be bit-identical"
    ref, ref_cnt = orc.update_centroids_fast(x, lab.view(-1, 1), k)
    assert torch.equal(cnt.cpu(), ref_cnt)
    assert int(cnt.sum()) == n
    assert orc.rel_err_centers(c_new.cpu(), ref) <= 1e-5
    if k >= 2:
        assert torch.all(c_new[k // 2] == 0)
    if n * k <= 2_000_000:
        lit = orc.update_centroids_literal(x, lab.view(-1, 1), torch.zeros((k, d)))
        assert orc.rel_err_centers(c_new.cpu(), lit) <= 1e-5


def test_update_ignores_out_of_range_labels(cuda):
    x = torch.arange(40, dtype=torch.float32).view(10, 4)
    lab = torch.tensor([0, 1, -1, 5, 1, 0, 99, 1, 0, 1], dtype=torch.int32)
    c_new = torch.empty((2, 4), device=cuda)
    cnt = torch.empty((2,), dtype=torch.int64, device=cuda)
    _native.update(x.to(cuda), lab.to(cuda), c_new, cnt, _native.Workspace(cuda))
    assert cnt.tolist() == [3, 4]
    assert torch.allclose(c_new.cpu()[0], x[[0, 5, 8]].mean(0))
    assert torch.allclose(c_new.cpu()[1], x[[1, 4, 7, 9]].mean(0))


@pytest.mark.parametrize("n,d,k", [(20000, 3, 8), (20000, 8, 16), (30000, 32, 256), (5000, 64, 1024), (4000, 512, 96),
                                   (20000, 16, 8), (15000, 12, 10), (10000, 9, 20), (12000, 15, 4)])
def test_lloyd_step_matches_oracle_and_is_deterministic(cuda, n, d, k):
    print(f"lloyd n={n} d={d} k={k}", flush=True)
    x, _ = _data(n, d, k, seed=11 * n + k)
    c0 = x[torch.randperm(n, generator=torch.Generator().manual_seed(3))[:k]].contiguous()
    xs, cs = x.to(cuda), c0.to(cuda)
    outs = []
    for _ in range(2):
        c_new = torch.empty_like(cs)
        lab = torch.empty((n,), dtype=torch.int32, device=cuda)
        shift = torch.empty((), device=cuda)
        sse = torch.empty((), device=cuda)
        _native.lloyd_step(xs, cs, c_new, lab, shift, sse, _native.Workspace(cuda))
        torch.cuda.synchronize()
        outs.append((c_new.cpu(), lab.cpu(), shift.cpu(), sse.cpu()))
    for a, b in zip(outs[0], outs[1]):
        assert torch.equal(a, b), "two runs must be bit-identical"
    c_new, lab, shift, sse = outs[0]
    ref_lab, _ = orc.assign_to_cluster_literal(x, c0)
    rep = orc.label_agreement(x, c0, lab, ref_lab)
    assert rep["n_unexcused"] == 0 and rep["agreement"] >= 0.9999, rep
    ref_c, _ = orc.update_centroids_fast(x, lab.view(-1, 1).long(), k)  # same labels -> isolates the update
    assert orc.rel_err_centers(c_new, ref_c) <= 1e-5
    ref_shift = orc.centroid_shift(c0, c_new)
    assert orc.rel_err_scalar(float(shift), float(ref_shift), floor=1e-12) <= 1e-5
    ref_sse = orc.sse(x, c0, lab.long())
    assert orc.rel_err_scalar(float(sse), ref_sse) <= 1e-4


def _step_and_two_pass(xs, cs, dev, lists=False):
    """One hkm_lloyd_step_f32 and, from the same inputs, hkm_assign_f32 + hkm_update_f32 (``lists``:
    with the list-based update kernels, which are also what the one-sweep step falls back to)."""
    import os

    if lists:
        os.environ["HKM_UPDATE_LISTS"] = "1"
    try:
        return _step_and_two_pass_impl(xs, cs, dev)
    finally:
        os.environ.pop("HKM_UPDATE_LISTS", None)


def _step_and_two_pass_impl(xs, cs, dev):
    n, k = xs.shape[0], cs.shape[0]
    ws = _native.Workspace(dev)
    c_step = torch.empty_like(cs)
    lab_step = torch.empty((n,), dtype=torch.int32, device=dev)
    shift = torch.empty((), device=dev)
    _native.lloyd_step(xs, cs, c_step, lab_step, shift, None, ws)
    lab2 = torch.empty_like(lab_step)
    _native.assign(xs, cs, lab2, None, ws)
    c2 = torch.empty_like(cs)
    cnt2 = torch.empty((k,), dtype=torch.int64, device=dev)
    _native.update(xs, lab2, c2, cnt2, ws)
    torch.cuda.synchronize()
    return c_step, lab_step, shift, c2, lab2, cnt2


# shapes of the one-sweep MFMA step (up to 128 features, centroids + fp64 accumulators fit in LDS):
# ragged N, K not a multiple of 32, D not a multiple of 4 (scalar loads), every padded width
@pytest.mark.parametrize("n,d,k", [(100003, 32, 256), (50000, 20, 37), (1537, 24, 3), (40000, 30, 100),
                                   (70001, 40, 129), (30000, 64, 128), (768, 17, 5), (100, 48, 7),
                                   (50000, 16, 64), (40000, 8, 40), (30001, 12, 100), (20000, 5, 60), (9000, 4, 256),
                                   (40000, 128, 8), (30001, 100, 16), (20000, 96, 32), (10000, 65, 3), (25000, 128, 90),
                                   (5000, 77, 1),
                                   (30000, 64, 16), (20000, 48, 13),
                                   # few clusters of 17 to 64 features: the vector kernel with the same sums, in each
                                   # of its launch geometries (workgroups of 256, 512, 1024 lanes; 32 or fewer copies
                                   # of the accumulators), rows that are no whole 16-byte groups
                                   (60001, 32, 8), (30000, 64, 12), (20001, 21, 2), (7000, 63, 11), (4000, 36, 16),
                                   (1000, 64, 1), (300000, 20, 3), (50000, 40, 9), (40000, 48, 12), (25000, 28, 16),
                                   (33333, 52, 11), (9000, 17, 16)])
def test_one_sweep_mfma_step_equals_assign_plus_update(cuda, n, d, k):
    few = 16 < d <= 64 and k <= (16 if d <= 40 else 12)
    assert _native.lloyd_kernel_name(n, d, k) == ("lloyd_few" if few else "lloyd_mfma_resident")
    print(f"one-sweep n={n} d={d} k={k}", flush=True)
    x, _ = _data(n, d, k, seed=5 * n + d)
    x[::97] = 0.0  # all-zero rows only count
    c0 = x[torch.randperm(n, generator=torch.Generator().manual_seed(4))[:k]].contiguous()
    xs, cs = x.to(cuda), c0.to(cuda)
    c_step, lab_step, shift, c2, lab2, cnt2 = _step_and_two_pass(xs, cs, cuda)
    assert torch.equal(lab_step, lab2)
    assert orc.rel_err_centers(c_step.cpu(), c2.cpu()) <= 1e-6
    # the fp64 sums of the one-sweep step are exact up to 2^-29 per row: compare with fp64 directly
    ref = torch.zeros((k, d), dtype=torch.float64).index_add_(0, lab2.cpu().long(), x.double())
    ref = (ref / cnt2.cpu().clamp(min=1).double().unsqueeze(1)).float()
    assert (c_step.cpu() - ref).abs().max() <= 2e-7 * float(x.abs().max())
    again = _step_and_two_pass(xs, cs, cuda)
    assert torch.equal(again[0], c_step) and torch.equal(again[2], shift)


@pytest.mark.parametrize("n,d,k", [(100003, 32, 256), (50000, 20, 37), (1537, 24, 3), (768, 17, 5), (50000, 16, 64),
                                   (40000, 8, 40), (30000, 13, 7)])
def test_one_point_block_per_wave_gives_the_same_labels(cuda, n, d, k, monkeypatch):
    # HKM_POINT_BLOCKS=1 (16 < D <= 32): another launch geometry of the same kernels
    print(f"point blocks n={n} d={d} k={k}", flush=True)
    x, _ = _data(n, d, k, seed=3 * n + d)
    c0 = x[torch.randperm(n, generator=torch.Generator().manual_seed(9))[:k]].contiguous()
    xs, cs = x.to(cuda), c0.to(cuda)
    ws = _native.Workspace(cuda)

    def run():
        lab = torch.empty((n,), dtype=torch.int32, device=cuda)
        md = torch.empty((n,), device=cuda)
        _native.assign(xs, cs, lab, md, ws)
        cn = torch.empty_like(cs)
        lab2 = torch.empty_like(lab)
        shift = torch.empty((), device=cuda)
        _native.lloyd_step(xs, cs, cn, lab2, shift, None, ws)
        torch.cuda.synchronize()
        return lab.cpu(), md.cpu(), lab2.cpu(), cn.cpu(), float(shift)

    two = run()
    monkeypatch.setenv("HKM_POINT_BLOCKS", "1")
    one = run()
    # both geometries cut the rows into the same tiles for the same workgroups: every output bit for bit
    assert torch.equal(one[0], two[0]) and torch.equal(one[1], two[1]) and torch.equal(one[2], two[2])
    assert torch.equal(one[3], two[3]) and one[4] == two[4]


def test_geometry_trial_runs_on_the_callers_own_steps(cuda, monkeypatch):
    """The choice between the two launch geometries of the resident matrix-core kernels is made on the steps a
    large fit issues anyway: no extra launch, no wait, the same bits whichever geometry a step ran in, and a
    verdict for the device once three windows of consecutive steps have been timed."""
    from heat_amd.cluster._lloyd import LloydLoop
    from heat_amd.utils import benchhooks

    monkeypatch.delenv("HKM_POINT_BLOCKS", raising=False)
    n, d, k = 1 << 20, 16, 32
    assert _native.lloyd_kernel_name(n, d, k) == "lloyd_mfma_resident"
    x, _ = _data(n, d, k, seed=77)
    c0 = x[torch.randperm(n, generator=torch.Generator().manual_seed(2))[:k]].contiguous()
    xs, cs = x.to(cuda), c0.to(cuda)
    # what a run pinned to one geometry gives
    monkeypatch.setenv("HKM_POINT_BLOCKS", "2")
    pinned = LloydLoop(xs, cs, _native.Workspace(cuda))
    assert pinned.run(12, None) == 12
    want_c, want_lab = pinned.centers.clone(), pinned.labels.clone()
    assert benchhooks.point_blocks(d) == (2, False)
    monkeypatch.setenv("HKM_POINT_BLOCKS", "1")
    assert benchhooks.point_blocks(d) == (1, False)
    monkeypatch.delenv("HKM_POINT_BLOCKS")
    # steps in a row, as a fit issues them: the windows fill, then a later call finds the verdict
    verdict = benchhooks.point_blocks_trial()[0]
    loop = LloydLoop(xs, cs, _native.Workspace(cuda))
    assert loop.run(12, None) == 12
    assert torch.equal(loop.centers, want_c) and torch.equal(loop.labels, want_lab)
    for _ in range(40):
        if verdict:
            break
        assert loop.run(100, None) == 100
        torch.cuda.synchronize()
        assert loop.run(1, None) == 1  # looks at the last window's event
        verdict = benchhooks.point_blocks_trial()[0]
    v, ms_two, ms_one = benchhooks.point_blocks_trial()
    print(f"geometry trial: verdict {v} point block(s) per wave, {ms_two:.4f} ms per step with two, "
          f"{ms_one:.4f} ms with one", flush=True)
    assert v in (1, 2) and benchhooks.point_blocks(d) == (v, True)
    after = LloydLoop(xs, cs, _native.Workspace(cuda))
    assert after.run(12, None) == 12
    assert torch.equal(after.centers, want_c) and torch.equal(after.labels, want_lab)
    # shapes without the choice: wider rows have one geometry, rows beyond 128 features no resident kernel
    assert benchhooks.point_blocks(48)[0] == 1 and benchhooks.point_blocks(100)[0] == 1
    assert benchhooks.point_blocks(130)[0] == 0


@pytest.mark.parametrize("n,d,k", [(30000, 16, 15), (20000, 9, 25), (25000, 12, 20), (10000, 10, 22), (40000, 4, 50), (30000, 7, 31),
                                   (50000, 2, 90), (40000, 3, 256), (30000, 3, 70)])
def test_one_sweep_mfma_step_with_few_centroids_and_narrow_rows(cuda, n, d, k):
    # From 2 features on the step runs on the matrix cores whatever K is, while the assignment alone stays
    # on the vector kernel below 32 centroids: the two may break a tie at the resolution of the formula
    # differently, so the step is checked against the oracle, and its means against its own labels.
    assert _native.lloyd_kernel_name(n, d, k) == "lloyd_mfma_resident"
    print(f"one-sweep narrow n={n} d={d} k={k}", flush=True)
    x, _ = _data(n, d, k, seed=7 * n + d)
    c0 = x[torch.randperm(n, generator=torch.Generator().manual_seed(4))[:k]].contiguous()
    xs, cs = x.to(cuda), c0.to(cuda)
    c_step, lab_step, shift, _, _, _ = _step_and_two_pass(xs, cs, cuda)
    lab = lab_step.cpu()
    ref_lab, _ = orc.assign_to_cluster_literal(x, c0)
    rep = orc.label_agreement(x, c0, lab, ref_lab)
    assert rep["n_unexcused"] == 0 and rep["n_strict"] == 0 and rep["agreement"] >= 0.9999, rep
    ref = torch.zeros((k, d), dtype=torch.float64).index_add_(0, lab.long(), x.double())
    cnt = torch.bincount(lab.long(), minlength=k).clamp(min=1).double().unsqueeze(1)
    assert (c_step.cpu() - (ref / cnt).float()).abs().max() <= 2e-7 * float(x.abs().max())
    assert orc.rel_err_scalar(float(shift), float(orc.centroid_shift(c0, c_step.cpu())), floor=1e-12) <= 1e-5


@pytest.mark.parametrize("n,d,k", [(60000, 2, 90), (50000, 4, 60), (40000, 32, 64)])
def test_one_sweep_mfma_step_keeps_its_exact_sums_with_rows_near_the_origin(cuda, n, d, k):
    # Rows far smaller than the centroids -- the rule in two or three dimensions, where a blob around the origin
    # has points at any distance from it -- are rounded to a quantum derived from the largest centroid norm
    # instead of their own, so they no longer break the range in which the fp64 sums are exact: the step stays
    # on its own sums (equal to the fp64 means, which the fp32 partials of the two-pass update only approximate).
    x, _ = _data(n, d, k, seed=13 * n + d)
    g = torch.Generator().manual_seed(9)
    tiny = torch.randperm(n, generator=g)[: n // 50]
    x[tiny] *= torch.pow(2.0, -torch.randint(10, 40, (tiny.numel(), 1), generator=g).float())
    c0 = _data(n, d, k, seed=13 * n + d)[0][torch.randperm(n, generator=g)[:k]].contiguous()
    xs, cs = x.to(cuda), c0.to(cuda)
    c_step, lab_step, shift, c2, lab2, cnt2 = _step_and_two_pass(xs, cs, cuda)
    lab = lab_step.cpu()
    ref = torch.zeros((k, d), dtype=torch.float64).index_add_(0, lab.long(), x.double())
    cnt = torch.bincount(lab.long(), minlength=k).clamp(min=1).double().unsqueeze(1)
    assert (c_step.cpu() - (ref / cnt).float()).abs().max() <= 1.2e-7 * float(c0.abs().max())
    again = _step_and_two_pass(xs, cs, cuda)
    assert torch.equal(again[0], c_step) and torch.equal(again[2], shift)


def test_one_sweep_mfma_step_falls_back_outside_the_exact_range(cuda):
    # Row magnitudes spread over 2^60 (or rows holding inf / NaN) break the condition under which the
    # fp64 LDS sums are independent of the order of additions: the step must then produce exactly
    # what assign + update produce (their fp32 partials, fixed order), run after run.
    n, d, k = 60000, 32, 64
    x, _ = _data(n, d, k, seed=77)
    g = torch.Generator().manual_seed(2)
    scale = torch.pow(2.0, torch.randint(-30, 31, (n, 1), generator=g).float())
    for variant in ("wide", "nonfinite", "allhuge", "allnan"):
        xv = x * scale if variant == "wide" else x.clone()
        if variant == "nonfinite":
            xv[5, 3] = float("inf")
            xv[4000, 0] = float("nan")
        if variant == "allhuge":   # every |x|^2 overflows: no row has a usable magnitude bound, none differs from another
            xv = xv * 3e19
        if variant == "allnan":
            xv[:, 1] = float("nan")
        c0 = xv[torch.randperm(n, generator=g)[:k]].contiguous()
        c0 = torch.nan_to_num(c0, nan=0.0, posinf=1.0, neginf=-1.0)
        xs, cs = xv.to(cuda), c0.to(cuda)
        c_step, lab_step, shift, c2, lab2, _ = _step_and_two_pass(xs, cs, cuda, lists=True)
        assert torch.equal(lab_step, lab2)
        assert torch.equal(c_step.isnan(), c2.isnan())
        assert torch.equal(torch.nan_to_num(c_step), torch.nan_to_num(c2)), variant
        again = _step_and_two_pass(xs, cs, cuda, lists=True)
        assert torch.equal(torch.nan_to_num(again[0]), torch.nan_to_num(c_step))
    # moderate spread (2^+-3) stays on the exact path: the result is the fp64 mean, which the fp32
    # partials of the two-pass update only approximate
    xv = x * torch.pow(2.0, torch.randint(-3, 4, (n, 1), generator=g).float())
    c0 = xv[torch.randperm(n, generator=g)[:k]].contiguous()
    c_step, lab_step, _, c2, lab2, cnt2 = _step_and_two_pass(xv.to(cuda), c0.to(cuda), cuda)
    ref = torch.zeros((k, d), dtype=torch.float64).index_add_(0, lab2.cpu().long(), xv.double())
    ref = (ref / cnt2.cpu().clamp(min=1).double().unsqueeze(1)).float()
    assert (c_step.cpu() - ref).abs().max() <= 2e-7 * float(xv.abs().max())


@pytest.mark.parametrize("n,d,k", [(60001, 32, 8), (30000, 64, 12), (20001, 21, 2), (25000, 28, 16)])
def test_few_cluster_step_without_labels_equals_the_step_with_labels(cuda, n, d, k):
    """The fit's steps on few clusters of 17 to 64 features store no labels.  Same centroids and shift bit for bit
    as the step that stores them -- on the exact path, and where a workgroup raises its flag (row magnitudes
    spread over 2^60, non-finite rows): there the labels the two-pass update needs are computed into the
    workspace by one more launch, which otherwise returns at once."""
    assert _native.lloyd_kernel_name(n, d, k) == "lloyd_few" and _native.lloyd_step_labels_optional(n, d, k)
    x, _ = _data(n, d, k, seed=3 * n + d)
    g = torch.Generator().manual_seed(5)
    for variant in ("plain", "wide", "nonfinite"):
        xv = x.clone()
        if variant == "wide":
            xv = xv * torch.pow(2.0, torch.randint(-30, 31, (n, 1), generator=g).float())
        if variant == "nonfinite":
            xv[7, 2] = float("inf")
            xv[n // 2, 0] = float("nan")
        c0 = torch.nan_to_num(xv[torch.randperm(n, generator=g)[:k]].contiguous(), nan=0.0, posinf=1.0, neginf=-1.0)
        xs, cs = xv.to(cuda), c0.to(cuda)
        ws = _native.Workspace(cuda)
        out = []
        for lab in (torch.full((n,), -7, dtype=torch.int32, device=cuda), None, None):
            c_new = torch.full_like(cs, -3.0)
            shift = torch.empty((), device=cuda)
            _native.lloyd_step(xs, cs, c_new, lab, shift, None, ws)
            torch.cuda.synchronize()
            out.append((c_new.cpu(), shift.cpu()))
        for c_new, shift in out[1:]:
            assert torch.equal(torch.nan_to_num(c_new), torch.nan_to_num(out[0][0])), variant
            assert torch.equal(c_new.isnan(), out[0][0].isnan()), variant
            assert torch.equal(torch.nan_to_num(shift), torch.nan_to_num(out[0][1])), variant
        if variant != "plain":
            # a flagged step's means are those of the (list-based) two-pass update of its labels; the spread of
            # magnitudes alone need not raise a flag (rows far below the centroids are rounded to a floor derived
            # from the centroid norms), and then the means are the fp64 ones
            _, _, _, c2, lab2, cnt2 = _step_and_two_pass(xs, cs, cuda, lists=True)
            flagged = torch.equal(torch.nan_to_num(c2.cpu()), torch.nan_to_num(out[1][0]))
            assert flagged or variant == "wide", variant
            if not flagged:
                ref = torch.zeros((k, d), dtype=torch.float64).index_add_(0, lab2.cpu().long(), xv.double())
                ref = (ref / cnt2.cpu().clamp(min=1).double().unsqueeze(1)).float()
                assert (out[1][0] - ref).abs().max() <= 2e-7 * float(ref.abs().max())


def _narrow_step(xs, cs, dev, sums, monkeypatch, want_sse=True):
    """One hkm_lloyd_step_f32 on a narrow shape with the per-cluster sums formed the given way."""
    monkeypatch.setenv("HKM_SMALL_SUMS", sums)
    n = xs.shape[0]
    c_new = torch.empty_like(cs)
    lab = torch.full((n,), -7, dtype=torch.int32, device=dev)
    shift = torch.empty((), device=dev)
    sse = torch.empty((), device=dev) if want_sse else None
    _native.lloyd_step(xs, cs, c_new, lab, shift, sse, _native.Workspace(dev))
    torch.cuda.synchronize()
    return c_new.cpu(), lab.cpu(), shift.cpu(), (sse.cpu() if want_sse else None)


# narrow shapes beyond 48 accumulator slots: every D, K up to the limit of 240 slots, ragged N
NARROW_SHAPES = [(20000, 8, 16), (30011, 8, 26), (50000, 4, 32), (40001, 6, 20), (25000, 7, 30), (60000, 2, 64),
                 (60002, 3, 40), (50000, 1, 100), (33333, 5, 40), (300, 8, 16), (7, 2, 20), (45001, 4, 15), (30000, 8, 14),
                 # 9 to 16 features, up to 240 accumulator slots
                 (30000, 16, 8), (25001, 12, 18), (10000, 10, 3), (20000, 9, 24), (40000, 13, 17), (33001, 15, 15),
                 (20000, 16, 14), (5000, 11, 1), (20002, 14, 16)]


@pytest.mark.parametrize("n,d,k", NARROW_SHAPES)
def test_integer_sums_of_the_narrow_step_equal_the_ordered_ones(cuda, n, d, k, monkeypatch):
    # Large fits form the per-cluster sums of the narrow one-sweep step as exact 64-bit integer sums (LDS
    # atomics, any order); small ones in a fixed order on the matrix cores or with a wave-wide tree.  Forced
    # either way on the same input: same labels, same sum of distances, centroids equal to fp32 rounding
    # and equal to the fp64 means of the labels; the integer way gives the same bits run after run.
    assert _native.lloyd_kernel_name(n, d, k) == "lloyd_small" and (k * (d + 1) > 48 or d > 8)
    print(f"narrow sums n={n} d={d} k={k}", flush=True)
    x, _ = _data(n, d, k, seed=3 * n + d)
    x[::97] = 0.0
    c0 = x[torch.randperm(n, generator=torch.Generator().manual_seed(5))[:k]].contiguous()
    if n < k:
        c0 = _data(k, d, k, seed=1)[0]
    xs, cs = x.to(cuda), c0.to(cuda)
    c_o, lab_o, shift_o, sse_o = _narrow_step(xs, cs, cuda, "ordered", monkeypatch)
    c_i, lab_i, shift_i, sse_i = _narrow_step(xs, cs, cuda, "integer", monkeypatch)
    assert torch.equal(lab_o, lab_i) and torch.equal(sse_o, sse_i)
    cmax = float(c0.abs().max())
    assert (c_i - c_o).abs().max() <= 2.4e-7 * cmax
    ref = torch.zeros((k, d), dtype=torch.float64).index_add_(0, lab_i.long(), x.double())
    cnt = torch.bincount(lab_i.long(), minlength=k).clamp(min=1).double().unsqueeze(1)
    ref = (ref / cnt).float()
    # exact sums of rows rounded to 2^-32 of the largest centroid coordinate, one rounding at the end
    assert (c_i - ref).abs().max() <= 6e-8 * max(cmax, float(ref.abs().max())) + 2.0 ** -31 * cmax
    again = _narrow_step(xs, cs, cuda, "integer", monkeypatch)
    assert torch.equal(again[0], c_i) and torch.equal(again[2], shift_i)
    # rows with a leading dimension and no alignment: the guarded rounds
    big = torch.zeros((n, d + 3), device=cuda)
    big[:, 1:d + 1] = xs
    c_s, lab_s, shift_s, _ = _narrow_step(big[:, 1:d + 1], cs, cuda, "integer", monkeypatch)
    assert torch.equal(lab_s, lab_i)
    assert (c_s - ref).abs().max() <= 6e-8 * max(cmax, float(ref.abs().max())) + 2.0 ** -31 * cmax


def test_integer_sums_of_the_narrow_step_fall_back_outside_their_range(cuda, monkeypatch):
    # The integer scale comes from the largest centroid coordinate.  A row too large for it, a row or a
    # centroid that is not finite, or centroids that are all zero leave no exact integer sum: the step must
    # then give exactly what the ordered way gives.  A row 2^10 times larger than the centroids is inside.
    n, d, k = 30000, 8, 16
    x, _ = _data(n, d, k, seed=41)
    g = torch.Generator().manual_seed(6)
    c_base = x[torch.randperm(n, generator=g)[:k]].contiguous()
    for variant in ("huge_row", "inf_row", "nan_row", "zero_centroids", "inf_centroid", "large_row_inside"):
        xv, c0 = x.clone(), c_base.clone()
        if variant == "huge_row":
            xv[12345] *= 2.0 ** 40
        if variant == "inf_row":
            xv[77, 3] = float("inf")
        if variant == "nan_row":
            xv[29999, 0] = float("nan")
        if variant == "zero_centroids":
            c0.zero_()
        if variant == "inf_centroid":
            c0[3, 2] = float("inf")
        if variant == "large_row_inside":
            xv[222] *= 2.0 ** 10
        xs, cs = xv.to(cuda), c0.to(cuda)
        c_o, lab_o, shift_o, sse_o = _narrow_step(xs, cs, cuda, "ordered", monkeypatch)
        c_i, lab_i, shift_i, sse_i = _narrow_step(xs, cs, cuda, "integer", monkeypatch)
        assert torch.equal(lab_o, lab_i), variant
        if variant == "large_row_inside":
            ref = torch.zeros((k, d), dtype=torch.float64).index_add_(0, lab_i.long(), xv.double())
            cnt = torch.bincount(lab_i.long(), minlength=k).clamp(min=1).double().unsqueeze(1)
            ref = (ref / cnt).float()
            assert (c_i - ref).abs().max() <= 6e-8 * float(ref.abs().max()) + 2.0 ** -31 * float(c0.abs().max())
            continue
        assert torch.equal(c_o.isnan(), c_i.isnan()), variant
        assert torch.equal(torch.nan_to_num(c_o), torch.nan_to_num(c_i)), variant
        assert torch.equal(torch.nan_to_num(shift_o), torch.nan_to_num(shift_i)), variant


@pytest.mark.parametrize("d", [1, 4, 8])
def test_narrow_kernels_take_centroid_rows_at_any_four_byte_address(cuda, d):
    # For these widths the narrow kernels fetch a centroid row as one scalar load of 1, 4 or 8 values;
    # the rows of C are only required to be 4-byte aligned.
    n, k = 20000, 24
    x, _ = _data(n, d, k, seed=91 + d)
    c0 = x[torch.randperm(n, generator=torch.Generator().manual_seed(8))[:k]].contiguous()
    xs = x.to(cuda)
    flat = torch.zeros((k * d + 8,), device=cuda)
    ref_lab, ref_min = _assign_gpu(x, c0, cuda)
    for off in (1, 2, 3):
        flat[off:off + k * d] = c0.to(cuda).reshape(-1)
        cs = flat[off:off + k * d].view(k, d)
        assert cs.data_ptr() % 16 == 4 * off
        lab = torch.full((n,), -7, dtype=torch.int32, device=cuda)
        md = torch.empty((n,), device=cuda)
        _native.assign(xs, cs, lab, md, _native.Workspace(cuda))
        c_new = torch.empty((k, d), device=cuda)
        lab2 = torch.empty_like(lab)
        _native.lloyd_step(xs, cs, c_new, lab2, torch.empty((), device=cuda), None, _native.Workspace(cuda))
        torch.cuda.synchronize()
        assert torch.equal(lab.cpu(), ref_lab) and torch.equal(md.cpu(), ref_min)
        assert torch.equal(lab2.cpu(), ref_lab)


def test_shift_and_functional_value(cuda):
    g = torch.Generator().manual_seed(9)
    a, b = torch.randn((37, 19), generator=g), torch.randn((37, 19), generator=g)
    out = torch.empty((), device=cuda)
    _native.shift(a.to(cuda), b.to(cuda), out)
    assert orc.rel_err_scalar(float(out), float(orc.centroid_shift(a, b))) <= 1e-6
    _native.shift(a.to(cuda), a.to(cuda), out)
    assert float(out) == 0.0
    md = torch.rand((100003,), generator=g) * 7
    _native.functional_value(md.to(cuda), out, _native.Workspace(cuda))
    m = torch.sqrt(md)
    ref = torch.sqrt(torch.dot(m, m)) ** 2
    assert orc.rel_err_scalar(float(out), float(ref)) <= 1e-5


def test_cdist_known_answers_and_oracle(cuda):
    # known answers of the reference's tests/spatial/test_distances.py:16-58
    X, Y = torch.ones((4, 4)), torch.zeros((4, 4))
    out = torch.empty((4, 4), device=cuda)
    _native.cdist(X.to(cuda), Y.to(cuda), out, sqrt=True)
    assert torch.equal(out.cpu(), torch.full((4, 4), 2.0))
    _native.cdist(X.to(cuda), X.to(cuda), out, sqrt=True)
    assert torch.equal(out.cpu(), torch.zeros((4, 4)))
    g = torch.Generator().manual_seed(10)
    for m, n, d in ((100, 70, 3), (130, 257, 64), (65, 64, 200), (1, 1, 1)):
        a, b = torch.randn((m, d), generator=g) * 3, torch.randn((n, d), generator=g) * 3
        out = torch.empty((m, n), device=cuda)
        _native.cdist(a.to(cuda), b.to(cuda), out, sqrt=False)
        ref = orc.quadratic_expand(a, b)
        scale = float((a.double() ** 2).sum(1).max() + (b.double() ** 2).sum(1).max())
        assert float((out.cpu() - ref).abs().max()) <= 2e-6 * scale
        _native.cdist(a.to(cuda), b.to(cuda), out, sqrt=True)
        bf = orc.brute_force_d2(a, b).sqrt()
        assert float((out.cpu().double() - bf).abs().max()) <= 1e-3


@pytest.mark.parametrize("m,n,d", [(300, 257, 40), (129, 1, 64), (1000, 700, 100), (128, 128, 32), (5, 3, 18),
                                   (200, 333, 16), (64, 513, 130)])
def test_cdist_matrix_core_path(cuda, m, n, d):
    """Quadratic-expansion full matrices from 16 features on take the matrix-core kernel: ragged tiles,
    feature counts that are no multiple of the chunk or of 4, strided rows, every epilogue."""
    g = torch.Generator().manual_seed(m * 7 + n * 3 + d)
    a, b = torch.randn((m, d), generator=g) * 3, torch.randn((n, d), generator=g) * 3
    scale = float((a.double() ** 2).sum(1).max() + (b.double() ** 2).sum(1).max())
    ref = orc.quadratic_expand(a, b)
    bf = orc.brute_force_d2(a, b)
    ag, bg = a.to(cuda), b.to(cuda)
    out = torch.full((m, n + 5), -7.0, device=cuda)[:, :n]  # strided output, guard columns behind it
    _native.cdist(ag, bg, out, sqrt=False)
    assert float((out.cpu() - ref).abs().max()) <= 2e-6 * scale
    assert float(out.min()) >= 0.0
    assert torch.all(out._base[:, n:] == -7.0), "stores beyond the last column"
    _native.pairwise(ag, bg, out, _native.METRIC_EUCLID_QE)
    assert float((out.cpu().double() ** 2 - bf).abs().max()) <= 4e-6 * scale
    _native.pairwise(ag, bg, out, _native.METRIC_GAUSS_QE, 2.5)
    want = torch.exp(-bf / (2 * 2.5 ** 2))
    assert float((out.cpu().double() - want).abs().max()) <= 1e-5 + 4e-6 * scale / (2 * 2.5 ** 2)
    # strided inputs (rows embedded in wider matrices, 16-byte alignment lost for odd strides)
    wide_a = torch.zeros((m, d + 3), device=cuda)
    wide_a[:, 1:d + 1] = ag
    wide_b = torch.zeros((n, d + 8), device=cuda)
    wide_b[:, 4:d + 4] = bg
    dense = torch.empty((m, n), device=cuda)
    _native.cdist(wide_a[:, 1:d + 1], wide_b[:, 4:d + 4], dense, sqrt=False)
    assert float((dense.cpu() - ref).abs().max()) <= 2e-6 * scale
    # X against itself: symmetric to rounding, diagonal zero within the resolution of the formula
    sq = torch.empty((m, m), device=cuda)
    _native.cdist(ag, ag, sq, sqrt=False)
    assert float(sq.diagonal().abs().max()) <= 2e-6 * scale
    assert float((sq - sq.T).abs().max()) <= 2e-6 * scale
    # NaN rows pass through the clamp
    a2 = ag.clone()
    a2[0, 0] = float("nan")
    _native.cdist(a2, bg, dense, sqrt=True)
    assert bool(torch.isnan(dense[0]).all()) and not bool(torch.isnan(dense[1:]).any())


@pytest.mark.parametrize("scale", [1.0, 1e-3, 1e-15, 1e-18, 1e-22])
def test_cdist_matrix_core_sqrt_is_correctly_rounded(cuda, scale):
    """The kernel's square root is the correctly rounded one at every magnitude: the short form for
    ordinary values, the library routine for sub-tiles that hold positive values below 2^-96
    (squared distances of rows scaled by 1e-15 and less, denormals included), zeros on the diagonal,
    infinities and NaN.  Checked against the square root, taken in float64 by numpy and rounded to
    float32 (innocuous double rounding: 53 >= 2 * 24 + 2 bits), of the kernel's own squared output --
    not against torch's CPU square root, which goes through a vector math library that is only
    accurate to an ulp on some hosts."""
    m, n, d = 300, 260, 48
    g = torch.Generator().manual_seed(int(-torch.log10(torch.tensor(scale))) + 5)
    a, b = torch.randn((m, d), generator=g) * scale, torch.randn((n, d), generator=g) * scale
    b[:100] = a[:100]  # exact zeros
    a[200:, :] *= 1e6 / scale if scale < 1e-10 else 1.0  # ordinary and tiny values in one matrix
    a[299, 0] = float("inf")
    b[259, 1] = float("nan")
    ag, bg = a.to(cuda), b.to(cuda)
    sq = torch.empty((m, n), device=cuda)
    rt = torch.empty((m, n), device=cuda)
    _native.cdist(ag, bg, sq, sqrt=False)
    _native.cdist(ag, bg, rt, sqrt=True)
    with np.errstate(invalid="ignore"):
        want = torch.from_numpy(np.sqrt(sq.cpu().numpy().astype(np.float64)).astype(np.float32))
    got = rt.cpu()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    assert torch.equal(got[~nan].view(torch.int32), want[~nan].view(torch.int32))
    assert int((sq[:100, :100].diagonal() == 0).sum()) > 0 or scale >= 1e-3


def test_cdist_matrix_core_known_answers(cuda):
    # the reference's known answers (tests/spatial/test_distances.py:16-58) at a width that takes the
    # matrix-core kernel: ones against zeros -> sqrt(D), a matrix against itself -> 0, exactly
    for d in (16, 36, 64):
        X, Y = torch.ones((40, d), device=cuda), torch.zeros((150, d), device=cuda)
        out = torch.empty((40, 150), device=cuda)
        _native.cdist(X, Y, out, sqrt=True)
        assert torch.equal(out.cpu(), torch.full((40, 150), float(d)).sqrt())
        sq = torch.empty((40, 40), device=cuda)
        _native.cdist(X, X, sq, sqrt=True)
        assert torch.equal(sq.cpu(), torch.zeros((40, 40)))


def test_widen_and_empty_inputs(cuda):
    lab = torch.tensor([3, 0, 2147483647, 5], dtype=torch.int32, device=cuda)
    out = torch.empty((4,), dtype=torch.int64, device=cuda)
    _native.widen_labels(lab, out)
    assert out.tolist() == [3, 0, 2147483647, 5]
    # N = 0: nothing to do, no launch, no error
    x = torch.empty((0, 8), device=cuda)
    c = torch.randn((4, 8), device=cuda)
    _native.assign(x, c, torch.empty((0,), dtype=torch.int32, device=cuda), None, _native.Workspace(cuda))
    c_new = torch.full((4, 8), 9.0, device=cuda)
    _native.update(x, torch.empty((0,), dtype=torch.int32, device=cuda), c_new, None, _native.Workspace(cuda))
    assert torch.all(c_new == 0)
    # the reductions and the selection of the initialiser on empty vectors: sums 0, nothing selected
    ws = _native.Workspace(cuda)
    e = torch.empty((0,), device=cuda)
    s = torch.full((), 7.0, device=cuda)
    _native.min_dist_sum(e, s, ws)
    assert float(s) == 0.0
    s.fill_(7.0)
    _native.min_merge_sum(e, e.clone(), s, ws)
    assert float(s) == 0.0
    s.fill_(7.0)
    _native.functional_value(e, s, ws)
    assert float(s) == 0.0
    cnt = torch.full((), 5, dtype=torch.int64, device=cuda)
    idx = torch.empty((4,), dtype=torch.int64, device=cuda)
    _native.sample_select(e, e.clone(), torch.ones((), device=cuda), 2.0, idx, cnt, ws)
    assert int(cnt) == 0


def test_binding_refuses_matrices_it_would_misread(cuda):
    """Rows must have unit stride inside (a transposed view would be read as other numbers), and the
    centroid matrices of the step, which the C ABI takes without a leading dimension, must be dense."""
    ws = _native.Workspace(cuda)
    xt = torch.randn((8, 100), device=cuda).T            # (100, 8) with stride (1, 100)
    c = torch.randn((4, 8), device=cuda)
    lab = torch.empty((100,), dtype=torch.int32, device=cuda)
    with pytest.raises(ValueError, match="contiguous"):
        _native.assign(xt, c, lab, None, ws)
    with pytest.raises(ValueError, match="contiguous"):
        _native.pairwise(xt, c, torch.empty((100, 4), device=cuda), _native.METRIC_EUCLID)
    x = xt.contiguous()
    wide = torch.randn((4, 12), device=cuda)
    shift = torch.empty((), device=cuda)
    with pytest.raises(ValueError, match="dense"):
        _native.lloyd_step(x, wide[:, :8], torch.empty_like(c), lab, shift, None, ws)
    # a padded X is fine: it has a leading dimension
    xp = torch.randn((100, 12), device=cuda)[:, :8]
    _native.lloyd_step(xp, c, torch.empty_like(c), lab, shift, None, ws)
    _native.assign(xp, wide[:, :8], lab, None, ws)
