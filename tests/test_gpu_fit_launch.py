"""
hkm_lloyd_fit_f32 -- the whole loop of KMeans.fit as one launch, for data that stays in registers -- against the
step-by-step loop (one hkm_lloyd_step_f32 per iteration, HKM_FIT=steps) and the CPU oracle.

The two paths form their sums differently (exact integers there, the one-sweep kernels' sums here), so centroids
are compared to 1e-6 and labels under the tie rule, iteration counts exactly; against the oracle the bars of
tests/test_gpu_kmeans.py apply.  The waits between the kernel's workgroups are bounded: with a limit of zero the
first workgroup that has to wait gives up, every workgroup leaves, the status says so and the estimator falls back.
"""
import warnings

import pytest
import torch

import heat_amd as ht
from heat_amd import _native
from heat_amd.utils import synthetic
from oracle import heat_oracle as orc

pytestmark = pytest.mark.gpu


def _blobs(n, d, k, seed, spread=10.0):
    g = torch.Generator().manual_seed(seed)
    c = (torch.rand((k, d), generator=g) - 0.5) * 2.0 * spread
    x = (torch.randn((n, d), generator=g) + c[torch.randint(0, k, (n,), generator=g)]).contiguous()
    return x, x[torch.randperm(n, generator=g)[:k]].contiguous()


def _fit(x, init, k, iters, tol, dev):
    km = ht.cluster.KMeans(n_clusters=k, init=ht.array(init.to(dev)), max_iter=iters, tol=tol)
    km.fit(ht.array(x.to(dev), split=0))
    torch.cuda.synchronize()
    return km


SHAPES = [(100000, 8, 16), (5000, 3, 8), (70000, 2, 30), (262144, 4, 5), (131072, 8, 26), (65536, 16, 14),
          (1000, 11, 20), (33, 5, 7), (7, 1, 3), (250000, 1, 100), (40000, 13, 17), (2049, 6, 1)]


@pytest.mark.parametrize("n,d,k", SHAPES)
def test_one_launch_fit_equals_the_step_loop(cuda, n, d, k, monkeypatch):
    assert _native.lloyd_fit_supported(n, d, k)
    print(f"one-launch fit n={n} d={d} k={k}", flush=True)
    x, init = _blobs(n, d, k, seed=n + 7 * d + k)
    for tol, iters in ((0.0, 25), (1e-3, 25), (None, 4)):
        monkeypatch.delenv("HKM_FIT", raising=False)
        a = _fit(x, init, k, iters, tol, cuda)
        a2 = _fit(x, init, k, iters, tol, cuda)
        monkeypatch.setenv("HKM_FIT", "steps")
        b = _fit(x, init, k, iters, tol, cuda)
        assert torch.equal(a.cluster_centers_.larray, a2.cluster_centers_.larray)
        assert torch.equal(a.labels_.larray, a2.labels_.larray) and float(a.inertia_) == float(a2.inertia_)
        assert a.n_iter_ == a2.n_iter_
        la, lb = a.labels_.larray.cpu().view(-1), b.labels_.larray.cpu().view(-1)
        same = float((la == lb).float().mean())
        if a.n_iter_ == b.n_iter_ and same == 1.0:
            assert orc.rel_err_centers(a.cluster_centers_.larray.cpu(), b.cluster_centers_.larray.cpu()) <= 1e-6
            floor = 1e-6 * float((b.cluster_centers_.larray.double() ** 2).sum(1).mean())
            assert orc.rel_err_scalar(float(a.inertia_), float(b.inertia_), floor=floor) <= 1e-4
        else:
            # a tie resolved differently somewhere along the way: same objective, (nearly) the same partition
            sa = orc.sse(x, a.cluster_centers_.larray.cpu(), orc.assign_to_cluster_fast(x, a.cluster_centers_.larray.cpu())[0])
            sb = orc.sse(x, b.cluster_centers_.larray.cpu(), orc.assign_to_cluster_fast(x, b.cluster_centers_.larray.cpu())[0])
            assert orc.rel_err_scalar(sa, sb) <= 1e-4 and same >= 0.99, (a.n_iter_, b.n_iter_, same)
        # the means of the returned labels are the returned centroids
        want, _ = orc.update_centroids_fast(x, la.view(-1, 1), k)
        assert orc.rel_err_centers(a.cluster_centers_.larray.cpu(), want) <= 1e-6


@pytest.mark.parametrize("n,d,k", [(100000, 8, 16), (20000, 3, 8), (30000, 12, 9)])
def test_one_launch_fit_against_the_oracle(cuda, n, d, k, parity_report):
    x, init = _blobs(n, d, k, seed=3 * n + d)
    ref = orc.kmeans_fit(x, init, 30, 0.0, literal=True)
    km = _fit(x, init, k, 30, 0.0, cuda)
    lab = km.labels_.larray.cpu().view(-1)
    agree = float((lab == ref["labels"].view(-1)).float().mean())
    parity_report(f"one-launch fit N={n} D={d} K={k}: n_iter_ {km.n_iter_} (oracle {ref['n_iter']}), labels equal on "
                  f"{agree:.6f}, centroids {orc.rel_err_centers(km.cluster_centers_.larray.cpu(), ref['cluster_centers']):.2e}")
    if agree == 1.0:
        assert km.n_iter_ == ref["n_iter"]
        assert orc.rel_err_centers(km.cluster_centers_.larray.cpu(), ref["cluster_centers"]) <= 1e-5
    else:
        a = orc.sse(x, km.cluster_centers_.larray.cpu(), lab.view(-1, 1))
        b = orc.sse(x, ref["cluster_centers"], ref["labels"])
        assert orc.rel_err_scalar(a, b) <= 1e-4 and agree >= 0.999


def test_one_launch_fit_gives_up_instead_of_hanging(cuda):
    """A wait limit of zero: the first workgroup that has to wait raises the abort flag, every workgroup leaves, the
    status word says -1; nothing hangs, and the estimator's fallback gives the step loop's result."""
    n, d, k = 100000, 8, 16
    x, init = _blobs(n, d, k, seed=5)
    xs, cs = x.to(cuda), init.to(cuda)
    c_out = torch.empty_like(cs)
    lab = torch.empty((n,), dtype=torch.int64, device=cuda)
    shift = torch.zeros((), device=cuda)
    info = torch.zeros((2,), dtype=torch.int32, pin_memory=True)
    ws = _native.Workspace(cuda)
    _native.lloyd_fit(xs, cs, 10, 0.0, c_out, lab, shift, info, ws, wait_limit_us=0)
    torch.cuda.synchronize()
    assert int(info[0]) == -1
    # the same call with the ordinary limit delivers
    _native.lloyd_fit(xs, cs, 10, 0.0, c_out, lab, shift, info, ws)
    torch.cuda.synchronize()
    assert int(info[0]) >= 1 and int(lab.min()) >= 0 and int(lab.max()) < k


def test_one_launch_fit_leaves_non_finite_data_to_the_step_loop(cuda, monkeypatch):
    n, d, k = 5000, 4, 6
    x, init = _blobs(n, d, k, seed=9)
    x[123, 2] = float("inf")
    xs, cs = x.to(cuda), init.to(cuda)
    info = torch.zeros((2,), dtype=torch.int32, pin_memory=True)
    _native.lloyd_fit(xs, cs, 5, 0.0, torch.empty_like(cs), torch.empty((n,), dtype=torch.int64, device=cuda),
                      torch.zeros((), device=cuda), info, _native.Workspace(cuda))
    torch.cuda.synchronize()
    assert int(info[0]) == -2
    monkeypatch.delenv("HKM_FIT", raising=False)
    with warnings.catch_warnings():
        warnings.simplefilter("error")  # the fallback for such data is silent: nothing went wrong
        a = _fit(x, init, k, 5, 0.0, cuda)
    monkeypatch.setenv("HKM_FIT", "steps")
    b = _fit(x, init, k, 5, 0.0, cuda)
    assert a.n_iter_ == b.n_iter_ and torch.equal(a.labels_.larray, b.labels_.larray)
    assert torch.equal(a.cluster_centers_.larray.isnan(), b.cluster_centers_.larray.isnan())


def test_one_launch_fit_refuses_what_it_does_not_hold():
    assert not _native.lloyd_fit_supported(262145, 4, 5)
    assert not _native.lloyd_fit_supported(131073, 8, 5)
    assert not _native.lloyd_fit_supported(1000, 17, 5)
    assert not _native.lloyd_fit_supported(1000, 8, 27)
    assert _native.workspace_bytes(1000, 17, 5, _native.WS_FIT) == 0
    assert _native.workspace_bytes(1000, 8, 16, _native.WS_FIT) > 0
