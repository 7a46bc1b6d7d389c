"""
Buffers beyond 4 GiB: every kernel family once with an X (or an output matrix) whose byte offsets do
not fit 32 bits, so that an index computed in 32-bit arithmetic anywhere on the way shows up.

No CPU oracle at these sizes.  The checks are size-independent properties:
  * a row's label and minimum depend on that row only, so a call on the whole array and calls on row
    slices (each below 4 GiB) must agree bit for bit;
  * rows on both sides of the 4 GiB byte offset and at the very end are compared with a float64
    evaluation on the GPU under the gap rule of the parity bar (a different label is excused only where
    best and second-best squared distance differ by less than 1e-5 relative);
  * the new centroids equal the float64 per-cluster means of the labels the step returned (1e-6), and
    the counts sum to N.
Data are generated on the device in chunks (blobs around K centres, sigma 0.5).
"""
import pytest
import torch

from heat_amd import _native

pytestmark = pytest.mark.gpu

GIB4 = 1 << 32


def _blobs(n, d, k, dev, seed, dtype=torch.float32):
    g = torch.Generator(device=dev).manual_seed(seed)
    c = (torch.rand((k, d), device=dev, generator=g) * 10.0 - 5.0).to(dtype)
    x = torch.empty((n, d), device=dev, dtype=dtype)
    step = max(1, (1 << 28) // d)
    for a in range(0, n, step):
        b = min(n, a + step)
        which = torch.randint(0, k, (b - a,), device=dev, generator=g)
        x[a:b] = c[which] + 0.5 * torch.randn((b - a, d), device=dev, generator=g, dtype=dtype)
    assert x.numel() * x.element_size() > GIB4
    return x, c


def _probe_rows(n, d, dev):
    """Rows around the 4 GiB byte offset of a float32 (n, d) array, and the last rows."""
    r4 = GIB4 // (4 * d)
    assert 4096 < r4 < n - 8192
    return torch.cat([torch.arange(r4 - 2048, r4 + 2048, device=dev), torch.arange(n - 8192, n, device=dev)])


def _gap_rule(x, c, rows, lab, md=None):
    xr = x[rows].double()
    cd = c.double()
    d2 = ((xr * xr).sum(1, keepdim=True) + (cd * cd).sum(1)[None, :] - 2.0 * (xr @ cd.T)).clamp_min(0.0)
    best2, idx2 = torch.topk(d2, 2, dim=1, largest=False)
    got = lab[rows].long()
    diff = got != idx2[:, 0]
    tied = (best2[:, 1] - best2[:, 0]) <= 1e-5 * best2[:, 0]
    assert int((diff & ~tied).sum()) == 0, int((diff & ~tied).sum())
    assert float(diff.float().mean()) <= 1e-4
    if md is not None:
        ok = ~diff
        assert torch.allclose(md[rows][ok].double(), best2[ok, 0], rtol=1e-4, atol=1e-3)


def _slices(n, parts=3):
    step = ((n + parts - 1) // parts + 63) // 64 * 64
    return [(a, min(n, a + step)) for a in range(0, n, step)]


def _assign_whole_equals_slices(x, c, dev, fn=None):
    n = x.shape[0]
    ws = _native.Workspace(dev)
    fn = fn or (lambda xs, lab, md: _native.assign(xs, c, lab, md, ws))
    lab = torch.full((n,), -7, dtype=torch.int32, device=dev)
    md = torch.full((n,), -7.0, device=dev)
    fn(x, lab, md)
    for a, b in _slices(n):
        assert (b - a) * x.shape[1] * 4 < GIB4
        lab_s = torch.empty((b - a,), dtype=torch.int32, device=dev)
        md_s = torch.empty((b - a,), device=dev)
        fn(x[a:b], lab_s, md_s)
        assert torch.equal(lab[a:b], lab_s), (a, b)
        assert torch.equal(md[a:b].view(torch.int32), md_s.view(torch.int32)), (a, b)
    assert int(lab.min()) >= 0 and int(lab.max()) < c.shape[0]
    return lab, md


def _means_f64(x, lab, k):
    n, d = x.shape
    # one-hot product per chunk: a scatter-add onto a handful of rows would serialise on its atomics
    sums = torch.zeros((k, d), dtype=torch.float64, device=x.device)
    step = max(1, min((1 << 27) // d, (1 << 28) // k))
    for a in range(0, n, step):
        b = min(n, a + step)
        onehot = torch.zeros((b - a, k), dtype=torch.float64, device=x.device)
        onehot.scatter_(1, lab[a:b].long().view(-1, 1), 1.0)
        sums += onehot.T @ x[a:b].double()
    cnt = torch.bincount(lab.long(), minlength=k)
    return (sums / cnt.clamp_min(1).view(-1, 1).double()).float(), cnt


def _step_matches_its_labels(x, c, dev, expect_kernel):
    n, d = x.shape
    k = c.shape[0]
    assert _native.lloyd_kernel_name(n, d, k) == expect_kernel, _native.lloyd_kernel_name(n, d, k)
    ws = _native.Workspace(dev)
    lab = torch.full((n,), -7, dtype=torch.int32, device=dev)
    c_new = torch.empty_like(c)
    shift = torch.empty((), device=dev)
    sse = torch.empty((), device=dev)
    _native.lloyd_step(x, c, c_new, lab, shift, sse, ws)
    ref, cnt = _means_f64(x, lab, k)
    assert int(cnt.sum()) == n
    err = float((c_new - ref).abs().max()) / float(ref.abs().max())
    assert err <= 1e-6, err
    ref_shift = float(((c.double() - c_new.double()) ** 2).sum())
    assert abs(float(shift) - ref_shift) <= 1e-4 * ref_shift + 1e-12
    return lab


def test_wide_rows_beyond_4gib(cuda):
    """2-D streaming kernel + sorted two-pass update (D > 64)."""
    x, c = _blobs(2_400_000, 512, 1024, cuda, 41)
    lab, md = _assign_whole_equals_slices(x, c, cuda)
    _gap_rule(x, c, _probe_rows(*x.shape, cuda), lab, md)
    lab2 = _step_matches_its_labels(x, c, cuda, _native.lloyd_kernel_name(*x.shape, 1024))
    assert torch.equal(lab, lab2)


def test_resident_mfma_beyond_4gib(cuda):
    """Centroids resident in LDS, per-cluster sums in the same sweep (16 < D <= 64)."""
    x, c = _blobs(40_000_000, 32, 256, cuda, 42)
    lab, md = _assign_whole_equals_slices(x, c, cuda)
    _gap_rule(x, c, _probe_rows(*x.shape, cuda), lab, md)
    lab2 = _step_matches_its_labels(x, c, cuda, "lloyd_mfma_resident")
    assert torch.equal(lab, lab2)


def test_tiled_mfma_beyond_4gib(cuda):
    """Centroid tiles streamed through LDS (more centroids than LDS holds)."""
    x, c = _blobs(20_000_000, 64, 1024, cuda, 43)
    lab, md = _assign_whole_equals_slices(x, c, cuda)
    _gap_rule(x, c, _probe_rows(*x.shape, cuda), lab, md)
    lab2 = _step_matches_its_labels(x, c, cuda, _native.lloyd_kernel_name(*x.shape, 1024))
    assert torch.equal(lab, lab2)


def test_narrow_one_sweep_beyond_4gib(cuda):
    """One-sweep vector kernel (D <= 8)."""
    x, c = _blobs(450_000_000, 3, 8, cuda, 44)
    lab, md = _assign_whole_equals_slices(x, c, cuda)
    _gap_rule(x, c, _probe_rows(*x.shape, cuda), lab, md)
    lab2 = _step_matches_its_labels(x, c, cuda, "lloyd_small")
    assert torch.equal(lab, lab2)


def test_narrow_rows_on_the_matrix_cores_beyond_4gib(cuda):
    """4 <= D <= 16 outside the narrow kernel's limits: the matrix-core kernels with the features padded to 16."""
    x, c = _blobs(100_000_000, 12, 64, cuda, 45)
    lab, md = _assign_whole_equals_slices(x, c, cuda)
    _gap_rule(x, c, _probe_rows(*x.shape, cuda), lab, md)
    lab2 = _step_matches_its_labels(x, c, cuda, "lloyd_mfma_resident")
    assert torch.equal(lab, lab2)


def test_narrow_one_sweep_with_integer_sums_beyond_4gib(cuda):
    """One-sweep vector kernel beyond 48 accumulator slots at a size where it takes the integer sums by itself
    (and, with 16 centroids of 8 coordinates, the cross terms from the matrix cores)."""
    x, c = _blobs(150_000_000, 8, 16, cuda, 46)
    lab, md = _assign_whole_equals_slices(x, c, cuda)
    _gap_rule(x, c, _probe_rows(*x.shape, cuda), lab, md)
    lab2 = _step_matches_its_labels(x, c, cuda, "lloyd_small")
    assert torch.equal(lab, lab2)


def test_two_features_on_the_matrix_cores_beyond_4gib(cuda):
    """Fewer than 4 features outside the narrow kernel's limits: the assignment alone on the generic vector
    kernel, the step on the matrix cores (features padded to 8); the two may part on ties, so each is held to
    the gap rule."""
    x, c = _blobs(600_000_000, 2, 100, cuda, 47)
    lab, md = _assign_whole_equals_slices(x, c, cuda)
    rows = _probe_rows(*x.shape, cuda)
    _gap_rule(x, c, rows, lab, md)
    lab2 = _step_matches_its_labels(x, c, cuda, "lloyd_mfma_resident")
    _gap_rule(x, c, rows, lab2)
    assert int((lab != lab2).sum()) <= x.shape[0] // 100_000


def test_manhattan_beyond_4gib(cuda):
    """Fused Manhattan distance + argmin and the radix-selection median."""
    n, d, k = 40_000_000, 32, 256
    x, c = _blobs(n, d, k, cuda, 46)
    lab, md = _assign_whole_equals_slices(x, c, cuda, fn=lambda xs, l, m: _native.assign_l1(xs, c, l, m))
    rows = _probe_rows(n, d, cuda)
    d1 = (x[rows].double()[:, None, :] - c.double()[None, :, :]).abs().sum(-1)
    best2, idx2 = torch.topk(d1, 2, dim=1, largest=False)
    diff = lab[rows].long() != idx2[:, 0]
    assert int((diff & ((best2[:, 1] - best2[:, 0]) > 1e-5 * best2[:, 0])).sum()) == 0
    med = torch.empty_like(c)
    _native.update_median(x, lab, med, _native.Workspace(cuda), lower=True)
    for kk, dd in ((0, 0), (k // 2, d - 1), (k - 1, 7)):
        col = x[:, dd][lab == kk]
        assert col.numel() > 0
        assert float(med[kk, dd]) == float(torch.median(col)), (kk, dd)


@pytest.mark.parametrize("d,metric", [(32, _native.METRIC_EUCLID_QE), (8, _native.METRIC_EUCLID_QE),
                                      (16, _native.METRIC_MANHATTAN)])
def test_full_matrix_output_beyond_4gib(cuda, d, metric):
    """An output matrix beyond 4 GiB: its last rows equal a separate call on those rows, bit for bit,
    and a float64 evaluation to fp32 accuracy."""
    m = 36_864
    g = torch.Generator(device=cuda).manual_seed(47 + d)
    x = torch.randn((m, d), device=cuda, generator=g)
    y = torch.randn((m, d), device=cuda, generator=g)
    out = torch.full((m, m), -7.0, device=cuda)
    assert out.numel() * 4 > GIB4
    _native.pairwise(x, y, out, metric)
    tail = torch.empty((256, m), device=cuda)
    _native.pairwise(x[-256:], y, tail, metric)
    assert torch.equal(out[-256:].view(torch.int32), tail.view(torch.int32))
    r4 = GIB4 // (4 * m)
    mid = torch.empty((128, m), device=cuda)
    _native.pairwise(x[r4 - 64:r4 + 64], y, mid, metric)
    assert torch.equal(out[r4 - 64:r4 + 64].view(torch.int32), mid.view(torch.int32))
    p = 1.0 if metric == _native.METRIC_MANHATTAN else 2.0
    ref = torch.cdist(x[-256:].double(), y.double(), p=p)
    assert torch.allclose(tail.double(), ref, rtol=1e-4, atol=2e-3)
    assert float(out.min()) >= 0.0
