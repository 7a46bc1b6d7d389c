"""
hkm_assign_static_f32 -- the assignment on the library's built-in scratch array, for callers that cannot
allocate -- against hkm_assign_f32 with a caller-owned workspace: labels and minimum squared distances
must be bit-identical (same kernels, same launch geometry, only the scratch address differs), on two calls
in a row of which the second has the smaller input, so anything a call leaves behind in the shared array
would show.  Shapes are chosen to use the scratch: the tiled kernel reads the squared centroid norms from
it, the streaming kernel (D > 128, or more centroids than LDS holds) also merges its partial minima through 8-byte keys kept there.
"""
import pytest
import torch

from heat_amd import _native

pytestmark = pytest.mark.gpu


def _data(n, d, k, seed):
    g = torch.Generator().manual_seed(seed)
    c = torch.randn((k, d), generator=g) * 3.0
    x = c[torch.randint(0, k, (n,), generator=g)] + torch.randn((n, d), generator=g)
    return x.contiguous(), c.contiguous()


def _both(x, c, dev):
    xs, cs = x.to(dev), c.to(dev)
    n = x.shape[0]
    out = []
    for static in (False, True):
        lab = torch.full((n,), -7, dtype=torch.int32, device=dev)
        md = torch.full((n,), -1.0, dtype=torch.float32, device=dev)
        if static:
            _native.assign_static(xs, cs, lab, md)
        else:
            _native.assign(xs, cs, lab, md, _native.Workspace(dev))
        torch.cuda.synchronize()
        out.append((lab.cpu(), md.cpu()))
    return out


# (first call, second smaller call) per kernel family that keeps something in the scratch
CASES = [
    ((6000, 64, 1024), (1500, 48, 700)),      # tiled matrix-core kernel: norms
    ((5000, 130, 300), (900, 100, 70)),       # streaming matrix-core kernel: norms + merge keys
    ((5000, 130, 300), (3000, 64, 1024)),     # streaming, then tiled over the same bytes
    ((4096, 32, 256), (1000, 3, 8)),          # kernels that need no scratch at all
]


@pytest.mark.parametrize("first,second", CASES)
def test_static_scratch_assign_equals_workspace_assign(cuda, first, second):
    assert _native.load().hkm_static_scratch_bytes() == 16 << 20
    for i, (n, d, k) in enumerate((first, second)):
        print(f"assign_static call {i}: n={n} d={d} k={k} kernel={_native.assign_kernel_name(n, d, k)}", flush=True)
        x, c = _data(n, d, k, seed=11 * n + d + k)
        (lab_w, md_w), (lab_s, md_s) = _both(x, c, cuda)
        assert lab_w.min() >= 0 and lab_w.max() < k
        assert torch.equal(lab_s, lab_w)
        assert torch.equal(md_s.view(torch.int32), md_w.view(torch.int32))


def test_static_scratch_assign_without_min_d2_and_strided_rows(cuda):
    n, d, k = 3000, 100, 257
    x, c = _data(n, d + 4, k, seed=5)
    xs, cs = x.to(cuda)[:, :d], c.to(cuda)[:, :d]
    lab_w = torch.full((n,), -7, dtype=torch.int32, device=cuda)
    lab_s = torch.full((n,), -7, dtype=torch.int32, device=cuda)
    _native.assign(xs, cs, lab_w, None, _native.Workspace(cuda))
    _native.assign_static(xs, cs, lab_s, None)
    torch.cuda.synchronize()
    assert torch.equal(lab_s, lab_w)


def test_static_scratch_assign_rejects_what_does_not_fit(cuda):
    # D > 128 keeps 8 bytes per row in the scratch: 3M rows need 24 MB, the array holds 16 MiB
    n, d, k = 3_000_000, 130, 4
    assert _native.workspace_bytes(n, d, k, _native.WS_ASSIGN) > 16 << 20
    x = torch.zeros((n, d), dtype=torch.float32, device=cuda)
    c = torch.zeros((k, d), dtype=torch.float32, device=cuda)
    lab = torch.zeros((n,), dtype=torch.int32, device=cuda)
    with pytest.raises(_native.HkmError) as e:
        _native.assign_static(x, c, lab, None)
    assert e.value.code == _native.HKM_EUNSUPPORTED
    assert "scratch" in str(e.value)
    # the same rows with D <= 128 need no per-row scratch and run
    _native.assign_static(x[:, :64], c[:, :64], lab, None)
    torch.cuda.synchronize()
    assert int(lab.max()) == 0


@pytest.mark.parametrize("n,d,k", [(6000, 64, 1024), (4096, 32, 256), (5000, 130, 300)])
def test_static_scratch_assign_under_graph_capture(cuda, n, d, k):
    """After the documented warm-up (hkm_static_scratch_bytes resolves the array's address outside capture)
    the entry point only enqueues kernels: one call captured into a HIP graph and replayed several times, with
    eager work and synchronisations between the replays, gives the workspace path's bits every time."""
    assert _native.load().hkm_static_scratch_bytes() == 16 << 20  # the warm-up, device current
    print(f"assign_static under capture: n={n} d={d} k={k} kernel={_native.assign_kernel_name(n, d, k)}", flush=True)
    x, c = _data(n, d, k, seed=3 * n + d)
    xs, cs = x.to(cuda), c.to(cuda)
    lab_w = torch.empty((n,), dtype=torch.int32, device=cuda)
    md_w = torch.empty((n,), dtype=torch.float32, device=cuda)
    _native.assign(xs, cs, lab_w, md_w, _native.Workspace(cuda))
    lab = torch.empty((n,), dtype=torch.int32, device=cuda)
    md = torch.empty((n,), dtype=torch.float32, device=cuda)
    _native.assign_static(xs, cs, lab, md)  # every kernel of the call has run once before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _native.assign_static(xs, cs, lab, md)
    for rep in range(4):
        lab.fill_(-7)
        md.fill_(-1.0)
        if rep % 2:
            # eager work of the same library in between, on the shared scratch array
            other = torch.empty((1000,), dtype=torch.int32, device=cuda)
            _native.assign_static(xs[:1000], cs, other, None)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(lab, lab_w), rep
        assert torch.equal(md.view(torch.int32), md_w.view(torch.int32)), rep
