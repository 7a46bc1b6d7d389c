"""
Host-side tests that need no GPU: the estimator protocol and exception matrix of the reference's
tests/cluster/test_kmeans.py:18-34,68-100 and tests/spatial/test_distances.py:190-205 restated for
heat_amd, the DNDarray/array surface callers use, and the C ABI (every symbol of include/hkm.h is
exported; argument validation returns the documented codes before anything is launched).
"""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import heat_amd as ht
from heat_amd import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
IRIS = np.loadtxt(os.path.join(ROOT, "tests", "golden", "iris.csv"), delimiter=";", dtype=np.float32)


# ---- estimator protocol -----------------------------------------------------------------------
def test_clusterer_protocol():
    km = ht.cluster.KMeans()
    assert ht.is_estimator(km) and ht.is_clusterer(km)
    assert isinstance(km, ht.BaseEstimator) and isinstance(km, ht.ClusteringMixin)


def test_get_and_set_params():
    km = ht.cluster.KMeans()
    params = km.get_params()
    assert params == {"n_clusters": 8, "init": "random", "max_iter": 300, "tol": 1e-4, "random_state": None}
    params["n_clusters"] = 10
    km.set_params(**params)
    assert km.n_clusters == 10
    with pytest.raises(ValueError):
        km.set_params(foo="bar")
    assert "KMeans(" in repr(km)
    assert ht.cluster.KMeans(init="kmeans++").init == "probability_based"
    for attr in ("cluster_centers_", "labels_", "inertia_", "n_iter_", "functional_value_"):
        assert getattr(km, attr) is None


def test_exception_matrix():
    iris_split1 = ht.array(torch.from_numpy(IRIS), split=1)
    iris = ht.array(torch.from_numpy(IRIS), split=0)
    k = 3
    with pytest.raises(NotImplementedError):  # split = 1 is refused by the distance
        ht.cluster.KMeans(n_clusters=k).fit(iris_split1)
    with pytest.raises(ValueError):
        ht.cluster.KMeans(n_clusters=k, init="random_number").fit(iris_split1)
    with pytest.raises(NotImplementedError):
        ht.cluster.KMeans(n_clusters=k, init="batchparallel").fit(iris_split1)
    with pytest.raises(ValueError):
        ht.cluster.KMeans(n_clusters=k, init=np.array([1, 2, 3])).fit(iris_split1)
    with pytest.raises(ValueError):
        ht.cluster.KMeans(n_clusters=k).fit(iris_split1, oversampling=-1)
    with pytest.raises(ValueError):
        ht.cluster.KMeans(n_clusters=k).fit(iris_split1, iter_multiplier=-1)
    with pytest.raises(ValueError):
        ht.cluster.KMeans(n_clusters=k, init=ht.array([1, 2])).fit(iris_split1)
    with pytest.raises(NotImplementedError):
        ht.cluster.KMeans(n_clusters=k, init="probability_based").fit(iris_split1)
    with pytest.raises(ValueError):  # (K, D) mismatch
        ht.cluster.KMeans(n_clusters=k, init=ht.array(torch.zeros((2, 4)))).fit(iris)
    with pytest.raises(ValueError):
        ht.cluster.KMeans(n_clusters=k, init=ht.array(torch.zeros((3, 5)))).fit(iris)
    with pytest.raises(TypeError):  # fit wants a DNDarray
        ht.cluster.KMeans(n_clusters=k).fit(IRIS)
    with pytest.raises(ValueError):  # predict wants a DNDarray
        ht.cluster.KMeans(n_clusters=k).predict(IRIS)


def test_no_cpu_fallback():
    # data on the host: the product must refuse, not compute on the CPU
    iris = ht.array(torch.from_numpy(IRIS), split=0)
    init = ht.array(torch.from_numpy(IRIS[:3].copy()))
    with pytest.raises(RuntimeError, match="GPU only"):
        ht.cluster.KMeans(n_clusters=3, init=init, max_iter=2).fit(iris)
    with pytest.raises(RuntimeError, match="GPU only"):
        ht.spatial.cdist(iris, init, quadratic_expansion=True)


def test_cdist_exceptions():
    X = ht.ones((4, 4), split=1)
    Y = ht.zeros((4, 4))
    with pytest.raises(NotImplementedError):
        ht.spatial.cdist(X, quadratic_expansion=True)
    with pytest.raises(NotImplementedError):
        ht.spatial.cdist(X, Y, quadratic_expansion=True)
    with pytest.raises(NotImplementedError):
        ht.spatial.cdist(ht.ones((4, 4)), ht.zeros((4, 4), split=1), quadratic_expansion=True)
    Z = ht.ones((4, 6, 3))
    with pytest.raises(NotImplementedError):
        ht.spatial.cdist(Z, quadratic_expansion=True)
    with pytest.raises(NotImplementedError):
        ht.spatial.cdist(ht.ones((4, 4)), Z, quadratic_expansion=True)
    with pytest.raises(ValueError):
        ht.spatial.cdist(ht.ones((4, 4)), ht.ones((4, 5)), quadratic_expansion=True)
    with pytest.raises(RuntimeError):  # float64 has kernels of its own, but host data is still refused
        ht.spatial.cdist(ht.ones((4, 4), dtype=ht.float64), quadratic_expansion=True)
    with pytest.raises(NotImplementedError):
        ht.spatial.rbf(X)
    with pytest.raises(NotImplementedError):
        ht.spatial.manhattan(ht.ones((4, 4)), Z)


# ---- array surface ----------------------------------------------------------------------------
def test_array_and_dndarray_surface():
    t = torch.arange(12, dtype=torch.float32).view(4, 3)
    a = ht.array(t, split=0)
    assert a.larray.data_ptr() == t.data_ptr()  # shared, not copied
    assert a.shape == (4, 3) == a.gshape == a.lshape and a.split == 0 and a.dtype is ht.float32
    assert a.device == ht.cpu and a.comm.size == 1 and a.comm.rank == 0 and a.balanced
    assert not a.is_distributed() and a.ndim == 2 and a.size == 12 and len(a) == 4
    b = a.resplit(None)
    assert b.split is None and b.larray.data_ptr() != t.data_ptr()  # resplit copies
    c = a.astype(ht.int64)
    assert c.dtype is ht.int64 and c.larray.dtype == torch.int64
    assert a.copy().larray.data_ptr() != t.data_ptr()
    # DNDarray == "string" is False instead of raising (the reference relies on this)
    assert (a == "kmeans++") is False
    assert bool(ht.array(3.0) <= 4.0) and not bool(ht.array(5.0) <= 4.0)
    with pytest.raises(TypeError):
        bool(a)
    assert ht.array([1, 2]).shape == (2,)
    assert ht.zeros((2, 2)).larray.sum() == 0 and ht.ones((2, 2), dtype=ht.int32).dtype is ht.int32
    with pytest.raises(ValueError):
        ht.array(t, split=0, is_split=0)
    assert a[1:3].shape == (2, 3) and a[1:3].split == 0


def test_type_promotion():
    assert ht.promote_types(ht.int32, ht.float32) is ht.float32
    assert ht.promote_types(ht.int64, ht.float32) is ht.float64
    assert ht.promote_types(ht.int8, ht.uint8) is ht.int16
    assert ht.promote_types(ht.uint8, ht.uint8) is ht.uint8
    assert ht.promote_types("i8", "f4") is ht.float64
    assert ht.float32.torch_type() == torch.float32
    assert ht.iinfo(ht.int64).max == 9223372036854775807
    assert ht.heat_type_of(torch.zeros(1, dtype=torch.int16)) is ht.int16


def test_devices():
    assert str(ht.cpu) == "cpu:0" and ht.cpu.torch_device == "cpu"
    assert ht.get_device() == ht.cpu
    assert ht.sanitize_device("cpu") is ht.cpu
    with pytest.raises(ValueError):
        ht.sanitize_device("tpu")


# ---- C ABI -----------------------------------------------------------------------------------
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "hkm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hkm_[a-z0-9_]+)\s*\(", text)))


def test_bench_hooks_are_declared_apart_and_exported():
    """include/hkm_bench.h: the measuring hooks live in libhkm.so, the microbenchmarks in a library of their own
    that the product never loads; include/hkm.h declares none of them."""
    from heat_amd.utils import benchhooks

    text = open(os.path.join(ROOT, "include", "hkm_bench.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(hkm_[a-z0-9_]+)\s*\(", text)))
    assert names == sorted(benchhooks.SIGNATURES)
    assert not set(names) & set(_declared_symbols())
    lib, blib = benchhooks.hkm(), benchhooks.bench()
    for name, (home, _, _) in benchhooks.SIGNATURES.items():
        assert hasattr(lib if home == "hkm" else blib, name), name
        if home == "bench":
            assert not hasattr(lib, name), f"{name} must not be part of the product library"


def test_library_exports_every_declared_symbol():
    lib = _native.load()
    names = _declared_symbols()
    assert len(names) >= 25
    for name in names:
        assert hasattr(lib, name), name
        assert name in _native.SIGNATURES, f"{name} has no ctypes signature"
    assert sorted(_native.SIGNATURES) == names
    assert lib.hkm_version() >= 100


def test_workspace_and_kernel_selection():
    assert _native.workspace_bytes(-1, 3, 8, 3) == 0
    assert _native.workspace_bytes(10, 0, 8, 3) == 0
    a = _native.workspace_bytes(10_000_000, 32, 256, _native.WS_LLOYD)
    b = _native.workspace_bytes(10_000_000, 32, 256, _native.WS_LLOYD | _native.WS_SSE)
    assert 0 < a < b and b - a >= 40_000_000 and a % 256 == 0
    assert _native.assign_kernel_name(200_000_000, 3, 8).startswith("valu")
    assert _native.assign_kernel_name(100_000, 8, 16).startswith("valu")
    assert _native.assign_kernel_name(10_000_000, 32, 256) == "mfma_resident"
    assert _native.assign_kernel_name(1 << 20, 64, 1024) == "mfma_tiled"
    assert _native.assign_kernel_name(2_000_000, 512, 1024) == "mfma_stream"
    assert _native.lloyd_kernel_name(200_000_000, 3, 8) == "lloyd_small"
    assert _native.lloyd_kernel_name(10_000_000, 32, 256) == "lloyd_mfma_resident"
    assert _native.lloyd_kernel_name(10_000_000, 64, 512) == "mfma_tiled+update"  # accumulators exceed LDS
    # steps that may run without storing labels: those of the two vector kernels
    for d, k, opt in ((3, 8, True), (8, 16, True), (32, 8, True), (64, 12, True), (128, 8, False), (96, 32, False),
                      (32, 32, False), (32, 256, False), (16, 32, False), (512, 8, False), (8, 64, False)):
        assert _native.lloyd_step_labels_optional(10_000_000, d, k) == opt, (d, k)
    # few clusters of 17 to 64 features: the vector kernel, for the step and for the assignment alone
    for d, k, few in ((32, 8, True), (17, 1, True), (40, 16, True), (64, 12, True), (64, 13, False), (44, 16, False),
                      (16, 8, False), (65, 8, False), (32, 17, False)):
        assert (_native.lloyd_kernel_name(10_000_000, d, k) == "lloyd_few") == few, (d, k)
        assert (_native.assign_kernel_name(10_000_000, d, k) == "valu_wide") == few, (d, k)
    assert _native.lloyd_kernel_name(2_000_000, 512, 1024) == "mfma_stream+update"


def test_argument_validation_happens_on_the_host():
    lib = _native.load()
    P = ctypes.c_void_p
    good, ws = P(4096), P(1 << 20)  # never dereferenced: every call below fails validation first
    big = 1 << 30

    def err():
        return lib.hkm_last_error().decode()

    assert lib.hkm_assign_f32(None, 10, 3, 3, good, 8, 3, good, None, ws, big, None) == _native.HKM_EINVAL
    assert "X is NULL" in err()
    assert lib.hkm_assign_f32(good, -1, 3, 3, good, 8, 3, good, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_assign_f32(good, 10, 0, 3, good, 8, 3, good, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_assign_f32(good, 10, 3, 3, good, 0, 3, good, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_assign_f32(good, 10, 3, 2, good, 8, 3, good, None, ws, big, None) == _native.HKM_EINVAL
    assert "leading dimension" in err()
    assert lib.hkm_assign_f32(P(4098), 10, 3, 3, good, 8, 3, good, None, ws, big, None) == _native.HKM_EINVAL
    assert "aligned" in err()
    assert lib.hkm_assign_f32(good, 10, 3, 3, good, 8, 3, None, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_assign_f32(good, 10, 3, 3, good, 8, 3, good, None, None, 0, None) == _native.HKM_EWORKSPACE
    assert lib.hkm_assign_f32(good, 10, 3, 3, good, 8, 3, good, None, ws, 16, None) == _native.HKM_EWORKSPACE
    assert "too small" in err()
    assert lib.hkm_assign_f32(good, 10, 3, 3, good, 8, 3, good, None, P((1 << 20) + 8), big, None) == _native.HKM_EWORKSPACE
    assert lib.hkm_update_f32(good, 10, 3, 3, None, 8, good, 3, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_update_f32(good, 10, 3, 3, good, 8, good, 2, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_update_f32(good, 10, 3, 3, good, 8, good, 3, None, ws, 8, None) == _native.HKM_EWORKSPACE
    assert lib.hkm_lloyd_step_f32(good, 10, 3, 3, good, good, 8, good, good, None, ws, big, None) == _native.HKM_EINVAL
    assert "alias" in err()
    assert lib.hkm_lloyd_step_f32(good, 10, 3, 3, good, P(8192), 8, good, None, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_shift_f32(None, good, 8, 3, good, None) == _native.HKM_EINVAL
    assert lib.hkm_shift_f32(good, good, 0, 3, good, None) == _native.HKM_EINVAL
    assert lib.hkm_cdist_f32(good, 4, 3, good, 4, 3, 3, good, 3, 1, None) == _native.HKM_EINVAL  # ldo < Nn
    assert lib.hkm_cdist_f32(good, -4, 3, good, 4, 3, 3, good, 4, 1, None) == _native.HKM_EINVAL
    assert lib.hkm_pairwise_f32(good, 4, 3, good, 4, 3, 3, good, 4, 9, 1.0, None) == _native.HKM_EINVAL  # metric
    assert lib.hkm_pairwise_f32(good, 4, 3, good, 4, 3, 3, good, 4, _native.METRIC_GAUSS, 0.0, None) == _native.HKM_EINVAL
    assert "sigma" in err()
    assert lib.hkm_widen_labels_i64(None, 4, good, None) == _native.HKM_EINVAL
    assert lib.hkm_assign_f64(P(4100), 10, 3, 3, good, 8, 3, good, None, None) == _native.HKM_EINVAL
    assert "8-byte" in err()
    assert lib.hkm_assign_f64(good, 10, 3, 2, good, 8, 3, good, None, None) == _native.HKM_EINVAL
    assert lib.hkm_update_f64(good, 10, 3, 3, good, 8, good, 3, None, ws, 8, None) == _native.HKM_EWORKSPACE
    assert lib.hkm_lloyd_step_f64(good, 10, 3, 3, good, good, 8, good, good, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_shift_f64(None, good, 8, 3, good, None) == _native.HKM_EINVAL
    assert lib.hkm_functional_value_f64(good, -1, good, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_pairwise_f64(good, 4, 3, good, 4, 3, 3, good, 4, 9, 1.0, None) == _native.HKM_EINVAL
    assert lib.hkm_min_dist_sum_f32(good, -1, good, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_min_dist_sum_f32(good, 8, good, None, 0, None) == _native.HKM_EWORKSPACE
    assert lib.hkm_sample_select_f32(good, good, 8, good, 0.0, good, 4, good, ws, big, None) == _native.HKM_EINVAL
    assert "oversampling" in err()
    assert lib.hkm_sample_select_f32(good, None, 8, good, 2.0, good, 4, good, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_sample_select_f32(good, good, 8, good, 2.0, good, -4, good, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_sample_select_f32(good, good, 8, good, 2.0, good, 4, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_label_counts_i64(good, 8, 0, good, None) == _native.HKM_EINVAL
    assert lib.hkm_label_counts_i64(None, 8, 4, good, None) == _native.HKM_EINVAL
    assert lib.hkm_assign_l1_f32(None, 10, 3, 3, good, 8, 3, good, None, None) == _native.HKM_EINVAL
    assert lib.hkm_assign_l1_f32(good, 10, 3, 2, good, 8, 3, good, None, None) == _native.HKM_EINVAL
    assert lib.hkm_assign_l1_f32(good, 10, 3, 3, good, 8, 3, None, None, None) == _native.HKM_EINVAL
    assert lib.hkm_assign_l1_f32(good, 0, 3, 3, good, 8, 3, None, None, None) == _native.HKM_OK
    assert lib.hkm_closest_rows_l1_f32(good, 0, 3, 3, good, 2, 3, good, None, ws, big, None) == _native.HKM_EINVAL
    assert "empty" in err()
    assert lib.hkm_closest_rows_l1_f32(good, 10, 3, 3, good, 2, 3, None, None, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_closest_rows_l1_f32(good, 10, 3, 3, good, 2, 3, good, None, ws, 16, None) == _native.HKM_EWORKSPACE
    assert lib.hkm_update_median_f32(good, 10, 3, 3, good, 4, None, None, good, 3, None, 2, 0, ws, big, None) == _native.HKM_EINVAL
    assert "mode" in err()
    assert lib.hkm_update_median_f32(good, 10, 3, 3, None, 4, None, None, good, 3, None, 0, 0, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_update_median_f32(good, 10, 3, 3, good, 4, None, None, good, 2, None, 0, 0, ws, big, None) == _native.HKM_EINVAL
    assert lib.hkm_update_median_f32(good, 10, 3, 3, good, 4, None, None, good, 3, None, 0, 0, ws, 64, None) == _native.HKM_EWORKSPACE
    assert lib.hkm_update_median_f32(good, 1 << 31, 3, 3, good, 4, None, None, good, 3, None, 0, 0, ws, big, None) == _native.HKM_EUNSUPPORTED
    assert lib.hkm_functional_value_f32(good, -1, good, ws, big, None) == _native.HKM_EINVAL
    # zero-sized problems succeed without touching the device
    assert lib.hkm_widen_labels_i64(good, 0, good, None) == _native.HKM_OK
    assert lib.hkm_cdist_f32(None, 0, 3, good, 4, 3, 3, good, 4, 1, None) == _native.HKM_OK
    assert err() == ""


def test_validation_layer_under_address_sanitizer():
    # heat_amd/csrc/Makefile, target asan-host: hkm_api.hip with its host code instrumented, linked with the
    # objects of the ordinary build and driven by tests/host/hkm_api_check.cpp, which only makes calls the
    # library refuses (or finishes) before anything reaches the device
    import shutil
    import subprocess

    csrc = os.path.join(os.path.dirname(_native.lib_path()))
    if not shutil.which("make") or not os.path.exists("/opt/rocm/bin/hipcc"):
        pytest.skip("no toolchain to build the instrumented library with")
    if not os.path.exists(os.path.join(csrc, "hkm_knn.o")):
        pytest.skip("the objects of the ordinary build are not there (make -C heat_amd/csrc)")
    run = subprocess.run(["make", "-C", csrc, "asan-host"], capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-2000:]
    assert "all checks passed" in run.stdout
    assert "AddressSanitizer" not in run.stdout + run.stderr


def test_sizes_no_device_holds_are_refused():
    lib = _native.load()
    P = ctypes.c_void_p
    good, ws = P(4096), P(1 << 20)
    assert lib.hkm_assign_f32(good, (1 << 40) + 1, 3, 3, good, 8, 3, good, None, ws, 1 << 30, None) == _native.HKM_EUNSUPPORTED
    assert "2^40" in lib.hkm_last_error().decode()
    assert lib.hkm_assign_f32(good, 10, 1 << 21, 1 << 21, good, 1 << 20, 1 << 21, good, None, ws, 1 << 30, None) == _native.HKM_EUNSUPPORTED
    assert lib.hkm_workspace_bytes((1 << 40) + 1, 3, 8, 1) == 0
    assert lib.hkm_workspace_bytes(1 << 62, (1 << 31) - 1, (1 << 31) - 1, 3) == 0
    assert lib.hkm_workspace_bytes(1 << 40, 3, 8, 3) > (1 << 40)


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "_LIB_PATH", "/nonexistent/libhkm.so")
    with pytest.raises(ImportError, match="no CPU fallback"):
        _native.load()


def test_batchparallel_kmeans_surface():
    # tests/cluster/test_batchparallelclustering.py:46-84,135-190 of the reference (constructor part)
    from heat_amd.cluster.batchparallelclustering import _BatchParallelKCluster

    bp = ht.cluster.BatchParallelKMeans()
    assert ht.is_estimator(bp) and ht.is_clusterer(bp)
    params = bp.get_params()
    assert params == {"n_clusters": 8, "init": "k-means++", "max_iter": 300, "tol": 1e-4, "random_state": None,
                      "n_procs_to_merge": None}
    params["n_clusters"] = 10
    params["n_procs_to_merge"] = 4
    bp.set_params(**params)
    assert bp.n_clusters == 10
    with pytest.raises(TypeError):
        _BatchParallelKCluster(2, 10, "++", 100, 1e-2, random_state=3.14, n_procs_to_merge=None)
    with pytest.warns(UserWarning):
        _BatchParallelKCluster(3, 10, "++", 100, 1e-2, random_state=None, n_procs_to_merge=None)
    with pytest.raises(TypeError):
        _BatchParallelKCluster(2, 10, "++", 100, 1e-2, random_state=None, n_procs_to_merge=2.7183)
    with pytest.raises(ValueError):
        _BatchParallelKCluster(2, 10, "++", 100, 1e-2, random_state=None, n_procs_to_merge=1)
    for kwargs, exc in (({"n_clusters": -1}, ValueError), ({"n_clusters": "abc"}, TypeError),
                        ({"max_iter": -10}, ValueError), ({"max_iter": 0.1}, TypeError),
                        ({"tol": -0.5}, ValueError), ({"tol": "abc"}, TypeError), ({"init": "abc"}, ValueError),
                        ({"init": 3.14}, TypeError), ({"init": "random"}, NotImplementedError)):
        with pytest.raises(exc):
            ht.cluster.BatchParallelKMeans(**kwargs)
    with pytest.raises(TypeError):
        bp.fit("abc")
    with pytest.raises(RuntimeError):  # host data: refused, not computed on the CPU
        ht.cluster.BatchParallelKMeans(n_clusters=2).fit(ht.array(torch.rand(16, 2), split=0))
    with pytest.raises(RuntimeError):
        ht.cluster.KMeans(n_clusters=2, init="probability_based").fit(ht.array(torch.rand(16, 2), split=0))


def test_manhattan_estimators_surface():
    # tests/cluster/test_kmedians.py / test_kmedoids.py of the reference: protocol and parameters
    kmed = ht.cluster.KMedians()
    assert ht.is_estimator(kmed) and ht.is_clusterer(kmed)
    assert kmed.get_params() == {"n_clusters": 8, "init": "random", "max_iter": 300, "tol": 1e-4, "random_state": None}
    kmedoid = ht.cluster.KMedoids()
    assert ht.is_estimator(kmedoid) and ht.is_clusterer(kmedoid)
    params = kmedoid.get_params()
    assert params == {"n_clusters": 8, "init": "random", "max_iter": 300, "random_state": None}
    params["n_clusters"] = 10
    kmedoid.set_params(**params)
    assert kmedoid.n_clusters == 10 and kmedoid.tol == 0.0
    assert ht.cluster.KMedians(init="kmedians++").init == "probability_based"
    assert ht.cluster.KMedoids(init="kmedoids++").init == "probability_based"
    bp = ht.cluster.BatchParallelKMedians()
    assert bp.get_params()["init"] == "k-medians++" and bp._p == 1
    with pytest.raises(NotImplementedError):
        ht.cluster.BatchParallelKMedians(init="random")
    with pytest.raises(ValueError):
        ht.cluster.BatchParallelKMedians(init="k-means++")
    host = ht.array(torch.rand(16, 2), split=0)
    for est in (ht.cluster.KMedians(n_clusters=2), ht.cluster.KMedoids(n_clusters=2),
                ht.cluster.BatchParallelKMedians(n_clusters=2)):
        with pytest.raises(RuntimeError):  # host data is refused, never computed on the CPU
            est.fit(host)
    assert _native.workspace_bytes(1000, 4, 8, _native.WS_MEDIAN) > 8 * 4 * 256 * 4


def test_load_csv():
    # the reference's clustering tests start from ht.load(<iris.csv>, sep=";", split=...)
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "iris.csv")
    a = ht.load(path, sep=";", split=0)
    assert a.shape == (150, 4) and a.dtype is ht.float32 and a.split == 0
    assert np.allclose(a.larray.numpy(), IRIS)
    b = ht.load_csv(path, sep=";", header_lines=10, dtype=ht.float64, split=1)
    assert b.shape == (140, 4) and b.dtype is ht.float64 and b.split == 1
    with pytest.raises(TypeError):
        ht.load_csv(12)
    with pytest.raises(TypeError):
        ht.load_csv(path, sep=3)
    with pytest.raises(TypeError):
        ht.load_csv(path, header_lines="3")
    with pytest.raises(ValueError):
        ht.load("data.txt")
    with pytest.raises(RuntimeError):
        ht.load("data.h5")


def test_knn_classifier_surface():
    """tests/classification/test_knn.py:50-76 of the reference: the exception matrix of fit and the one-hot
    utility, plus the estimator protocol.  No kernel runs."""
    knn_cls = ht.classification.KNeighborsClassifier
    a, b, c = ht.zeros((3,)), ht.zeros((3, 2)), ht.zeros((2, 2, 2))
    for x, y in ((a, b), (b, c), (c, a)):
        with pytest.raises(ValueError):
            knn_cls(n_neighbors=1).fit(x, y)
    with pytest.raises(TypeError):
        knn_cls().fit(torch.zeros((3, 2)), b)
    one_hot = knn_cls.one_hot_encoding(ht.array([1, 2, 3, 4]))
    want = torch.tensor([[0, 1, 0, 0, 0], [0, 0, 1, 0, 0], [0, 0, 0, 1, 0], [0, 0, 0, 0, 1]], dtype=torch.float32)
    assert torch.equal(one_hot.larray, want)
    knn = knn_cls(n_neighbors=3)
    assert ht.is_estimator(knn) and ht.is_classifier(knn) and not ht.is_clusterer(knn)
    assert knn.get_params()["n_neighbors"] == 3 and knn.get_params()["effective_metric_"] is ht.spatial.cdist
    with pytest.raises(RuntimeError):
        knn.predict(b)
    # any metric callable is accepted (the full-matrix route of the reference); on host tensors it ends where
    # every compute call ends: there is no CPU path
    other = knn_cls(n_neighbors=1, effective_metric_=ht.spatial.manhattan)
    other.fit(b, ht.zeros((3,)))
    with pytest.raises(RuntimeError):
        other.predict(b)


def test_argument_validation_of_the_neighbour_silhouette_and_laplacian_entry_points():
    """Every call fails validation on the host, before anything touches a device."""
    lib = _native.load()
    P = ctypes.c_void_p
    good, other, ws = P(4096), P(8192), P(1 << 20)
    big = 1 << 30

    def err():
        return lib.hkm_last_error().decode()

    einval, eunsup, ews = _native.HKM_EINVAL, _native.HKM_EUNSUPPORTED, _native.HKM_EWORKSPACE
    # hkm_knn_f32(Q, M, ldq, X, N, ldx, D, k, idx, ldi, dist, ldd, ws, ws_bytes, stream)
    assert lib.hkm_knn_f32(good, 4, 3, other, 10, 3, 3, 11, good, 11, None, 11, ws, big, None) == einval
    assert "k = 11" in err()
    assert lib.hkm_knn_f32(good, 4, 3, other, 10, 3, 3, 0, good, 1, None, 1, ws, big, None) == einval
    assert lib.hkm_knn_f32(good, 4, 3, other, 0, 3, 3, 1, good, 1, None, 1, ws, big, None) == einval
    assert "empty" in err()
    assert lib.hkm_knn_f32(good, 4, 2, other, 10, 3, 3, 2, good, 2, None, 2, ws, big, None) == einval
    assert "leading dimension of Q" in err()
    assert lib.hkm_knn_f32(good, 4, 3, other, 10, 3, 3, 2, good, 1, None, 2, ws, big, None) == einval
    assert "leading dimension of idx" in err()
    assert lib.hkm_knn_f32(good, 4, 3, other, 10, 3, 3, 2, None, 2, None, 2, ws, big, None) == einval
    assert lib.hkm_knn_f32(good, 4, 3, other, 3000, 3, 3, 2000, good, 2000, None, 2000, ws, big, None) == eunsup
    assert lib.hkm_knn_f32(good, 4, 3, other, 10, 3, 3, 2, good, 2, None, 2, ws, 16, None) == ews
    assert lib.hkm_knn_f32(good, 4, 3, other, 10, 3, 3, 2, good, 2, None, 2, None, 0, None) == ews
    assert lib.hkm_knn_workspace_bytes(4, 0) == 0 and lib.hkm_knn_workspace_bytes(4, 10) >= 4 * 8
    # a few query rows against many reference rows: room for the per-split lists
    assert lib.hkm_knn_workspace_bytes(64, 1 << 20) > lib.hkm_knn_workspace_bytes(64, 100)
    # hkm_knn_vote_f32(idx, M, k, ldi, Y, N, C, ldy, classes, stream)
    assert lib.hkm_knn_vote_f32(good, 4, 2, 1, other, 10, 3, 3, good, None) == einval
    assert lib.hkm_knn_vote_f32(good, 4, 2, 2, other, 10, 3, 2, good, None) == einval
    assert lib.hkm_knn_vote_f32(good, 4, 2, 2, other, 10, 0, 3, good, None) == einval
    assert lib.hkm_knn_vote_f32(good, 4, 2, 2, other, 10, 3, 3, None, None) == einval
    # hkm_cluster_distance_sums_f32(X, N, D, ldx, perm, offsets, K, S, lds, stream)
    assert lib.hkm_cluster_distance_sums_f32(good, 10, 3, 3, None, other, 2, good, 2, None) == einval
    assert lib.hkm_cluster_distance_sums_f32(good, 10, 3, 3, other, other, 2, good, 1, None) == einval
    assert lib.hkm_cluster_distance_sums_f32(good, 10, 3, 3, other, other, 70000, good, 70000, None) == eunsup
    # hkm_silhouette_finish_f32(S, N, K, lds, labels, counts, out, stream)
    assert lib.hkm_silhouette_finish_f32(good, 10, 3, 2, other, other, good, None) == einval
    assert lib.hkm_silhouette_finish_f32(good, 10, 3, 3, other, None, good, None) == einval
    # hkm_laplacian_f32(S, N, lds, definition, mode, weighted, eps, L, ldl, degree, stream)
    assert lib.hkm_laplacian_f32(good, 10, 10, 2, 0, 1, 1.0, good, 10, other, None) == einval
    assert "definition" in err()
    assert lib.hkm_laplacian_f32(good, 10, 10, 0, 3, 1, 1.0, good, 10, other, None) == einval
    assert lib.hkm_laplacian_f32(good, 10, 9, 0, 0, 1, 1.0, good, 10, other, None) == einval
    assert lib.hkm_laplacian_f32(good, 10, 10, 0, 0, 1, 1.0, good, 10, None, None) == einval
    big = 65535 * 256 + 1
    assert lib.hkm_laplacian_f32(good, big, big, 0, 0, 1, 1.0, good, big, other, None) == eunsup
    assert lib.hkm_laplacian_f64(good, big, big, 0, 0, 1, 1.0, good, big, other, None) == eunsup
    assert lib.hkm_laplacian_f64(good, 10, 10, 0, 0, 1, 1.0, good, 10, None, None) == einval
