"""
ctypes binding of libhkm, the C-ABI library holding the gfx950 kernels (see include/hkm.h).

The library is built in-tree (``heat_amd/csrc/libhkm.so``) by ``heat_amd/csrc/Makefile``.  There
is no fallback: if the library is missing, every compute entry point raises.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_int32, c_int64, c_size_t, c_void_p
from typing import Optional

import torch

from . import _f64_paths

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libhkm.so")
_lib: Optional[ctypes.CDLL] = None

LIB_VERSION = 308  # hkm_version() this binding was written for: major * 10000 + minor * 100 + patch
HKM_OK, HKM_EINVAL, HKM_EWORKSPACE, HKM_EHIP, HKM_EUNSUPPORTED = 0, -1, -2, -3, -4
WS_ASSIGN, WS_UPDATE, WS_LLOYD, WS_SSE, WS_MEDIAN, WS_F64, WS_FIT = 1, 2, 3, 4, 8, 16, 32

# name -> (restype, argtypes); must list every symbol declared in include/hkm.h
SIGNATURES = {
    "hkm_version": (ctypes.c_int, []),
    "hkm_last_error": (c_char_p, []),
    "hkm_workspace_bytes": (c_size_t, [c_int64, c_int32, c_int32, c_int32]),
    "hkm_assign_kernel_name": (c_char_p, [c_int64, c_int32, c_int32]),
    "hkm_lloyd_kernel_name": (c_char_p, [c_int64, c_int32, c_int32]),
    "hkm_assign_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_int64,
                                      c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_assign_labels64_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_int64,
                                               c_void_p, c_void_p, c_void_p]),
    "hkm_static_scratch_bytes": (c_size_t, []),
    "hkm_assign_static_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_int64,
                                             c_void_p, c_void_p, c_void_p]),
    "hkm_update_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_void_p,
                                      c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_lloyd_step_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_void_p, c_int32,
                                          c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_lloyd_step_labels64_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_void_p, c_int32,
                                                   c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_lloyd_fit_supported": (ctypes.c_int, [c_int64, c_int32, c_int32]),
    "hkm_lloyd_step_labels_optional": (ctypes.c_int, [c_int64, c_int32, c_int32]),
    "hkm_lloyd_fit_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_int32, c_int32,
                                         ctypes.c_double, c_void_p, c_void_p, c_void_p, c_void_p, ctypes.c_uint64,
                                         c_void_p, c_size_t, c_void_p]),
    "hkm_shift_f32": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p]),
    "hkm_functional_value_f32": (ctypes.c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_cdist_f32": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int32,
                                     c_void_p, c_int64, c_int32, c_void_p]),
    "hkm_pairwise_f32": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int32,
                                        c_void_p, c_int64, c_int32, ctypes.c_float, c_void_p]),
    "hkm_min_dist_sum_f32": (ctypes.c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_min_merge_sum_f32": (ctypes.c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_sample_select_f32": (ctypes.c_int, [c_void_p, c_void_p, c_int64, c_void_p, ctypes.c_float, c_void_p,
                                             c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_label_counts_i64": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_void_p, c_void_p]),
    "hkm_seed_plus_plus_f32": (ctypes.c_int, [c_void_p, c_int32, c_int32, c_int64, c_void_p, c_int32, c_void_p,
                                              c_int32, c_int32, c_void_p, c_void_p]),
    "hkm_seed_plus_plus_rows_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int64, c_void_p,
                                                   c_int32, c_int32, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_assign_l1_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_int64,
                                         c_void_p, c_void_p, c_void_p]),
    "hkm_closest_rows_l1_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_int64,
                                               c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_update_median_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_void_p,
                                             c_void_p, c_void_p, c_int64, c_void_p, c_int32, c_int32, c_void_p,
                                             c_size_t, c_void_p]),
    "hkm_update_median_q64_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_void_p,
                                                 c_void_p, c_void_p, c_int64, c_void_p, c_int32, c_int32, c_void_p,
                                                 c_void_p, c_size_t, c_void_p]),
    "hkm_closest_rows_l1_q64_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_void_p,
                                                   c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_knn_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "hkm_knn_f32": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int32, c_int32, c_void_p,
                                   c_int64, c_void_p, c_int64, c_void_p, c_size_t, c_void_p]),
    "hkm_knn_vote_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int64, c_int32, c_int64,
                                        c_void_p, c_void_p]),
    "hkm_cluster_distance_sums_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_void_p, c_int32,
                                                     c_void_p, c_int64, c_void_p]),
    "hkm_silhouette_finish_f32": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_void_p, c_void_p,
                                                 c_void_p]),
    "hkm_laplacian_f32": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_int32, c_int32, c_int32, ctypes.c_float,
                                         c_void_p, c_int64, c_void_p, c_void_p]),
    "hkm_laplacian_f64": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_int32, c_int32, c_int32, ctypes.c_double,
                                         c_void_p, c_int64, c_void_p, c_void_p]),
    "hkm_assign_f64": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_int64,
                                      c_void_p, c_void_p, c_void_p]),
    "hkm_update_f64": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_int32, c_void_p,
                                      c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_lloyd_step_f64": (ctypes.c_int, [c_void_p, c_int64, c_int32, c_int64, c_void_p, c_void_p, c_int32,
                                          c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_shift_f64": (ctypes.c_int, [c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p]),
    "hkm_functional_value_f64": (ctypes.c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hkm_pairwise_f64": (ctypes.c_int, [c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64, c_int32,
                                        c_void_p, c_int64, c_int32, ctypes.c_double, c_void_p]),
    "hkm_widen_labels_i64": (ctypes.c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
}


class HkmError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"libhkm error {code}: {message}")
        self.code = code


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load libhkm once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                f"{_LIB_PATH} is missing: build it with `make -C heat_amd/csrc` "
                "(or __graft_entry__.build()). heat_amd has no CPU fallback."
            )
        lib = ctypes.CDLL(_LIB_PATH)
        lib.hkm_version.restype = ctypes.c_int
        have = int(lib.hkm_version())
        missing = [name for name in SIGNATURES if not hasattr(lib, name)]
        if have != LIB_VERSION or missing:
            raise ImportError(
                f"{_LIB_PATH} is version {have} but this binding needs {LIB_VERSION}"
                + (f" (missing: {', '.join(missing[:5])})" if missing else "")
                + ": rebuild it with `make -C heat_amd/csrc`."
            )
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def last_error() -> str:
    return load().hkm_last_error().decode()


def check(rc: int) -> None:
    if rc != HKM_OK:
        raise HkmError(rc, last_error())


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else c_void_p(t.data_ptr())


def _stream():
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "heat_amd computes on the GPU only: got a tensor on "
                f"'{t.device}'. Create the DNDarray with device='gpu'."
            )


def _require_rows(*mats: Optional[torch.Tensor]) -> None:
    """The library reads matrices row by row with unit stride inside a row: anything else (a transposed
    view, a column slice with a step) would be read as different numbers, so it is refused here."""
    for t in mats:
        if t is None or t.dim() != 2:
            continue
        if t.shape[1] > 1 and t.stride(1) != 1:
            raise ValueError("matrix rows must be contiguous (stride 1 along the last axis); call .contiguous()")
        if t.shape[0] > 1 and t.stride(0) < t.shape[1]:
            raise ValueError("matrix rows overlap (row stride below the row length)")


def _require_dense(*mats: Optional[torch.Tensor]) -> None:
    """For the arguments the C ABI takes without a leading dimension (centroid matrices of the step)."""
    for t in mats:
        if t is not None and not t.is_contiguous():
            raise ValueError("this matrix must be dense (row stride equal to the row length); call .contiguous()")


class Workspace:
    """A reusable device scratch buffer, grown on demand."""

    def __init__(self, device: torch.device):
        self.device = device
        self.buf: Optional[torch.Tensor] = None

    def get(self, nbytes: int) -> torch.Tensor:
        if self.buf is None or self.buf.numel() < nbytes:
            self.buf = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=self.device)
        return self.buf


def workspace_bytes(n: int, d: int, k: int, flags: int) -> int:
    return int(load().hkm_workspace_bytes(n, d, k, flags))


def assign_kernel_name(n: int, d: int, k: int) -> str:
    return load().hkm_assign_kernel_name(n, d, k).decode()


def lloyd_kernel_name(n: int, d: int, k: int) -> str:
    return load().hkm_lloyd_kernel_name(n, d, k).decode()


def _is_f64(*tensors: Optional[torch.Tensor]) -> bool:
    """True if the floating-point operands are float64 (all of them must then be)."""
    kinds = {t.dtype for t in tensors if t is not None and t.dtype in (torch.float32, torch.float64)}
    if len(kinds) > 1:
        raise TypeError("float32 and float64 operands cannot be mixed")
    return kinds == {torch.float64}


def assign(x: torch.Tensor, c: torch.Tensor, labels: torch.Tensor, min_d2: Optional[torch.Tensor],
           ws: Workspace) -> None:
    _require_gpu(x, c, labels, min_d2)
    _require_rows(x, c)
    n, d = x.shape
    k = c.shape[0]
    if _is_f64(x, c, min_d2):
        check(load().hkm_assign_f64(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(c), k,
                                    c.stride(0) if k > 1 else d, _ptr(labels), _ptr(min_d2), _stream()))
        return
    need = workspace_bytes(n, d, k, WS_ASSIGN)
    buf = ws.get(need)
    check(load().hkm_assign_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(c), k, c.stride(0) if k > 1 else d,
                                _ptr(labels), _ptr(min_d2), _ptr(buf), buf.numel(), _stream()))


def assign_labels64(x: torch.Tensor, c: torch.Tensor, labels64: torch.Tensor, min_d2: Optional[torch.Tensor]) -> None:
    """:func:`assign` for the narrow shapes (assign_kernel_name() == "valu_fused") with int64 labels stored at once."""
    _require_gpu(x, c, labels64, min_d2)
    _require_rows(x, c)
    if labels64.dtype != torch.int64 or not labels64.is_contiguous() or labels64.numel() != x.shape[0]:
        raise ValueError("labels64 must hold one contiguous int64 per row")
    n, d = x.shape
    k = c.shape[0]
    check(load().hkm_assign_labels64_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(c), k,
                                         c.stride(0) if k > 1 else d, _ptr(labels64), _ptr(min_d2), _stream()))


def assign_static(x: torch.Tensor, c: torch.Tensor, labels: torch.Tensor, min_d2: Optional[torch.Tensor]) -> None:
    """:func:`assign` (float32) on the library's built-in scratch array: no workspace, no allocation."""
    _require_gpu(x, c, labels, min_d2)
    _require_rows(x, c)
    n, d = x.shape
    k = c.shape[0]
    check(load().hkm_assign_static_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(c), k,
                                       c.stride(0) if k > 1 else d, _ptr(labels), _ptr(min_d2), _stream()))


def update(x: torch.Tensor, labels: torch.Tensor, c_new: torch.Tensor, counts: Optional[torch.Tensor],
           ws: Workspace) -> None:
    _require_gpu(x, labels, c_new, counts)
    _require_rows(x, c_new)
    n, d = x.shape
    k = c_new.shape[0]
    if _is_f64(x, c_new):
        buf = ws.get(workspace_bytes(n, d, k, WS_UPDATE | WS_F64))
        check(load().hkm_update_f64(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(labels), k, _ptr(c_new),
                                    c_new.stride(0) if k > 1 else d, _ptr(counts), _ptr(buf), buf.numel(), _stream()))
        return
    need = workspace_bytes(n, d, k, WS_UPDATE)
    buf = ws.get(need)
    check(load().hkm_update_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(labels), k, _ptr(c_new),
                                c_new.stride(0) if k > 1 else d, _ptr(counts), _ptr(buf), buf.numel(), _stream()))


def lloyd_step(x: torch.Tensor, c: torch.Tensor, c_new: torch.Tensor, labels: Optional[torch.Tensor],
               shift: torch.Tensor, sse: Optional[torch.Tensor], ws: Workspace) -> None:
    _require_gpu(x, c, c_new, labels, sse)
    _require_rows(x, c, c_new)
    _require_dense(c, c_new)
    if not (shift.is_cuda or shift.is_pinned()):
        # a pinned host scalar is written by the kernel itself over the bus: no copy engine, no
        # extra stream operation between two steps
        raise RuntimeError("shift must live on the GPU or in pinned host memory")
    n, d = x.shape
    k = c.shape[0]
    if _is_f64(x, c, c_new, shift, sse):
        flags = WS_LLOYD | WS_F64 | (WS_SSE if sse is not None else 0)
        buf = ws.get(workspace_bytes(n, d, k, flags))
        check(load().hkm_lloyd_step_f64(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(c), _ptr(c_new), k,
                                        _ptr(labels), _ptr(shift), _ptr(sse), _ptr(buf), buf.numel(), _stream()))
        return
    flags = WS_LLOYD | (WS_SSE if sse is not None else 0)
    need = workspace_bytes(n, d, k, flags)
    buf = ws.get(need)
    check(load().hkm_lloyd_step_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(c), _ptr(c_new), k,
                                    _ptr(labels), _ptr(shift), _ptr(sse), _ptr(buf), buf.numel(), _stream()))


def lloyd_step_labels_optional(n: int, d: int, k: int) -> bool:
    """Whether :func:`lloyd_step` accepts ``labels=None`` for this shape (float32 only)."""
    return bool(load().hkm_lloyd_step_labels_optional(n, d, k))


def lloyd_fit_supported(n: int, d: int, k: int) -> bool:
    """True where the whole Lloyd loop runs as one launch (hkm_lloyd_fit_f32 in include/hkm.h)."""
    return bool(load().hkm_lloyd_fit_supported(n, d, k))


FIT_WAIT_LIMIT_US = 2_000_000  # how long a workgroup of the one-launch fit waits for the others before it gives up


def lloyd_fit(x: torch.Tensor, c0: torch.Tensor, max_iter: int, tol: Optional[float], c_out: torch.Tensor,
              labels64: torch.Tensor, shift: torch.Tensor, info: torch.Tensor, ws: Workspace,
              wait_limit_us: Optional[int] = None) -> None:
    """Enqueue the whole loop (see hkm_lloyd_fit_f32 in include/hkm.h).  ``info`` (two int32, device or pinned
    host memory) holds the iteration count or a negative status once the stream has finished."""
    _require_gpu(x, c0, c_out, labels64, shift)
    _require_rows(x, c0, c_out)
    _require_dense(c0, c_out)
    if not (info.is_cuda or info.is_pinned()) or info.dtype != torch.int32 or info.numel() < 2:
        raise RuntimeError("info must be two int32 on the GPU or in pinned host memory")
    if labels64.dtype != torch.int64 or not labels64.is_contiguous() or labels64.numel() != x.shape[0]:
        raise ValueError("labels64 must hold one contiguous int64 per row")
    n, d = x.shape
    k = c0.shape[0]
    buf = ws.get(workspace_bytes(n, d, k, WS_FIT))
    check(load().hkm_lloyd_fit_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(c0), k, int(max_iter),
                                   0 if tol is None else 1, 0.0 if tol is None else float(tol), _ptr(c_out),
                                   _ptr(labels64), _ptr(shift), _ptr(info),
                                   FIT_WAIT_LIMIT_US if wait_limit_us is None else int(wait_limit_us),
                                   _ptr(buf), buf.numel(), _stream()))


def prepare_lloyd_step(x: torch.Tensor, c: torch.Tensor, c_new: torch.Tensor, labels: Optional[torch.Tensor],
                       shift: torch.Tensor, sse: Optional[torch.Tensor], ws: Workspace, labels64: bool = False):
    """The same call as :func:`lloyd_step` with every argument converted once: returns a function
    without arguments that enqueues the step on the stream that was current when it was prepared.
    For loops that issue thousands of steps on small problems, where building the argument list costs
    as much as the step.  The tensors are kept alive by the returned function.  ``labels64``: ``labels`` is an
    int64 vector that the step fills itself (the narrow one-sweep step only)."""
    _require_gpu(x, c, c_new, labels, sse)
    _require_rows(x, c, c_new)
    _require_dense(c, c_new)
    if not (shift.is_cuda or shift.is_pinned()):
        raise RuntimeError("shift must live on the GPU or in pinned host memory")
    n, d = x.shape
    k = c.shape[0]
    f64 = _is_f64(x, c, c_new, shift, sse)
    flags = WS_LLOYD | (WS_F64 if f64 else 0) | (WS_SSE if sse is not None else 0)
    buf = ws.get(workspace_bytes(n, d, k, flags))
    fn = load().hkm_lloyd_step_f64 if f64 else load().hkm_lloyd_step_f32
    if labels64:
        if f64 or labels is None or labels.dtype != torch.int64 or not labels.is_contiguous() or labels.numel() != n:
            raise ValueError("labels64 needs float32 data and a contiguous int64 vector of N labels")
        fn = load().hkm_lloyd_step_labels64_f32
    elif labels is not None and labels.dtype != torch.int32:
        raise ValueError("labels must be int32")
    args = (_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(c), _ptr(c_new), k, _ptr(labels), _ptr(shift),
            _ptr(sse), _ptr(buf), buf.numel(), _stream())
    keep = (x, c, c_new, labels, shift, sse, buf)

    def enqueue(_fn=fn, _args=args, _keep=keep) -> None:
        rc = _fn(*_args)
        if rc != HKM_OK:
            raise HkmError(rc, last_error())

    return enqueue


def shift(c_old: torch.Tensor, c_new: torch.Tensor, out: torch.Tensor) -> None:
    _require_gpu(c_old, c_new, out)
    _require_rows(c_old, c_new)
    _require_dense(c_old, c_new)
    k, d = c_old.shape
    if _is_f64(c_old, c_new, out):
        check(load().hkm_shift_f64(_ptr(c_old), _ptr(c_new), k, d, _ptr(out), _stream()))
        return
    check(load().hkm_shift_f32(_ptr(c_old), _ptr(c_new), k, d, _ptr(out), _stream()))


def functional_value(min_d2: torch.Tensor, out: torch.Tensor, ws: Workspace) -> None:
    _require_gpu(min_d2, out)
    n = min_d2.numel()
    need = workspace_bytes(n, 1, 1, WS_ASSIGN)
    buf = ws.get(need)
    if _is_f64(min_d2, out):
        check(load().hkm_functional_value_f64(_ptr(min_d2), n, _ptr(out), _ptr(buf), buf.numel(), _stream()))
        return
    check(load().hkm_functional_value_f32(_ptr(min_d2), n, _ptr(out), _ptr(buf), buf.numel(), _stream()))


def cdist(x: torch.Tensor, y: torch.Tensor, out: torch.Tensor, sqrt: bool = True) -> None:
    _require_gpu(x, y, out)
    _require_rows(x, y, out)
    m, d = x.shape
    nn = y.shape[0]
    check(load().hkm_cdist_f32(_ptr(x), m, x.stride(0) if m > 1 else d, _ptr(y), nn, y.stride(0) if nn > 1 else d,
                               d, _ptr(out), out.stride(0) if m > 1 else nn, 1 if sqrt else 0, _stream()))


METRIC_EUCLID_QE, METRIC_EUCLID, METRIC_GAUSS_QE, METRIC_GAUSS, METRIC_MANHATTAN = 0, 1, 2, 3, 4


def pairwise(x: torch.Tensor, y: torch.Tensor, out: torch.Tensor, metric: int, sigma: float = 1.0) -> None:
    _require_gpu(x, y, out)
    _require_rows(x, y, out)
    m, d = x.shape
    nn = y.shape[0]
    if _is_f64(x, y, out):
        check(load().hkm_pairwise_f64(_ptr(x), m, x.stride(0) if m > 1 else d, _ptr(y), nn,
                                      y.stride(0) if nn > 1 else d, d, _ptr(out), out.stride(0) if m > 1 else nn,
                                      metric, float(sigma), _stream()))
        return
    check(load().hkm_pairwise_f32(_ptr(x), m, x.stride(0) if m > 1 else d, _ptr(y), nn,
                                  y.stride(0) if nn > 1 else d, d, _ptr(out), out.stride(0) if m > 1 else nn,
                                  metric, float(sigma), _stream()))


def min_dist_sum(min_d2: torch.Tensor, out: torch.Tensor, ws: Workspace) -> None:
    """out = sum_i sqrt(min_d2[i]) (device scalar)."""
    _require_gpu(min_d2, out)
    n = min_d2.numel()
    buf = ws.get(workspace_bytes(n, 1, 1, WS_ASSIGN))
    check(load().hkm_min_dist_sum_f32(_ptr(min_d2), n, _ptr(out), _ptr(buf), buf.numel(), _stream()))


def min_merge_sum(min_d2: torch.Tensor, new_d2: torch.Tensor, out: torch.Tensor, ws: Workspace) -> None:
    """min_d2 = min(min_d2, new_d2) in place and out = sum(sqrt(min_d2)) of the result, one pass."""
    _require_gpu(min_d2, new_d2, out)
    if min_d2.numel() != new_d2.numel() or min_d2.dtype != torch.float32 or new_d2.dtype != torch.float32:
        raise ValueError("min_d2 and new_d2 must be float32 vectors of one length")
    buf = ws.get(workspace_bytes(min_d2.numel(), 1, 1, WS_ASSIGN))
    check(load().hkm_min_merge_sum_f32(_ptr(min_d2), _ptr(new_d2), min_d2.numel(), _ptr(out), _ptr(buf),
                                       buf.numel(), _stream()))


def sample_select(min_d2: torch.Tensor, u: torch.Tensor, cost: torch.Tensor, oversampling: float,
                  idx: torch.Tensor, count: torch.Tensor, ws: Workspace) -> None:
    """idx[:count] = ascending rows i with u[i] <= oversampling * sqrt(min_d2[i]) / max(cost, 1e-12)."""
    _require_gpu(min_d2, u, cost, idx, count)
    n = min_d2.numel()
    if u.numel() != n:
        raise ValueError(f"u has {u.numel()} elements, expected {n}")
    buf = ws.get(workspace_bytes(n, 1, 1, WS_ASSIGN))
    check(load().hkm_sample_select_f32(_ptr(min_d2), _ptr(u), n, _ptr(cost), float(oversampling), _ptr(idx),
                                       idx.numel(), _ptr(count), _ptr(buf), buf.numel(), _stream()))


def label_counts(labels32: torch.Tensor, k: int, counts: torch.Tensor) -> None:
    _require_gpu(labels32, counts)
    if counts.numel() != k:
        raise ValueError(f"counts has {counts.numel()} elements, expected {k}")
    check(load().hkm_label_counts_i64(_ptr(labels32), labels32.numel(), k, _ptr(counts), _stream()))


SEED_MAX_ROWS = 16384  # HKM_SEED_MAX_ROWS


def seed_plus_plus(x: torch.Tensor, weights: Optional[torch.Tensor], first: int, u: torch.Tensor, k: int, p: int,
                   idx: torch.Tensor) -> None:
    """k-means++ seeding of at most SEED_MAX_ROWS rows in one launch (see hkm_seed_plus_plus_f32 in
    include/hkm.h): idx[0] = first, idx[j] drawn by inverse CDF from u[j - 1]; -1 where no row has mass."""
    _require_gpu(x, weights, u, idx)
    _require_rows(x)
    m, d = x.shape
    if idx.numel() != k or idx.dtype != torch.int64:
        raise ValueError("idx must hold k int64 entries")
    if u.numel() < k - 1 or u.dtype != torch.float32:
        raise ValueError("u must hold k - 1 float32 numbers")
    if weights is not None and (weights.numel() != m or weights.dtype != torch.float32 or not weights.is_contiguous()):
        raise ValueError("weights must be a contiguous float32 vector with one entry per row")
    check(load().hkm_seed_plus_plus_f32(_ptr(x), m, d, x.stride(0) if m > 1 else d, _ptr(weights), int(first),
                                        _ptr(u), k, p, _ptr(idx), _stream()))


SEED_ROWS_MAX = 1 << 24  # HKM_SEED_ROWS_MAX


def seed_plus_plus_rows(x: torch.Tensor, weights: Optional[torch.Tensor], first: int, u: torch.Tensor, k: int, p: int,
                        idx: torch.Tensor, ws: Workspace) -> None:
    """The draws of :func:`seed_plus_plus` for up to SEED_ROWS_MAX rows: two launches per centre, none of
    them waits for the host (see hkm_seed_plus_plus_rows_f32 in include/hkm.h)."""
    _require_gpu(x, weights, u, idx)
    _require_rows(x)
    m, d = x.shape
    if idx.numel() != k or idx.dtype != torch.int64:
        raise ValueError("idx must hold k int64 entries")
    if u.numel() < k - 1 or u.dtype != torch.float32:
        raise ValueError("u must hold k - 1 float32 numbers")
    if weights is not None and (weights.numel() != m or weights.dtype != torch.float32 or not weights.is_contiguous()):
        raise ValueError("weights must be a contiguous float32 vector with one entry per row")
    buf = ws.get(workspace_bytes(m, 1, 1, WS_ASSIGN | WS_SSE))
    check(load().hkm_seed_plus_plus_rows_f32(_ptr(x), m, d, x.stride(0) if m > 1 else d, _ptr(weights), int(first),
                                             _ptr(u), k, p, _ptr(idx), _ptr(buf), buf.numel(), _stream()))


def assign_l1(x: torch.Tensor, c: torch.Tensor, labels: torch.Tensor, min_dist: Optional[torch.Tensor]) -> None:
    """labels[i] = argmin_k sum|x_i - c_k| (Manhattan), optional minimum distance."""
    _require_gpu(x, c, labels, min_dist)
    _require_rows(x, c)
    n, d = x.shape
    k = c.shape[0]
    if _is_f64(x, c, min_dist):
        _f64_paths.assign_l1(x, c, labels, min_dist)
        return
    check(load().hkm_assign_l1_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(c), k,
                                   c.stride(0) if k > 1 else d, _ptr(labels), _ptr(min_dist), _stream()))


def closest_rows_l1(x: torch.Tensor, q: torch.Tensor, idx: torch.Tensor, dist: Optional[torch.Tensor],
                    ws: Workspace) -> None:
    """idx[m] = row of x closest to q[m] in the Manhattan metric (first index on ties)."""
    _require_gpu(x, q, idx, dist)
    _require_rows(x, q)
    n, d = x.shape
    m = q.shape[0]
    if _is_f64(x, q, dist):
        _f64_paths.closest_rows_l1(x, q, idx, dist)
        return
    buf = ws.get(workspace_bytes(n, d, m, WS_MEDIAN))
    check(load().hkm_closest_rows_l1_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(q), m,
                                         q.stride(0) if m > 1 else d, _ptr(idx), _ptr(dist), _ptr(buf),
                                         buf.numel(), _stream()))


def closest_rows_l1_q64(x: torch.Tensor, q64: torch.Tensor, idx: torch.Tensor, dist64: Optional[torch.Tensor],
                        ws: Workspace) -> None:
    """idx[m] = row of the float32 x closest to the float64 q64[m] in the Manhattan metric, distances in
    float64, first index on exact ties (see hkm_closest_rows_l1_q64_f32 in include/hkm.h)."""
    _require_gpu(x, q64, idx, dist64)
    _require_rows(x)
    _require_dense(q64)
    if q64.dtype == torch.float64 and x.dtype == torch.float64:
        _f64_paths.closest_rows_l1(x, q64, idx, dist64)
        return
    if q64.dtype != torch.float64 or x.dtype != torch.float32:
        raise TypeError("x must be float32 (or float64) and q64 float64")
    n, d = x.shape
    m = q64.shape[0]
    buf = ws.get(workspace_bytes(n, d, m, WS_MEDIAN))
    check(load().hkm_closest_rows_l1_q64_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(q64), m, _ptr(idx),
                                             _ptr(dist64), _ptr(buf), buf.numel(), _stream()))


def update_median(x: torch.Tensor, labels: torch.Tensor, c_new: torch.Tensor, ws: Workspace,
                  fallback_rows: Optional[torch.Tensor] = None, c_old: Optional[torch.Tensor] = None,
                  counts: Optional[torch.Tensor] = None, lower: bool = False, skip_zero_rows: bool = False,
                  median64: Optional[torch.Tensor] = None) -> None:
    """Per-cluster, per-coordinate median (see hkm_update_median_f32 in include/hkm.h); ``median64``
    (K x D float64) additionally receives every median before its rounding to float32."""
    _require_gpu(x, labels, c_new, fallback_rows, c_old, counts, median64)
    if median64 is not None:
        _require_dense(median64)
        if median64.dtype != torch.float64 or tuple(median64.shape) != tuple(c_new.shape):
            raise ValueError("median64 must be a float64 matrix of the shape of c_new")
    _require_rows(x, c_new, c_old)
    _require_dense(c_old)
    n, d = x.shape
    k = c_new.shape[0]
    if _is_f64(x, c_new, c_old):
        _f64_paths.update_median(x, labels, c_new, fallback_rows, c_old, counts, lower, skip_zero_rows, median64)
        return
    buf = ws.get(workspace_bytes(n, d, k, WS_MEDIAN))
    if median64 is not None:
        check(load().hkm_update_median_q64_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(labels), k,
                                               _ptr(fallback_rows), _ptr(c_old), _ptr(c_new),
                                               c_new.stride(0) if k > 1 else d, _ptr(counts), 1 if lower else 0,
                                               1 if skip_zero_rows else 0, _ptr(median64), _ptr(buf), buf.numel(),
                                               _stream()))
        return
    check(load().hkm_update_median_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(labels), k,
                                       _ptr(fallback_rows), _ptr(c_old), _ptr(c_new),
                                       c_new.stride(0) if k > 1 else d, _ptr(counts), 1 if lower else 0,
                                       1 if skip_zero_rows else 0, _ptr(buf), buf.numel(), _stream()))


def widen_labels(labels32: torch.Tensor, out64: torch.Tensor) -> None:
    _require_gpu(labels32, out64)
    check(load().hkm_widen_labels_i64(_ptr(labels32), labels32.numel(), _ptr(out64), _stream()))


KNN_MAX_K = 1024  # HKM_KNN_MAX_K


def knn(q: torch.Tensor, x: torch.Tensor, k: int, idx: torch.Tensor, dist: Optional[torch.Tensor],
        ws: Workspace) -> None:
    """idx[m, :k] = the k rows of x closest (Euclidean) to q[m], ascending in (distance, row index);
    dist[m, :k] their distances (see hkm_knn_f32 in include/hkm.h)."""
    _require_gpu(q, x, idx, dist)
    _require_rows(q, x, idx, dist)
    if q.dtype == torch.float64 and x.dtype == torch.float64 and idx.dtype == torch.int64:
        if q.shape[1] != x.shape[1] or tuple(idx.shape) != (q.shape[0], k) or not 1 <= k <= x.shape[0]:
            raise ValueError("shapes of q, x and idx do not fit together")
        _f64_paths.knn(q, x, k, idx, dist)
        return
    if q.dtype != torch.float32 or x.dtype != torch.float32:
        raise TypeError("q and x must both be float32 or both be float64")
    if idx.dtype != torch.int64 or (dist is not None and dist.dtype != torch.float32):
        raise TypeError("idx must be int64 and dist float32")
    m, d = q.shape
    n = x.shape[0]
    if x.shape[1] != d:
        raise ValueError(f"feature counts differ: {d} != {x.shape[1]}")
    if tuple(idx.shape) != (m, k) or (dist is not None and tuple(dist.shape) != (m, k)):
        raise ValueError(f"idx and dist must have shape ({m}, {k})")
    lib = load()
    buf = ws.get(lib.hkm_knn_workspace_bytes(m, n))
    check(lib.hkm_knn_f32(_ptr(q), m, q.stride(0) if m > 1 else d, _ptr(x), n, x.stride(0) if n > 1 else d, d, k,
                          _ptr(idx), idx.stride(0) if m > 1 else k, _ptr(dist),
                          (dist.stride(0) if m > 1 else k) if dist is not None else k, _ptr(buf), buf.numel(),
                          _stream()))


def knn_vote(idx: torch.Tensor, y: torch.Tensor, classes: torch.Tensor) -> None:
    """classes[m] = first index of the largest entry of the sum of the label rows y[idx[m, j]]
    (see hkm_knn_vote_f32 in include/hkm.h)."""
    _require_gpu(idx, y, classes)
    _require_rows(idx, y)
    if idx.dtype != torch.int64 or classes.dtype != torch.int64 or y.dtype != torch.float32:
        raise TypeError("idx and classes must be int64, y float32")
    m, k = idx.shape
    n, c = y.shape
    if classes.numel() != m or not classes.is_contiguous():
        raise ValueError(f"classes must hold {m} contiguous entries")
    check(load().hkm_knn_vote_f32(_ptr(idx), m, k, idx.stride(0) if m > 1 else k, _ptr(y), n, c,
                                  y.stride(0) if n > 1 else c, _ptr(classes), _stream()))


def cluster_distance_sums(x: torch.Tensor, perm: torch.Tensor, offsets: torch.Tensor, out: torch.Tensor) -> None:
    """out[i, c] = sum of the Euclidean distances from row i to the rows perm[offsets[c]:offsets[c + 1]]
    (see hkm_cluster_distance_sums_f32 in include/hkm.h).  perm and offsets are checked here, on the
    device, because the kernel gathers rows through them."""
    _require_gpu(x, perm, offsets, out)
    _require_rows(x, out)
    if x.dtype != torch.float32 or out.dtype != torch.float32:
        raise TypeError("x and out must be float32")
    if perm.dtype != torch.int64 or offsets.dtype != torch.int64 or not perm.is_contiguous() or not offsets.is_contiguous():
        raise TypeError("perm and offsets must be contiguous int64 vectors")
    n, d = x.shape
    k = offsets.numel() - 1
    if k < 1 or perm.numel() != n or tuple(out.shape) != (n, k):
        raise ValueError(f"perm must hold {n} entries and out must be ({n}, {k})")
    if n:
        ok = (int(perm.min()) >= 0 and int(perm.max()) < n and int(offsets[0]) == 0 and int(offsets[-1]) == n
              and bool((offsets[1:] >= offsets[:-1]).all()))
        if not ok:
            raise ValueError("perm must index rows of x and offsets must rise from 0 to the number of rows")
    check(load().hkm_cluster_distance_sums_f32(_ptr(x), n, d, x.stride(0) if n > 1 else d, _ptr(perm), _ptr(offsets), k,
                                               _ptr(out), out.stride(0) if n > 1 else k, _stream()))


def silhouette_finish(sums: torch.Tensor, labels: torch.Tensor, counts: torch.Tensor, out: torch.Tensor) -> None:
    """out[i] = silhouette coefficient of sample i from its per-cluster distance sums (see
    hkm_silhouette_finish_f32 in include/hkm.h); labels are checked here against the number of clusters."""
    _require_gpu(sums, labels, counts, out)
    _require_rows(sums)
    n, k = sums.shape
    if sums.dtype != torch.float32 or out.dtype != torch.float32:
        raise TypeError("sums and out must be float32")
    if labels.dtype != torch.int64 or counts.dtype != torch.int64:
        raise TypeError("labels and counts must be int64")
    if labels.numel() != n or counts.numel() != k or out.numel() != n:
        raise ValueError("labels and out need one entry per sample, counts one per cluster")
    if not (labels.is_contiguous() and counts.is_contiguous() and out.is_contiguous()):
        raise ValueError("labels, counts and out must be contiguous")
    if n and (int(labels.min()) < 0 or int(labels.max()) >= k):
        raise ValueError("labels must lie in [0, number of clusters)")
    check(load().hkm_silhouette_finish_f32(_ptr(sums), n, k, sums.stride(0) if n > 1 else k, _ptr(labels), _ptr(counts),
                                           _ptr(out), _stream()))


def laplacian(sim: torch.Tensor, out: torch.Tensor, definition: int, mode: int, weighted: bool, eps: float,
              degree: torch.Tensor) -> None:
    """out = graph Laplacian of the similarity matrix sim (see hkm_laplacian_f32 in include/hkm.h):
    definition 0 simple / 1 norm_sym, mode 0 fully connected / 1 keep below eps / 2 keep above eps."""
    _require_gpu(sim, out, degree)
    _require_rows(sim, out)
    n = sim.shape[0]
    if sim.dim() != 2 or sim.shape[1] != n or tuple(out.shape) != (n, n):
        raise ValueError("sim and out must be square matrices of the same size")
    if sim.dtype not in (torch.float32, torch.float64) or out.dtype != sim.dtype or degree.dtype != sim.dtype:
        raise TypeError("sim, out and degree must all be float32 or all be float64")
    if degree.numel() != n or not degree.is_contiguous():
        raise ValueError(f"degree must hold {n} contiguous entries")
    fn = load().hkm_laplacian_f64 if sim.dtype == torch.float64 else load().hkm_laplacian_f32
    check(fn(_ptr(sim), n, sim.stride(0) if n > 1 else n, definition, mode, 1 if weighted else 0,
                                   float(eps), _ptr(out), out.stride(0) if n > 1 else n, _ptr(degree), _stream()))
