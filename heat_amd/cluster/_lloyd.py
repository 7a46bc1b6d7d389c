"""
The Lloyd iteration loop of KMeans.fit (heat/cluster/kmeans.py:131-143) as a pipeline on one stream.

The reference looks at ``inertia <= tol`` on the host after every iteration, which leaves the GPU
idle while the 4 bytes travel and the next launches are issued.  Here step i+1 is enqueued BEFORE the
host waits for the shift of step i: if the loop goes on (the usual case) the GPU never idles, if it
stops the extra step is simply not used -- it writes to buffers the results of step i do not live
in (three centroid buffers, two label buffers, two shift scalars in rotation).  The shift scalars
live in pinned host memory and are written by the finishing kernel itself, so no copy-engine
operation sits between two steps on the stream -- and no event either: before a step is enqueued its
scalar is set to a value no shift can take (-1: a shift is a sum of squares or NaN), and the host
waits for the step by reading the scalar until it has changed.  For a step of a few microseconds the
record and the wait of an event were a third of the host's time per iteration, and the host is what
bounds such fits.  For the narrow shapes whose step is one sweep of a
vector kernel (D <= 16, few clusters), writing N labels is a quarter of the step's memory traffic, so the steps run
without storing labels and those of the last iteration are computed once, on demand, against the
centroids that iteration started from -- the same kernel code, hence the same bits.  The values
returned are exactly those of the sequential loop.

The stop decision.  The two one-sweep kernels form their per-cluster sums on the way (rows pre-rounded
to 28 bits below their largest coordinate, or below a floor taken from the centroid norms, on the matrix cores; fp32 partial sums per lane, or rows rounded
to 32 bits below the largest centroid coordinate, in the narrow kernel), so their means can differ from the fp64 divide-then-sum of heat/cluster/kmeans.py:76-103 in the
last bit.  That is far inside the 1e-4 bar on the centroids but it decides ``shift <= tol`` when the shift
is (nearly) zero: a fit sitting on a fixed point of the reference's arithmetic would run one iteration
longer.  So whenever a one-sweep step reports a shift within its own rounding error of the tolerance --
in particular before EVERY stop -- the means of that iteration are recomputed from its labels with the
two-pass update (fp64 from the first addition to the division, fixed order: bit-identical to the
reference's means in all but about one coordinate in a thousand), and the decision is taken on that
shift.  If the loop goes on, the step enqueued ahead is re-issued from the recomputed centroids.
One case is decided before that: a one-sweep step whose centroids equal the ones it started from bit for
bit saw the labels of the step before it, and two iterations with the same labels are where the
reference stops with a shift of exactly 0 -- the recomputed means are stored, the shift is 0.
"""

from __future__ import annotations

import os
import time
from typing import Optional

import torch

from .. import _native

_PENDING = -1.0  # what a shift scalar holds while its step has not delivered: no sum of squares is negative


class LloydLoop:
    def __init__(self, xt: torch.Tensor, c0: torch.Tensor, ws: _native.Workspace):
        _native._require_gpu(xt, c0)
        dev = xt.device
        self.x = xt
        self.ws = ws
        self.c = [c0.clone(), torch.empty_like(c0), torch.empty_like(c0)]
        n, d = xt.shape
        kernel = _native.lloyd_kernel_name(n, d, c0.shape[0]) if xt.dtype == torch.float32 else ""
        self.lazy_labels = kernel == "lloyd_small"
        # relative size (against sum |c|^2) of the squared centroid movement below which a one-sweep step's
        # shift is within the rounding error of its own sums; 0 for the shapes that run the two-pass update
        self._fuzz = {"lloyd_small": 1e-11 * d, "lloyd_mfma_resident": 1e-13 * d}.get(kernel, 0.0)
        self._cscale: Optional[float] = None
        self.rechecks = 0  # iterations whose means were recomputed by the two-pass update
        nbuf = 1 if self.lazy_labels else 2
        self.lab = [torch.empty((n,), dtype=torch.int32, device=dev) for _ in range(nbuf)]
        self._lab_of = -1  # iteration whose labels self.lab[0] holds (lazy mode)
        self.shift_host = torch.zeros((2,), dtype=xt.dtype, pin_memory=True)
        self._shift_np = self.shift_host.numpy()  # the same two scalars, read without building a tensor
        self._free_running = False  # steps were enqueued that nobody waited for (tol is None)
        self.enqueued = 0  # steps handed to the stream
        self.done = 0      # steps whose results count
        self._plans = {}   # prepared calls, one per rotation of the buffers (and stream)
        # Large fits on the resident matrix-core kernels: let the library measure once per device which of
        # its two launch geometries this chip runs faster (the results do not depend on it).  The call is a
        # step from c[0] into c[1] that the loop's own first step then repeats.
        if kernel == "lloyd_mfma_resident" and n >= (1 << 20):
            pb, tuned = _native.point_blocks(d)
            if pb and d <= 32 and not tuned and not os.environ.get("HKM_POINT_BLOCKS"):
                _native.tune_lloyd_step(self.x, self.c[0], self.c[1], self.lab[0], self.shift_host[0], self.ws)

    def _enqueue(self) -> None:
        j = self.enqueued
        key = (j % 6, torch.cuda.current_stream().cuda_stream)
        plan = self._plans.get(key)
        if plan is None:
            # the argument list of a step only depends on which buffers of the rotation it uses
            plan = _native.prepare_lloyd_step(self.x, self.c[j % 3], self.c[(j + 1) % 3],
                                              None if self.lazy_labels else self.lab[j % 2],
                                              self.shift_host[j % 2], None, self.ws)
            self._plans[key] = plan
        self._shift_np[j % 2] = _PENDING
        plan()
        self.enqueued = j + 1

    def _wait(self, i: int) -> float:
        """The shift of step i, once its finishing kernel has written it."""
        slot = i % 2
        spins = 0
        while self._shift_np[slot] == _PENDING:
            spins += 1
            if spins == 1 << 16:
                t0 = time.monotonic()
            elif spins > 1 << 16 and (spins & 0xFFF) == 0 and time.monotonic() - t0 > 60.0:
                torch.cuda.current_stream().synchronize()  # raises what the device has to report
                if self._shift_np[slot] == _PENDING:
                    raise RuntimeError(f"Lloyd step {i} finished without delivering its centroid shift")
        return float(self._shift_np[slot])

    def run(self, max_iter: int, tol: Optional[float]) -> int:
        """Up to ``max_iter`` further iterations; stops after the first whose shift is <= tol
        (never if ``tol`` is None, and then without any host read).  Returns the number run."""
        ran = 0
        if tol is not None and self._free_running:
            # steps nobody waited for may still be on their way and write the two scalars after a later step
            # has marked them pending
            torch.cuda.current_stream().synchronize()
            self._free_running = False
        for _ in range(max_iter):
            i = self.done
            if self.enqueued == i:
                self._enqueue()
            if tol is None:
                self._free_running = True
                self.done = i + 1
                ran += 1
                continue
            if ran + 1 < max_iter and self.enqueued == i + 1:
                self._enqueue()  # ahead of the host's look at step i
            shift = self._wait(i)
            self.done = i + 1
            ran += 1
            if self._fuzz and shift <= tol + self._margin(tol):
                unchanged = shift == 0.0
                shift = self._recompute(i)
                if unchanged:
                    # Bit-identical centroids from a one-sweep step: it saw the labels of the step before it.
                    # The reference forms the exact means in every iteration and finds no movement between
                    # two iterations with the same labels (kmeans.py:141-143); the centroids this step
                    # started from carry the one-sweep rounding, so the exact means just stored would show
                    # a movement of that size and cost an iteration the reference does not run.
                    shift = 0.0
                    self.shift_host[i % 2] = 0.0
            if shift <= tol:
                break
        return ran

    def _margin(self, tol: float) -> float:
        """How far above ``tol`` a one-sweep step's shift may sit while the exact one is <= tol: with
        e = the rounding error of the step's centroids, |shift - exact| <= 2 sqrt(exact) |e| + |e|^2."""
        if self._cscale is None:
            self._cscale = float((self.c[0].double() ** 2).sum())
        e2 = self._fuzz * self._cscale
        return 2.0 * (max(tol, 0.0) * e2) ** 0.5 + e2

    def _recompute(self, i: int) -> float:
        """Replace the centroids step i produced by the two-pass means of its labels; returns the shift."""
        if self.lazy_labels:
            if self._lab_of != i:
                _native.assign(self.x, self.c[i % 3], self.lab[0], None, self.ws)
                self._lab_of = i
            lab = self.lab[0]
        else:
            lab = self.lab[i % 2]
        _native.update(self.x, lab, self.c[(i + 1) % 3], None, self.ws)
        out = torch.empty((), dtype=self.x.dtype, device=self.x.device)
        _native.shift(self.c[i % 3], self.c[(i + 1) % 3], out)
        self.shift_host[i % 2] = out.cpu()  # synchronises: a step enqueued ahead has run and written its scalar
        self.enqueued = i + 1  # that step started from the centroids just replaced
        self.rechecks += 1
        return float(self.shift_host[i % 2])

    # results of the last iteration that counts
    @property
    def centers(self) -> torch.Tensor:
        return self.c[self.done % 3]

    @property
    def labels(self) -> torch.Tensor:
        """int32 labels of the last iteration that counts (against the centroids it started from)."""
        i = self.done - 1
        if not self.lazy_labels:
            return self.lab[i % 2]
        if self._lab_of != i:
            _native.assign(self.x, self.c[i % 3], self.lab[0], None, self.ws)
            self._lab_of = i
        return self.lab[0]

    @property
    def last_shift(self) -> torch.Tensor:
        """0-d device tensor; waits for the step that produced it."""
        i = self.done - 1
        torch.cuda.current_stream().synchronize()
        return self.shift_host[i % 2].to(self.x.device)
