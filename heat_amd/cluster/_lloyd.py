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
bounds such fits.  For the shapes whose step is one sweep of a vector kernel (few clusters of at most 64
features), writing N labels is up to a quarter of the step's memory traffic and, next to the stream of
reads, costs more time than its share, so the steps run without storing labels and those of the last iteration are computed once, on demand, against the
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
        # the one-sweep steps that memory bounds: the two vector kernels'
        self.lazy_labels = bool(kernel) and _native.lloyd_step_labels_optional(n, d, c0.shape[0])
        # A step known to be the last of a run (the max_iter-th) stores its labels after all: one more stream of
        # writes in one step instead of one more pass over X afterwards.  (The narrow shapes' last step writes the
        # int64 labels the caller wants, see below.)
        self._label_last = self.lazy_labels and kernel != "lloyd_small"
        # The narrow shapes' last step can store the int64 labels the caller wants at once, into the caller's own
        # vector (final_labels64): neither the pass over X nor the widening pass is left.
        self._narrow = kernel == "lloyd_small"
        self._lab64_out: Optional[torch.Tensor] = None
        self._lab64_of = -1  # iteration whose labels self._lab64_out holds
        # Relative size (against sum |c|^2) of the squared rounding error of a one-sweep step's centroids; 0 for the
        # shapes that run the two-pass update.  From the kernels' quanta: the matrix-core step rounds a row to
        # 2^-28 of its largest coordinate or, for rows below the floor it derives from the centroid norms, to at
        # most 2^-23 of the smallest centroid's norm -- squared and summed over K clusters of D coordinates that is
        # at most D * 2^-46 * sum |c|^2, taken eight times over.  The narrow step sums fp32 partials per lane, or
        # integers with a quantum of 2^-33 of the largest centroid coordinate: a mean is good to a few dozen ulps,
        # (2^-18)^2 of its magnitude per coordinate.
        self._fuzz = {"lloyd_small": d * 2.0 ** -36, "lloyd_mfma_resident": d * 2.0 ** -43,
                      "lloyd_few": d * 2.0 ** -43}.get(kernel, 0.0)  # (lloyd_few rounds its rows as the matrix-core step)
        # Upper bound on the Frobenius norm of the current centroids, kept from the shifts the host reads (see
        # _margin).  It starts at the norm of the init, taken here from a copy on the host, before anything is
        # in flight: no reduction kernel of the tensor library is loaded or launched for sixteen numbers.
        self._cnorm: Optional[float] = self._host_norm(c0) if self._fuzz else None
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

    def final_labels64(self, out: Optional[torch.Tensor]) -> None:
        """A contiguous int64 vector of N entries that the last step of a run may fill with its labels (the narrow
        shapes only; ignored otherwise).  labels64_into(out) then finds them there."""
        self._lab64_out = out if self._narrow else None
        self._lab64_of = -1
        self._plans = {k: v for k, v in self._plans.items() if k[1] != 2}

    def _enqueue(self, last: bool = False) -> None:
        j = self.enqueued
        # 0: no labels; 1: int32 labels; 2: int64 labels into the caller's vector
        mode = 1 if not self.lazy_labels or (last and self._label_last) else 0
        if last and self._lab64_out is not None:
            mode = 2
        key = (j % 6, mode, torch.cuda.current_stream().cuda_stream)
        plan = self._plans.get(key)
        if plan is None:
            # the argument list of a step only depends on which buffers of the rotation it uses
            if mode == 2:
                lab = self._lab64_out
            else:
                lab = None if mode == 0 else self.lab[0] if self.lazy_labels else self.lab[j % 2]
            plan = _native.prepare_lloyd_step(self.x, self.c[j % 3], self.c[(j + 1) % 3], lab,
                                              self.shift_host[j % 2], None, self.ws, labels64=mode == 2)
            self._plans[key] = plan
        self._shift_np[j % 2] = _PENDING
        plan()
        if mode == 2:
            self._lab64_of = j
        elif self.lazy_labels and mode == 1:
            self._lab_of = j
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
                self._enqueue(last=ran + 1 == max_iter)
            if tol is None:
                self._free_running = True
                self._cnorm = None  # nobody reads these shifts: the bound is taken again when it is needed
                self.done = i + 1
                ran += 1
                continue
            if ran + 1 < max_iter and self.enqueued == i + 1:
                self._enqueue(last=ran + 2 == max_iter)  # ahead of the host's look at step i
            shift = self._wait(i)
            self.done = i + 1
            ran += 1
            if self._fuzz:
                if shift <= tol + self._margin(tol, shift):
                    # Bit-identical centroids from a one-sweep step (looked at before they are replaced): the step
                    # saw the labels of the step before it.  The reference forms the exact means in every
                    # iteration and finds no movement between two iterations with the same labels
                    # (kmeans.py:141-143); the centroids this step started from carry the one-sweep rounding,
                    # so the exact means stored below would show a movement of that size and cost an iteration
                    # the reference does not run.  Not at the first step: nothing came before it, and an init
                    # that reproduces itself under the one-sweep rounding still moves by the last bit in the
                    # reference.
                    unchanged = i > 0 and torch.equal(self.c[i % 3], self.c[(i + 1) % 3])
                    shift = self._recompute(i)
                    if unchanged:
                        shift = 0.0
                        self.shift_host[i % 2] = 0.0
                # |c_new| <= |c_old| + sqrt(shift): the bound follows the centroids without a look at them
                if self._cnorm is not None and shift == shift:
                    self._cnorm += max(shift, 0.0) ** 0.5
            if shift <= tol:
                break
        return ran

    def _margin(self, tol: float, shift: float) -> float:
        """How far above ``tol`` the shift of the one-sweep step just waited for may sit while the exact one is
        <= tol: with e = the rounding error of the step's centroids, |shift - exact| <= 2 sqrt(exact) |e| + |e|^2.
        e^2 is priced against an upper bound on sum |c|^2 that holds for the centroids the step started from and
        for those it produced: the norm of the initial centroids (one look at the device, at the first call) plus
        the square roots of every shift since, so centroids that grow -- an init near the origin, data far from
        it -- raise the margin with them."""
        if self._cnorm is None:  # after steps nobody waited for: one look at the device
            self._cnorm = self._host_norm(self.c[(self.done - 1) % 3])
        bound = self._cnorm + (max(shift, 0.0) ** 0.5 if shift == shift else 0.0)
        e2 = self._fuzz * bound * bound
        return 2.0 * (max(tol, 0.0) * e2) ** 0.5 + e2

    @staticmethod
    def _host_norm(c: torch.Tensor) -> float:
        """Frobenius norm of a (small) device matrix, computed on the host in float64; waits for the stream."""
        v = c.detach().cpu().double().numpy()
        return float((v * v).sum()) ** 0.5

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

    def labels64_into(self, out: torch.Tensor) -> None:
        """The labels of the last iteration that counts as the (N, 1) int64 matrix the reference returns.  Where
        the steps stored none (the narrow shapes) and none have been computed since, the one assignment pass
        writes int64 at once instead of int32 labels that a second pass would widen."""
        i = self.done - 1
        n, d = self.x.shape
        if self._lab64_out is not None and self._lab64_of == i and out.data_ptr() == self._lab64_out.data_ptr():
            return  # the last step wrote them
        if self.lazy_labels and self._lab_of != i and _native.assign_kernel_name(n, d, self.c[0].shape[0]) == "valu_fused":
            _native.assign_labels64(self.x, self.c[i % 3], out.view(-1), None)
        else:
            _native.widen_labels(self.labels, out)

    @property
    def last_shift(self) -> torch.Tensor:
        """0-d device tensor; waits for the step that produced it."""
        i = self.done - 1
        torch.cuda.current_stream().synchronize()
        return self.shift_host[i % 2].to(self.x.device)
