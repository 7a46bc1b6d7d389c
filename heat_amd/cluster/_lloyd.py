"""
The Lloyd iteration loop of KMeans.fit (heat/cluster/kmeans.py:131-143) as a pipeline on one stream.

The reference looks at ``inertia <= tol`` on the host after every iteration, which leaves the GPU
idle while the 4 bytes travel and the next launches are issued.  Here step i+1 is enqueued BEFORE the
host waits for the shift of step i: if the loop goes on (the usual case) the GPU never idles, if it
stops the extra step is simply not used -- it writes to buffers the results of step i do not live
in (three centroid buffers, two label buffers, two shift scalars in rotation).  The shift scalars
live in pinned host memory and are written by the finishing kernel itself, so no copy-engine
operation sits between two steps on the stream.  For the narrow shapes whose step is one sweep of a
vector kernel (D <= 8), writing N labels is a quarter of the step's memory traffic, so the steps run
without storing labels and those of the last iteration are computed once, on demand, against the
centroids that iteration started from -- the same kernel code, hence the same bits.  The values
returned are exactly those of the sequential loop.
"""

from __future__ import annotations

from typing import Optional

import torch

from .. import _native


class LloydLoop:
    def __init__(self, xt: torch.Tensor, c0: torch.Tensor, ws: _native.Workspace):
        _native._require_gpu(xt, c0)
        dev = xt.device
        self.x = xt
        self.ws = ws
        self.c = [c0.clone(), torch.empty_like(c0), torch.empty_like(c0)]
        n, d = xt.shape
        self.lazy_labels = xt.dtype == torch.float32 and _native.lloyd_kernel_name(n, d, c0.shape[0]) == "lloyd_small"
        nbuf = 1 if self.lazy_labels else 2
        self.lab = [torch.empty((n,), dtype=torch.int32, device=dev) for _ in range(nbuf)]
        self._lab_of = -1  # iteration whose labels self.lab[0] holds (lazy mode)
        self.shift_host = torch.zeros((2,), dtype=xt.dtype, pin_memory=True)
        self.ev = [torch.cuda.Event(), torch.cuda.Event()]
        self.enqueued = 0  # steps handed to the stream
        self.done = 0      # steps whose results count
        self._plans = {}   # prepared calls, one per rotation of the buffers (and stream)

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
        plan()
        self.ev[j % 2].record()
        self.enqueued = j + 1

    def run(self, max_iter: int, tol: Optional[float]) -> int:
        """Up to ``max_iter`` further iterations; stops after the first whose shift is <= tol
        (never if ``tol`` is None, and then without any host read).  Returns the number run."""
        ran = 0
        for _ in range(max_iter):
            i = self.done
            if self.enqueued == i:
                self._enqueue()
            if tol is None:
                self.done = i + 1
                ran += 1
                continue
            if ran + 1 < max_iter and self.enqueued == i + 1:
                self._enqueue()  # ahead of the host's look at step i
            self.ev[i % 2].synchronize()
            self.done = i + 1
            ran += 1
            if float(self.shift_host[i % 2]) <= tol:
                break
        return ran

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
        self.ev[i % 2].synchronize()
        return self.shift_host[i % 2].to(self.x.device)
