"""
Writes the golden vectors of tests/golden/*.npz.

The reference cannot be imported in the build environment (it needs mpi4py at import time), so the
vectors come from the CPU restatement in oracle/heat_oracle.py, whose functions are pinned
separately (tests/test_oracle_pins.py) against the known answers of the reference's own tests and
against closed forms.  The vectors freeze those results so that a later change to the oracle or to
the kernels shows up as a diff.  ``iris.csv`` is the data file the reference's KMeans tests load
(heat/datasets/iris.csv, ';'-separated, 150 x 4).

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import heat_oracle as orc  # noqa: E402


def fit_case(x, c0, iters, tol):
    r = orc.kmeans_fit(x, c0, iters, tol, literal=True)
    lab_pred, fval = orc.predict(x, r["cluster_centers"])
    return dict(
        x=x.numpy(), init=c0.numpy(), max_iter=np.int64(iters),
        centers=r["cluster_centers"].numpy(), labels=r["labels"].numpy(),
        inertia=np.float32(r["inertia"]), n_iter=np.int64(r["n_iter"]),
        shifts=np.asarray(r["shifts"], dtype=np.float64),
        predict_labels=lab_pred.numpy(), functional_value=np.float32(fval),
        d2_first=orc.quadratic_expand(x, c0).numpy(),
    )


def main():
    torch.set_num_threads(1)
    # 1. iris, K = 3, init = first three rows, 5 iterations, tol = 0
    iris = torch.from_numpy(np.loadtxt(os.path.join(HERE, "iris.csv"), delimiter=";", dtype=np.float32))
    np.savez(os.path.join(HERE, "iris_k3.npz"), **fit_case(iris, iris[:3].clone(), 5, 0.0))

    # 2. 64 x 5, K = 4 with: an exact tie (two identical centroids), a cluster that stays empty
    #    (a centroid far away from all points), and duplicated points equal to a centroid
    #    (negative expansion before the clamp)
    g = torch.Generator().manual_seed(20240)
    x = torch.randn((64, 5), generator=g)
    x[10] = x[3]
    x[11] = x[3]
    c0 = torch.stack([x[3], x[40], x[40], torch.full((5,), 1000.0)])
    np.savez(os.path.join(HERE, "edge_k4.npz"), **fit_case(x, c0, 4, 0.0))

    # 3. two translated copies of one cloud (the invariant of the reference's clustering tutorial):
    #    centroids differ by exactly the translation, counts are equal
    base = 0.4 * torch.randn((100, 2), generator=g)
    x = torch.cat([base + 2.0, base - 2.0])
    c0 = torch.stack([x[0], x[150]])
    np.savez(os.path.join(HERE, "translated_k2.npz"), **fit_case(x, c0, 10, 0.0))


if __name__ == "__main__":
    main()
