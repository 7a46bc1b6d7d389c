"""
k-nearest-neighbours classifier with the interface of heat/classification/kneighborsclassifier.py.

``predict`` there is ``cdist -> topk(largest=False) -> y[indices] -> sum -> argmax`` (:114-132) over the
full (test rows x training rows) distance matrix.  Here the matrix is never formed: ``hkm_knn_f32`` keeps
the k best rows per test row while it walks the training rows, ``hkm_knn_vote_f32`` adds up their label
rows and takes the first maximum.
"""

from __future__ import annotations

from typing import Callable, Optional

import torch

from .. import _native
from ..core import types
from ..core.base import BaseEstimator, ClassificationMixin
from ..core.dndarray import DNDarray
from ..spatial import distance


class KNeighborsClassifier(BaseEstimator, ClassificationMixin):
    def __init__(self, n_neighbors: int = 5, effective_metric_: Optional[Callable] = None):  # noqa: D107
        self.n_neighbors = n_neighbors
        self.effective_metric_ = effective_metric_ if effective_metric_ is not None else distance.cdist
        self.x = None
        self.y = None
        self.n_samples_fit_ = -1
        self.outputs_2d_ = True
        self.classes_ = None
        self.kneighbors_ = None
        self._ws = None

    @staticmethod
    def one_hot_encoding(x: DNDarray) -> DNDarray:
        """heat/classification/kneighborsclassifier.py:44-61: (n, max + 1) float32 matrix with a one per row."""
        lab = x.larray.reshape(-1).long()
        n = lab.shape[0]
        n_features = int(lab.max().item()) + 1 if n else 0
        one_hot = torch.zeros((n, n_features), dtype=torch.float32, device=lab.device)
        if n:
            one_hot.scatter_(1, lab.view(-1, 1), 1.0)
        return DNDarray(one_hot, (n, n_features), types.float32, x.split, x.device, x.comm, True)

    def fit(self, x: DNDarray, y: DNDarray):
        """Checks and label encoding of heat/classification/kneighborsclassifier.py:63-112."""
        if not isinstance(x, DNDarray) or not isinstance(y, DNDarray):
            raise TypeError(f"x and y must be DNDarrays but were {type(x)} {type(y)}")
        if len(x.shape) != 2:
            raise ValueError(f"x must be two-dimensional, but was {len(x.shape)}")
        self.x = x
        self.n_samples_fit_ = x.shape[0]
        if x.shape[0] != y.shape[0]:
            raise ValueError(f"Number of samples x and y samples mismatch, got {x.shape[0]}, {y.shape[0]}")
        if len(y.shape) == 1:
            self.y = self.one_hot_encoding(y)
            self.outputs_2d_ = False
        elif len(y.shape) == 2:
            self.y = y
            self.outputs_2d_ = True
        else:
            raise ValueError(f"y needs to be one- or two-dimensional, but was {len(y.shape)}")

    def predict(self, x: DNDarray) -> DNDarray:
        """
        heat/classification/kneighborsclassifier.py:114-132.  With the default metric ``ht.spatial.cdist`` on
        float32 data the distance matrix is never formed.  Arithmetic of that path: below 16 and above 128
        features squared distances are summed directly as sum (a - b)^2, in between they are the clamped
        expansion (|a|^2 + |b|^2) - 2 a.b with the products on the matrix cores -- the form the reference's
        ``torch.cdist`` itself takes above 25 rows; it carries an absolute error of up to about
        4e-7 (|a|^2 + |b|^2), so training rows closer together than that may swap places.  Ties between
        training rows at exactly the same distance go to the smaller row index (``torch.topk`` leaves their
        order open), and the label rows are added in float32 (exact for one-hot labels and integer weights
        below 2^24).  Any other metric callable, and float64 / int64 data, take the reference's own route:
        the full matrix from the callable, ``topk(largest=False)``, the label rows summed, ``argmax``.
        The neighbours found are kept in ``kneighbors_``.
        """
        if self.x is None or self.y is None:
            raise RuntimeError("fit needs to be called before predict")
        if not isinstance(x, DNDarray):
            raise TypeError(f"x must be a DNDarray but was {type(x)}")
        if len(x.shape) != 2 or x.shape[1] != self.x.shape[1]:
            raise ValueError(f"x must be two-dimensional with {self.x.shape[1]} features, but was {x.shape}")
        k = int(self.n_neighbors)
        if k < 1 or k > self.n_samples_fit_:
            raise ValueError(f"n_neighbors = {k} must be in [1, {self.n_samples_fit_}]")
        promoted = types.promote_types(types.promote_types(x.dtype, self.x.dtype), types.float32)
        if self.effective_metric_ is not distance.cdist or promoted is not types.float32:
            return self._predict_full_matrix(x, k)
        q = distance._as_f32_matrix(x, promoted)
        train = distance._as_f32_matrix(self.x, promoted)
        dev = q.device
        yt = self.y.larray.to(device=dev, dtype=torch.float32)
        if yt.stride(-1) != 1:
            yt = yt.contiguous()
        if self._ws is None or self._ws.device != dev:
            self._ws = _native.Workspace(dev)
        m = q.shape[0]
        idx = torch.empty((m, k), dtype=torch.int64, device=dev)
        _native.knn(q, train, k, idx, None, self._ws)
        classes = torch.empty((m,), dtype=torch.int64, device=dev)
        _native.knn_vote(idx, yt, classes)
        self.kneighbors_ = DNDarray(idx, (m, k), types.int64, x.split, x.device, x.comm, True)
        self.classes_ = DNDarray(classes, (m,), types.int64, x.split, x.device, x.comm, True)
        return self.classes_

    def _predict_full_matrix(self, x: DNDarray, k: int) -> DNDarray:
        """The reference's op sequence on the device: distances from the metric callable (the library's
        full-matrix kernels when it is one of ht.spatial's), then torch's selection and reductions."""
        distances = self.effective_metric_(x, self.x)
        if not isinstance(distances, DNDarray) or tuple(distances.shape) != (x.shape[0], self.x.shape[0]):
            raise ValueError("the metric must return a (test rows x training rows) DNDarray")
        d = distances.larray
        _, idx = torch.topk(d, k, dim=1, largest=False)
        yt = self.y.larray.to(device=d.device)
        votes = yt[idx.reshape(-1)].reshape(idx.shape[0], k, yt.shape[1]).sum(dim=1)
        classes = torch.argmax(votes, dim=1)
        m = idx.shape[0]
        self.kneighbors_ = DNDarray(idx, (m, k), types.int64, x.split, x.device, x.comm, True)
        self.classes_ = DNDarray(classes, (m,), types.int64, x.split, x.device, x.comm, True)
        return self.classes_
