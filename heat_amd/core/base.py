"""
Estimator protocol, mirroring heat/core/base.py:13-93 (BaseEstimator), :96-140 (ClassificationMixin),
:184-212 (ClusteringMixin) and :260-306 (is_classifier / is_estimator / is_clusterer).
"""

from __future__ import annotations

import inspect
import json
from typing import Dict, List


class BaseEstimator:
    @classmethod
    def _parameter_names(cls) -> List[str]:
        ctor = cls.__init__
        if ctor is object.__init__:
            return []
        sig = inspect.signature(ctor)
        return [p.name for p in sig.parameters.values()
                if p.name != "self" and p.kind == p.POSITIONAL_OR_KEYWORD]

    def get_params(self, deep: bool = True) -> Dict[str, object]:
        out = {}
        for name in self._parameter_names():
            val = getattr(self, name)
            if deep and hasattr(val, "get_params"):
                val = val.get_params()
            out[name] = val
        return out

    def set_params(self, **params):
        if not params:
            return self
        names = self._parameter_names()
        for key, val in params.items():
            if key not in names:
                raise ValueError(
                    f"Invalid parameter {key} for estimator {self}. Check the list of available "
                    "parameters with `estimator.get_params().keys()`."
                )
            if isinstance(val, dict):
                getattr(self, key).set_params(val)
            else:
                setattr(self, key, val)
        return self

    def __repr__(self, indent: int = 1) -> str:
        return f"{self.__class__.__name__}({json.dumps(self.get_params(), indent=4, default=str)})"


class ClusteringMixin:
    def fit(self, x):
        raise NotImplementedError()

    def fit_predict(self, x):
        self.fit(x)
        return self.predict(x)


class ClassificationMixin:
    def fit(self, x, y):
        raise NotImplementedError()

    def fit_predict(self, x, y):
        self.fit(x, y)
        return self.predict(x)

    def predict(self, x):
        raise NotImplementedError()


def is_classifier(obj: object) -> bool:
    return isinstance(obj, ClassificationMixin)


def is_estimator(obj: object) -> bool:
    return isinstance(obj, BaseEstimator)


def is_clusterer(obj: object) -> bool:
    return isinstance(obj, ClusteringMixin)


__all__ = ["BaseEstimator", "ClassificationMixin", "ClusteringMixin", "is_classifier", "is_estimator", "is_clusterer"]
