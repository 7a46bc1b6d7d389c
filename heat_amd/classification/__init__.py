"""Classification estimators on the distance kernels (heat/classification/__init__.py)."""
from .kneighborsclassifier import KNeighborsClassifier  # noqa: F401

__all__ = ["KNeighborsClassifier"]
