"""Graph tools on the distance kernels (heat/graph/__init__.py)."""
from .laplacian import Laplacian  # noqa: F401

__all__ = ["Laplacian"]
