"""
heat_amd -- the k-means Lloyd path of Heat (cdist -> argmin -> per-cluster mean) on MI355X.

Same call surface as the reference for this path::

    import heat_amd as ht
    x = ht.array(torch_tensor_on_gpu, split=0)
    km = ht.cluster.KMeans(n_clusters=8, init=c0, max_iter=10, tol=0.0).fit(x)
    km.cluster_centers_, km.labels_, km.inertia_, km.n_iter_
    d = ht.spatial.cdist(x, y, quadratic_expansion=True)

Arithmetic runs in hand-written gfx950 kernels loaded through ctypes (``heat_amd/_native.py``).
"""
from .core import *  # noqa: F401,F403
from .core import types, devices, communication, factories, base, dndarray  # noqa: F401
from . import classification, cluster, graph, spatial, utils  # noqa: F401
from . import _native  # noqa: F401

__version__ = "0.3.2"  # = hkm_version() of the library this binding was written for (_native.LIB_VERSION)
