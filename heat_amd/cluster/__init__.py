"""Clustering estimators (subset of heat/cluster)."""
from .kmeans import KMeans  # noqa: F401
from ._kcluster import _KCluster  # noqa: F401
from .batchparallelclustering import BatchParallelKMeans  # noqa: F401
