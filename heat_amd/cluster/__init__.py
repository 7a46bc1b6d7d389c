"""Clustering estimators (subset of heat/cluster)."""
from .kmeans import KMeans  # noqa: F401
from ._kcluster import _KCluster  # noqa: F401
from .kmedians import KMedians  # noqa: F401
from .kmedoids import KMedoids  # noqa: F401
from .batchparallelclustering import BatchParallelKMeans, BatchParallelKMedians  # noqa: F401
from .metrics import silhouette_samples, silhouette_score  # noqa: F401
