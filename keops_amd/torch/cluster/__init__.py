"""Block-sparse reduction helpers on torch tensors: cluster labelling, sorting, ranges.

Same functions, argument meaning and return values as pykeops/pykeops/torch/cluster
(utils.py:4-245, matrix.py:4-130, grid_cluster.py:4-53)."""
from .utils import (  # noqa: F401
    cluster_centroids, cluster_ranges, cluster_ranges_centroids, from_matrix, grid_cluster, sort_clusters, swap_axes,
)
