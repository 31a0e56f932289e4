import torch


def grid_cluster(x, size):
    """Labels of the cubic cells of side ``size`` that contain the points x (M,D), D <= 3.
    Labels are compact integers in [0,C), ordered like the lexicographic order of the cells
    (pykeops/torch/cluster/grid_cluster.py:4-53; docstring example: x=[0,.1,.9,.05,.5], size .2 ->
    [0,0,2,0,1])."""
    if x.shape[1] > 3:
        raise NotImplementedError("grid_cluster handles points of dimension 1, 2 or 3")
    with torch.no_grad():
        cells = ((x - x.min(dim=0, keepdim=True).values) / size).floor().to(torch.int64)
        key = torch.zeros(x.shape[0], dtype=torch.int64, device=x.device)
        for d in range(x.shape[1]):
            key = key * 1024 + cells[:, d]  # 10 bits per axis, as the reference's 2**10 / 2**20 weights
        _, lab = torch.unique(key, sorted=True, return_inverse=True)
    return lab.to(torch.int32)


def sort_clusters(x, lab):
    """Sort points (a tensor, or a tuple / list of tensors) and labels so that clusters are
    contiguous in memory (utils.py:4-47)."""
    lab, perm = torch.sort(lab.view(-1))
    if isinstance(x, tuple):
        return tuple(a[perm] for a in x), lab
    if isinstance(x, list):
        return [a[perm] for a in x], lab
    return x[perm], lab


def cluster_ranges(lab, Nlab=None):
    """(C,2) int64 [start,end) slices of the C clusters of a label-sorted cloud (utils.py:50-98)."""
    if Nlab is None:
        Nlab = torch.bincount(lab)
    ends = torch.cumsum(Nlab.to(torch.int64), 0)
    return torch.stack((ends - Nlab.to(torch.int64), ends), dim=1)


def cluster_centroids(x, lab, Nlab=None, weights=None, weights_c=None):
    """(C,D) weighted barycentres of the classes given by ``lab`` (utils.py:101-150)."""
    lab = lab.to(torch.int64)
    C = int(lab.max()) + 1 if Nlab is None else len(Nlab)
    w = torch.ones(x.shape[0], dtype=x.dtype, device=x.device) if weights is None else weights.view(-1).to(x.dtype)
    if weights_c is None:
        weights_c = torch.zeros(C, dtype=x.dtype, device=x.device).index_add_(0, lab, w)
    sums = torch.zeros((C, x.shape[1]), dtype=x.dtype, device=x.device).index_add_(0, lab, x * w[:, None])
    return sums / weights_c.view(-1, 1).to(x.dtype)


def cluster_ranges_centroids(x, lab, weights=None, min_weight=1e-9):
    """(ranges, centroids, total weight per cluster) of a labelled cloud (utils.py:153-232)."""
    Nlab = torch.bincount(lab)
    if weights is None:
        return cluster_ranges(lab, Nlab), cluster_centroids(x, lab, Nlab), Nlab.to(x.dtype)
    weights = weights.clone()
    weights[weights <= min_weight] = min_weight
    w_c = torch.bincount(lab, weights=weights).view(-1)
    return cluster_ranges(lab, Nlab), cluster_centroids(x, lab, Nlab, weights=weights, weights_c=w_c), w_c


def swap_axes(ranges):
    """Exchange the i and j halves of a 6-tuple of ranges (utils.py:235-245)."""
    if ranges is None:
        return None
    return (*ranges[3:6], *ranges[0:3])


def from_matrix(ranges_i, ranges_j, keep):
    """Turn a boolean (Mc,Nc) cluster-to-cluster mask into the 6-tuple
    (ranges_i, slices_i, redranges_j, ranges_j, slices_j, redranges_i) of Genred's ``ranges``
    argument (matrix.py:4-130)."""
    keep = keep.to(torch.bool)
    rows, cols = torch.nonzero(keep, as_tuple=True)          # row-major order: grouped by i-cluster
    cols_t, rows_t = torch.nonzero(keep.t(), as_tuple=True)  # grouped by j-cluster
    redranges_j = ranges_j[cols]
    redranges_i = ranges_i[rows_t]
    slices_i = keep.sum(1).cumsum(0).to(torch.int64)
    slices_j = keep.sum(0).cumsum(0).to(torch.int64)
    return (ranges_i, slices_i, redranges_j, ranges_j, slices_j, redranges_i)
