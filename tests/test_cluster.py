"""Known-answer tests of the block-sparse helpers: the literal examples of the reference's
docstrings (pykeops/pykeops/torch/cluster/matrix.py:62-111, utils.py:26-37,74-93,127-134,198-217,
grid_cluster.py:19-23)."""
import torch

from keops_amd.torch.cluster import (
    cluster_centroids, cluster_ranges, cluster_ranges_centroids, from_matrix, grid_cluster, sort_clusters, swap_axes,
)


def test_from_matrix_docstring_example():
    r_i = torch.tensor([[2, 5], [7, 12]])
    r_j = torch.tensor([[1, 4], [4, 9], [20, 30]])
    x, y = torch.tensor([1.0, 0.0]), torch.tensor([1.5, 0.5, 2.5])
    keep = (x[:, None] - y[None, :]) ** 2 <= 1
    assert keep.tolist() == [[True, True, False], [False, True, False]]
    ranges_i, slices_i, redranges_j, ranges_j, slices_j, redranges_i = from_matrix(r_i, r_j, keep)
    assert ranges_i.tolist() == [[2, 5], [7, 12]]
    assert slices_i.tolist() == [2, 3]
    assert redranges_j.tolist() == [[1, 4], [4, 9], [4, 9]]
    assert ranges_j.tolist() == [[1, 4], [4, 9], [20, 30]]
    assert slices_j.tolist() == [1, 3, 3]
    assert redranges_i.tolist() == [[2, 5], [2, 5], [7, 12]]
    sw = swap_axes((ranges_i, slices_i, redranges_j, ranges_j, slices_j, redranges_i))
    assert sw[0] is ranges_j and sw[3] is ranges_i and swap_axes(None) is None


def test_sort_clusters_and_ranges_docstring_example():
    x = torch.tensor([[0.0], [5.0], [0.4], [0.3], [2.0]])
    lab = torch.tensor([0, 2, 0, 0, 1], dtype=torch.int32)
    xs, labs = sort_clusters(x, lab)
    assert labs.tolist() == [0, 0, 0, 1, 2]
    assert sorted(xs[:3, 0].tolist()) == [0.0, 0.30000001192092896, 0.4000000059604645] and xs[3:, 0].tolist() == [2.0, 5.0]
    assert cluster_ranges(lab).tolist() == [[0, 3], [3, 4], [4, 5]]
    (a, b), _ = sort_clusters((x, 2 * x), lab)
    assert torch.equal(b, 2 * a)


def test_centroids_docstring_examples():
    x = torch.tensor([[0.0], [1.0], [4.0], [5.0], [6.0]])
    lab = torch.tensor([0, 0, 1, 1, 1], dtype=torch.int32)
    w = torch.tensor([0.5, 0.5, 2.0, 1.0, 1.0])
    assert torch.allclose(cluster_centroids(x, lab, weights=w), torch.tensor([[0.5], [4.75]]))
    x = torch.tensor([[0.0], [0.5], [1.0], [2.0], [3.0]])
    ranges, c, wc = cluster_ranges_centroids(x, lab)
    assert ranges.tolist() == [[0, 2], [2, 5]]
    assert torch.allclose(c, torch.tensor([[0.25], [2.0]])) and wc.tolist() == [2.0, 3.0]
    w = torch.tensor([1.0, 0.5, 1.0, 1.0, 10.0])
    ranges, c, wc = cluster_ranges_centroids(x, lab, weights=w)
    assert torch.allclose(c, torch.tensor([[1 / 6], [2.75]])) and torch.allclose(wc, torch.tensor([1.5, 12.0]))


def test_grid_cluster_docstring_example():
    x = torch.tensor([[0.0], [0.1], [0.9], [0.05], [0.5]])
    assert grid_cluster(x, 0.2).tolist() == [0, 0, 2, 0, 1]
    x3 = torch.rand(500, 3)
    lab = grid_cluster(x3, 0.25)
    cells = (x3 - x3.min(0, keepdim=True).values).div(0.25).floor()
    same = (cells[:, None, :] == cells[None, :, :]).all(-1)
    assert torch.equal(same, lab[:, None] == lab[None, :])
    assert lab.min() == 0 and lab.max() == len(torch.unique(lab)) - 1
