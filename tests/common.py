"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch


def to_dev(*arrays):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrays]


def rel_l2(got, ref):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    return np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-300)


def assert_sum_parity(got, ref, scale, tol=1e-5):
    """Parity metric for floating-point sums: norm-wise relative error <= tol and element-wise
    |a_i - ref_i| <= tol * sum_j |F_ij| (condition-aware: signed weights can make |ref_i| tiny)."""
    got, ref, scale = (np.asarray(t, np.float64) for t in (got, ref, scale))
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert rel_l2(got, ref) <= tol, f"norm-wise error {rel_l2(got, ref):.3e}"
    worst = np.max(np.abs(got - ref) / np.maximum(scale, 1e-30))
    assert worst <= tol, f"element-wise error {worst:.3e} (relative to sum |F_ij|)"
