"""GPU parity of the block-sparse (ranges) and batched schemes (keops_conv_ranges)."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity, rel_l2, to_dev
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu

GAUSS = "Exp(-g*SqDist(x,y))*b"
AL = ["x=Vi(3)", "y=Vj(3)", "b=Vj(1)", "g=Pm(1)"]


def _clustered(nclusters, per, seed, sigma=0.05):
    """Config-4 style data: points N(c_k, sigma^2) around centres c_k ~ U[0,10)^3, label-sorted."""
    rng = np.random.default_rng(seed)
    c = (10 * rng.random((nclusters, 3))).astype(np.float32)
    x = (np.repeat(c, per, 0) + sigma * rng.standard_normal((nclusters * per, 3))).astype(np.float32)
    y = (np.repeat(c, per, 0) + sigma * rng.standard_normal((nclusters * per, 3))).astype(np.float32)
    b = rng.standard_normal((nclusters * per, 1)).astype(np.float32)
    return c, x, y, b


def _ranges(c, per, thr=1.0):
    from keops_amd.torch.cluster import from_matrix

    C = c.shape[0]
    r = torch.tensor([[per * k, per * (k + 1)] for k in range(C)], dtype=torch.int64)
    ct = torch.from_numpy(c)
    keep = torch.cdist(ct, ct) < thr
    return from_matrix(r, r, keep), keep


@pytest.mark.parametrize("nclusters,per", [(12, 700), (100, 1000)])
def test_block_sparse_gaussian(nclusters, per):
    from keops_amd.torch import Genred

    c, x, y, b = _clustered(nclusters, per, 3)
    g = np.array([1 / 0.1**2], np.float32)
    ranges, keep = _ranges(c, per)
    M = N = nclusters * per
    conv = Genred(GAUSS, AL, reduction_op="Sum", axis=1)
    got = conv(*to_dev(x, y, b, g), ranges=tuple(r.cuda() for r in ranges)).cpu().numpy()
    rows = np.sort(np.random.default_rng(1).choice(M, min(M, 2048), replace=False)).astype(np.int64)
    r3 = tuple(r.numpy() for r in ranges[:3])
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1, ranges=r3, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 1, ranges=r3, rows=rows)
    assert_sum_parity(got[rows], ref, scale)
    # axis=0 uses the last three ranges; the kept pattern is symmetric here so compare with the transpose problem
    conv0 = Genred("Exp(-g*SqDist(x,y))*a", ["x=Vi(3)", "y=Vj(3)", "a=Vi(1)", "g=Pm(1)"], reduction_op="Sum", axis=0)
    got0 = conv0(*to_dev(x, y, b, g), ranges=tuple(r.cuda() for r in ranges)).cpu().numpy()
    r3t = tuple(r.numpy() for r in ranges[3:])
    ref0 = cpu_reduc("gauss", [y, x, b, g], N, M, 1, ranges=r3t, rows=rows)
    scale0 = cpu_reduc("gauss", [y, x, np.abs(b), g], N, M, 1, ranges=r3t, rows=rows)
    assert_sum_parity(got0[rows], ref0, scale0)


def test_config4_block_sparse_100x10k_row_subset():
    """Headline configuration 4 at its full size: 100 clusters x 10,000 points, seed 3, sigma = 0.1, cluster pairs
    kept when their centres are closer than 1.0; the oracle evaluates 2048 random rows (CpuReduc_ranges.py:150-228)."""
    from keops_amd.torch import Genred

    nclusters, per = 100, 10_000
    c, x, y, b = _clustered(nclusters, per, 3)
    g = np.array([1 / 0.1**2], np.float32)
    ranges, keep = _ranges(c, per)
    M = N = nclusters * per
    conv = Genred(GAUSS, AL, reduction_op="Sum", axis=1)
    dev = to_dev(x, y, b, g)
    rd = tuple(r.cuda() for r in ranges)
    got = conv(*dev, ranges=rd)
    from keops_amd import keops_io

    # the clusters are about three kernel widths across: every row range passes the device-side check and the
    # exponents come from the matrix cores (kernels/keops_radial_ranges.h)
    assert keops_io.last_loader.module.path_status() == 1
    rows = np.sort(np.random.default_rng(1).choice(M, 2048, replace=False)).astype(np.int64)
    r3 = tuple(r.numpy() for r in ranges[:3])
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1, ranges=r3, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 1, ranges=r3, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    # size-independent properties on the full output: exact linearity in b; dropping every range of one row
    # cluster zeroes exactly its rows and leaves the others bit-identical
    assert torch.equal(conv(dev[0], dev[1], 2 * dev[2], dev[3], ranges=rd), 2 * got)
    keep2 = keep.clone()
    keep2[7, :] = False
    from keops_amd.torch.cluster import from_matrix

    r = torch.tensor([[per * k, per * (k + 1)] for k in range(nclusters)], dtype=torch.int64)
    got2 = conv(*dev, ranges=tuple(t.cuda() for t in from_matrix(r, r, keep2)))
    assert torch.all(got2[7 * per:8 * per] == 0)
    assert torch.equal(got2[:7 * per], got[:7 * per]) and torch.equal(got2[8 * per:], got[8 * per:])


def test_config5a_lse_b16_50k_row_subset():
    """Headline configuration 5a at its full size: B = 16 batches of 50,000 x 50,000, eps = 0.05, seed 4; the oracle
    evaluates 128 random rows of every batch."""
    from keops_amd.torch import Genred

    B, M, N = 16, 50_000, 50_000
    rng = np.random.default_rng(4)
    x = rng.standard_normal((B, M, 3)).astype(np.float32)
    y = rng.standard_normal((B, N, 3)).astype(np.float32)
    l = rng.standard_normal((B, N, 1)).astype(np.float32)
    e = np.array([1 / 0.05], np.float32)
    lse = Genred("l-SqDist(x,y)*e", ["x=Vi(3)", "y=Vj(3)", "l=Vj(1)", "e=Pm(1)"], reduction_op="LogSumExp", axis=1)
    xd, yd, ld, ed = to_dev(x, y, l, e)
    got = lse(xd, yd, ld, ed)
    assert tuple(got.shape) == (B, M, 1)
    pick = np.random.default_rng(44)
    for bidx in range(B):
        rows = np.sort(pick.choice(M, 128, replace=False)).astype(np.int64)
        ms = cpu_reduc("lse_gauss", [x[bidx], y[bidx], l[bidx], e], M, N, 2, reduction="Max_SumShiftExp", rows=rows)
        ref = ms[:, 0].astype(np.float64) + np.log(ms[:, 1].astype(np.float64))
        g = got[bidx, torch.from_numpy(rows).cuda(), 0].cpu().numpy()
        assert np.max(np.abs(g - ref) / np.maximum(1, np.abs(ref))) <= 1e-5, bidx
    # size-independent property on the full output: LSE(l + c) = LSE(l) + c (c = 4 is exact on these magnitudes up
    # to one rounding of the sum), and batches are independent: batch 3 alone gives the same bits
    shifted = lse(xd, yd, ld + 4.0, ed)
    assert float((shifted - got - 4.0).abs().max()) <= 2e-5
    alone = lse(xd[3], yd[3], ld[3], ed)
    assert float((alone - got[3]).abs().max()) <= 2e-5


def test_ranges_uncovered_rows_unsorted_and_adjacent_ranges():
    from keops_amd.torch import Genred

    M, N = 5000, 6000
    rng = np.random.default_rng(5)
    x, y = rng.standard_normal((M, 3)).astype(np.float32), rng.standard_normal((N, 3)).astype(np.float32)
    b, g = rng.standard_normal((N, 1)).astype(np.float32), np.array([0.5], np.float32)
    # rows 1200..1999 and 4500.. uncovered; second row range longer than one workgroup; column ranges
    # [0,1000)+[1000,2500) are adjacent (merged by the kernel), [4000,6000) separate, one empty slice
    ranges_i = np.array([[0, 1200], [2000, 4500], [4500, 4500]], np.int64)
    slices_i = np.array([2, 3, 3], np.int64)
    redranges_j = np.array([[0, 1000], [1000, 2500], [4000, 6000]], np.int64)
    dummy = np.zeros((1, 2), np.int64)
    ranges = (ranges_i, slices_i, redranges_j, dummy, np.array([0], np.int64), dummy)
    conv = Genred(GAUSS, AL, reduction_op="Sum", axis=1)
    got = conv(*to_dev(x, y, b, g), ranges=tuple(torch.from_numpy(r).cuda() for r in ranges)).cpu().numpy()
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1, ranges=(ranges_i, slices_i, redranges_j))
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 1, ranges=(ranges_i, slices_i, redranges_j)) + 1e-30
    assert_sum_parity(got, ref, scale)
    assert np.all(got[1200:2000] == 0) and np.all(got[4500:] == 0)
    # index-carrying reduction: global column indices, (inf, 0) on uncovered rows
    vals, idx = Genred("SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], reduction_op="Min_ArgMin", axis=1)(
        *to_dev(x, y), ranges=tuple(torch.from_numpy(r).cuda() for r in ranges))
    refm = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="Min_ArgMin", scheme="direct_sum",
                     ranges=(ranges_i, slices_i, redranges_j))
    assert np.array_equal(vals.cpu().numpy(), refm[:, :1]) and np.array_equal(idx.cpu().numpy(), refm[:, 1:].astype(np.int64))
    assert torch.isinf(vals[1500]).all() and idx[1500].item() == 0


def test_batched_logsumexp_config5a_shape():
    """B batches of an LSE softmin; oracle = loop over batches of the non-batched oracle."""
    from keops_amd.torch import Genred

    B, M, N = 4, 3000, 2500
    rng = np.random.default_rng(4)
    x = rng.standard_normal((B, M, 3)).astype(np.float32)
    y = rng.standard_normal((B, N, 3)).astype(np.float32)
    l = rng.standard_normal((B, N, 1)).astype(np.float32)
    e = np.array([1 / 0.05], np.float32)
    lse = Genred("l-SqDist(x,y)*e", ["x=Vi(3)", "y=Vj(3)", "l=Vj(1)", "e=Pm(1)"], reduction_op="LogSumExp", axis=1)
    got = lse(*to_dev(x, y, l, e)).cpu().numpy()
    assert got.shape == (B, M, 1)
    for bidx in range(B):
        ms = cpu_reduc("lse_gauss", [x[bidx], y[bidx], l[bidx], e], M, N, 2, reduction="Max_SumShiftExp")
        ref = ms[:, 0].astype(np.float64) + np.log(ms[:, 1].astype(np.float64))
        assert np.max(np.abs(got[bidx, :, 0] - ref) / np.maximum(1, np.abs(ref))) <= 1e-5


def test_batch_broadcasting_two_batch_dims_and_gradients():
    """(A,B) batch dims with size-1 broadcasting on x, y and the parameter (cf. the reference's
    pykeops/test/test_torch.py:478-581), forward and gradients against dense torch in float64."""
    from keops_amd.torch import Genred

    A, B, M, N = 2, 3, 150, 170
    rng = np.random.default_rng(6)
    x = torch.from_numpy(rng.standard_normal((A, 1, M, 3))).cuda().requires_grad_(True)
    y = torch.from_numpy(rng.standard_normal((1, B, N, 3))).cuda().requires_grad_(True)
    b = torch.from_numpy(rng.standard_normal((A, B, N, 2))).cuda().requires_grad_(True)
    g = torch.from_numpy(rng.random((1, B, 1)) + 0.5).cuda().requires_grad_(True)
    conv = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)", "g=Pm(1)"], reduction_op="Sum", axis=1)
    out = conv(x, y, b, g)
    assert tuple(out.shape) == (A, B, M, 2)
    K = torch.exp(-g[:, :, None, None, :] * ((x[:, :, :, None, :] - y[:, :, None, :, :]) ** 2).sum(-1, keepdim=True))
    ref = (K * b[:, :, None, :, :]).sum(3)
    assert rel_l2(out.detach().cpu().numpy(), ref.detach().cpu().numpy()) < 1e-12
    E = torch.from_numpy(rng.standard_normal((A, B, M, 2))).cuda()
    got = torch.autograd.grad((out * E).sum(), [x, y, b, g])
    want = torch.autograd.grad((ref * E).sum(), [x, y, b, g])
    for a_, b_ in zip(got, want):
        assert a_.shape == b_.shape
        assert rel_l2(a_.cpu().numpy(), b_.cpu().numpy()) < 1e-11
    # batch-relative indices for Arg reductions
    idx = Genred("SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], reduction_op="ArgMin", axis=1)(x.detach().float(), y.detach().float())
    d = ((x.detach().float()[:, :, :, None, :] - y.detach().float()[:, :, None, :, :]) ** 2).sum(-1)
    assert tuple(idx.shape) == (A, B, M, 1)
    assert (idx[..., 0] == d.argmin(-1)).float().mean() > 0.999  # fp32 near-ties aside


def test_ranges_with_batch_is_rejected():
    from keops_amd.torch import Genred

    x = torch.randn(2, 10, 3, device="cuda")
    y = torch.randn(2, 12, 3, device="cuda")
    r = torch.tensor([[0, 10]], device="cuda")
    rr = (r, torch.tensor([1], device="cuda"), torch.tensor([[0, 12]], device="cuda")) * 2
    with pytest.raises(Exception):
        Genred("SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], reduction_op="Sum", axis=1)(x, y, ranges=rr)
