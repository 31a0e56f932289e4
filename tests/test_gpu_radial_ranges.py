"""GPU parity of block-sparse Gaussian-type sums whose exponents come from the matrix cores
(kernels/keops_radial_ranges.h: one centre per row range, the columns of every range formatted relative to it)
against the CPU oracle (CpuReduc_ranges.py:150-228).  Tolerances: float32 sums 1e-5, norm-wise and relative to
sum_j |F_ij|.  `Module.path_status()` tells which kernel family served a launch."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity, to_dev
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu


def _genred(D, Dv, axis=1, **kw):
    from keops_amd.torch import Genred

    if axis == 1:
        return Genred("Exp(-g*SqDist(x,y))*b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})", "g=Pm(1)"], reduction_op="Sum", axis=1, **kw)
    return Genred("Exp(-g*SqDist(x,y))*a", [f"x=Vi({D})", f"y=Vj({D})", f"a=Vi({Dv})", "g=Pm(1)"], reduction_op="Sum", axis=0, **kw)


def _module():
    from keops_amd import keops_io

    return keops_io.last_loader.module


def _clusters(D, Dv, nclusters, seed, sigma=0.05, box=4.0, lo=2500, hi=4500):
    """Label-sorted points N(c_k, sigma^2) around centres c_k ~ U[0, box)^D, clusters of unequal sizes (not multiples
    of the workgroup's rows or of the column tile)."""
    rng = np.random.default_rng(seed)
    c = (box * rng.random((nclusters, D))).astype(np.float32)
    nx_k, ny_k = rng.integers(lo, hi, nclusters), rng.integers(lo, hi, nclusters)
    x = (np.repeat(c, nx_k, 0) + sigma * rng.standard_normal((nx_k.sum(), D))).astype(np.float32)
    y = (np.repeat(c, ny_k, 0) + sigma * rng.standard_normal((ny_k.sum(), D))).astype(np.float32)
    b = rng.standard_normal((ny_k.sum(), Dv)).astype(np.float32)
    bounds = lambda n: torch.from_numpy(np.stack([np.cumsum(n) - n, np.cumsum(n)], 1).astype(np.int64))
    return c, x, y, b, bounds(nx_k), bounds(ny_k)


def _pattern(c, rx, ry, thr=1.0):
    from keops_amd.torch.cluster import from_matrix

    ct = torch.from_numpy(c)
    keep = torch.cdist(ct, ct) < thr
    return from_matrix(rx, ry, keep), keep


@pytest.mark.parametrize("D,Dv,sigma", [(3, 1, 0.05), (3, 3, 0.05), (2, 8, 0.05), (5, 2, 0.04), (8, 1, 0.03), (3, 12, 0.05)])
def test_block_sparse_gaussian_sums_on_the_matrix_cores_vs_oracle(D, Dv, sigma):
    c, x, y, b, rx, ry = _clusters(D, Dv, 64, 10 * D + Dv, sigma=sigma, box=4.0 if D <= 3 else 2.0)
    g = np.array([100.0], np.float32)
    ranges, keep = _pattern(c, rx, ry)
    M, N = x.shape[0], y.shape[0]
    dev = to_dev(x, y, b, g)
    rd = tuple(r.cuda() for r in ranges)
    conv = _genred(D, Dv)
    got = conv(*dev, ranges=rd)                        # the ranges are read back and validated on the host
    assert _module().meta("rad_ranges") == "1" and _module().path_status() == 1
    again = conv(*dev, ranges=rd)                      # workgroup table built on the device
    assert _module().path_status() == 1 and _module().ranges_status() == 0
    assert torch.equal(again, got)
    rows = np.sort(np.random.default_rng(1).choice(M, 1500, replace=False)).astype(np.int64)
    r3 = tuple(r.numpy() for r in ranges[:3])
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, ranges=r3, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv, ranges=r3, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    assert torch.equal(conv(dev[0], dev[1], 2 * dev[2], dev[3], ranges=rd), 2 * got)   # exact linearity in b


@pytest.mark.parametrize("case", ["inf_row", "nan_row", "huge_column"])
def test_values_that_are_not_finite_or_huge_send_the_call_to_the_general_purpose_kernel(case):
    """A row range that holds an infinite, NaN or huge coordinate fails the per-range check (its largest centred norm is
    not finite, or far beyond the bound), so the general-purpose kernel serves the call: NaN where the reference's
    loops give NaN and nowhere else."""
    D, Dv = 3, 2
    c, x, y, b, rx, ry = _clusters(D, Dv, 64, 23)
    g = np.array([100.0], np.float32)
    ranges, keep = _pattern(c, rx, ry)
    i, j = int(rx[7, 0]) + 5, int(ry[9, 0]) + 3
    if case == "inf_row":
        x[i, 1] = np.inf
    elif case == "nan_row":
        x[i, 1] = np.nan
    else:
        y[j, 2] = 1e30
    dev = to_dev(x, y, b, g)
    rd = tuple(r.cuda() for r in ranges)
    conv = _genred(D, Dv)
    for _ in range(2):                                  # host-validated launch, then device-built tables
        got = conv(*dev, ranges=rd)
        assert _module().meta("rad_ranges") == "1" and _module().path_status() == 0
        want = _genred(D, Dv, enable_chunks=False)(*dev, ranges=rd)
        assert torch.equal(torch.isnan(got), torch.isnan(want))
        assert int(torch.isnan(want).any(dim=1).sum()) == (1 if case == "nan_row" else 0)
        assert torch.equal(torch.nan_to_num(got), torch.nan_to_num(want))


def test_reduction_over_i_uses_the_last_three_ranges():
    D, Dv = 3, 2
    c, x, y, a, rx, ry = _clusters(D, Dv, 64, 5)
    # (here `a` is indexed like x: draw it with the right number of rows)
    a = np.random.default_rng(6).standard_normal((x.shape[0], Dv)).astype(np.float32)
    g = np.array([100.0], np.float32)
    ranges, keep = _pattern(c, rx, ry)
    M, N = x.shape[0], y.shape[0]
    got = _genred(D, Dv, axis=0)(*to_dev(x, y, a, g), ranges=tuple(r.cuda() for r in ranges))
    assert got.shape == (N, Dv) and _module().path_status() == 1
    cols = np.sort(np.random.default_rng(2).choice(N, 1500, replace=False)).astype(np.int64)
    r3t = tuple(r.numpy() for r in ranges[3:])
    ref = cpu_reduc("gauss", [y, x, a, g], N, M, Dv, ranges=r3t, rows=cols)   # roles of i and j exchanged
    scale = cpu_reduc("gauss", [y, x, np.abs(a), g], N, M, Dv, ranges=r3t, rows=cols)
    assert_sum_parity(got[torch.from_numpy(cols).cuda()].cpu().numpy(), ref, scale)


def test_rows_without_columns_and_rows_outside_every_range_are_zero():
    from keops_amd.torch.cluster import from_matrix

    D, Dv = 3, 1
    c, x, y, b, rx, ry = _clusters(D, Dv, 64, 9)
    g = np.array([100.0], np.float32)
    keep = torch.cdist(torch.from_numpy(c), torch.from_numpy(c)) < 1.0
    keep[5, :] = False                                  # row cluster 5 keeps no column cluster
    sel = torch.tensor([k for k in range(64) if k != 11])
    ranges = from_matrix(rx[sel], ry, keep[sel])        # row cluster 11 is in no range at all
    M, N = x.shape[0], y.shape[0]
    dev = to_dev(x, y, b, g)
    out = torch.full((M, Dv), 7.0, device="cuda")
    got = _genred(D, Dv)(*dev, ranges=tuple(r.cuda() for r in ranges), out=out)
    assert _module().path_status() == 1
    for k in (5, 11):
        assert torch.all(got[int(rx[k, 0]):int(rx[k, 1])] == 0)
    rows = np.sort(np.random.default_rng(3).choice(M, 1500, replace=False)).astype(np.int64)
    r3 = tuple(r.numpy() for r in ranges[:3])
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, ranges=r3, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv, ranges=r3, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)


def test_gradient_with_respect_to_the_points_under_ranges_vs_oracle():
    """autograd hands the same ranges to the gradient formula (generic_red.py:152-259): the difference factor
    (x_i - y_j) is formed around the centre of every row range."""
    D = 3
    c, x, y, b, rx, ry = _clusters(D, 1, 64, 21)
    g = np.array([100.0], np.float32)
    ranges, keep = _pattern(c, rx, ry)
    M, N = x.shape[0], y.shape[0]
    xd, yd, bd, gd = to_dev(x, y, b, g)
    xd.requires_grad_(True)
    rd = tuple(r.cuda() for r in ranges)
    a = _genred(D, 1)(xd, yd, bd, gd, ranges=rd)
    e = np.random.default_rng(4).standard_normal((M, 1)).astype(np.float32)
    (gx,) = torch.autograd.grad(a, [xd], torch.from_numpy(e).cuda())
    assert _module().meta("rad_ranges") == "1" and _module().path_status() == 1
    rows = np.sort(np.random.default_rng(5).choice(M, 1500, replace=False)).astype(np.int64)
    r3 = tuple(r.numpy() for r in ranges[:3])
    ref = cpu_reduc("gauss_gradx", [x, y, b, g, e], M, N, D, ranges=r3, rows=rows)
    scale = cpu_reduc("gauss_gradx_abs", [x, y, b, g, e], M, N, D, ranges=r3, rows=rows)
    assert_sum_parity(gx[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)


def test_kernel_too_narrow_for_the_clusters_falls_back_to_exact_differences():
    """sqrt(g) times the radius of a cluster is about 20: the device-side check fails for the ranges, the
    general-purpose kernel of the module runs and the result is bit-identical to a module built without the scheme."""
    D, Dv = 3, 2
    c, x, y, b, rx, ry = _clusters(D, Dv, 64, 31)
    g = np.array([1.0e4], np.float32)
    ranges, keep = _pattern(c, rx, ry)
    M, N = x.shape[0], y.shape[0]
    dev = to_dev(x, y, b, g)
    rd = tuple(r.cuda() for r in ranges)
    got = _genred(D, Dv)(*dev, ranges=rd)
    assert _module().meta("rad_ranges") == "1" and _module().path_status() == 0
    plain = _genred(D, Dv, enable_chunks=False)(*dev, ranges=rd)   # matrix-core schemes switched off
    assert _module().meta("radial") is None
    assert torch.equal(got, plain)
    rows = np.sort(np.random.default_rng(7).choice(M, 1000, replace=False)).astype(np.int64)
    r3 = tuple(r.numpy() for r in ranges[:3])
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, ranges=r3, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv, ranges=r3, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)


def test_short_row_ranges_and_small_patterns_stay_on_the_general_purpose_kernel():
    D, Dv = 3, 1
    c, x, y, b, rx, ry = _clusters(D, Dv, 200, 41, lo=40, hi=90)   # 65-row ranges: formatting a column per range would dominate
    g = np.array([100.0], np.float32)
    ranges, keep = _pattern(c, rx, ry)
    M, N = x.shape[0], y.shape[0]
    got = _genred(D, Dv)(*to_dev(x, y, b, g), ranges=tuple(r.cuda() for r in ranges))
    assert _module().path_status() == 0
    r3 = tuple(r.numpy() for r in ranges[:3])
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, ranges=r3)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv, ranges=r3)
    assert_sum_parity(got.cpu().numpy(), ref, scale)


def test_ranges_edited_in_place_follow_and_an_outgrown_workspace_falls_back():
    """Later launches with the same range tensors read their current contents on the device.  A pattern that loses
    column ranges is followed on the matrix cores; one that grows beyond what the validating launch measured does not
    fit the formatted operand: the general-purpose kernel takes over, same result class."""
    D, Dv = 3, 1
    c, x, y, b, rx, ry = _clusters(D, Dv, 64, 51)
    g = np.array([100.0], np.float32)
    ranges, keep = _pattern(c, rx, ry)
    M, N = x.shape[0], y.shape[0]
    dev = to_dev(x, y, b, g)
    rd = tuple(r.cuda() for r in ranges)
    conv = _genred(D, Dv)
    conv(*dev, ranges=rd)
    assert _module().path_status() == 1
    rows = np.sort(np.random.default_rng(8).choice(M, 800, replace=False)).astype(np.int64)

    def check(expect_taken):
        got = conv(*dev, ranges=rd)
        assert _module().path_status() == expect_taken and _module().ranges_status() == 0
        r3 = tuple(r.cpu().numpy() for r in rd[:3])
        ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, ranges=r3, rows=rows)
        scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv, ranges=r3, rows=rows)
        assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)

    rd[2][::3] = 0                                      # every third reduced-index range becomes [0, 0)
    check(1)
    rd[2][:, 0], rd[2][:, 1] = 0, N                     # every reduced-index range becomes the whole axis
    check(0)


def test_block_sparse_matrix_core_sums_under_graph_capture():
    D, Dv = 3, 2
    c, x, y, b, rx, ry = _clusters(D, Dv, 64, 61)
    g = np.array([100.0], np.float32)
    ranges, keep = _pattern(c, rx, ry)
    xd, yd, bd, gd = to_dev(x, y, b, g)
    rd = tuple(r.cuda() for r in ranges)
    conv = _genred(D, Dv)
    conv(xd, yd, bd, gd, ranges=rd)
    eager = conv(xd, yd, bd, gd, ranges=rd)
    assert _module().path_status() == 1
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        conv(xd, yd, bd, gd, ranges=rd)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = conv(xd, yd, bd, gd, ranges=rd)
    gen = torch.Generator(device="cuda").manual_seed(3)
    for k in range(3):
        bd.copy_(torch.randn(bd.shape, device="cuda", generator=gen))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        assert torch.equal(got, conv(xd, yd, bd, gd, ranges=rd))   # eager launches between the replays


def test_batches_are_served_as_row_ranges_with_one_centre_each():
    """Batch dimensions that no variable is broadcast over (GpuReduc1D_ranges.py:74-173 with the block-diagonal
    ranges of Ranges.h:40-86): every batch is one row range of the flattened arrays with its own centre.  Batches far
    from each other (offsets of 50 kernel widths) would fail a check on one common centre."""
    D, Dv, B, M, N = 3, 2, 7, 9500, 6700   # (at least one workgroup per compute unit: 7 x 38 row blocks)
    rng = np.random.default_rng(61)
    off = (50.0 * rng.standard_normal((B, 1, D))).astype(np.float32)
    x = (rng.standard_normal((B, M, D)) + off).astype(np.float32)
    y = (rng.standard_normal((B, N, D)) + off).astype(np.float32)
    b = rng.standard_normal((B, N, Dv)).astype(np.float32)
    g = np.array([0.6], np.float32)
    dev = to_dev(x, y, b, g)
    got = _genred(D, Dv)(*dev)
    assert got.shape == (B, M, Dv)
    assert _module().meta("rad_ranges") == "1" and _module().path_status() == 1
    rows = np.sort(rng.choice(M, 400, replace=False)).astype(np.int64)
    for k in range(B):
        ref = cpu_reduc("gauss", [x[k], y[k], b[k], g], M, N, Dv, rows=rows)
        scale = cpu_reduc("gauss", [x[k], y[k], np.abs(b[k]), g], M, N, Dv, rows=rows)
        assert_sum_parity(got[k][torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    # the general-purpose kernel gives (slightly) different bits; deterministic from call to call
    plain = _genred(D, Dv, enable_chunks=False)(*dev)
    assert _module().meta("radial") is None and not torch.equal(plain, got)
    assert torch.equal(_genred(D, Dv)(*dev), got)
    # a variable shared by the batches (broadcast) or a parameter per batch keeps the call on the general-purpose kernel
    shared = _genred(D, Dv)(dev[0], dev[1][:1], dev[2], dev[3])
    assert _module().path_status() == 0
    ref = cpu_reduc("gauss", [x[3], y[0], b[3], g], M, N, Dv, rows=rows)
    scale = cpu_reduc("gauss", [x[3], y[0], np.abs(b[3]), g], M, N, Dv, rows=rows)
    assert_sum_parity(shared[3][torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    gs = torch.full((B, 1), 0.6, device="cuda")
    per_batch = _genred(D, Dv)(dev[0], dev[1], dev[2], gs)
    assert _module().path_status() == 0
    assert_sum_parity(per_batch[2][torch.from_numpy(rows).cuda()].cpu().numpy(),
                      cpu_reduc("gauss", [x[2], y[2], b[2], g], M, N, Dv, rows=rows),
                      cpu_reduc("gauss", [x[2], y[2], np.abs(b[2]), g], M, N, Dv, rows=rows))


def test_batched_reduction_over_i_and_two_batch_dimensions():
    D, Dv, B1, B2, M, N = 2, 1, 3, 4, 5200, 5700     # 12 batches of 23 workgroups (the output is indexed by j)
    rng = np.random.default_rng(63)
    x = rng.standard_normal((B1, B2, M, D)).astype(np.float32)
    y = rng.standard_normal((B1, B2, N, D)).astype(np.float32)
    a = rng.standard_normal((B1, B2, M, Dv)).astype(np.float32)
    g = np.array([0.8], np.float32)
    got = _genred(D, Dv, axis=0)(*to_dev(x, y, a, g))
    assert got.shape == (B1, B2, N, Dv) and _module().path_status() == 1
    cols = np.sort(rng.choice(N, 300, replace=False)).astype(np.int64)
    for k1, k2 in ((0, 0), (2, 3), (1, 2)):
        ref = cpu_reduc("gauss", [y[k1, k2], x[k1, k2], a[k1, k2], g], N, M, Dv, rows=cols)   # roles of i and j exchanged
        scale = cpu_reduc("gauss", [y[k1, k2], x[k1, k2], np.abs(a[k1, k2]), g], N, M, Dv, rows=cols)
        assert_sum_parity(got[k1, k2][torch.from_numpy(cols).cuda()].cpu().numpy(), ref, scale)


def test_batches_with_a_kernel_too_narrow_for_them_fall_back():
    D, Dv, B, M, N = 3, 1, 5, 14000, 7800
    rng = np.random.default_rng(62)
    x = rng.standard_normal((B, M, D)).astype(np.float32)
    y = rng.standard_normal((B, N, D)).astype(np.float32)
    b = rng.standard_normal((B, N, Dv)).astype(np.float32)
    g = np.array([400.0], np.float32)
    dev = to_dev(x, y, b, g)
    got = _genred(D, Dv)(*dev)
    assert _module().meta("rad_ranges") == "1" and _module().path_status() == 0
    plain = _genred(D, Dv, enable_chunks=False)(*dev)
    assert torch.equal(got, plain)


def test_batched_matrix_core_sums_under_graph_capture():
    D, Dv, B, M, N = 3, 1, 8, 8448, 8200
    rng = np.random.default_rng(64)
    x = rng.standard_normal((B, M, D)).astype(np.float32)
    y = rng.standard_normal((B, N, D)).astype(np.float32)
    b = rng.standard_normal((B, N, Dv)).astype(np.float32)
    xd, yd, bd, gd = to_dev(x, y, b, np.array([0.5], np.float32))
    conv = _genred(D, Dv)
    conv(xd, yd, bd, gd)
    assert _module().path_status() == 1
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        conv(xd, yd, bd, gd)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = conv(xd, yd, bd, gd)
    gen = torch.Generator(device="cuda").manual_seed(5)
    for k in range(3):
        bd.copy_(torch.randn(bd.shape, device="cuda", generator=gen))
        xd.add_(0.01)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        assert torch.equal(got, conv(xd, yd, bd, gd))   # eager launches between the replays


def test_gradient_with_respect_to_the_points_of_batched_sums_vs_dense_float64():
    """The gradient is another batched map-reduce (generic_red.py:165-214) of the same family: it takes the same
    kernels, one centre per batch."""
    D, Dv, B, M, N = 3, 1, 8, 8448, 8300   # (scalar weights: <b_j, e_i> is then a product of a row and a column factor)
    gen = torch.Generator(device="cuda").manual_seed(65)
    x = torch.randn(B, M, D, device="cuda", generator=gen) + 30.0 * torch.randn(B, 1, D, device="cuda", generator=gen)
    y = x[:, :N].clone() + 0.3 * torch.randn(B, N, D, device="cuda", generator=gen)
    b = torch.randn(B, N, Dv, device="cuda", generator=gen)
    e = torch.randn(B, M, Dv, device="cuda", generator=gen)
    g = torch.tensor([0.7], device="cuda")
    x.requires_grad_(True)
    (_genred(D, Dv)(x, y, b, g) * e).sum().backward()
    assert _module().meta("rad_ranges") == "1" and _module().path_status() == 1
    for k in (0, 5):
        xk = x[k].detach().double().requires_grad_(True)
        K = torch.exp(-0.7 * torch.cdist(xk, y[k].double()) ** 2)
        ((K @ b[k].double()) * e[k].double()).sum().backward()
        err = (x.grad[k].double() - xk.grad).norm() / xk.grad.norm()
        assert float(err) <= 1e-5, float(err)


def test_batched_gradient_with_vector_weights_forms_the_scalar_product_per_pair():
    """Momentum-weighted gradient of shape models, batched: sum_j K_ij <e_i, b_j> (x_i - y_j) with three-component
    e and b; the range kernels read e_i of their rows from the arguments (rows of a batch, clamped to its end)."""
    D, Dv, B, M, N = 3, 3, 9, 7500, 7600     # 7500 rows: the last workgroup of every batch is ragged
    gen = torch.Generator(device="cuda").manual_seed(66)
    x = torch.randn(B, M, D, device="cuda", generator=gen) + 20.0 * torch.randn(B, 1, D, device="cuda", generator=gen)
    y = x[:, :N].clone() if N <= M else torch.randn(B, N, D, device="cuda", generator=gen) + x.mean(1, keepdim=True)
    b = torch.randn(B, N, Dv, device="cuda", generator=gen)
    e = torch.randn(B, M, Dv, device="cuda", generator=gen)
    g = torch.tensor([0.7], device="cuda")
    x.requires_grad_(True)
    (_genred(D, Dv)(x, y, b, g) * e).sum().backward()
    assert _module().meta("rad_ranges") == "1" and _module().meta("rad_dv") == "4" and _module().path_status() == 1
    for k in (0, 8):
        xk = x[k].detach().double().requires_grad_(True)
        K = torch.exp(-0.7 * torch.cdist(xk, y[k].double()) ** 2)
        ((K @ b[k].double()) * e[k].double()).sum().backward()
        err = (x.grad[k].double() - xk.grad).norm() / xk.grad.norm()
        assert float(err) <= 1e-5, float(err)
