"""Gaussian kernel sums whose exponents come from the matrix cores (kernels/keops_radial_mfma.h): parity with the CPU
oracle where the device takes that path, and bit-identity with the general-purpose kernel where the device decides
against it (kernels much narrower than the cloud, clouds far from their mean)."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity, to_dev
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu

GAUSS = "Exp(-g*SqDist(x,y))*b"


@pytest.fixture(autouse=True)
def _scheme_from_2_to_the_28_pairs(monkeypatch):
    """By default the scheme takes dense calls from 2**29 pairs on, where it is the faster one; the cases below are a
    little above 2**28 pairs, which keeps their oracle comparisons short and exercises the same kernels."""
    from keops_amd import config

    monkeypatch.setattr(config, "radial_min_pairs_log2", 29)


def _genred(D, Dv, axis=1, **kw):
    from keops_amd.torch import Genred

    bcat = "Vj" if axis == 1 else "Vi"
    return Genred(GAUSS, [f"x=Vi({D})", f"y=Vj({D})", f"b={bcat}({Dv})", "g=Pm(1)"], reduction_op="Sum", axis=axis, **kw)


def _plain(D, Dv, axis=1):
    """The same reduction with the matrix-core schemes switched off: the general-purpose kernel alone."""
    return _genred(D, Dv, axis, enable_chunks=False)


def _last_meta(key):
    from keops_amd import keops_io

    return keops_io.last_loader.module.meta(key)


def _path_status():
    """1 when the device let the matrix-core kernels serve the last launch, 0 when the general-purpose kernel did."""
    from keops_amd import keops_io

    return keops_io.last_loader.module.path_status()


@pytest.mark.parametrize("D,Dv,M,N", [(3, 1, 30011, 30500), (3, 8, 20000, 21000), (3, 2, 300000, 1001), (5, 3, 17000, 23001),
                                      (8, 1, 16000, 18000), (2, 4, 33333, 10001), (6, 7, 18011, 19003), (3, 10, 17000, 16500),
                                      (3, 16, 16400, 16700), (4, 23, 16500, 16400)])
def test_gaussian_sums_with_matrix_core_exponents_vs_oracle(D, Dv, M, N):
    rng = np.random.default_rng(100 * D + Dv)
    x = rng.standard_normal((M, D)).astype(np.float32)
    y = (rng.standard_normal((N, D)) + 0.3).astype(np.float32)   # not centred on the origin: the kernels centre on mean(y)
    b = rng.standard_normal((N, Dv)).astype(np.float32)
    g = np.array([0.7], np.float32)
    dev = to_dev(x, y, b, g)
    got = _genred(D, Dv)(*dev)
    assert _last_meta("radial") == "1"
    # from seven components on, the weighted sum runs on the matrix cores too (three-term operands; beyond ten components
    # the operand columns take two or three blocks)
    assert _last_meta("rad_mm") == ("1" if Dv >= 7 else "0")
    rows = np.sort(rng.choice(M, 1500, replace=False)).astype(np.int64)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    # the matrix-core path really ran: the general-purpose kernel gives (slightly) different bits
    plain = _plain(D, Dv)(*dev)
    assert _last_meta("radial") is None
    assert not torch.equal(plain, got)
    assert_sum_parity(plain[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    # exact linearity in the weights, deterministic from call to call
    assert torch.equal(_genred(D, Dv)(dev[0], dev[1], 2 * dev[2], dev[3]), 2 * got)
    assert torch.equal(_genred(D, Dv)(*dev), got)


def test_default_threshold_of_the_scheme(monkeypatch):
    from keops_amd import config

    monkeypatch.setattr(config, "radial_min_pairs_log2", 30)      # the library's default
    gen = torch.Generator(device="cuda").manual_seed(5)
    for n, served in ((17000, None), (24000, "1")):                # 2**28.1 and 2**29.1 pairs
        x, y = torch.randn(n, 3, device="cuda", generator=gen), torch.randn(n, 3, device="cuda", generator=gen)
        b, g = torch.randn(n, 1, device="cuda", generator=gen), torch.tensor([0.7], device="cuda")
        got = _genred(3, 1)(x, y, b, g)
        assert _last_meta("radial") == served
        ref = torch.exp(-0.7 * torch.cdist(x[:512].double(), y.double()) ** 2) @ b.double()
        assert torch.allclose(got[:512].double(), ref, rtol=0, atol=1e-5 * float(ref.abs().max()))


def test_reduction_over_i_and_formula_spellings():
    from keops_amd.torch import Genred

    M, N, D = 21000, 19000, 3
    rng = np.random.default_rng(9)
    x, y = rng.standard_normal((M, D)).astype(np.float32), rng.standard_normal((N, D)).astype(np.float32)
    a = rng.standard_normal((M, 2)).astype(np.float32)
    s = np.array([1.3], np.float32)
    conv = Genred("Exp(-SqDist(x,y)/(2*s*s))*a", [f"x=Vi({D})", f"y=Vj({D})", "a=Vi(2)", "s=Pm(1)"], reduction_op="Sum", axis=0)
    got = conv(*to_dev(x, y, a, s)).cpu().numpy()
    assert _last_meta("radial") == "1" and got.shape == (N, 2)
    g = np.array([1 / (2 * 1.3 ** 2)], np.float32)
    rows = np.arange(0, N, 13, dtype=np.int64)
    ref = cpu_reduc("gauss", [y, x, a, g], N, M, 2, rows=rows)   # roles of i and j exchanged
    scale = cpu_reduc("gauss", [y, x, np.abs(a), g], N, M, 2, rows=rows)
    assert_sum_parity(got[rows], ref, scale)
    # no weights at all: sum_j exp(-|x - y|^2)
    ones = Genred("Exp(-SqDist(x,y))", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="Sum", axis=1)(*to_dev(x, y)).cpu().numpy()
    assert _last_meta("radial") == "1"
    ref1 = cpu_reduc("gauss", [x, y, np.ones((N, 1), np.float32), np.ones(1, np.float32)], M, N, 1, rows=rows[:800])
    assert_sum_parity(ones[rows[:800]], ref1, ref1)


@pytest.mark.parametrize("case", ["narrow", "far"])
def test_device_side_decision_falls_back_to_exact_differences(case):
    """Where most pairs have |c| log2(e) (|x^|^2 + |y^|^2) beyond the bound (a kernel much narrower than the cloud, a
    cloud much wider than the kernel), taking them one sub-tile at a time from exact differences would be slower than
    the general-purpose kernel: the device skips the matrix-core kernels and the general-purpose kernel of the same
    module runs.  Same code, same slabs: bit-identical to the module built without the matrix-core kernels."""
    M, N, D = 20000, 20000, 3
    rng = np.random.default_rng(3)
    x, y = rng.random((M, D)).astype(np.float32), rng.random((N, D)).astype(np.float32)
    if case == "narrow":
        g = np.array([1 / 0.05 ** 2], np.float32)              # kernel width 0.05 in the unit cube
    else:
        x, y, g = x * 100, y * 100, np.array([0.5], np.float32)  # width 1 in a cube of side 100
    b = rng.standard_normal((N, 1)).astype(np.float32)
    dev = to_dev(x, y, b, g)
    got = _genred(D, 1)(*dev)
    assert _last_meta("radial") == "1" and _path_status() == 0
    plain = _plain(D, 1)(*dev)
    assert torch.equal(got, plain)
    rows = np.arange(0, M, 17, dtype=np.int64)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 1, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale + 1e-30)


@pytest.mark.parametrize("D,Dv", [(3, 1), (3, 8), (7, 2)])
def test_outliers_cost_their_own_tiles_only(D, Dv):
    """A few far points on either side used to send the whole call to the general-purpose kernel (the check was on
    the cloud-wide largest norms).  The clouds are sorted by their centred norms and the choice is made per tile: the
    outliers' tiles are computed from exact differences, everything else keeps the matrix-core exponents.  The rows
    of the outliers themselves (all their pairs far in the tail, or a single near neighbour) are part of the check."""
    M, N = 21000, 20000
    rng = np.random.default_rng(30 + D)
    x, y = rng.standard_normal((M, D)).astype(np.float32), rng.standard_normal((N, D)).astype(np.float32)
    x[5] += 40.0
    x[777] -= 25.0
    y[11] = x[5] + 0.3      # y[11] and x[5] are neighbours, far from everything else
    y[4000] = x[777] + 0.1
    b = (0.1 + np.abs(rng.standard_normal((N, Dv)))).astype(np.float32)
    g = np.array([0.9], np.float32)
    dev = to_dev(x, y, b, g)
    got = _genred(D, Dv)(*dev)
    assert _last_meta("radial") == "1" and _path_status() == 1
    rows = np.unique(np.concatenate([np.array([5, 777]), rng.choice(M, 1500, replace=False)])).astype(np.int64)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows)
    assert ref[list(rows).index(5)].max() > 1e-3 and ref[list(rows).index(777)].max() > 1e-3   # their near neighbours count
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, ref)
    assert torch.equal(_genred(D, Dv)(*dev), got)


def _shell_case(D, Dv, q_lo, q_hi, seed, M=16500, N=16400, g=1.0):
    """Rows with one to three effective neighbours and positive weights: the columns lie on spheres around the centre
    whose radii put |c| log2(e) |y^|^2 in [q_lo, q_hi]; row i sits at a kernel width from column j(i) (and, for a third
    of the rows, from a second column placed beside it), and everything else is tens of widths away.  A row's sum is
    one or two kernel values: its error is the error of a single exponent, nothing averages out."""
    rng = np.random.default_rng(seed)
    kappa = g * 1.4426950408889634
    q = rng.uniform(q_lo, q_hi, (N, 1))
    y = rng.standard_normal((N, D))
    y *= np.sqrt(q / kappa) / np.linalg.norm(y, axis=1, keepdims=True)
    twin = rng.choice(N, N // 3, replace=False)
    y[twin] = y[(twin + 1) % N] + 0.3 * rng.standard_normal((len(twin), D)) / np.sqrt(D)
    y -= y.mean(0)
    j = rng.integers(0, N, M)
    delta = rng.standard_normal((M, D))
    delta *= np.sqrt(rng.uniform(0.2, 2.0, (M, 1)) / g) / np.linalg.norm(delta, axis=1, keepdims=True)
    x = y[j] + delta
    b = rng.uniform(0.5, 1.5, (N, Dv))
    return x.astype(np.float32), y.astype(np.float32), b.astype(np.float32), np.array([g], np.float32)


@pytest.mark.parametrize("D,Dv,q_lo,q_hi,path", [
    (8, 1, 10.0, 12.5, 1),    # |c| log2(e) (|x^|^2 + |y^|^2) just under the bound for every pair that counts: matrix cores
    (7, 3, 10.0, 12.5, 1),
    (3, 8, 10.0, 12.5, 1),    # (weighted sum on the matrix cores too)
    (8, 1, 2.0, 17.0, 1),     # a shell of the cloud beyond the bound: its tiles from exact differences, the rest as above
    (7, 2, 2.0, 17.0, 1),
    (8, 1, 55.0, 65.0, 0),    # everything far beyond (the old cloud-wide bound of 128 let this through): general-purpose kernel
    (7, 1, 55.0, 65.0, 0),
])
def test_rows_with_one_to_three_effective_neighbours(D, Dv, q_lo, q_hi, path):
    """The a-priori bound of the matrix-core exponents (3.3e-7 times |c| log2(e) (|x^|^2 + |y^|^2) <= 1e-5 under the
    per-tile bound of 30) tested where nothing hides an error: every row is one or two pairs, all weights positive."""
    x, y, b, g = _shell_case(D, Dv, q_lo, q_hi, seed=1000 * D + int(q_hi))
    M, N = len(x), len(y)
    dev = to_dev(x, y, b, g)
    got = _genred(D, Dv)(*dev)
    assert _last_meta("radial") == "1" and _path_status() == path
    rows = np.arange(0, M, 3, dtype=np.int64)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows)
    out = got[torch.from_numpy(rows).cuda()].cpu().numpy()
    # positive weights: sum |K b| is the sum itself, the bar is a plain relative one, row by row
    assert ref.min() > 0
    worst = float(np.max(np.abs(out.astype(np.float64) - ref) / ref))
    assert worst <= 1e-5, f"element-wise relative error {worst:.3e}"
    # float64 truth: the same bar (the oracle's own float32 rounding is far below it here: every exponent is small)
    xd, yd = (torch.from_numpy(a).double().cuda() for a in (x, y))
    truth = (torch.exp(-float(g[0]) * torch.cdist(xd[torch.from_numpy(rows).cuda()], yd) ** 2) @ torch.from_numpy(b).double().cuda()).cpu().numpy()
    assert float(np.max(np.abs(out - truth) / truth)) <= 1e-5


def test_one_far_outlier_in_a_large_cloud_keeps_the_matrix_core_path():
    """10^6 x 10^6 with one row and one column thirty cloud radii away: the outliers' tiles are computed from exact
    differences, the launch stays on the matrix cores (the time is the benchmark's business: bench.py --workload
    gauss_1m_dv1 measures the same call without outliers) and the outliers' own rows meet the bar."""
    M = N = 1_000_000
    rng = np.random.default_rng(77)
    x, y = rng.standard_normal((M, 3)).astype(np.float32), rng.standard_normal((N, 3)).astype(np.float32)
    x[123456] += 100.0
    y[654321] = x[123456] + 0.5
    y[7] -= 80.0
    b = rng.standard_normal((N, 1)).astype(np.float32)
    g = np.array([1.0], np.float32)
    got = _genred(3, 1)(*to_dev(x, y, b, g))
    assert _last_meta("radial") == "1" and _path_status() == 1
    rows = np.unique(np.concatenate([[123456], rng.choice(M, 700, replace=False)])).astype(np.int64)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 1, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)


@pytest.mark.parametrize("case", ["nan_row", "inf_row", "huge_row", "inf_column", "huge_column", "nan_column", "nan_weight"])
def test_values_that_are_not_finite_or_huge_behave_as_on_the_general_purpose_kernel(case):
    """The reference's loops give a NaN or infinite coordinate of x_i to row i alone, an infinite or huge y_j a kernel
    value of zero in every row, a NaN in y_j or b_j to every row: the sort, the centre and the device-side choice of
    the matrix-core family must not change that."""
    M, N, Dv = 17000, 16500, 2
    gen = torch.Generator(device="cuda").manual_seed(12)
    x, y = torch.randn(M, 3, device="cuda", generator=gen), torch.randn(N, 3, device="cuda", generator=gen)
    b, g = torch.randn(N, Dv, device="cuda", generator=gen), torch.tensor([0.7], device="cuda")
    if case == "nan_row":
        x[4321, 1] = float("nan")
    elif case == "inf_row":
        x[4321, 1] = float("inf")
    elif case == "huge_row":
        x[4321, 1] = 3e19          # its square overflows float32
    elif case == "inf_column":
        y[1234, 2] = float("-inf")
    elif case == "huge_column":
        y[1234, 2] = 1e30
    elif case == "nan_column":
        y[1234, 0] = float("nan")
    else:
        b[1234, 1] = float("nan")
    got = _genred(3, Dv)(x, y, b, g)
    assert _last_meta("radial") == "1"
    want = _plain(3, Dv)(x, y, b, g)
    assert _last_meta("radial") is None
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    ok = ~torch.isnan(want)
    if case in ("nan_row", "inf_row", "huge_row"):
        assert int((~ok).any(dim=1).sum()) == (1 if case == "nan_row" else 0) and bool(ok[:4321].all()) and bool(ok[4322:].all())
        if case != "nan_row":
            assert float(got[4321].abs().max()) == 0.0     # exp(-inf): no neighbour
    elif case in ("inf_column", "huge_column"):
        assert bool(ok.all())
    elif case == "nan_column":
        assert not bool(ok.any())
    else:
        assert not bool(ok[:, 1].any()) and bool(ok[:, 0].all())
    if ok.any():
        scale = _plain(3, Dv)(x, y, torch.nan_to_num(b).abs(), g)
        err = ((got - want).abs() / scale.clamp_min(1e-30))[ok]
        assert float(err.max()) <= 1e-5


@pytest.mark.parametrize("D,Dv,M,N,ratio,offset", [
    (7, 23, 24918, 13490, 0.101, 0.0),     # every live term of a row has an exponent of -50 ... -87
    (8, 20, 16004, 18283, 0.0448, 30.0),
    (7, 1, 17000, 16500, 0.16, 0.0),
    (8, 3, 6000, 7000, 0.08, 1.0),         # (a small call: the module has no matrix-core kernels at all)
    (3, 1, 9000, 8000, 0.02, 0.0),
])
def test_kernels_far_narrower_than_the_cloud_keep_parity_in_the_deep_tail(D, Dv, M, N, ratio, offset):
    """A kernel 5 to 50 times narrower than the cloud in 7-8 dimensions: nearly every pair is tens of widths apart, the
    rows sum kernel values of 1e-22 ... 1e-38, and an exponential magnifies the relative error of its argument 50 to
    87 times.  The general-purpose kernel (these calls end there: the device-side estimate finds nearly every tile
    beyond the matrix cores' bound) forms the argument as the reference does, rounding for rounding, so the values
    agree with the oracle to the bar where they are not denormal; against float64 the error is the reference's own
    plus a few 1e-6."""
    rng = np.random.default_rng(int(1000 * ratio) + D)
    spread = 0.3
    x = (rng.standard_normal((M, D)) * spread + offset * spread).astype(np.float32)
    y = (rng.standard_normal((N, D)) * spread + offset * spread).astype(np.float32)
    b = np.abs(rng.standard_normal((N, Dv))).astype(np.float32)
    width = ratio * spread
    g = np.array([1.0 / (2 * width * width)], np.float32)
    got = _genred(D, Dv)(*to_dev(x, y, b, g))
    if M * N >= 1 << 28:
        assert _last_meta("radial") == "1" and _path_status() == 0
    rows = np.sort(rng.choice(M, 4000, replace=False)).astype(np.int64)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows)
    out = got[torch.from_numpy(rows).cuda()].cpu().numpy().astype(np.float64)
    live = ref.min(axis=1) > 1e-30                # (positive weights: the sum is its own scale)
    assert live.sum() >= 50
    deep = -np.log(ref[live].max(axis=1) / b.max()) # at least this deep in the tail
    assert np.median(deep) > 10
    worst = float(np.max(np.abs(out[live] - ref[live]) / ref[live]))
    assert worst <= 1e-5, f"against the oracle: {worst:.3e}"
    sel = torch.from_numpy(rows[live]).cuda()
    xd, yd = torch.from_numpy(x).double().cuda(), torch.from_numpy(y).double().cuda()
    d2 = ((xd[sel][:, None, :] - yd[None, :, :]) ** 2).sum(-1)
    truth = (torch.exp(-float(g[0]) * d2) @ torch.from_numpy(b).double().cuda()).cpu().numpy()
    own = float(np.max(np.abs(ref[live] - truth) / truth))
    vs_truth = float(np.max(np.abs(out[live] - truth) / truth))
    assert vs_truth <= own + 6e-6, f"against float64: {vs_truth:.3e} (the reference's own float32 evaluation: {own:.3e})"


def test_small_calls_other_sum_schemes_and_dtypes_stay_on_the_general_purpose_kernel():
    rng = np.random.default_rng(4)
    x, y = rng.standard_normal((2000, 3)).astype(np.float32), rng.standard_normal((3000, 3)).astype(np.float32)
    b, g = rng.standard_normal((3000, 1)).astype(np.float32), np.array([1.0], np.float32)
    _genred(3, 1)(*to_dev(x, y, b, g))
    assert _last_meta("radial") is None                                   # 6e6 pairs: not worth the pre-pass
    big = [np.repeat(a, 12, 0) for a in (x, y, b)]
    _genred(3, 1, sum_scheme="kahan_scheme")(*to_dev(*big, g))
    assert _last_meta("radial") is None
    _genred(3, 1, use_fast_math=False)(*to_dev(*big, g))
    assert _last_meta("radial") is None
    _genred(3, 1)(*[t.double() for t in to_dev(*big, g)])
    assert _last_meta("radial") is None


def test_matrix_core_exponents_under_graph_capture():
    gen = torch.Generator(device="cuda").manual_seed(0)
    r = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    x, y, b, g = r(20000, 3), r(21000, 3), r(21000, 2), torch.tensor([0.5], device="cuda")
    conv = _genred(3, 2)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        conv(x, y, b, g)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = conv(x, y, b, g)
    for scale in (1.0, 0.5, 30.0):   # the last one flips the device-side decision inside the same graph
        x.copy_(r(20000, 3) * scale)
        y.copy_(r(21000, 3) * scale)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        assert torch.equal(got, conv(x, y, b, g))


@pytest.mark.parametrize("D", [3, 2, 7])
def test_gradients_wrt_points_and_weights_with_matrix_core_exponents(D):
    """Backward pass of the Gaussian kernel sum: the gradients with respect to x, y and b are again Gaussian sums
    (with a difference factor for the points) and take the same path; against the oracle's gradient body.  (D = 7:
    eight sums per row, which the variant with the weighted sum on the matrix cores accumulates.)"""
    from keops_amd import keops_io

    M, N = 24000, 26000
    rng = np.random.default_rng(50 + D)
    x = rng.standard_normal((M, D)).astype(np.float32)
    y = (rng.standard_normal((N, D)) - 0.2).astype(np.float32)
    b = rng.standard_normal((N, 1)).astype(np.float32)
    e = rng.standard_normal((M, 1)).astype(np.float32)     # incoming gradient
    g = np.array([0.6], np.float32)
    xd, yd, bd, gd = to_dev(x, y, b, g)
    xd.requires_grad_(True), yd.requires_grad_(True), bd.requires_grad_(True)
    out = _genred(D, 1)(xd, yd, bd, gd)
    gx, gy, gb = torch.autograd.grad(out, [xd, yd, bd], torch.from_numpy(e).cuda())
    # the two gradients with respect to the points accumulate D + 1 sums per row on the matrix-core path
    assert sum(m.meta("rad_dv") == str(D + 1) and m.meta("rad_d") == str(D) for m in keops_io._modules.values()) >= 2
    rows = np.sort(rng.choice(M, 1200, replace=False)).astype(np.int64)
    ref = cpu_reduc("gauss_gradx", [x, y, b, g, e], M, N, D, rows=rows)
    scale = cpu_reduc("gauss_gradx_abs", [x, y, b, g, e], M, N, D, rows=rows)
    assert_sum_parity(gx[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    # gradient with respect to y_j: the same body with the roles of the two clouds (and of b and e) exchanged
    cols = np.sort(rng.choice(N, 1200, replace=False)).astype(np.int64)
    refy = cpu_reduc("gauss_gradx", [y, x, e, g, b], N, M, D, rows=cols)
    scaley = cpu_reduc("gauss_gradx_abs", [y, x, e, g, b], N, M, D, rows=cols)
    assert_sum_parity(gy[torch.from_numpy(cols).cuda()].cpu().numpy(), refy, scaley)
    # gradient with respect to b_j: sum_i e_i K_ij
    refb = cpu_reduc("gauss", [y, x, e, g], N, M, 1, rows=cols)
    scaleb = cpu_reduc("gauss", [y, x, np.abs(e), g], N, M, 1, rows=cols)
    assert_sum_parity(gb[torch.from_numpy(cols).cuda()].cpu().numpy(), refb, scaleb)


@pytest.mark.parametrize("seed", [0, 7])
def test_random_clouds_and_kernel_widths_vs_oracle(seed):
    """Seeded sweep over dimensions, cloud shapes (anisotropic, two clumps, far from the origin), weight scales and
    kernel widths from 25 times narrower to 30 times wider than the cloud: the device-side check sends each case to
    the matrix-core exponents or to the exact differences, and every one meets the parity bar against the oracle
    (rows whose whole sum underflows in float32 are left out)."""
    rng = np.random.default_rng(seed)
    served = 0
    for case in range(20):
        D, Dv = int(rng.integers(2, 9)), int(rng.integers(1, 9))
        M = int(rng.integers(12000, 40000))
        N = max(1, (1 << 28) // M + int(rng.integers(1, 3000)))
        spread = float(10 ** rng.uniform(-2, 1.5))
        offset = float(rng.choice([0, 0, 1, 30, 1000])) * spread
        aniso = rng.uniform(0.05, 1, D) if rng.random() < 0.5 else np.ones(D)
        x = (rng.standard_normal((M, D)) * aniso * spread + offset).astype(np.float32)
        y = (rng.standard_normal((N, D)) * aniso * spread + offset * (1 + 0.01 * rng.random())).astype(np.float32)
        if rng.random() < 0.3:
            y[: N // 2] += 5 * spread
        b = rng.standard_normal((N, Dv)).astype(np.float32) * float(10 ** rng.uniform(-3, 3))
        if rng.random() < 0.3:
            b = np.abs(b)
        width = float(10 ** rng.uniform(-1.4, 1.5)) * spread   # from 25 times narrower than the cloud to 30 times wider
        g = np.array([1.0 / (2 * width * width)], np.float32)
        got = _genred(D, Dv)(*to_dev(x, y, b, g))
        served += _path_status() == 1
        rows = np.sort(rng.choice(M, 400, replace=False)).astype(np.int64)
        ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows)
        scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv, rows=rows)
        live = scale.max(axis=1) > 1e-30
        if not live.any():
            continue
        out = got[torch.from_numpy(rows).cuda()].cpu().numpy()
        try:
            assert_sum_parity(out[live], ref[live], np.maximum(scale[live], 1e-30))
        except AssertionError as e:
            raise AssertionError(f"case {case}: D={D} Dv={Dv} M={M} N={N} spread={spread:.3g} offset={offset:.3g} "
                                 f"width={width:.3g}: {e}") from None
    assert served >= 10


@pytest.mark.parametrize("D,Dw", [(3, 4), (3, 8), (2, 13)])
def test_scalar_product_of_a_row_and_a_column_vector_as_weight(D, Dw):
    """sum_j K_ij <u_i, v_j> (the kernel energy of shape models): one factor depends on both indices, but it is a
    scalar product, so the sums are accumulated per component of v_j and contracted with u_i once per row.  Reference:
    dense float64."""
    from keops_amd.torch import Genred

    M, N = 17000, 16500
    gen = torch.Generator(device="cuda").manual_seed(70 + Dw)
    x, y = torch.randn(M, D, device="cuda", generator=gen), torch.randn(N, D, device="cuda", generator=gen) + 0.2
    u, v = torch.randn(M, Dw, device="cuda", generator=gen), torch.randn(N, Dw, device="cuda", generator=gen)
    g = torch.tensor([0.6], device="cuda")
    f = Genred("Exp(-g*SqDist(x,y))*(u|v)", [f"x=Vi({D})", f"y=Vj({D})", f"u=Vi({Dw})", f"v=Vj({Dw})", "g=Pm(1)"],
               reduction_op="Sum", axis=1)
    got = f(x, y, u, v, g)
    assert got.shape == (M, 1)
    assert _last_meta("radial") == "1" and _last_meta("rad_mm") == ("1" if Dw >= 7 else "0")
    assert _path_status() == 1
    K = torch.exp(-0.6 * torch.cdist(x.double(), y.double()) ** 2)
    ref = ((K @ v.double()) * u.double()).sum(1, keepdim=True)
    scale = ((K @ v.double().abs()) * u.double().abs()).sum(1, keepdim=True)
    assert_sum_parity(got.cpu().numpy(), ref.cpu().numpy(), scale.cpu().numpy())
    plain = Genred("Exp(-g*SqDist(x,y))*(u|v)", [f"x=Vi({D})", f"y=Vj({D})", f"u=Vi({Dw})", f"v=Vj({Dw})", "g=Pm(1)"],
                   reduction_op="Sum", axis=1, enable_chunks=False)(x, y, u, v, g)
    assert _last_meta("radial") is None
    assert_sum_parity(plain.cpu().numpy(), ref.cpu().numpy(), scale.cpu().numpy())


def test_gradient_with_respect_to_the_points_with_vector_weights():
    """sum_j K_ij <e_i, b_j> (x_i - y_j) with two-component weights in the plane: 2 x 3 sums per pair, contracted with
    e_i at the end; with more components the sweep forms <e_i, b_j> per pair, as the general-purpose kernel does."""
    D, Dv, M, N = 2, 2, 17000, 16500
    gen = torch.Generator(device="cuda").manual_seed(81)
    x, y = torch.randn(M, D, device="cuda", generator=gen), torch.randn(N, D, device="cuda", generator=gen)
    b, e = torch.randn(N, Dv, device="cuda", generator=gen), torch.randn(M, Dv, device="cuda", generator=gen)
    g = torch.tensor([0.6], device="cuda")
    xr = x.clone().requires_grad_(True)
    (_genred(D, Dv)(xr, y, b, g) * e).sum().backward()
    assert _last_meta("radial") == "1" and _last_meta("rad_dv") == "3" and _path_status() == 1
    xd = x.double().requires_grad_(True)
    ((torch.exp(-0.6 * torch.cdist(xd, y.double()) ** 2) @ b.double()) * e.double()).sum().backward()
    assert float((xr.grad.double() - xd.grad).norm() / xd.grad.norm()) <= 1e-5
    assert _last_meta("rad_bil") == "1"   # <e_i, b_j> out of the matrix cores, next to the exponent
    # the same with the expanded sums (2 x 3 per pair, contracted with e_i at the end)
    import keops_amd.config as cfg
    cfg.radial_bilinear = False
    try:
        xe = x.clone().requires_grad_(True)
        (_genred(D, Dv, sum_scheme="direct_sum")(xe, y, b, g) * e).sum().backward()   # (another module: the option is part of its key)
        assert _last_meta("radial") == "1" and _last_meta("rad_bil") == "0" and _last_meta("rad_dv") == "6" and _path_status() == 1
        assert float((xe.grad.double() - xd.grad).norm() / xd.grad.norm()) <= 1e-5
    finally:
        cfg.radial_bilinear = True
    # three components in space: 4 sums per pair either way; in six dimensions the slot vectors have no room for the
    # second product and the sweep forms <e_i, b_j> per pair on the vector ALU
    for D3, mode in ((3, "bil"), (6, "upair")):
        x3, y3 = torch.randn(M, D3, device="cuda", generator=gen), torch.randn(N, D3, device="cuda", generator=gen)
        b3, e3 = torch.randn(N, 3, device="cuda", generator=gen), torch.randn(M, 3, device="cuda", generator=gen)
        xr3 = x3.clone().requires_grad_(True)
        (_genred(D3, 3)(xr3, y3, b3, g) * e3).sum().backward()
        assert _last_meta("radial") == "1" and _last_meta("rad_dv") == str(D3 + 1) and _path_status() == 1
        assert _last_meta("rad_bil") == ("1" if mode == "bil" else "0")
        xd3 = x3.double().requires_grad_(True)
        ((torch.exp(-0.6 * torch.cdist(xd3, y3.double()) ** 2) @ b3.double()) * e3.double()).sum().backward()
        assert float((xr3.grad.double() - xd3.grad).norm() / xd3.grad.norm()) <= 1e-5
    x3, y3 = torch.randn(M, 3, device="cuda", generator=gen), torch.randn(N, 3, device="cuda", generator=gen)
    # eight components: three more k blocks, five in all; twelve: the general-purpose kernel
    for Dv8, radial in ((8, "1"), (12, None)):
        b8, e8 = torch.randn(N, Dv8, device="cuda", generator=gen), torch.randn(M, Dv8, device="cuda", generator=gen)
        xr8 = x3.clone().requires_grad_(True)
        (_genred(3, Dv8)(xr8, y3, b8, g) * e8).sum().backward()
        assert _last_meta("radial") == radial
        xd8 = x3.double().requires_grad_(True)
        ((torch.exp(-0.6 * torch.cdist(xd8, y3.double()) ** 2) @ b8.double()) * e8.double()).sum().backward()
        assert float((xr8.grad.double() - xd8.grad).norm() / xd8.grad.norm()) <= 1e-5
