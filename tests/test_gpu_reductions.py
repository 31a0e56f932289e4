"""GPU parity of every reduction policy against the CPU oracle: log-sum-exp family, Min/Max/Arg*,
KMin/ArgKMin/KMin_ArgKMin (bit-exact indices and values, ties keep the lower index)."""
import numpy as np
import pytest
import torch

from common import rel_l2, to_dev
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu


def _xy(M, N, D, seed, uniform=False):
    rng = np.random.default_rng(seed)
    draw = (lambda s: rng.random(s)) if uniform else (lambda s: rng.standard_normal(s))
    return draw((M, D)).astype(np.float32), draw((N, D)).astype(np.float32), rng


@pytest.mark.parametrize("M,N", [(1000, 3000), (50, 20011)])
@pytest.mark.parametrize("scheme", ["block_sum", "direct_sum", "kahan_scheme"])
def test_logsumexp_sinkhorn_style(M, N, scheme):
    from keops_amd.torch import Genred

    x, y, rng = _xy(M, N, 3, 4)
    l = rng.standard_normal((N, 1)).astype(np.float32)
    e = np.array([1 / 0.05], np.float32)
    lse = Genred("l-SqDist(x,y)*e", ["x=Vi(3)", "y=Vj(3)", "l=Vj(1)", "e=Pm(1)"], reduction_op="LogSumExp", axis=1,
                 sum_scheme=scheme)
    got = lse(*to_dev(x, y, l, e)).cpu().numpy()
    ms = cpu_reduc("lse_gauss", [x, y, l, e], M, N, 2, reduction="Max_SumShiftExp", scheme=scheme)
    ref = (ms[:, 0].astype(np.float64) + np.log(ms[:, 1].astype(np.float64)))[:, None]
    assert got.shape == (M, 1)
    # values are O(1)..O(100): absolute error of the log-sum-exp below 1e-5 * max(1, |ref|)
    assert np.max(np.abs(got - ref) / np.maximum(1.0, np.abs(ref))) <= 1e-5


@pytest.mark.parametrize("D", [3, 64])
@pytest.mark.parametrize("scheme", ["block_sum", "kahan_scheme"])
@pytest.mark.parametrize("where", [0, 5, 1000, 1019, 1022])
def test_logsumexp_of_a_value_that_is_not_a_number_is_not_a_number(where, scheme, D):
    """The reference's update (Max_SumShiftExpWeight_Reduction.py:35-61) turns the running sum into NaN for good when a
    pair value is NaN, wherever the column sits: in a group of eight, among the last columns of a tile that are folded
    one by one, first or last (the per-pair update used to drop such a value, and the sum so far with it)."""
    from keops_amd.torch import Genred

    M, N = 300, 1023
    x, y, rng = _xy(M, N, D, 6)
    x, y = x / np.sqrt(D), y / np.sqrt(D)
    y[where, 1] = np.nan
    lse = Genred("-SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="LogSumExp", axis=1, sum_scheme=scheme)
    got = lse(*to_dev(x, y))
    assert bool(torch.isnan(got).all())


def test_logsumexp_weighted_and_softmax():
    from keops_amd.torch import Genred

    M, N = 700, 900
    x, y, rng = _xy(M, N, 3, 5)
    w = rng.random((N, 2)).astype(np.float32) + 0.5
    xd, yd, wd = to_dev(x, y, w)
    f = -((torch.from_numpy(x)[:, None] - torch.from_numpy(y)[None]) ** 2).sum(-1).double()  # (M,N)
    lsew = Genred("-SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)", "w=Vj(2)"], reduction_op="LogSumExp", axis=1, formula2="w")
    got = lsew(xd, yd, wd).cpu().double()
    ref = torch.logsumexp(f[:, :, None] + torch.log(torch.from_numpy(w).double())[None], dim=1)
    assert torch.allclose(got, ref, rtol=1e-5, atol=1e-5)
    sm = Genred("-SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)", "w=Vj(2)"], reduction_op="SumSoftMaxWeight", axis=1, formula2="w")
    got = sm(xd, yd, wd).cpu().double()
    ref = torch.softmax(f, dim=1) @ torch.from_numpy(w).double()
    assert torch.allclose(got, ref, rtol=1e-5, atol=1e-6)


def test_logsumexp_gradient():
    from keops_amd.torch import Genred

    M, N = 300, 400
    x, y, rng = _xy(M, N, 3, 6)
    xd, yd = to_dev(x.astype(np.float64), y.astype(np.float64))
    xd.requires_grad_(True)
    yd.requires_grad_(True)
    lse = Genred("-SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], reduction_op="LogSumExp", axis=1)
    out = lse(xd, yd)
    E = torch.from_numpy(rng.standard_normal((M, 1))).cuda()
    gx, gy = torch.autograd.grad((out * E).sum(), [xd, yd])
    xt, yt = xd.detach().clone().requires_grad_(True), yd.detach().clone().requires_grad_(True)
    ref = torch.logsumexp(-((xt[:, None] - yt[None]) ** 2).sum(-1), dim=1, keepdim=True)
    rx, ry = torch.autograd.grad((ref * E).sum(), [xt, yt])
    assert rel_l2(gx.cpu().numpy(), rx.cpu().numpy()) < 1e-10
    assert rel_l2(gy.cpu().numpy(), ry.cpu().numpy()) < 1e-10


@pytest.mark.parametrize("op", ["Min", "ArgMin", "Min_ArgMin", "Max", "ArgMax", "Max_ArgMax"])
def test_min_max_family_bit_exact(op):
    from keops_amd.torch import Genred

    M, N, D = 900, 5000, 5
    x, y, rng = _xy(M, N, D, 7, uniform=True)
    y[100] = y[7]
    y[4000] = y[7]  # exact ties
    x[3] = y[7]
    red = Genred("SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op=op, axis=1)
    got = red(*to_dev(x, y))
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction=op, scheme="direct_sum")
    if op in ("Min", "Max"):
        assert np.array_equal(got.cpu().numpy(), ref)
    elif op in ("ArgMin", "ArgMax"):
        assert got.dtype == torch.int64 and np.array_equal(got.cpu().numpy(), ref.astype(np.int64))
    else:
        vals, idx = got
        assert np.array_equal(vals.cpu().numpy(), ref[:, :1]) and np.array_equal(idx.cpu().numpy(), ref[:, 1:].astype(np.int64))
    if op == "ArgMin":
        assert got[3, 0].item() == 7


@pytest.mark.parametrize("M,N,D,K", [(500, 4000, 8, 5), (300, 70000, 3, 10), (64, 1500, 20, 1), (100, 7, 4, 10)])
def test_kmin_argkmin_bit_exact(M, N, D, K):
    from keops_amd.torch import Genred

    x, y, rng = _xy(M, N, D, 8, uniform=True)
    if N > 50:
        y[17] = y[3]
        y[50] = y[3]
        x[0] = y[3]
    al = [f"x=Vi({D})", f"y=Vj({D})"]
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    rv, ri = ref[:, 0::2], ref[:, 1::2].astype(np.int64)
    vals, idx = Genred("SqDist(x,y)", al, reduction_op="KMin_ArgKMin", axis=1, opt_arg=K)(*to_dev(x, y))
    assert idx.dtype == torch.int64 and tuple(idx.shape) == (M, K)
    assert np.array_equal(idx.cpu().numpy(), ri)
    assert np.array_equal(vals.cpu().numpy(), rv)
    only_idx = Genred("SqDist(x,y)", al, reduction_op="ArgKMin", axis=1, opt_arg=K)(*to_dev(x, y))
    only_val = Genred("SqDist(x,y)", al, reduction_op="KMin", axis=1, opt_arg=K)(*to_dev(x, y))
    assert np.array_equal(only_idx.cpu().numpy(), ri) and np.array_equal(only_val.cpu().numpy(), rv)
    if N > 50 and K >= 3:
        assert idx[0, :3].tolist() == [3, 17, 50]


def test_kmin_column_slabs_and_axis0():
    """Few rows, many columns: the slab scheme merges sorted K-lists in slab order (ties included)."""
    from keops_amd.torch import Genred

    M, N, D, K = 40, 300000, 4, 6
    x, y, rng = _xy(M, N, D, 9, uniform=True)
    y[250000] = y[11]
    x[5] = y[11]
    ref = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="KMin_ArgKMin", K=K, scheme="direct_sum")
    for backend in ("GPU_1D", "GPU_2D"):
        vals, idx = Genred("SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="KMin_ArgKMin", axis=1, opt_arg=K)(
            *to_dev(x, y), backend=backend)
        assert np.array_equal(idx.cpu().numpy(), ref[:, 1::2].astype(np.int64)), backend
        assert np.array_equal(vals.cpu().numpy(), ref[:, 0::2]), backend
    assert idx[5, :2].tolist() == [11, 250000]
    # reduction over i (axis=0): nearest x for every y
    idx0 = Genred("SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="ArgKMin", axis=0, opt_arg=3)(*to_dev(x, y[:5000]))
    ref0 = cpu_reduc("sqdist", [y[:5000], x], 5000, M, 1, reduction="ArgKMin", K=3, scheme="direct_sum")
    assert np.array_equal(idx0.cpu().numpy(), ref0.astype(np.int64))


def test_vector_valued_min_and_kmin():
    from keops_amd.torch import Genred

    M, N = 200, 1000
    x, y, rng = _xy(M, N, 3, 10)
    F = (x[:, None, :] - y[None, :, :]).astype(np.float32)  # formula x - y, dim 3
    al = ["x=Vi(3)", "y=Vj(3)"]
    vals, idx = Genred("x-y", al, reduction_op="Min_ArgMin", axis=1)(*to_dev(x, y))
    ref = cpu_reduc("dense", [F], M, N, 3, reduction="Min_ArgMin", scheme="direct_sum")
    assert np.array_equal(vals.cpu().numpy(), ref[:, :3]) and np.array_equal(idx.cpu().numpy(), ref[:, 3:].astype(np.int64))
    vals, idx = Genred("x-y", al, reduction_op="KMin_ArgKMin", axis=1, opt_arg=4)(*to_dev(x, y))
    ref = cpu_reduc("dense", [F], M, N, 3, reduction="KMin_ArgKMin", K=4, scheme="direct_sum").reshape(M, 4, 2, 3)
    assert tuple(vals.shape) == (M, 4, 3)
    assert np.array_equal(vals.cpu().numpy(), ref[:, :, 0, :]) and np.array_equal(idx.cpu().numpy(), ref[:, :, 1, :].astype(np.int64))


def test_arg_reduction_size_guard_and_autodiff_error():
    from keops_amd.torch import Genred

    x, y, _ = _xy(10, 10, 3, 0)
    xd, yd = to_dev(x, y)
    xd.requires_grad_(True)
    out = Genred("SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], reduction_op="Min", axis=1)(xd, yd)
    with pytest.raises(NotImplementedError):
        out.sum().backward()
