"""Seeded random shapes across the schemes (general-purpose, chunked matrix-core, chunked vector-ALU, nearest
neighbours with exact re-rank): ragged sizes, dimensions around every threshold of the engine, vectors whose length
is not a multiple of the load width.  References: the CPU oracle (float32 sums in the reference's order) for the
kernel sums and the indices, dense float64 torch formulas for the others."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity
from keops_amd.torch import Genred
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu

DIMS = [24, 25, 31, 32, 33, 47, 64, 100, 101, 129, 200, 257, 300, 511, 784, 1025, 1100]


def _case(seed):
    rng = np.random.default_rng(seed)
    M, N = int(rng.integers(1, 1500)), int(rng.integers(1, 1500))
    D = int(rng.choice(DIMS))
    kind = ["sum_sq", "sum_l1", "lse_sq", "knn_sq", "knn_l1", "sum_dot64"][seed % 6]
    x = torch.from_numpy(rng.standard_normal((M, D))).float() / D ** 0.5
    y = torch.from_numpy(rng.standard_normal((N, D))).float() / D ** 0.5
    b = torch.from_numpy(rng.standard_normal((N, 2))).float()
    return kind, M, N, D, x, y, b, rng


@pytest.mark.parametrize("seed", range(48))
def test_random_shape(seed):
    kind, M, N, D, x, y, b, rng = _case(seed)
    xd, yd, bd = x.cuda(), y.cuda(), b.cuda()
    x64, y64, b64 = x.double(), y.double(), b.double()
    var = [f"x=Vi({D})", f"y=Vj({D})"]
    if kind in ("sum_sq", "sum_l1"):
        f = "Exp(-SqDist(x,y))*b" if kind == "sum_sq" else "Exp(-Sum(Abs(x-y)))*b"
        out = Genred(f, var + ["b=Vj(2)"], reduction_op="Sum", axis=1)(xd, yd, bd).cpu().double()
        # the oracle sums the D terms of the exponent in float32, in the reference's order: 1e-5 against that
        body, args = ("gauss", [x.numpy(), y.numpy(), b.numpy(), np.ones(1, np.float32)]) if kind == "sum_sq" else ("exp_l1", [x.numpy(), y.numpy(), b.numpy()])
        ref = cpu_reduc(body, args, M, N, 2)
        args[2] = np.abs(b.numpy())
        scale = cpu_reduc(body, args, M, N, 2)
        assert_sum_parity(out.numpy(), ref, scale)
    elif kind == "lse_sq":
        out = Genred("-SqDist(x,y)", var, reduction_op="LogSumExp", axis=1)(xd, yd).cpu().double()[:, 0]
        ref = torch.logsumexp(-torch.cdist(x64, y64) ** 2, 1)
        assert float((out - ref).abs().max()) < 2e-5 * max(1.0, float(ref.abs().max()))
    elif kind in ("knn_sq", "knn_l1"):
        K = int(rng.integers(1, 12))
        f = "SqDist(x,y)" if kind == "knn_sq" else "Sum(Abs(x-y))"
        idx = Genred(f, var, reduction_op="ArgKMin", axis=1, opt_arg=K)(xd, yd).cpu().numpy()
        d = np.zeros((M, N), np.float32)
        xn, yn = x.numpy(), y.numpy()
        for k in range(D):
            t = xn[:, None, k] - yn[None, :, k]
            d += t * t if kind == "knn_sq" else np.abs(t)
        # with fewer than K reduced rows the unused slots keep their initial index 0 (KMin_ArgKMin_Reduction.py:34-45)
        want = np.zeros((M, K), np.int64)
        want[:, :min(K, N)] = np.argsort(d, axis=1, kind="stable")[:, :K]
        assert np.array_equal(idx.astype(np.int64), want)
    else:
        out = Genred("(x|y)*b", var + ["b=Vj(2)"], reduction_op="Sum", axis=1)(xd.double(), yd.double(), bd.double()).cpu()
        ref = (x64 @ y64.T) @ b64
        assert float((out - ref).abs().max()) < 1e-11 * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("M,N", [(0, 5), (5, 0), (0, 0)])
def test_no_rows_or_nothing_to_reduce_over(M, N):
    """An empty output gives an empty result; an empty reduced axis gives every row the reduction's neutral element, as
    the reference's loops leave it (CpuReduc.py:43-64: Initialize, no pair, Finalize): 0 for a sum, -inf for a
    log-sum-exp, (+inf, 0) for a minimum with its index, index 0 for the K nearest neighbours.  (The library used to
    divide by the number of column tiles.)"""
    import torch

    from keops_amd.torch import Genred

    x, y = torch.randn(M, 3, device="cuda"), torch.randn(N, 3, device="cuda")
    b, g = torch.randn(N, 2, device="cuda"), torch.tensor([0.5], device="cuda")
    s = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)", "g=Pm(1)"], reduction_op="Sum", axis=1)(x, y, b, g)
    lse = Genred("-g*SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)", "g=Pm(1)"], reduction_op="LogSumExp", axis=1)(x, y, g)
    idx = Genred("SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], reduction_op="ArgKMin", axis=1, opt_arg=3)(x, y)
    vmin, imin = Genred("SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], reduction_op="Min_ArgMin", axis=1)(x, y)
    xh, yh = torch.randn(M, 64, device="cuda"), torch.randn(N, 64, device="cuda")
    hd = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(64)", "y=Vj(64)", "b=Vj(2)"], reduction_op="Sum", axis=1)(xh, yh, b)
    kd = Genred("SqDist(x,y)", ["x=Vi(64)", "y=Vj(64)"], reduction_op="KMin_ArgKMin", axis=1, opt_arg=2)(xh, yh)
    assert tuple(s.shape) == (M, 2) and tuple(lse.shape) == (M, 1) and tuple(idx.shape) == (M, 3)
    assert tuple(vmin.shape) == (M, 1) and tuple(imin.shape) == (M, 1) and tuple(hd.shape) == (M, 2)
    assert tuple(kd[0].shape) == (M, 2) and tuple(kd[1].shape) == (M, 2)
    if M > 0:       # N = 0
        assert bool((s == 0).all()) and bool((hd == 0).all()) and bool(torch.isneginf(lse).all())
        assert bool((idx == 0).all()) and bool(torch.isposinf(vmin).all()) and bool((imin == 0).all())
        assert bool(torch.isposinf(kd[0]).all()) and bool((kd[1] == 0).all())

