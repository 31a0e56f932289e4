"""Seeded sweep over shapes, reductions, axes and schemes against dense float64 torch evaluations:
exercises the launch heuristics (column slabs, rows per lane, matrix-core scheme selection) at
awkward sizes (1, primes, just above / below tile and slab boundaries)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 7, 63, 64, 65, 255, 257, 1000, 1025, 4099, 20011]


def _dense(x, y, b, g):
    K = torch.exp(-g * ((x[:, None, :] - y[None, :, :]) ** 2).sum(-1))
    return K, K @ b


@pytest.mark.parametrize("seed", range(12))
def test_sum_and_lse_shapes(seed):
    from keops_amd.torch import Genred

    rng = np.random.default_rng(100 + seed)
    M, N = (int(v) for v in rng.choice(SIZES, 2))
    D, Dv = int(rng.choice([1, 3, 5])), int(rng.choice([1, 2, 7, 33]))
    axis = int(rng.integers(0, 2))
    backend = str(rng.choice(["GPU_1D", "GPU_2D", "auto"]))
    scheme = str(rng.choice(["auto", "direct_sum", "kahan_scheme"]))
    x = torch.from_numpy(rng.standard_normal((M, D))).float().cuda()
    y = torch.from_numpy(rng.standard_normal((N, D))).float().cuda()
    nb = N if axis == 1 else M
    b = torch.from_numpy(rng.standard_normal((nb, Dv))).float().cuda()
    g = torch.tensor([0.5], device="cuda")
    bcat = "Vj" if axis == 1 else "Vi"
    conv = Genred("Exp(-g*SqDist(x,y))*b", [f"x=Vi({D})", f"y=Vj({D})", f"b={bcat}({Dv})", "g=Pm(1)"], reduction_op="Sum",
                  axis=axis, sum_scheme=scheme)
    got = conv(x, y, b, g, backend=backend).double()
    K = torch.exp(-0.5 * ((x.double()[:, None, :] - y.double()[None, :, :]) ** 2).sum(-1))
    ref = K @ b.double() if axis == 1 else K.T @ b.double()
    scale = (K @ b.double().abs() if axis == 1 else K.T @ b.double().abs()) + 1e-30
    assert got.shape == ref.shape
    assert float(((got - ref).abs() / scale).max()) <= 1e-5, (M, N, D, Dv, axis, backend, scheme)
    # log-sum-exp of -g|x-y|^2 + first column of b
    lse = Genred("w-g*SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})", f"w={bcat}(1)", "g=Pm(1)"], reduction_op="LogSumExp",
                 axis=axis, sum_scheme="auto" if scheme == "kahan_scheme" else scheme)
    w = b[:, :1].contiguous()
    gl = lse(x, y, w, g, backend=backend).double()
    d2 = ((x.double()[:, None, :] - y.double()[None, :, :]) ** 2).sum(-1)
    ref_l = torch.logsumexp(w.double().T - 0.5 * d2, dim=1) if axis == 1 else torch.logsumexp(w.double() - 0.5 * d2, dim=0)
    assert float((gl[:, 0] - ref_l).abs().max()) <= 1e-5 * max(1.0, float(ref_l.abs().max())), (M, N, D, axis, backend)


@pytest.mark.parametrize("seed", range(10))
def test_index_reductions_shapes(seed):
    from keops_amd.torch import Genred

    rng = np.random.default_rng(200 + seed)
    M, N = (int(v) for v in rng.choice(SIZES, 2))
    D = int(rng.choice([1, 2, 3, 17, 40, 64]))
    K = int(rng.choice([1, 3, 10]))
    x = torch.from_numpy(rng.random((M, D))).float().cuda()
    y = torch.from_numpy(rng.random((N, D))).float().cuda()
    if N > 3:
        y[N - 1] = y[0]  # an exact tie: the lower index must come first
    # exact float32 distances in the reference's operation order (sequential sum of squared differences)
    d2 = torch.zeros(M, N, device="cuda")
    for k in range(D):
        diff = x[:, k:k + 1] - y[None, :, k]
        d2 = d2 + diff * diff
    order = torch.sort(d2, dim=1, stable=True)
    Ke = min(K, N)
    knn = Genred("SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="KMin_ArgKMin", axis=1, opt_arg=K)
    vals, idx = knn(x, y)
    assert torch.equal(idx[:, :Ke], order.indices[:, :Ke]), (M, N, D, K)
    assert torch.equal(vals[:, :Ke], order.values[:, :Ke]), (M, N, D, K)
    am = Genred("SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="ArgMin", axis=1)(x, y)
    assert torch.equal(am[:, 0], order.indices[:, 0])
    mx, amx = Genred("SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="Max_ArgMax", axis=0)(x, y)
    ref0 = torch.sort(d2, dim=0, descending=True, stable=True)
    assert torch.equal(mx[:, 0], ref0.values[0])
    # ties for the maximum resolve to the lower index as well
    first_max = (d2 == ref0.values[0][None, :]).float().argmax(dim=0)
    assert torch.equal(amx[:, 0], first_max)
