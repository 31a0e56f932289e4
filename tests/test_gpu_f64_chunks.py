"""Double-precision contractions on the float64 matrix instruction (kernels/keops_chunk_f64.h): Sum and log-sum-exp
reductions whose formula holds one SqDist(x_i, y_j) or <x_i, y_j> of 32..256 components, with enough output rows to
fill the chip.  References: dense float64 torch evaluations (the accuracy bar of float64 in this suite: 1e-12)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _last_module():
    from keops_amd import keops_io

    return keops_io.last_loader.module


def _rel(got, ref):
    return float((got - ref).abs().max() / ref.abs().max())


def _sqdist(x, y):
    """Squared distances from the differences (torch.cdist goes through a matrix product for large inputs and loses
    the digits this test is about when the clouds are far from the origin)."""
    out = torch.empty(x.shape[0], y.shape[0], device=x.device, dtype=torch.float64)
    step = max(1, (1 << 25) // (y.shape[0] * x.shape[1]))
    for i0 in range(0, x.shape[0], step):
        out[i0:i0 + step] = (x[i0:i0 + step, None, :] - y[None, :, :]).pow(2).sum(-1)
    return out


@pytest.mark.parametrize("D,M,N", [(64, 5000, 6001), (256, 4100, 3000), (37, 4500, 2000), (129, 4096, 777)])
def test_float64_gaussian_sum_on_the_matrix_cores(D, M, N):
    from keops_amd.torch import Genred

    gen = torch.Generator(device="cuda").manual_seed(D)
    x = torch.randn(M, D, device="cuda", dtype=torch.float64, generator=gen) / D ** 0.5 + 3.0   # far from the origin
    y = torch.randn(N, D, device="cuda", dtype=torch.float64, generator=gen) / D ** 0.5 + 3.0
    b = torch.randn(N, 3, device="cuda", dtype=torch.float64, generator=gen)
    g = torch.tensor([0.7], device="cuda", dtype=torch.float64)
    conv = Genred("Exp(-g*SqDist(x,y))*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vj(3)", "g=Pm(1)"], reduction_op="Sum", axis=1)
    got = conv(x, y, b, g)
    assert _last_module().meta("scheme") == "chunk64"
    ref = torch.exp(-0.7 * _sqdist(x, y)) @ b
    assert _rel(got, ref) < 1e-12
    assert torch.equal(conv(x, y, b, g), got)                       # deterministic
    # few output rows: the vector-ALU chunked kernel, which cuts the reduced axis in slabs
    small = conv(x[:300].contiguous(), y, b, g)
    assert _last_module().meta("scheme") != "chunk64"
    assert _rel(small, ref[:300]) < 1e-12


def test_float64_laplace_lse_scalar_products_and_self_interaction():
    from keops_amd.torch import Genred

    gen = torch.Generator(device="cuda").manual_seed(1)
    r = lambda *s: torch.randn(*s, device="cuda", dtype=torch.float64, generator=gen)
    D = 96
    x = r(4200, D) / D ** 0.5
    # x against itself (zero distances on the diagonal) through a square root, and tight clusters: the pairs whose
    # expansion has lost its digits are recomputed from the differences
    x[1000:2000] = x[0] + 1e-6 * r(1000, D)
    b = r(4200, 2)
    lap = Genred("Exp(-Norm2(x-y))*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vj(2)"], reduction_op="Sum", axis=1)
    got = lap(x, x, b)
    assert _last_module().meta("scheme") == "chunk64"
    # (torch.cdist loses the same digits: plain differences as the reference value)
    dist = _sqdist(x, x).sqrt()
    ref = torch.exp(-dist) @ b
    assert _rel(got, ref) < 1e-12
    lse = Genred("-Norm2(x-y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="LogSumExp", axis=0)
    got = lse(x, x)
    assert _last_module().meta("scheme") == "chunk64"
    assert _rel(got[:, 0], torch.logsumexp(-dist, dim=0)) < 1e-12
    lin = Genred("(x|y)*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vi(2)"], reduction_op="Sum", axis=0)
    y = r(5000, D)
    got = lin(x, y, b)
    assert _last_module().meta("scheme") == "chunk64"
    assert _rel(got, (x @ y.T).T @ b) < 1e-12


def test_float64_matrix_core_scheme_with_ranges_and_batches():
    from keops_amd.torch import Genred, LazyTensor

    gen = torch.Generator(device="cuda").manual_seed(2)
    r = lambda *s: torch.randn(*s, device="cuda", dtype=torch.float64, generator=gen)
    D, M, N = 48, 6000, 5000
    x, y, b = r(M, D) / D ** 0.5, r(N, D) / D ** 0.5, r(N, 1)
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    # three row ranges (rows 4000..4499 are covered by none), block-sparse columns
    ranges = (i64([[0, 2500], [2500, 4000], [4500, 6000]]), i64([2, 3, 4]), i64([[0, 1000], [3000, 5000], [1000, 3000], [0, 5000]]),
              i64([[0, 1000], [1000, 3000], [3000, 5000]]), i64([2, 4, 5]),
              i64([[0, 2500], [4500, 6000], [2500, 4000], [4500, 6000], [0, 2500], [4500, 6000]]))
    conv = Genred("Exp(-SqDist(x,y))*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vj(1)"], reduction_op="Sum", axis=1)
    got = conv(x, y, b, ranges=ranges)
    assert _last_module().meta("scheme") == "chunk64" and _last_module().meta("ranges") == "1"
    K = torch.exp(-_sqdist(x, y))
    mask = torch.zeros(M, N, device="cuda", dtype=torch.float64)
    mask[0:2500, 0:1000] = 1
    mask[0:2500, 3000:5000] = 1
    mask[2500:4000, 1000:3000] = 1
    mask[4500:6000, :] = 1
    ref = (K * mask) @ b
    assert float((got - ref).abs().max()) < 1e-12 * float(ref.abs().max())
    assert float(got[4000:4500].abs().max()) == 0.0
    # batch dimensions, one of them broadcast
    xb, yb, bb = r(3, 4200, D) / D ** 0.5, r(1, 900, D) / D ** 0.5, r(3, 900, 2)
    d2 = ((LazyTensor(xb[:, :, None, :]) - LazyTensor(yb[:, None, :, :])) ** 2).sum(-1)
    out = ((-d2).exp() * LazyTensor(bb[:, None, :, :])).sum(2)
    assert _last_module().meta("scheme") == "chunk64"
    refb = torch.stack([torch.exp(-_sqdist(xb[k], yb[0])) @ bb[k] for k in range(3)])
    assert _rel(out, refb) < 1e-12
