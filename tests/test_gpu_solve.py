"""KernelSolve / LazyTensor.solve on the GPU against dense linear algebra (the reference's
pykeops/test style: torch.linalg.solve on the explicit kernel matrix, autograd on the dense formula)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dense_kernel(x, y):
    return torch.exp(-((x[:, None, :] - y[None, :, :]) ** 2).sum(-1))


def test_kernelsolve_matches_dense_solve_and_gradients():
    from keops_amd.torch import Genred, KernelSolve

    torch.manual_seed(0)
    N, D, Dv, alpha = 400, 3, 2, 0.5
    x = torch.randn(N, D, dtype=torch.float64, device="cuda", requires_grad=True)
    b = torch.randn(N, Dv, dtype=torch.float64, device="cuda", requires_grad=True)
    formula, aliases = "Exp(-SqDist(x, y)) * a", [f"x = Vi({D})", f"y = Vj({D})", f"a = Vj({Dv})"]
    K_inv = KernelSolve(formula, aliases, "a", axis=1)
    a = K_inv(x, x, b, alpha=alpha, eps=1e-12)
    assert a.shape == (N, Dv)
    # residual of the linear system, evaluated with the map-reduce product
    K = Genred(formula, aliases, axis=1)
    assert torch.linalg.norm(alpha * a + K(x, x, a) - b) <= 1e-9 * torch.linalg.norm(b)
    # dense reference
    xd, bd = x.detach().clone().requires_grad_(True), b.detach().clone().requires_grad_(True)
    ad = torch.linalg.solve(alpha * torch.eye(N, dtype=torch.float64, device="cuda") + _dense_kernel(xd, xd), bd)
    assert torch.allclose(a, ad, rtol=1e-8, atol=1e-10)
    # gradients of a scalar loss with respect to the right-hand side and to the points
    w = torch.randn(N, Dv, dtype=torch.float64, device="cuda")
    gx, gb = torch.autograd.grad((a * w).sum(), [x, b])
    gxd, gbd = torch.autograd.grad((ad * w).sum(), [xd, bd])
    assert torch.allclose(gb, gbd, rtol=1e-7, atol=1e-9)
    # x enters both as the i- and the j-variable: KernelSolve was given x twice, autograd adds both parts
    assert torch.allclose(gx, gxd, rtol=1e-6, atol=1e-8)


def test_lazytensor_solve_float32():
    from keops_amd.torch import LazyTensor

    torch.manual_seed(1)
    N = 1500
    x = torch.rand(N, 2, device="cuda")
    b = torch.randn(N, 1, device="cuda")
    x_i, x_j = LazyTensor(x[:, None, :]), LazyTensor(x[None, :, :])
    K = (-((x_i - x_j) ** 2).sum(-1) / (2 * 0.1 ** 2)).exp()
    a = K.solve(b, alpha=0.1, eps=1e-6)
    dense = torch.exp(-torch.cdist(x.double(), x.double()) ** 2 / (2 * 0.1 ** 2))
    ref = torch.linalg.solve(0.1 * torch.eye(N, dtype=torch.float64, device="cuda") + dense, b.double())
    assert torch.linalg.norm(a.double() - ref) <= 1e-4 * torch.linalg.norm(ref)
    # the aliases of the reductions are the same functions
    d = ((x_i - x_j) ** 2).sum(-1)
    assert torch.equal(d.argKmin_reduction(3, dim=1), d.argKmin(3, dim=1))
    assert torch.equal(d.min_reduction(dim=1), d.min(dim=1))
