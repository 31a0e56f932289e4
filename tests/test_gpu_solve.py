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


def test_numpy_front_end():
    import numpy as np

    from keops_amd.numpy import Genred, KernelSolve, generic_argkmin

    rng = np.random.default_rng(0)
    x, y, b = rng.standard_normal((300, 3)), rng.standard_normal((500, 3)), rng.standard_normal((500, 2))
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)"], reduction_op="Sum", axis=1)
    got = conv(x, y, b)
    assert isinstance(got, np.ndarray) and got.dtype == np.float64
    ref = np.exp(-((x[:, None, :] - y[None, :, :]) ** 2).sum(-1)) @ b
    assert np.max(np.abs(got - ref)) < 1e-12
    knn = generic_argkmin("SqDist(x,y)", "a = Vi(4)", "x = Vi(3)", "y = Vj(3)")
    idx = knn(x.astype(np.float32), y.astype(np.float32))
    d2 = ((x.astype(np.float32)[:, None, :] - y.astype(np.float32)[None, :, :]) ** 2).sum(-1)
    assert np.array_equal(np.sort(idx, 1), np.sort(np.argsort(d2, 1, kind="stable")[:, :4], 1))
    a = KernelSolve("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)"], "b", axis=1)(x, x, b[:300], alpha=0.3, eps=1e-12)
    K = np.exp(-((x[:, None, :] - x[None, :, :]) ** 2).sum(-1))
    assert np.max(np.abs(a - np.linalg.solve(0.3 * np.eye(300) + K, b[:300]))) < 1e-8
