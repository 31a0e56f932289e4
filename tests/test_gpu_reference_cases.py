"""Cases of the reference's own LazyTensor test files, run on the HIP backend with device tensors and compared
with dense torch: pykeops/test/test_transpose.py, conv2d.py, test_lazytensor_clamp.py, test_sinc.py,
test_contiguous_torch.py, test_lazytensor_gaussian_inplace.py, test_lazytensor_grad.py (same shapes, seeds and
tolerances)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_transpose():
    from keops_amd.torch import LazyTensor

    torch.manual_seed(0)
    x, y = torch.randn(1000, 3, device="cuda"), torch.randn(2000, 3, device="cuda")
    K_keops = (-((LazyTensor(x[:, None, :]) - LazyTensor(y[None, :, :])) ** 2).sum(2)).exp()
    K_torch = (-((x[:, None, :] - y[None, :, :]) ** 2).sum(2)).exp()
    w = torch.rand(1000, 2, device="cuda")
    assert torch.allclose(K_keops.t() @ w, K_torch.t() @ w, rtol=1e-5, atol=1e-4)


def test_clamp_forward_and_backward():
    from keops_amd.torch import LazyTensor

    torch.manual_seed(0)
    M, N, D = 1000, 1000, 3
    x = torch.randn(M, 1, D, requires_grad=True, device="cuda")
    y = torch.randn(1, N, D, device="cuda")
    a, b = -1.23, 1.54

    def fun(x, y, keops):
        if keops:
            x, y = LazyTensor(x), LazyTensor(y)
        Dxy = ((x * y).clamp(a, b)).sum(dim=2)
        return (-(Dxy ** 2)).exp().sum(dim=1)

    out = [fun(x, y, k).squeeze() for k in (False, True)]
    assert torch.allclose(out[0], out[1], rtol=1e-5, atol=1e-4)
    g = [torch.autograd.grad((o ** 2).sum(), [x])[0] for o in out]
    assert torch.allclose(g[0], g[1], atol=0.01, rtol=0.001)


def test_sinc_and_its_gradient():
    from keops_amd.torch import LazyTensor

    torch.manual_seed(0)
    x = (torch.rand(5, 1, dtype=torch.float64) * 2 * math.pi).cuda().requires_grad_(True)
    y = x.detach().clone().requires_grad_(True)
    s1 = LazyTensor(x[:, None]).sinc().sum(0)
    s1.backward()
    s2 = torch.sum(torch.sinc(y))
    s2.backward()
    assert torch.allclose(s1, s2) and torch.allclose(x.grad, y.grad)


def test_non_contiguous_input_gives_the_same_result():
    from keops_amd.torch import LazyTensor

    torch.manual_seed(0)
    a1 = torch.rand(2, 1000, 5, device="cuda")
    a2 = a1.permute(2, 0, 1).contiguous().permute(1, 2, 0)   # same values, other strides
    b, c = torch.rand(2, 1000, 5, device="cuda"), torch.rand(2, 1000, 5, device="cuda")
    b_j = LazyTensor(b[:, None])
    d1 = LazyTensor(a1[:, :, None]).sqdist(b_j).exp() @ c
    with pytest.warns(UserWarning, match="not contiguous"):
        d2 = LazyTensor(a2[:, :, None]).sqdist(b_j).exp() @ c
    assert not a2.is_contiguous() and torch.equal(d2, d1)


def test_matmul_into_a_preallocated_output():
    from keops_amd.torch import LazyTensor

    torch.manual_seed(0)
    M, N, D, DV = 20, 30, 3, 1
    x = torch.rand(M, 1, D, device="cuda") / math.sqrt(D)
    y = torch.rand(1, N, D, device="cuda") / math.sqrt(D)
    b = torch.randn(N, DV, device="cuda")
    a = torch.empty(M, DV, device="cuda")
    Kxy = (-((LazyTensor(x) - LazyTensor(y)).square()).sum(dim=2)).exp()
    ret = Kxy.__matmul__(b, sum_scheme="block_sum", out=a)
    ref = (-((x - y).square()).sum(dim=2)).exp() @ b
    assert ret.data_ptr() == a.data_ptr() and torch.allclose(a, ref)


def test_first_and_second_order_gradients():
    from keops_amd.torch import LazyTensor

    torch.manual_seed(0)
    M, N, DV = 100, 100, 1
    x = torch.rand(M, 1, 3, requires_grad=True, device="cuda")
    y = torch.rand(1, N, 1, device="cuda")
    b = torch.randn(N, DV, device="cuda")

    def fun(x, y, keops):
        if keops:
            x, y = LazyTensor(x), LazyTensor(y)
        return ((x.cos() - y).sum(dim=2) @ b).squeeze()

    out = [fun(x, y, k) for k in (True, False)]
    assert torch.allclose(out[0], out[1], rtol=1e-4)
    g = [torch.autograd.grad((o ** 2).sum(), [x], create_graph=True)[0] for o in out]
    assert torch.allclose(g[0], g[1], rtol=1e-4, atol=1e-4)
    g2 = [torch.autograd.grad((gk ** 2).sum(), [x])[0] for gk in g]
    assert torch.allclose(g2[0], g2[1], rtol=1e-3, atol=1e-2)


def test_min_argmin_of_a_formula_on_990_components():
    """pykeops/test/test_torch.py::test_LazyTensor_min_chunked: vectors of 990 components, a formula that is not a
    contraction (its long straight-line body is compiled as a chain of bounded functions)."""
    from keops_amd.torch import LazyTensor

    torch.manual_seed(0)
    M, N, D = 120, 150, 990
    x, y = torch.rand(M, D, device="cuda"), torch.rand(N, D, device="cuda")
    K_ij = ((-((LazyTensor(x.unsqueeze(-2)) + LazyTensor(y.unsqueeze(-3))) ** 2)).exp()).sum(-1)
    m, am = K_ij.min_argmin(dim=0)
    dense = (-((x.unsqueeze(-2) + y.unsqueeze(-3)) ** 2)).exp().sum(-1, keepdim=True)
    rm, ram = dense.min(dim=0)
    assert m.shape == rm.shape and torch.allclose(m, rm, atol=1e-5, rtol=1e-5)
    assert torch.equal(am.long(), ram)


@pytest.mark.parametrize("shapes,in_dims,out_dims", [
    (((5, 10, 1, 2), (5, 1, 20, 2), (5, 1, 20, 1)), 0, 0),
    (((10, 5, 1, 2), (1, 5, 20, 2), (1, 5, 20, 1)), 1, 1),
    (((10, 5, 1, 2), (5, 1, 20, 2), (1, 5, 20, 1)), (1, 0, 1), 2),
])
def test_vmap_with_in_and_out_dims_and_gradient(shapes, in_dims, out_dims):
    """pykeops/test/test_vmap.py: torch.vmap over different positions of the mapped dimension, and a gradient
    taken through the mapped function."""
    from keops_amd.torch import LazyTensor

    torch.manual_seed(0)
    kw = dict(dtype=torch.float64, device="cuda")
    x_i = torch.randn(*shapes[0], requires_grad=True, **kw)
    x_j, y_j = torch.randn(*shapes[1], **kw), torch.randn(*shapes[2], **kw)

    def fn(x_i, x_j, y_j, use_keops=True):
        if use_keops:
            x_i, x_j, y_j = LazyTensor(x_i), LazyTensor(x_j), LazyTensor(y_j)
        K_ij = (-((x_i - x_j) ** 2).sum(-1)).exp()
        if not use_keops:
            K_ij = K_ij[..., None]
        return (K_ij * y_j).sum(1)

    res_keops = torch.vmap(fn, in_dims=in_dims, out_dims=out_dims)(x_i, x_j, y_j, use_keops=True)
    res_torch = torch.vmap(fn, in_dims=in_dims, out_dims=out_dims)(x_i, x_j, y_j, use_keops=False)
    assert torch.allclose(res_keops, res_torch)
    u = torch.rand(res_torch.shape, **kw)
    (g_torch,) = torch.autograd.grad(res_torch, x_i, u)
    (g_keops,) = torch.autograd.grad(res_keops, x_i, u)
    assert torch.allclose(g_keops, g_torch)


def test_host_resident_tensors_are_staged_through_the_device():
    """pykeops/test/test_lazytensor_gaussian_fromhost.py: tensors in host memory with the GPU backend, result
    back in host memory; gradient and a preallocated host output as well."""
    from keops_amd.torch import Genred, LazyTensor

    torch.manual_seed(0)
    M, N, D, DV = 2500, 2000, 3, 1
    x = (torch.rand(M, 1, D, dtype=torch.float64) / math.sqrt(D)).requires_grad_(True)
    y = torch.rand(1, N, D, dtype=torch.float64) / math.sqrt(D)
    b = torch.randn(N, DV, dtype=torch.float64)
    Kxy = (-((LazyTensor(x) - LazyTensor(y)).square()).sum(dim=2)).exp()
    out = Kxy.__matmul__(b, sum_scheme="block_sum", device_id=0)
    ref = (-((x - y).square()).sum(dim=2)).exp() @ b
    assert out.device.type == "cpu" and torch.allclose(out, ref)
    (g,) = torch.autograd.grad(out.sum(), [x])
    (gr,) = torch.autograd.grad(ref.sum(), [x])
    assert g.device.type == "cpu" and torch.allclose(g, gr)
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(1)"], reduction_op="Sum", axis=1)
    a = torch.empty(M, DV, dtype=torch.float64)
    ret = conv(x.detach()[:, 0], y[0], b, out=a)
    assert ret.data_ptr() == a.data_ptr() and torch.allclose(a, ref.detach())
    with pytest.raises(ValueError):
        conv(x.detach()[:, 0], y[0], b, backend="CPU")   # no CPU implementation behind this API


def test_softdtw_bspline_and_grad_matrix_on_the_device():
    """The three operations of keopscore/formulas/maths that are dynamic programs or operators on formulas
    (SoftDTW_SqDist.py, BSpline.py, GradMatrix.py), reduced on the device and compared with the host evaluation of
    the same formulas."""
    import numpy as np

    from host_eval import dense_eval
    from keops_amd.torch import LazyTensor

    torch.manual_seed(3)
    M, N = 60, 70
    x = torch.rand(M, 6, dtype=torch.float64, device="cuda")
    y = torch.rand(N, 5, dtype=torch.float64, device="cuda")
    x_i, y_j = LazyTensor(x[:, None, :]), LazyTensor(y[None, :, :])
    got = x_i.softdtw_sqdist(y_j, 0.5).sum(dim=1)
    al = ["x=Vi(0,6)", "y=Vj(1,5)"]
    ref = dense_eval("SoftDTW_SqDist(x,y,0.5)", al, [x.cpu().numpy(), y.cpu().numpy()], M, N).sum(1)
    assert np.allclose(got.cpu().numpy(), ref, rtol=1e-10)
    xg = x.clone().requires_grad_(True)
    (g,) = torch.autograd.grad(LazyTensor(xg[:, None, :]).softdtw_sqdist(y_j, 0.5).sum(dim=1).sum(), [xg])
    refg = dense_eval("Grad(SoftDTW_SqDist(x,y,0.5),x,Var(2,1,1))", al, [x.cpu().numpy(), y.cpu().numpy(), np.ones((N, 1))], M, N).sum(1)
    assert np.allclose(g.cpu().numpy(), refg, rtol=1e-9, atol=1e-12)

    knots = torch.tensor([0.0, 0.2, 0.35, 0.6, 0.8, 1.0, 1.3], dtype=torch.float64, device="cuda")
    t_i = LazyTensor(x[:, None, :1])
    spl = LazyTensor(knots.view(1, 1, -1)).bspline(t_i * y_j[0], 2).sum(dim=1)
    refs = dense_eval("BSpline(k,Elem(x,0)*Elem(y,0),2)", al + ["k=Pm(2,7)"], [x.cpu().numpy(), y.cpu().numpy(), knots.cpu().numpy()], M, N).sum(1)
    assert spl.shape == (M, 4) and np.allclose(spl.cpu().numpy(), refs, rtol=1e-10, atol=1e-12)

    u_i, v_j = LazyTensor(x[:, None, :3].contiguous()), LazyTensor(y[None, :, :3].contiguous())
    gm = (-(u_i - v_j) ** 2).exp().grad_matrix(u_i)
    assert gm.shape == (M, N, 9)
    refm = dense_eval("GradMatrix(Exp(-Square(u-v)),u)", ["u=Vi(0,3)", "v=Vj(1,3)"],
                      [x[:, :3].cpu().numpy(), y[:, :3].cpu().numpy()], M, N).sum(1)
    assert np.allclose(gm.sum(dim=1).cpu().numpy(), refm, rtol=1e-10, atol=1e-12)


def test_numpy_lazytensor_and_generic_ops():
    """The NumPy front end (pykeops.numpy: LazyTensor, Vi / Vj / Pm, generic_argkmin) on host arrays, cf.
    pykeops/test/test_numpy.py: arrays are staged through the device, results come back as NumPy arrays."""
    import numpy as np

    from keops_amd.numpy import LazyTensor, Pm, Vi, Vj, generic_argkmin

    rng = np.random.default_rng(0)
    x, y, b = rng.random((300, 3)), rng.random((500, 3)), rng.standard_normal((500, 2))
    K = (-((LazyTensor(x[:, None, :]) - LazyTensor(y[None, :, :])) ** 2).sum(-1) / 0.25).exp()
    a = K @ b
    ref = np.exp(-((x[:, None, :] - y[None, :, :]) ** 2).sum(-1) / 0.25) @ b
    assert isinstance(a, np.ndarray) and a.dtype == np.float64 and np.allclose(a, ref, rtol=1e-10)
    s = (Vi(x) - Vj(y)).sqnorm2()
    idx = s.argKmin(5, dim=1)
    refi = np.argsort(((x[:, None, :] - y[None, :, :]) ** 2).sum(-1), axis=1, kind="stable")[:, :5]
    assert isinstance(idx, np.ndarray) and np.array_equal(idx.astype(np.int64), refi)
    knn = generic_argkmin("SqDist(x,y)", "a = Vi(5)", "x = Vi(3)", "y = Vj(3)")
    assert np.array_equal(knn(x, y).astype(np.int64), refi)
    lse = ((Vi(x) * Vj(y)).sum(-1) * Pm(np.array([2.0]))).logsumexp(dim=1)
    refl = np.log(np.exp(2.0 * x @ y.T).sum(1))
    assert np.allclose(lse[:, 0], refl, rtol=1e-10)


def test_matmul_with_the_2d_backend_and_two_orders_of_gradients():
    """pykeops/test/conv2d.py: K @ b through LazyTensor.__matmul__(..., backend="GPU_2D") at 20000 x 30000, and the
    first and second order gradients with respect to b, against dense torch (same shapes and draws)."""
    import math

    from keops_amd.torch import LazyTensor

    M, N, D, DV = 20000, 30000, 3, 1
    torch.manual_seed(0)
    x = torch.rand(M, 1, D, device="cuda") / math.sqrt(D)
    y = torch.rand(1, N, D, device="cuda") / math.sqrt(D)
    b = torch.randn(N, DV, requires_grad=True, device="cuda")

    def fun(keops):
        if keops:
            Kxy = (-((LazyTensor(x) - LazyTensor(y)) ** 2).sum(dim=2)).exp()
            return LazyTensor.__matmul__(Kxy, b, backend="GPU_2D").squeeze()
        return ((-((x.double() - y.double()) ** 2).sum(dim=2)).exp() @ b.double()).squeeze()

    out = [fun(True), fun(False)]
    g1 = [torch.autograd.grad((o ** 2).sum(), [b], create_graph=True)[0] for o in out]
    g2 = [torch.autograd.grad((g ** 2).sum(), [b])[0] for g in g1]
    for got, ref in zip((out[0], g1[0], g2[0]), (out[1], g1[1], g2[1])):
        assert torch.allclose(got.double(), ref.double(), rtol=1e-4, atol=1e-5 * float(ref.detach().abs().max()))
