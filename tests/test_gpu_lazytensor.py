"""LazyTensor front end on the GPU, against dense torch (the reference's test style:
pykeops/test/test_lazytensor_gaussian_cpu.py, test_lazytensor_gaussian_batch.py, test_torch.py)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_gaussian_matvec_and_two_orders_of_gradients():
    from keops_amd.torch import LazyTensor

    torch.manual_seed(0)
    M, N, D, DV = 1000, 1001, 3, 2
    x = torch.randn(M, D, device="cuda", dtype=torch.float64, requires_grad=True)
    y = torch.randn(N, D, device="cuda", dtype=torch.float64)
    b = torch.randn(N, DV, device="cuda", dtype=torch.float64)

    def fun(x, y, b, lazy):
        if lazy:
            xi, yj = LazyTensor(x[:, None, :]), LazyTensor(y[None, :, :])
        else:
            xi, yj = x[:, None, :], y[None, :, :]
        K = (-((xi - yj) ** 2).sum(dim=2) / 2).exp()
        return K @ b if lazy else K @ b

    outs = []
    for lazy in (True, False):
        o = fun(x, y, b, lazy)
        (g1,) = torch.autograd.grad((o**2).sum(), [x], create_graph=True)
        (g2,) = torch.autograd.grad((g1**2).sum(), [x])
        outs.append((o, g1, g2))
    for a, r in zip(*outs):
        assert torch.allclose(a, r, rtol=1e-9, atol=1e-9)


def test_batch_lazytensor_logsumexp_argkmin_and_ops():
    from keops_amd.torch import LazyTensor, Pm, Vi, Vj

    torch.manual_seed(1)
    B, M, N = 3, 200, 300
    x = torch.randn(B, M, 1, 3, device="cuda")
    y = torch.randn(1, 1, N, 3, device="cuda")
    p = torch.rand(B, 1, 1, 1, device="cuda") + 0.5
    xi, yj, pp = LazyTensor(x), LazyTensor(y), LazyTensor(p)
    D = ((xi - yj) ** 2).sum(-1)
    lse = (-D * pp).logsumexp(dim=2)
    dd = ((x - y) ** 2).sum(-1)
    assert tuple(lse.shape) == (B, M, 1)
    assert torch.allclose(lse[..., 0], torch.logsumexp(-dd * p[..., 0], dim=2), rtol=1e-5, atol=1e-5)
    idx = D.argKmin(4, dim=2)
    assert tuple(idx.shape) == (B, M, 4)
    assert (idx == dd.topk(4, dim=2, largest=False).indices).float().mean() > 0.999
    # plain 2D constructors, scalar arithmetic, Scalprod, abs, clamp, elementwise ops, sum over i
    x2, y2 = torch.randn(M, 3, device="cuda"), torch.randn(N, 3, device="cuda")
    F = ((Vi(x2) | Vj(y2)).abs() * 0.5 + (Vi(x2) - Vj(y2)).clamp(-1, 1).sum(-1) - 2 * Pm(torch.tensor([0.25], device="cuda")))
    got = F.sum(dim=0)
    dense = ((x2 @ y2.T).abs() * 0.5 + (x2[:, None] - y2[None]).clamp(-1, 1).sum(-1) - 0.5).sum(0)[:, None]
    assert torch.allclose(got, dense, rtol=1e-4, atol=1e-3)
    vals, arg = (Vi(x2).sqdist(Vj(y2))).min_argmin(dim=1)
    d2 = ((x2[:, None] - y2[None]) ** 2).sum(-1)
    assert torch.allclose(vals[:, 0], d2.min(1).values, rtol=1e-5, atol=1e-6)


def test_lazytensor_ranges_and_symbolic_variables():
    from keops_amd.torch import LazyTensor, Vi, Vj
    from keops_amd.torch.cluster import cluster_ranges, from_matrix, grid_cluster, sort_clusters

    torch.manual_seed(2)
    x = torch.rand(3000, 2, device="cuda")
    b = torch.randn(3000, 1, device="cuda")
    lab = grid_cluster(x, 0.25).long()
    (x, b), lab = sort_clusters((x, b), lab)
    r = cluster_ranges(lab)
    keep = torch.ones(len(r), len(r), dtype=torch.bool, device="cuda")
    keep[0, 1:] = False
    K = (-Vi(x).sqdist(Vj(x)) * 10.0).exp()
    K.ranges = from_matrix(r, r, keep)
    got = K @ b
    dense = torch.exp(-10 * torch.cdist(x, x) ** 2)
    mask = keep[lab][:, lab]
    assert torch.allclose(got, (dense * mask) @ b, rtol=1e-4, atol=1e-4)
    # symbolic variables are bound at call time
    f = (-(LazyTensor((0, 2, 0)) - LazyTensor((1, 2, 1))).sqnorm2()).exp().reduction("Sum", axis=1)
    out = f(x, x)
    assert torch.allclose(out[:, 0], torch.exp(-torch.cdist(x, x) ** 2).sum(1), rtol=1e-4)


def test_tensordot_and_kron_lazytensors():
    """Matrix-valued variables contracted per pair (cf. the reference's test_lazytensor_tensordot.py)."""
    from keops_amd.torch import LazyTensor

    torch.manual_seed(3)
    M, N = 70, 90
    a = torch.randn(M, 2 * 3, dtype=torch.float64, device="cuda", requires_grad=True)
    b = torch.randn(N, 3 * 4, dtype=torch.float64, device="cuda")
    A, B = LazyTensor(a[:, None, :]), LazyTensor(b[None, :, :])
    out = A.keops_tensordot(B, (2, 3), (3, 4), (1,), (0,)).sum_reduction(dim=1)     # sum_j A_i @ B_j, (M, 8)
    ref = torch.einsum("mik,nkl->mil", a.reshape(M, 2, 3), b.reshape(N, 3, 4)).reshape(M, 8)
    assert torch.allclose(out, ref, rtol=1e-10, atol=1e-10)
    e = torch.randn(M, 8, dtype=torch.float64, device="cuda")
    (g,) = torch.autograd.grad((out * e).sum(), [a])
    (gr,) = torch.autograd.grad((ref * e).sum(), [a])
    assert torch.allclose(g, gr, rtol=1e-10, atol=1e-10)
    k = A.keops_kron(B, (2, 3), (3, 4)).sum_reduction(dim=1)                           # (M, 6*12)
    kref = torch.stack([torch.kron(a[i].reshape(2, 3), b.reshape(N, 3, 4).sum(0)) for i in range(M)]).reshape(M, 72)
    assert torch.allclose(k, kref, rtol=1e-10, atol=1e-10)


def test_laplacian_and_diff_lazytensors():
    from keops_amd.torch import LazyTensor

    torch.manual_seed(4)
    M, N = 60, 80
    x = torch.randn(M, 3, dtype=torch.float64, device="cuda")
    y = torch.randn(N, 3, dtype=torch.float64, device="cuda")
    u = torch.randn(M, 3, dtype=torch.float64, device="cuda")
    X, Y, U = LazyTensor(x[:, None, :]), LazyTensor(y[None, :, :]), LazyTensor(u[:, None, :])
    K = (-((X - Y) ** 2).sum(-1)).exp()
    lap = K.laplacian(X).sum_reduction(dim=1)
    r2 = torch.cdist(x, y) ** 2
    assert torch.allclose(lap, ((4 * r2 - 6) * torch.exp(-r2)).sum(1, keepdim=True), rtol=1e-10, atol=1e-10)
    d = K.diff(X, U).sum_reduction(dim=1)      # sum_j <grad_x K(x_i, y_j), u_i>
    ref = (torch.exp(-r2)[:, :, None] * (-2 * (x[:, None, :] - y[None, :, :])) * u[:, None, :]).sum((1, 2))
    assert torch.allclose(d[:, 0], ref, rtol=1e-10, atol=1e-10)


def test_forward_mode_jvp_through_genred():
    """torch.func.jvp through a Sum reduction (cf. the reference's pykeops/test/test_torch_func.py)."""
    from keops_amd.torch import Genred

    torch.manual_seed(5)
    M, N = 50, 70
    x = torch.randn(M, 3, dtype=torch.float64, device="cuda")
    y = torch.randn(N, 3, dtype=torch.float64, device="cuda")
    b = torch.randn(N, 2, dtype=torch.float64, device="cuda")
    ux, ub = torch.randn_like(x), torch.randn_like(b)
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)"], reduction_op="Sum", axis=1)

    def dense(x_, b_):
        return torch.exp(-((x_[:, None, :] - y[None, :, :]) ** 2).sum(-1)) @ b_

    out, tan = torch.func.jvp(lambda x_, b_: conv(x_, y, b_), (x, b), (ux, ub))
    ref, rtan = torch.func.jvp(dense, (x, b), (ux, ub))
    assert torch.allclose(out, ref, rtol=1e-10, atol=1e-10)
    assert torch.allclose(tan, rtan, rtol=1e-10, atol=1e-10)


def test_vmap_through_genred():
    from keops_amd.torch import Genred

    torch.manual_seed(6)
    B, M, N = 5, 40, 60
    xs = torch.randn(B, M, 3, dtype=torch.float64, device="cuda")
    y = torch.randn(N, 3, dtype=torch.float64, device="cuda")
    b = torch.randn(N, 2, dtype=torch.float64, device="cuda")
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)"], reduction_op="Sum", axis=1)
    out = torch.func.vmap(lambda x_: conv(x_, y, b))(xs)
    ref = torch.exp(-((xs[:, :, None, :] - y[None, None, :, :]) ** 2).sum(-1)) @ b
    assert out.shape == (B, M, 2) and torch.allclose(out, ref, rtol=1e-10, atol=1e-10)


def _func_cases():
    """Shapes and functions of the reference's pykeops/test/test_torch_func.py (Gaussian sum with a batched
    parameter) and test_torch_func_logsumexp.py (weighted log-sum-exp), in float64 on the device."""
    torch.manual_seed(0)
    B1, B2, M, N, D = 5, 4, 10, 20, 2
    kw = dict(dtype=torch.float64, device="cuda")
    x_i, y_j = torch.randn(B1, B2, M, 1, D, **kw), torch.randn(B1, 1, 1, N, D, **kw)
    b_j, p = torch.randn(B1, B2, 1, N, 1, **kw), torch.rand(B1, 1, 1, 1, 1, **kw)
    w_j = torch.rand(B1, B2, 1, N, 1, **kw) + 0.1

    def sum_torch(x_i, y_j, b_j, p):
        K_ij = (-p[..., 0] * ((x_i - y_j) ** 2).sum(-1)).exp()[..., None]
        return ((K_ij * b_j).sum(-3)).norm()

    def sum_keops(x_i, y_j, b_j, p):
        from keops_amd.torch import LazyTensor

        nb = x_i.dim() - 3
        K_ij = (-LazyTensor(p) * ((LazyTensor(x_i) - LazyTensor(y_j)) ** 2).sum(-1)).exp()
        return ((K_ij * LazyTensor(b_j)).sum(nb)).norm()

    def lse_torch(x_i, y_j, w_j):
        D2_ij = (0.3 * ((x_i - y_j) ** 2).sum(-1))[..., None]
        return ((D2_ij.exp() * w_j).sum(-3)).log().norm()

    def lse_keops(x_i, y_j, w_j):
        from keops_amd.torch import LazyTensor

        nb = x_i.dim() - 3
        D2_ij = 0.3 * ((LazyTensor(x_i) - LazyTensor(y_j)) ** 2).sum(-1)
        return D2_ij.logsumexp(axis=nb, other=LazyTensor(w_j)).norm()

    tangents = tuple(torch.randn_like(t) for t in (x_i, y_j, b_j, p))
    return (sum_torch, sum_keops, (x_i, y_j, b_j, p), tangents), (lse_torch, lse_keops, (x_i, y_j, w_j), tangents[:3])


@pytest.mark.parametrize("which", [0, 1])
def test_torch_func_transforms(which):
    """grad, vjp, jvp, jacrev, jacfwd, hessian and vmap of a scalar function of a reduction agree with dense torch,
    for a Sum and for a weighted log-sum-exp reduction (forward mode through the (max, sum) pair)."""
    f_torch, f_keops, args, tans = _func_cases()[which]
    idx = tuple(range(len(args)))
    close = lambda a, b: torch.allclose(a, b, rtol=1e-8, atol=1e-8)
    assert close(f_keops(*args), f_torch(*args))
    for a, b in zip(torch.func.grad(f_keops, idx)(*args), torch.func.grad(f_torch, idx)(*args)):
        assert close(a, b)
    one = torch.tensor(1.0, dtype=torch.float64, device="cuda")
    for a, b in zip(torch.func.vjp(f_keops, *args)[1](one), torch.func.vjp(f_torch, *args)[1](one)):
        assert close(a, b)
    assert close(torch.func.jvp(f_keops, args, tans)[1], torch.func.jvp(f_torch, args, tans)[1])
    for a, b in zip(torch.func.jacrev(f_keops, idx)(*args), torch.func.jacrev(f_torch, idx)(*args)):
        assert close(a, b)
    assert close(torch.func.jacfwd(f_keops)(*args), torch.func.jacfwd(f_torch)(*args))
    assert close(torch.func.hessian(f_keops)(*args), torch.func.hessian(f_torch)(*args))
    assert close(torch.func.vmap(f_keops)(*args), torch.func.vmap(f_torch)(*args))


def test_trace_operator_on_lazytensors():
    """x.trace_operator(v) (pykeops/common/lazy_tensor.py:2007-2035): self must be linear in the symbolic variable v,
    which leaves the formula and needs no data in the reduction."""
    from keops_amd.torch import LazyTensor, Vi, Vj

    gen = torch.Generator(device="cuda").manual_seed(12)
    A = torch.rand(300, 9, device="cuda", generator=gen)
    b = torch.rand(400, 1, device="cuda", generator=gen)
    Ai, bj = Vi(A), Vj(b)
    v = LazyTensor((7, 3, 1))                       # symbolic variable Var(7, 3, 1)
    F = Ai.matvecmult(v) * bj + 2 * v               # linear in v: trace = b_j tr(A_i) + 6
    T = F.trace_operator(v)
    out = T.sum(dim=1)
    tr = A[:, 0] + A[:, 4] + A[:, 8]
    assert torch.allclose(out[:, 0], tr * b.sum() + 6 * 400, rtol=1e-5)


def test_difference_matrix_on_lazytensors():
    """x.difference_matrix(y) (pykeops/common/lazy_tensor.py:1591-1597): the table x_i[a] - y_j[c] of size
    dim(x) * dim(y), entry (c, a) at c*dim(x)+a, forward and both gradients against dense torch in float64."""
    from keops_amd.torch import Vi, Vj

    gen = torch.Generator(device="cuda").manual_seed(13)
    x = torch.rand(300, 4, device="cuda", dtype=torch.float64, generator=gen, requires_grad=True)
    y = torch.rand(400, 3, device="cuda", dtype=torch.float64, generator=gen, requires_grad=True)
    w = torch.rand(400, 12, device="cuda", dtype=torch.float64, generator=gen)
    D = Vi(x).difference_matrix(Vj(y))
    assert D.ndim == 12
    out = ((-(D ** 2)).exp() * Vj(w)).sum(dim=1)
    dense = (torch.exp(-(x[:, None, None, :] - y[None, :, :, None]) ** 2).reshape(300, 400, 12) * w[None]).sum(1)
    assert torch.allclose(out, dense, rtol=1e-12)
    e = torch.rand(300, 12, device="cuda", dtype=torch.float64, generator=gen)
    for got, ref in zip(torch.autograd.grad(out, [x, y], e), torch.autograd.grad(dense, [x, y], e)):
        assert torch.allclose(got, ref, rtol=1e-10, atol=1e-12)
