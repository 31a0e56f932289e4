"""GPU parity of formulas with one long elementwise sum that has no matrix-core form (L1 distances, weighted or
transformed sums, float64 contractions): the general-purpose kernels built with KEOPS_VCHUNK, counterpart of the
reference's GpuReduc1D_chunks.py for such formulas.  References: dense float64 torch / NumPy evaluations, and
float32 sums in the reference's sequential order where indices are compared bit for bit."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity, rel_l2, to_dev

pytestmark = pytest.mark.gpu


def _last_module():
    from keops_amd import keops_io

    return list(keops_io._loaders.values())[-1].module


def test_l1_kernel_sum_and_its_gradient():
    from keops_amd.torch import Genred

    M, N, D, Dv = 700, 900, 300, 3
    gen = torch.Generator().manual_seed(0)
    x, y, b = torch.randn(M, D, generator=gen) / D, torch.randn(N, D, generator=gen) / D, torch.randn(N, Dv, generator=gen)
    conv = Genred("Exp(-Sum(Abs(x-y)))*b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"], reduction_op="Sum", axis=1)
    bd = b.cuda().requires_grad_(True)
    out = conv(x.cuda(), y.cuda(), bd)
    assert _last_module().meta("vchunk") == str(D)
    K = torch.exp(-torch.cdist(x.double(), y.double(), p=1))
    assert_sum_parity(out.detach().cpu().numpy(), (K @ b.double()).numpy(), (K @ b.double().abs()).numpy())
    e = torch.randn(M, Dv, generator=gen)
    (gb,) = torch.autograd.grad(out, [bd], e.cuda())
    assert rel_l2(gb.cpu().numpy(), (K.T @ e.double()).numpy()) < 1e-5
    # reduction over the other axis, few rows (column slabs)
    out0 = Genred("Exp(-Sum(Abs(x-y)))*b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vi({Dv})"], reduction_op="Sum", axis=0)(
        x.cuda(), y[:40].cuda(), e.cuda())
    assert rel_l2(out0.cpu().numpy(), (K[:, :40].T @ e.double()).numpy()) < 1e-5


@pytest.mark.parametrize("D", [784, 131])
def test_manhattan_nearest_neighbours_bit_exact(D):
    """ArgKMin of the L1 distance: indices must match a stable argsort of the float32 sums taken in the reference's
    order (component by component)."""
    from keops_amd.torch import Genred

    M, N, K = 200, 3000, 7
    rng = np.random.default_rng(D)
    x, y = rng.random((M, D), dtype=np.float32), rng.random((N, D), dtype=np.float32)
    knn = Genred("Sum(Abs(x-y))", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="KMin_ArgKMin", axis=1, opt_arg=K)
    vals, idx = knn(*to_dev(x, y))
    assert _last_module().meta("vchunk") == str(D)
    d = np.zeros((M, N), np.float32)
    for k in range(D):
        d += np.abs(x[:, None, k] - y[None, :, k])
    order = np.argsort(d, axis=1, kind="stable")[:, :K]
    assert np.array_equal(idx.cpu().numpy().astype(np.int64), order)
    assert np.array_equal(vals.cpu().numpy(), np.take_along_axis(d, order, 1))


def test_float64_gaussian_in_high_dimension():
    from keops_amd.torch import Genred

    M, N, D = 300, 500, 401
    gen = torch.Generator().manual_seed(3)
    x, y, b = (torch.randn(n, d, generator=gen, dtype=torch.float64) for n, d in ((M, D), (N, D), (N, 2)))
    x, y = x / D ** 0.5, y / D ** 0.5
    out = Genred("Exp(-SqDist(x,y))*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vj(2)"], reduction_op="Sum", axis=1)(
        x.cuda(), y.cuda(), b.cuda())
    assert _last_module().meta("vchunk") == str(D)
    ref = torch.exp(-torch.cdist(x, y) ** 2) @ b
    assert float((out.cpu() - ref).abs().max()) < 1e-12 * float(ref.abs().max())


def test_weighted_long_sum_with_batch_dimensions_and_logsumexp():
    """Short variables inside the long sum (a per-row weight and a parameter), batch dimensions with a broadcast one,
    log-sum-exp over the first index."""
    from keops_amd.torch import LazyTensor

    B, M, N, D = 3, 150, 220, 200
    gen = torch.Generator().manual_seed(4)
    x, y = torch.randn(B, M, D, generator=gen) / D, torch.randn(1, N, D, generator=gen) / D
    w, g = torch.rand(B, M, 1, generator=gen) + 0.5, torch.tensor([0.3])
    xd, yd, wd, gd = x.cuda(), y.cuda(), w.cuda(), g.cuda()
    x_i, y_j, w_i = LazyTensor(xd[:, :, None, :]), LazyTensor(yd[:, None, :, :]), LazyTensor(wd[:, :, None, :])
    F = -(((x_i - y_j).abs() * w_i).sum(-1)) * LazyTensor(gd)
    out = F.logsumexp(dim=1).cpu().double()[..., 0]                   # (B, N)
    assert _last_module().meta("vchunk") == str(D)
    dense = -(((x.double()[:, :, None, :] - y.double()[:, None, :, :]).abs() * w.double()[:, :, None, :]).sum(-1)) * 0.3
    ref = torch.logsumexp(dense, dim=1)
    assert float((out - ref).abs().max()) < 2e-5 * float(ref.abs().max())


def test_long_scalar_products_float64_and_transformed():
    """(a|b) is Sum(a*b): a float64 linear kernel and Sum(Exp(x*y)*z), which the engine rewrites as a scalar
    product with an elementwise operand."""
    from keops_amd.torch import Genred

    M, N, D = 260, 340, 300
    gen = torch.Generator().manual_seed(8)
    x, y, z = (torch.randn(n, D, generator=gen, dtype=torch.float64) / D ** 0.5 for n in (M, N, N))
    b = torch.randn(N, 2, generator=gen, dtype=torch.float64)
    lin = Genred("(x|y)*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vj(2)"], reduction_op="Sum", axis=1)
    out = lin(x.cuda(), y.cuda(), b.cuda()).cpu()
    assert _last_module().meta("vchunk") == str(D)
    ref = (x @ y.T) @ b
    assert float((out - ref).abs().max()) < 1e-12 * float(ref.abs().max())
    f32 = lambda t: t.float().cuda()
    tr = Genred("Sum(Exp(x*y)*z)", [f"x=Vi({D})", f"y=Vj({D})", f"z=Vj({D})"], reduction_op="Sum", axis=1)
    out2 = tr(f32(x), f32(y), f32(z)).cpu().double()
    assert _last_module().meta("vchunk") == str(D)
    ref2 = (torch.exp(x[:, None, :] * y[None, :, :]) * z[None, :, :]).sum(-1).sum(1, keepdim=True)
    assert float((out2 - ref2).abs().max()) < 1e-5 * float(ref2.abs().max())


def test_long_sum_over_the_first_index_with_block_sparse_ranges():
    """Reduction over i (axis=0) of an L1 kernel with block-sparse ranges: rows that no range covers give 0."""
    from keops_amd.torch import Genred

    M, N, D = 500, 640, 150
    gen = torch.Generator().manual_seed(12)
    x, y, e = torch.randn(M, D, generator=gen) / D, torch.randn(N, D, generator=gen) / D, torch.randn(M, 2, generator=gen)
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    # ranges_i, slices_i, redranges_j (for axis=1) and ranges_j, slices_j, redranges_i (used here, axis=0)
    ranges = (i64([[0, 200], [200, 500]]), i64([1, 2]), i64([[0, 300], [300, 600]]),
              i64([[0, 300], [300, 600]]), i64([1, 2]), i64([[0, 200], [200, 500]]))
    fn = Genred("Exp(-Sum(Abs(x-y)))*e", [f"x=Vi({D})", f"y=Vj({D})", "e=Vi(2)"], reduction_op="Sum", axis=0)
    out = fn(x.cuda(), y.cuda(), e.cuda(), ranges=ranges).cpu()
    assert _last_module().meta("vchunk") == str(D)
    mask = torch.zeros(M, N, dtype=torch.bool)
    mask[:200, :300] = True
    mask[200:, 300:600] = True
    K = torch.exp(-torch.cdist(x.double(), y.double(), p=1)) * mask
    assert rel_l2(out.numpy(), (K.T @ e.double()).numpy()) < 1e-5
    assert torch.all(out[600:] == 0)


def test_scalar_product_neighbours_keep_the_fused_multiply_add_chain(monkeypatch):
    """ArgKMin of 1 - (x|y) at D = 300 (angular neighbours of normalised rows): the chunked kernel folds the products
    with the reference's fma chain, so values and indices are bit-identical to the general-purpose kernel."""
    import keops_amd.get_keops_dll as engine
    from keops_amd import config, keops_io
    from keops_amd.torch import Genred

    M, N, D, K = 300, 5000, 300, 6
    rng = np.random.default_rng(17)
    x, y = rng.standard_normal((M, D)).astype(np.float32), rng.standard_normal((N, D)).astype(np.float32)
    x /= np.linalg.norm(x, axis=1, keepdims=True)
    y /= np.linalg.norm(y, axis=1, keepdims=True)
    knn = lambda: Genred("IntCst(1)-(x|y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="KMin_ArgKMin", axis=1, opt_arg=K)
    vals, idx = knn()(*to_dev(x, y))
    assert _last_module().meta("vchunk") == str(D)
    monkeypatch.setattr(config, "vchunk_min_dim", 1 << 20)
    engine._cache.clear()
    keops_io._loaders.clear()
    vals0, idx0 = knn()(*to_dev(x, y))
    assert _last_module().meta("vchunk") is None
    engine._cache.clear()
    keops_io._loaders.clear()
    assert torch.equal(vals, vals0) and torch.equal(idx, idx0)
    ref = np.argsort(1 - x.astype(np.float64) @ y.astype(np.float64).T, axis=1)[:, :K]
    assert (idx.cpu().numpy() == ref).mean() > 0.999
