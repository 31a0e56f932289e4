"""GPU parity of the matrix-core chunked scheme (keops_chunk_mfma.h) for high-dimensional formulas:
the result must equal the un-chunked formula (the scheme is only a schedule), cf. the reference's
pykeops/test/test_chunks.py (D=300-style tests, atol 1e-4)."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity, rel_l2, to_dev
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu


def _laplace_inputs(M, N, D, Dv, seed):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((M, D)) / np.sqrt(D)).astype(np.float32)
    y = (rng.standard_normal((N, D)) / np.sqrt(D)).astype(np.float32)
    b = rng.standard_normal((N, Dv)).astype(np.float32)
    return x, y, b


def _scheme_used(name):
    from keops_amd import keops_io

    return any(m.meta("scheme") == name for m in keops_io._modules.values())


@pytest.mark.parametrize("M,N,D,Dv", [(1000, 1500, 256, 16), (333, 4097, 64, 3), (2049, 31, 100, 1), (50, 70, 32, 2), (700, 1300, 24, 2)])
def test_laplace_chunked_vs_oracle(M, N, D, Dv):
    from keops_amd.torch import Genred

    x, y, b = _laplace_inputs(M, N, D, Dv, 5)
    conv = Genred("Exp(-Norm2(x-y))*b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"], reduction_op="Sum", axis=1)
    got = conv(*to_dev(x, y, b)).cpu().numpy()
    assert _scheme_used("chunk")
    ref = cpu_reduc("laplace", [x, y, b], M, N, Dv)
    scale = cpu_reduc("laplace", [x, y, np.abs(b)], M, N, Dv)
    assert_sum_parity(got, ref, scale)
    # without the matrix-core schemes (enable_chunks=False: exact float32 arithmetic) it is the same function
    plain = Genred("Exp(-Norm2(x-y))*b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"], reduction_op="Sum", axis=1,
                   enable_chunks=False)(*to_dev(x, y, b)).cpu().numpy()
    assert_sum_parity(plain, ref, scale)


def test_config5b_laplace_d256_row_subset():
    # headline configuration 5b: M=N=200,000, D=256, Dv=16, x,y ~ N(0,1/D), seed 5
    M = N = 200_000
    from keops_amd.torch import Genred

    x, y, b = _laplace_inputs(M, N, 256, 16, 5)
    conv = Genred("Exp(-Norm2(x-y))*b", ["x=Vi(256)", "y=Vj(256)", "b=Vj(16)"], reduction_op="Sum", axis=1)
    got = conv(*to_dev(x, y, b))
    rows = np.sort(np.random.default_rng(9).choice(M, 1024, replace=False)).astype(np.int64)
    ref = cpu_reduc("laplace", [x, y, b], M, N, 16, rows=rows)
    scale = cpu_reduc("laplace", [x, y, np.abs(b)], M, N, 16, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    twice = conv(*[t * s for t, s in zip(to_dev(x, y, b), (1, 1, 2))])
    assert torch.equal(twice, 2 * got)  # linearity in b holds exactly


def test_scalprod_mode_uncentred_data_axis0_and_lse():
    from keops_amd.torch import Genred

    M, N, D = 700, 900, 128
    rng = np.random.default_rng(7)
    x = (rng.standard_normal((M, D)) / np.sqrt(D) + 0.05).astype(np.float32)
    y = (rng.standard_normal((N, D)) / np.sqrt(D) + 0.05).astype(np.float32)
    b = rng.standard_normal((M, 2)).astype(np.float32)
    p = np.array([0.7], np.float32)
    xd, yd, bd, pd_ = to_dev(x, y, b, p)
    x64, y64, b64 = (torch.from_numpy(t).double() for t in (x, y, b))
    # reduction over i of exp(p * <x,y>) * b_i : Scalprod contraction, output indexed by j
    conv = Genred("Exp(p*(x|y))*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vi(2)", "p=Pm(1)"], reduction_op="Sum", axis=0)
    got = conv(xd, yd, bd, pd_).cpu().double()
    K = torch.exp(0.7 * (x64 @ y64.T))  # (M,N)
    ref = K.T @ b64
    scale = K.T @ b64.abs()
    assert_sum_parity(got.numpy(), ref.numpy(), scale.numpy())
    # log-sum-exp of -SqDist/ (2 sigma^2) over a high-dimensional feature space, far from the origin
    xs = (rng.standard_normal((M, D)) + 3.0).astype(np.float32)
    ys = (rng.standard_normal((N, D)) + 3.0).astype(np.float32)
    lse = Genred("-SqDist(x,y)*p", [f"x=Vi({D})", f"y=Vj({D})", "p=Pm(1)"], reduction_op="LogSumExp", axis=1)
    got = lse(*to_dev(xs, ys, np.array([0.01], np.float32))).cpu().double()
    d2 = torch.cdist(torch.from_numpy(xs).double(), torch.from_numpy(ys).double()) ** 2
    ref = torch.logsumexp(-0.01 * d2, dim=1, keepdim=True)
    assert float((got - ref).abs().max()) <= 1e-5 * max(1.0, float(ref.abs().max()))
    assert _scheme_used("chunk")


def test_gradient_through_chunked_formula():
    from keops_amd.torch import Genred

    M, N, D = 300, 400, 64
    rng = np.random.default_rng(8)
    x = torch.from_numpy((rng.standard_normal((M, D)) / 8).astype(np.float32)).cuda().requires_grad_(True)
    y = torch.from_numpy((rng.standard_normal((N, D)) / 8).astype(np.float32)).cuda()
    b = torch.from_numpy(rng.standard_normal((N, 1)).astype(np.float32)).cuda()
    conv = Genred("Exp(-SqDist(x,y))*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vj(1)"], reduction_op="Sum", axis=1)
    out = conv(x, y, b)
    (gx,) = torch.autograd.grad(out.sum(), [x])
    xt = x.detach().double().requires_grad_(True)
    ref = (torch.exp(-torch.cdist(xt, y.double()) ** 2) @ b.double()).sum()
    (rx,) = torch.autograd.grad(ref, [xt])
    assert rel_l2(gx.cpu().numpy(), rx.cpu().numpy()) < 1e-5


def test_final_product_variant_and_generic_variant():
    """Post-chunk formulas g(s)*b run their weighted sum on the matrix cores too (two 32-column blocks
    here, forced column slabs); other post-chunk formulas keep the per-lane accumulation."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    M, N, D, Dv = 300, 2100, 64, 40
    x, y, b = _laplace_inputs(M, N, D, Dv, 21)
    xd, yd, bd = to_dev(x, y, b)
    x64, y64, b64 = (torch.from_numpy(t).double() for t in (x, y, b))
    K = torch.exp(-torch.cdist(x64, y64))
    conv = Genred("Exp(-Norm2(x-y))*b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"], reduction_op="Sum", axis=1)
    for backend in ("GPU_1D", "GPU_2D"):
        got = conv(xd, yd, bd, backend=backend).cpu().numpy()
        assert_sum_parity(got, (K @ b64).numpy(), (K @ b64.abs()).numpy())
    assert any(m.meta("chk_final") == "1" for m in keops_io._modules.values())
    # not a plain product: generic accumulation in the formula's output dimension
    conv2 = Genred("Exp(-Norm2(x-y))*b+b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"], reduction_op="Sum", axis=1)
    got2 = conv2(xd, yd, bd).cpu().numpy()
    ref2 = (K @ b64 + b64.sum(0, keepdim=True)).numpy()
    scale2 = (K @ b64.abs() + b64.abs().sum(0, keepdim=True)).numpy()
    assert_sum_parity(got2, ref2, scale2)
    assert any(m.meta("scheme") == "chunk" and m.meta("chk_final") == "0" for m in keops_io._modules.values())


@pytest.mark.parametrize("M,N,D,Dv,axis", [(700, 900, 64, 64, 1), (333, 2100, 128, 40, 1), (500, 47, 32, 3, 1), (640, 500, 64, 16, 0),
                                          (300, 5000, 256, 64, 1)])
def test_softmax_weighted_sum_on_matrix_cores(M, N, D, Dv, axis):
    """SumSoftMaxWeight of a scaled inner product (attention-like): online softmax with the weighted sum on
    the matrix cores (keops_chk_softmax), against torch.softmax in float64; also the plain weighted
    log-sum-exp layout (no leading 1) and forced column slabs."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    rng = np.random.default_rng(31)
    q = (rng.standard_normal((M, D)) / D ** 0.25).astype(np.float32)
    k = (rng.standard_normal((N, D)) / D ** 0.25).astype(np.float32)
    nv = N if axis == 1 else M
    v = rng.standard_normal((nv, Dv)).astype(np.float32)
    qd, kd, vd = to_dev(q, k, v)
    vcat = "Vj" if axis == 1 else "Vi"
    att = Genred("p*(q|k)", [f"q=Vi({D})", f"k=Vj({D})", f"v={vcat}({Dv})", "p=Pm(1)"], reduction_op="SumSoftMaxWeight",
                 axis=axis, formula2="v")
    scale = torch.tensor([0.7], device="cuda")
    S = 0.7 * torch.from_numpy(q).double() @ torch.from_numpy(k).double().T
    if axis == 0:
        S = S.T
    ref = torch.softmax(S, dim=1) @ torch.from_numpy(v).double()
    for backend in ("GPU_1D", "GPU_2D"):
        got = att(qd, kd, vd, scale, backend=backend).cpu().double()
        assert got.shape == ref.shape
        assert float((got - ref).abs().max()) <= 2e-5 * float(ref.abs().max()), backend
    assert any(m.meta("chk_softmax") == "1" for m in keops_io._modules.values())
    # weighted log-sum-exp: log sum_j exp(S_ij) v_j with positive weights
    w = np.abs(v[:, :min(Dv, 5)]) + 0.1
    lse = Genred("p*(q|k)", [f"q=Vi({D})", f"k=Vj({D})", f"w={vcat}({w.shape[1]})", "p=Pm(1)"], reduction_op="LogSumExp",
                 axis=axis, formula2="w")
    gl = lse(qd, kd, to_dev(w)[0], scale).cpu().double()
    refl = torch.logsumexp(S[:, :, None] + torch.log(torch.from_numpy(w).double())[None, :, :], dim=1)
    assert float((gl - refl).abs().max()) <= 2e-5 * max(1.0, float(refl.abs().max()))


@pytest.mark.parametrize("M,N,D,Dv", [(200, 300, 300, 1), (700, 1000, 512, 16), (333, 777, 700, 3), (150, 260, 1024, 2)])
def test_contraction_beyond_256_components(M, N, D, Dv):
    """Several wavefronts share 32 output rows and split the contraction (D = 300 is the size of the reference's
    pykeops/test/test_chunks.py); Sum and log-sum-exp against dense float64."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    x, y, b = _laplace_inputs(M, N, D, Dv, 51)
    xd, yd, bd = to_dev(x, y, b)
    x64, y64, b64 = (torch.from_numpy(t).double() for t in (x, y, b))
    K = torch.exp(-torch.cdist(x64, y64))
    conv = Genred("Exp(-Norm2(x-y))*b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"], reduction_op="Sum", axis=1)
    got = conv(xd, yd, bd).cpu().numpy()
    assert any(m.meta("scheme") == "chunk" and m.meta("chk_d") == str(D) for m in keops_io._modules.values())
    assert_sum_parity(got, (K @ b64).numpy(), (K @ b64.abs()).numpy())
    # reduction over i, inner-product mode, log-sum-exp
    lse = Genred("p*(x|y)", [f"x=Vi({D})", f"y=Vj({D})", "p=Pm(1)"], reduction_op="LogSumExp", axis=0)
    gl = lse(xd, yd, torch.tensor([0.5], device="cuda")).cpu().double()[:, 0]
    refl = torch.logsumexp(0.5 * x64 @ y64.T, dim=0)
    assert float((gl - refl).abs().max()) <= 2e-5 * max(1.0, float(refl.abs().max()))


def test_contraction_beyond_256_components_batched():
    """Shapes of the reference's pykeops/test/test_chunks_ranges.py: two batch dimensions, D = 300."""
    from keops_amd.torch import LazyTensor

    B1, B2, M, N, D, Dv = 2, 3, 200, 300, 300, 1
    gen = torch.Generator().manual_seed(52)
    x = torch.randn(B1, B2, M, 1, D, generator=gen) / 8
    y = torch.randn(B1, 1, 1, N, D, generator=gen) / 8
    b = torch.randn(B1, B2, 1, N, Dv, generator=gen)
    got = ((-((LazyTensor(x.cuda()) - LazyTensor(y.cuda())) ** 2).sum(-1)).exp() * LazyTensor(b.cuda())).sum(dim=3).cpu()
    K = torch.exp(-((x.double() - y.double()) ** 2).sum(-1))          # (B1, B2, M, N)
    ref = K @ b.double()[:, :, 0]
    scale = K @ b.double()[:, :, 0].abs()
    assert_sum_parity(got.numpy(), ref.numpy(), scale.numpy())


@pytest.mark.parametrize("D,kernel", [(64, "gauss"), (256, "laplace"), (200, "expdot"), (640, "gauss"), (24, "laplace")])
def test_gradients_wrt_points_as_scalar_and_weighted_sums(D, kernel):
    """d/dx and d/dy of sum_ij e_i . K(x_i, y_j) b_j for radial and scalar-product kernels in high dimension:
    g_ij (x_i - y_j) (or g_ij y_j) is computed as x_i sum_j g_ij - sum_j g_ij y_j, chunked reductions only
    (get_keops_dll.plan_row_col_product).  Reference: torch.autograd on the dense float64 formula."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    M, N, Dv = 333, 450, 3
    gen = torch.Generator().manual_seed(D)
    x, y, b, e = (torch.randn(*s, generator=gen) for s in ((M, D), (N, D), (N, Dv), (M, Dv)))
    x, y = x / D ** 0.5, y / D ** 0.5 + 0.1
    formula = {"gauss": "Exp(-g*SqDist(x,y))*b", "laplace": "Exp(-g*Norm2(x-y))*b", "expdot": "Exp(g*(x|y))*b"}[kernel]
    conv = Genred(formula, [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})", "g=Pm(1)"], reduction_op="Sum", axis=1)
    xd, yd = x.cuda().requires_grad_(True), y.cuda().requires_grad_(True)
    g = torch.tensor([0.7])
    keops_io._loaders.clear()
    out = conv(xd, yd, b.cuda(), g.cuda())
    gx, gy = torch.autograd.grad(out, [xd, yd], e.cuda())
    planned = [ld for ld in keops_io._loaders.values() if ld.plan is not None]
    assert len(planned) == 2 and all(ld.module is None for ld in planned)
    subs = [s for ld in planned for s in ([ld.sub_scalar] if ld.sub_scalar else []) + [t[2] for t in ld.sub_slices]]
    assert all((ld.sub_scalar is None) == (ld.ones_column or kernel == "expdot") for ld in planned)
    assert subs and all(s.module.meta("scheme") == "chunk" for s in subs)
    x64, y64 = x.double().requires_grad_(True), y.double().requires_grad_(True)
    if kernel == "gauss":
        K = torch.exp(-0.7 * torch.cdist(x64, y64) ** 2)
    elif kernel == "laplace":
        K = torch.exp(-0.7 * torch.cdist(x64, y64))
    else:
        K = torch.exp(0.7 * x64 @ y64.T)
    rx, ry = torch.autograd.grad(((K @ b.double()) * e.double()).sum(), [x64, y64])
    assert rel_l2(gx.cpu().numpy(), rx.numpy()) < 2e-5, rel_l2(gx.cpu().numpy(), rx.numpy())
    assert rel_l2(gy.cpu().numpy(), ry.numpy()) < 2e-5, rel_l2(gy.cpu().numpy(), ry.numpy())


def test_gradient_wrt_points_with_batch_dimensions_and_out():
    from keops_amd.torch import LazyTensor

    B, M, N, D = 3, 200, 260, 96
    gen = torch.Generator().manual_seed(77)
    x, y, b = torch.randn(B, M, D, generator=gen) / D ** 0.5, torch.randn(1, N, D, generator=gen) / D ** 0.5, torch.randn(B, N, 2, generator=gen)
    xd, yd, bd = x.cuda().requires_grad_(True), y.cuda().requires_grad_(True), b.cuda()
    K_ij = (-((LazyTensor(xd[:, :, None, :]) - LazyTensor(yd[:, None, :, :])) ** 2).sum(-1)).exp()
    out = (K_ij * LazyTensor(bd[:, None, :, :])).sum(dim=2)
    gx, gy = torch.autograd.grad(out.sum(), [xd, yd])
    x64, y64 = x.double().requires_grad_(True), y.double().requires_grad_(True)
    K = torch.exp(-torch.cdist(x64, y64.expand(B, N, D)) ** 2)
    rx, ry = torch.autograd.grad((K @ b.double()).sum(), [x64, y64])
    assert gx.shape == rx.shape and gy.shape == ry.shape
    assert rel_l2(gx.cpu().numpy(), rx.numpy()) < 2e-5
    assert rel_l2(gy.cpu().numpy(), ry.numpy()) < 2e-5


def test_attention_backward_uses_chunked_reductions():
    """Gradients of softmax(q k^T) v and of a log-sum-exp with respect to queries and keys (D = 64): every
    reduction of the backward pass runs on the chunked scheme."""
    from keops_amd import keops_io
    from keops_amd.torch import LazyTensor

    M, N, D, Dv = 500, 700, 64, 32
    gen = torch.Generator().manual_seed(9)
    q, k, v = torch.randn(M, D, generator=gen) / D ** 0.25, torch.randn(N, D, generator=gen) / D ** 0.25, torch.randn(N, Dv, generator=gen)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    keops_io._loaders.clear()
    S_ij = (LazyTensor(qd[:, None, :]) * LazyTensor(kd[None, :, :])).sum(-1)
    out = S_ij.sumsoftmaxweight(LazyTensor(vd[None, :, :]), dim=1)
    lse = S_ij.logsumexp(dim=1)
    e = torch.randn(M, Dv, generator=gen)
    gq, gk, gv = torch.autograd.grad([out, lse], [qd, kd, vd], [e.cuda(), torch.ones(M, 1, device="cuda")])
    assert all(ld.plan is not None or ld.module.meta("scheme") == "chunk" for ld in keops_io._loaders.values())
    q64, k64, v64 = (t.double().requires_grad_(True) for t in (q, k, v))
    S = q64 @ k64.T
    rq, rk, rv = torch.autograd.grad([torch.softmax(S, 1) @ v64, torch.logsumexp(S, 1, keepdim=True)], [q64, k64, v64],
                                     [e.double(), torch.ones(M, 1, dtype=torch.float64)])
    for got, ref in ((gq, rq), (gk, rk), (gv, rv)):
        assert rel_l2(got.cpu().numpy(), ref.numpy()) < 3e-5, rel_l2(got.cpu().numpy(), ref.numpy())


def test_point_gradient_formula_with_block_sparse_ranges_and_out():
    """The formula g_ij (x_i - y_j) written by hand, with block-sparse ranges and a preallocated output: the
    scalar and weighted chunked reductions both receive the ranges."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    M, N, D = 600, 800, 72
    gen = torch.Generator().manual_seed(21)
    x, y = torch.randn(M, D, generator=gen) / D ** 0.5, torch.randn(N, D, generator=gen) / D ** 0.5
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    ranges = (i64([[0, 250], [250, 600]]), i64([1, 3]), i64([[0, 300], [100, 500], [500, 800]]),
              i64([[0, 300], [100, 500], [500, 800]]), i64([1, 2, 3]), i64([[0, 250], [250, 600], [250, 600]]))
    keops_io._loaders.clear()
    fn = Genred("Exp(-SqDist(x,y))*(x-y)", [f"x=Vi({D})", f"y=Vj({D})"], reduction_op="Sum", axis=1)
    out = torch.empty(M, D, device="cuda")
    res = fn(x.cuda(), y.cuda(), ranges=ranges, out=out)
    assert res.data_ptr() == out.data_ptr()
    assert any(ld.plan is not None for ld in keops_io._loaders.values())
    mask = torch.zeros(M, N, dtype=torch.bool)
    mask[:250, :300] = True
    mask[250:, 100:] = True
    x64, y64 = x.double(), y.double()
    K = torch.exp(-torch.cdist(x64, y64) ** 2) * mask
    ref = x64 * K.sum(1, keepdim=True) - K @ y64
    assert rel_l2(out.cpu().numpy(), ref.numpy()) < 2e-5


@pytest.mark.parametrize("reduction", ["Sum", "LogSumExp"])
def test_narrow_kernel_on_clustered_points_and_self_interaction(reduction):
    """Tight clusters far apart and a kernel as narrow as a cluster, x = y: every pair that matters is close compared
    with the norms, where the 16-bit expansion of |x - y|^2 alone would be off by 2^-17 of the squared norms (10 %
    of the kernel value here).  Such pairs are recomputed from the float32 rows: parity as everywhere else."""
    from keops_amd.torch import Genred

    D, C, per = 64, 20, 100
    gen = torch.Generator().manual_seed(31)
    centres = torch.randn(C, D, generator=gen)
    x = (centres[:, None, :] + 0.01 * torch.randn(C, per, D, generator=gen)).reshape(C * per, D)
    b = torch.randn(C * per, 5, generator=gen)
    g = torch.tensor([1.0 / (2 * 0.01 ** 2 * D)])                 # exp(-g s) ~ exp(-1) inside a cluster
    xd = x.cuda()
    x64 = x.double()
    S = torch.cdist(x64, x64) ** 2
    if reduction == "Sum":
        conv = Genred("Exp(-g*SqDist(x,y))*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vj(5)", "g=Pm(1)"], reduction_op="Sum", axis=1)
        out = conv(xd, xd, b.cuda(), g.cuda()).cpu()
        assert _scheme_used("chunk")
        K = torch.exp(-g.double() * S)
        assert_sum_parity(out.numpy(), (K @ b.double()).numpy(), (K @ b.double().abs()).numpy())
        # the diagonal alone: a kernel so narrow that only the self-interaction is left
        conv1 = Genred("Exp(-g*SqDist(x,y))", [f"x=Vi({D})", f"y=Vj({D})", "g=Pm(1)"], reduction_op="Sum", axis=1)
        ones = conv1(xd, xd, (1e4 * g).cuda()).cpu()
        assert float((ones - 1).abs().max()) < 1e-5
    else:
        lse = Genred("-g*SqDist(x,y)", [f"x=Vi({D})", f"y=Vj({D})", "g=Pm(1)"], reduction_op="LogSumExp", axis=1)
        out = lse(xd, xd, g.cuda()).cpu().double()[:, 0]
        ref = torch.logsumexp(-g.double() * S, dim=1)
        assert float((out - ref).abs().max()) < 1e-5 * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("N,D", [(12, 257), (3, 64), (9, 300), (1, 40)])
def test_log_sum_exp_with_fewer_columns_than_a_tile(N, D):
    """Fewer reduced rows than the lanes that share an output row can take: some of their accumulators stay empty
    (maximum -inf, sum 0) and merging two empty ones must stay empty, not NaN."""
    from keops_amd.torch import LazyTensor

    gen = torch.Generator().manual_seed(N * D)
    x, y, v = torch.randn(1, 300, D, generator=gen) / D ** 0.5, torch.randn(1, N, D, generator=gen) / D ** 0.5, torch.randn(1, N, 3, generator=gen)
    S_ij = (LazyTensor(x.cuda()[:, :, None, :]) * LazyTensor(y.cuda()[:, None, :, :])).sum(-1)
    out = S_ij.sumsoftmaxweight(LazyTensor(v.cuda()[:, None, :, :]), dim=2).cpu().double()
    lse = S_ij.logsumexp(dim=2).cpu().double()[..., 0]
    S = x.double() @ y.double().transpose(1, 2)
    assert float((out - torch.softmax(S, 2) @ v.double()).abs().max()) < 2e-5
    assert float((lse - torch.logsumexp(S, 2)).abs().max()) < 2e-5


@pytest.mark.parametrize("clustered", [False, True])
@pytest.mark.parametrize("reduction", ["Sum", "LogSumExp"])
@pytest.mark.parametrize("D", [24, 64, 256])
@pytest.mark.parametrize("width", [3, 10, 30, 100])
def test_narrow_but_not_local_kernels_meet_parity_on_the_default_path(width, D, reduction, clustered):
    """Kernels that are narrow compared with the cloud without being local: g (|x^|^2 + |y^|^2) = width for the
    centred points, where an error eps (|x^|^2 + |y^|^2) on the squared distance becomes width * eps on every
    kernel value and the pairs that matter are too far apart (s > 1/8 of the norms) to be recomputed in float32.
    Default flags (enable_chunks=True, use_fast_math=True): the matrix-core chunked scheme, against the CPU oracle
    (float32, the reference's operation order) at 1e-5."""
    from keops_amd.torch import Genred

    M, N = 600, 3000
    rng = np.random.default_rng(1000 * width + D + (7 if clustered else 0))
    if clustered:
        # 30 clusters of relative radius 1/2: inside a cluster s is about 1/5 of |x^|^2 + |y^|^2, above the 1/8 threshold
        c = rng.standard_normal((30, D)) / np.sqrt(D)
        x = (c[rng.integers(0, 30, M)] + 0.5 * rng.standard_normal((M, D)) / np.sqrt(D)).astype(np.float32)
        y = (c[rng.integers(0, 30, N)] + 0.5 * rng.standard_normal((N, D)) / np.sqrt(D)).astype(np.float32)
    else:
        x = (rng.standard_normal((M, D)) / np.sqrt(D)).astype(np.float32)
        y = (rng.standard_normal((N, D)) / np.sqrt(D)).astype(np.float32)
    mu = y.mean(0)
    norms = float(((x - mu) ** 2).sum(1).mean() + ((y - mu) ** 2).sum(1).mean())
    g = np.array([width / norms], np.float32)
    if reduction == "Sum":
        b = rng.standard_normal((N, 2)).astype(np.float32)
        conv = Genred("Exp(-g*SqDist(x,y))*b", [f"x=Vi({D})", f"y=Vj({D})", "b=Vj(2)", "g=Pm(1)"], reduction_op="Sum", axis=1)
        got = conv(*to_dev(x, y, b, g)).cpu().numpy()
        assert _scheme_used("chunk")
        ref = cpu_reduc("gauss", [x, y, b, g], M, N, 2)
        scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 2)
        if width <= 30:
            assert_sum_parity(got, ref, scale)
        else:
            # exp(-g s) with g s ~ 100 amplifies any rounding of s a hundredfold: the float32 arithmetic of the
            # reference itself (sum of D squared differences, about sqrt(D) 2^-24 s) is then 1e-5 .. 5e-5 away from
            # the exact kernel sum, and no independent float32 evaluation can agree with it more closely than that.
            # Measured here in float64: the chunked scheme must be as close to the exact value as the reference is.
            x64, y64, b64 = x.astype(np.float64), y.astype(np.float64), b.astype(np.float64)
            S = ((x64 ** 2).sum(1)[:, None] + (y64 ** 2).sum(1)[None, :] - 2 * x64 @ y64.T)
            S = np.maximum(S, 0)
            near = S < 1e-3 * S.mean()
            if near.any():  # the expansion is inexact for near-coincident points: direct differences there
                ii, jj = np.nonzero(near)
                S[ii, jj] = ((x64[ii] - y64[jj]) ** 2).sum(1)
            K = np.exp(-float(g[0]) * S)
            truth, scale64 = K @ b64, K @ np.abs(b64)
            # rows whose kernel values all lie below the float32 range (exp(-90) and less) are zero on the GPU, whose
            # exp flushes denormal results, and denormal in the reference: they are compared in absolute terms
            tiny = scale64 < 1e-30
            assert np.all(np.abs(got[tiny]) <= 1e-30)
            scale64 = np.where(tiny, np.inf, scale64)
            err_ref = np.max(np.abs(ref - truth) / scale64)
            err_got = np.max(np.abs(got - truth) / scale64)
            nrm_ref, nrm_got = rel_l2(ref, truth), rel_l2(got, truth)
            assert err_got <= max(1e-5, 2 * err_ref), f"chunked scheme {err_got:.2e} vs reference arithmetic {err_ref:.2e} from the exact sum"
            assert nrm_got <= max(1e-5, 2 * nrm_ref), f"norm-wise: chunked scheme {nrm_got:.2e} vs reference arithmetic {nrm_ref:.2e}"
            print(f"width {width} D {D} clustered {clustered}: element-wise {err_got:.2e} (reference {err_ref:.2e}), "
                  f"norm-wise {nrm_got:.2e} (reference {nrm_ref:.2e}), vs oracle {np.max(np.abs(got - ref) / scale):.2e}")
    else:
        l = rng.standard_normal((N, 1)).astype(np.float32)
        lse = Genred("l-SqDist(x,y)*g", [f"x=Vi({D})", f"y=Vj({D})", "l=Vj(1)", "g=Pm(1)"], reduction_op="LogSumExp", axis=1)
        got = lse(*to_dev(x, y, l, g)).cpu().numpy()[:, 0]
        assert _scheme_used("chunk")
        ms = cpu_reduc("lse_gauss", [x, y, l, g], M, N, 2, reduction="Max_SumShiftExp")
        ref = ms[:, 0].astype(np.float64) + np.log(ms[:, 1].astype(np.float64))
        assert np.max(np.abs(got - ref) / np.maximum(1, np.abs(ref))) <= 1e-5


@pytest.mark.parametrize("case", ["huge_row", "inf_row", "nan_row", "huge_column", "inf_column", "nan_column", "large_rows"])
@pytest.mark.parametrize("formula,D", [("Exp(-SqDist(x,y))*b", 64), ("Exp(-Norm2(x-y))*b", 256)])
def test_rows_far_beyond_the_others_keep_to_themselves(formula, D, case):
    """One operand scale for the whole cloud would let a single huge (or infinite, or NaN) component spoil every other
    row.  The scale follows the bulk of the rows, and a row that then leaves the half-precision range is computed pair
    by pair from the float32 data: the result is what the reference's loops give, row by row (zero kernel values for
    infinitely distant points, NaN only where a NaN enters)."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    M, N, Dv = 3000, 4000, 4
    gen = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(M, D, device="cuda", generator=gen) / D ** 0.5
    y = torch.randn(N, D, device="cuda", generator=gen) / D ** 0.5
    b = torch.randn(N, Dv, device="cuda", generator=gen)
    value = {"huge": 1e30, "inf": float("inf"), "nan": float("nan")}.get(case.split("_")[0])
    if case == "large_rows":
        x[70:73] *= 3e4          # three rows 30 000 times the others: finite, far away, kernel values zero
        y[99] *= 1e5
    elif case.endswith("row"):
        x[77, 5] = value
    else:
        y[99, 5] = value
    al = [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"]
    got = Genred(formula, al, reduction_op="Sum", axis=1)(x, y, b)
    assert keops_io.last_loader.module.meta("scheme") == "chunk" and keops_io.last_loader.module.meta("chk_robust") == "1"
    want = Genred(formula, al, reduction_op="Sum", axis=1, enable_chunks=False)(x, y, b)
    assert torch.equal(torch.isnan(got), torch.isnan(want))
    nan_rows = int(torch.isnan(want).any(dim=1).sum())
    assert nan_rows == {"nan_row": 1, "nan_column": M}.get(case, 0)
    if nan_rows < M:
        ok = ~torch.isnan(want)
        scale = Genred(formula, al, reduction_op="Sum", axis=1, enable_chunks=False)(x, torch.nan_to_num(y), b.abs())
        err = ((got - want).abs() / scale.clamp_min(1e-30))[ok]
        assert float(err.max()) <= 1e-5
        if case in ("huge_row", "inf_row"):
            assert float(got[77].abs().max()) == 0.0
        if case == "large_rows":
            assert float(got[70:73].abs().max()) == 0.0


@pytest.mark.parametrize("case", ["row_1e4_times_larger", "huge_row", "infinite_row"])
def test_scalar_product_formulas_keep_the_other_rows_when_one_row_is_far_larger(case):
    """Scalar products have no pair-by-pair path: their operand scale lets go of the largest component only when it is
    2^20 times the bulk's (one component of 1e30 used to leave every other row a quarter wrong); a row 10 000 times the
    others is still represented, rows beyond the ratio overflow in their own results only."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    M, N, D, Dv = 3000, 4000, 64, 4
    gen = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(M, D, device="cuda", generator=gen) / 8
    y = torch.randn(N, D, device="cuda", generator=gen) / 8
    b = torch.randn(N, Dv, device="cuda", generator=gen)
    if case == "row_1e4_times_larger":
        x[77] *= 1e4
    else:
        x[77, 5] = 1e30 if case == "huge_row" else float("inf")
    al = [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"]
    others = torch.ones(M, dtype=torch.bool, device="cuda")
    others[77] = False
    for formula, red, kw in (("Exp((x|y))*b", "Sum", {}), ("(x|y)", "SumSoftMaxWeight", dict(formula2="b"))):
        got = Genred(formula, al, reduction_op=red, axis=1, **kw)(x, y, b)
        assert keops_io.last_loader.module.meta("scheme") == "chunk"
        want = Genred(formula, al, reduction_op=red, axis=1, enable_chunks=False, **kw)(x, y, b)
        assert bool(torch.isfinite(want[others]).all()) and bool(torch.isfinite(got[others]).all())
        rel = (got - want).abs().max(dim=1).values / want.abs().max(dim=1).values
        assert float(rel[others].max()) <= 1e-5
        if case == "row_1e4_times_larger" and red == "SumSoftMaxWeight":
            assert float(rel[77]) <= 1e-5      # (the shift by the row maximum keeps this row finite)


def test_results_do_not_depend_on_what_the_workspace_held_before():
    """The pre-pass (column sums, operand copies) lives in a workspace that is reused from call to call: a call must
    give the same bits on a fresh workspace and after another call of the same module has left its data there."""
    from keops_amd.torch import Genred

    gen = torch.Generator(device="cuda").manual_seed(77)
    r = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    conv = Genred("Exp(-Norm2(x-y))*b", ["x=Vi(72)", "y=Vj(72)", "b=Vj(3)"], reduction_op="Sum", axis=1)
    x, y, b = r(900, 72) / 8, r(20000, 72) / 8, r(20000, 3)
    first = conv(x, y, b).clone()
    conv(5 + r(2000, 72), 3 + r(60000, 72), r(60000, 3))   # other sizes, other data, same module and workspace
    again = conv(x, y, b)
    assert torch.equal(first, again)
    assert _scheme_used("chunk")
