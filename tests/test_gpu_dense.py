"""GPU parity of the dense map-reduce path (keops_conv_dense / keops_reduce_partials) against the
CPU oracle, through Genred -> ctypes -> libkeops_hip.  Tolerances: float32 sums 1e-5 (norm-wise and
relative to sum_j |F_ij|), float64 1e-12, index outputs bit-exact."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity, rel_l2, to_dev
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu

GAUSS = "Exp(-g*SqDist(x,y))*b"


def _gauss_inputs(M, N, Dv, seed, dtype=np.float32):
    rng = np.random.default_rng(seed)  # draw order x, y, b
    x = rng.standard_normal((M, 3)).astype(dtype)
    y = rng.standard_normal((N, 3)).astype(dtype)
    b = rng.standard_normal((N, Dv)).astype(dtype)
    return x, y, b, np.array([1.0], dtype)


def _genred_gauss(Dv, D=3, **kw):
    from keops_amd.torch import Genred

    return Genred(GAUSS, [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})", "g=Pm(1)"], reduction_op="Sum", axis=1, **kw)


def test_config1_gaussian_10k_full_parity():
    # headline configuration 1: M=N=10,000, D=3, float32, seed 0
    M = N = 10000
    x, y, b, g = _gauss_inputs(M, N, 1, 0)
    got = _genred_gauss(1)(*to_dev(x, y, b, g)).cpu().numpy()
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 1)
    assert_sum_parity(got, ref, scale)


@pytest.mark.parametrize("M,N", [(1, 1), (1, 777), (777, 1), (255, 1025), (1030, 2049), (4099, 513)])
@pytest.mark.parametrize("Dv", [1, 3])
def test_ragged_sizes(M, N, Dv):
    x, y, b, g = _gauss_inputs(M, N, Dv, 11)
    got = _genred_gauss(Dv)(*to_dev(x, y, b, g)).cpu().numpy()
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv)
    assert_sum_parity(got, ref, scale)


@pytest.mark.parametrize("Dv", [1, 8])
def test_config2_gaussian_1M_row_subset(Dv):
    # headline configuration 2: M=N=1,000,000, seed 1; oracle on 2048 random rows (rows are independent)
    M = N = 1_000_000
    x, y, b, g = _gauss_inputs(M, N, Dv, 1)
    got = _genred_gauss(Dv)(*to_dev(x, y, b, g))
    rows = np.sort(np.random.default_rng(123).choice(M, 2048, replace=False)).astype(np.int64)
    # ... and the 128 rows farthest from the centre of the cloud: the exponents that the matrix cores produce are least
    # accurate where the norms are largest
    far = np.argsort(-(x.astype(np.float64) ** 2).sum(1))[:128]
    rows = np.unique(np.concatenate([rows, far])).astype(np.int64)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    # size-independent property at full size: linearity in b (doubling b doubles the result exactly)
    xd, yd, bd, gd = to_dev(x, y, b, g)
    twice = _genred_gauss(Dv)(xd, yd, 2 * bd, gd)
    assert torch.equal(twice, 2 * got)


def test_config2_gradient_wrt_x_row_subset():
    M = N = 1_000_000
    x, y, b, g = _gauss_inputs(M, N, 1, 1)
    xd, yd, bd, gd = to_dev(x, y, b, g)
    xd.requires_grad_(True)
    a = _genred_gauss(1)(xd, yd, bd, gd)
    (gx,) = torch.autograd.grad(a.sum(), [xd])  # G = ones
    rows = np.sort(np.random.default_rng(321).choice(M, 2048, replace=False)).astype(np.int64)
    G = np.ones((M, 1), np.float32)
    ref = cpu_reduc("gauss_gradx", [x, y, b, g, G], M, N, 3, rows=rows)
    scale = cpu_reduc("gauss_gradx_abs", [x, y, b, g, G], M, N, 3, rows=rows)  # sum_j |2 g K_ij b_j (x_i - y_j)|
    got = gx[torch.from_numpy(rows).cuda()].cpu().numpy()
    assert_sum_parity(got, ref, scale)


def test_gradients_small_all_variables():
    M, N, Dv = 500, 700, 2
    x, y, b, g = _gauss_inputs(M, N, Dv, 5, np.float64)
    td = [t.requires_grad_(True) for t in to_dev(x, y, b, g)]
    a = _genred_gauss(Dv)(*td)
    E = torch.from_numpy(np.random.default_rng(1).standard_normal((M, Dv))).cuda()
    grads = torch.autograd.grad((a * E).sum(), td)
    xt, yt, bt, gt = [t.detach().clone().requires_grad_(True) for t in td]
    K = torch.exp(-gt * ((xt[:, None] - yt[None]) ** 2).sum(-1))
    ref = torch.autograd.grad(((K @ bt) * E).sum(), [xt, yt, bt, gt])
    for got_k, ref_k in zip(grads, ref):
        assert got_k.shape == ref_k.shape
        assert rel_l2(got_k.cpu().numpy(), ref_k.cpu().numpy()) < 1e-12


def test_float64_and_double_accumulation():
    M, N = 2000, 3000
    x, y, b, g = _gauss_inputs(M, N, 1, 7, np.float64)
    got = _genred_gauss(1)(*to_dev(x, y, b, g)).cpu().numpy()
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1, dtype=np.float64)
    assert rel_l2(got, ref) <= 1e-12
    x, y, b, g = (t.astype(np.float32) for t in (x, y, b, g))
    got = _genred_gauss(1, dtype_acc="float64")(*to_dev(x, y, b, g)).cpu().numpy()
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1, acc_double=True)
    # per-pair values use the hardware exp2: the float32 floor (~1e-6), not 1e-12, is reachable here
    assert rel_l2(got, ref) <= 5e-6


@pytest.mark.parametrize("scheme", ["direct_sum", "block_sum", "kahan_scheme"])
def test_sum_schemes(scheme):
    M, N = 1500, 40000
    x, y, b, g = _gauss_inputs(M, N, 2, 9)
    got = _genred_gauss(2, sum_scheme=scheme)(*to_dev(x, y, b, g)).cpu().numpy()
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 2, scheme=scheme)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 2)
    # direct_sum: the oracle adds a row's 40 000 terms one after the other in float32, the kernel adds them in column
    # slabs and tiles; two orders of an uncompensated float32 sum of that length differ by about sqrt(N) 2^-24 = 1.2e-5
    # of sum |F_ij| whatever the kernel does, so the bar for this scheme is the sum's own accuracy
    assert_sum_parity(got, ref, scale, tol=1e-5 if scheme != "direct_sum" else 5e-5)


def test_no_fast_math_matches_libm_closely():
    M, N = 800, 900
    x, y, b, g = _gauss_inputs(M, N, 1, 13)
    got = _genred_gauss(1, use_fast_math=False)(*to_dev(x, y, b, g)).cpu().numpy()
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1)
    assert rel_l2(got, ref) <= 2e-6


def test_denormal_kernel_values_are_flushed_with_fast_math_and_kept_without():
    """exp(-d^2) for d = 9.4 ... 10: values of 4e-39 ... 4e-44, below the smallest normal float32.  v_exp_f32 returns
    zero there, as the reference's GPU build does under its default -use_fast_math (which implies -ftz=true,
    keopscore/binders/nvrtc/nvrtc_jit.cpp:87-88); use_fast_math=False calls the library exponential."""
    x = torch.zeros(4, 1, device="cuda")
    y = torch.tensor([[9.4], [9.6], [9.8], [10.0]], device="cuda")
    b, g = torch.ones(4, 1, device="cuda"), torch.tensor([1.0], device="cuda")
    truth = float(torch.exp(-(y.double() ** 2)).sum())
    assert 4e-39 < truth < 5e-39
    fast = _genred_gauss(1, D=1)(x, y, b, g)
    assert float(fast.abs().max()) == 0.0
    kept = _genred_gauss(1, D=1, use_fast_math=False)(x, y, b, g)
    assert abs(float(kept[0]) - truth) <= 1e-5 * truth + 2e-45      # one unit of the denormal grid


@pytest.mark.parametrize("backend", ["GPU_1D", "GPU_2D", "GPU"])
def test_backends_1d_2d(backend):
    # small M, long N: the column-slab scheme (the reference's GpuReduc2D) must agree with 1D
    M, N = 300, 200000
    x, y, b, g = _gauss_inputs(M, N, 1, 17)
    got = _genred_gauss(1)(*to_dev(x, y, b, g), backend=backend).cpu().numpy()
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 1)
    assert_sum_parity(got, ref, scale)


def test_axis0_reduction_over_i():
    from keops_amd.torch import Genred

    M, N = 1200, 900
    rng = np.random.default_rng(19)
    x, y = rng.standard_normal((M, 3)).astype(np.float32), rng.standard_normal((N, 3)).astype(np.float32)
    a = rng.standard_normal((M, 2)).astype(np.float32)
    g = np.array([0.5], np.float32)
    conv = Genred("Exp(-g*SqDist(x,y))*a", ["x=Vi(3)", "y=Vj(3)", "a=Vi(2)", "g=Pm(1)"], reduction_op="Sum", axis=0)
    got = conv(*to_dev(x, y, a, g)).cpu().numpy()
    assert got.shape == (N, 2)
    ref = cpu_reduc("gauss", [y, x, a, g], N, M, 2)  # roles of i and j exchanged
    scale = cpu_reduc("gauss", [y, x, np.abs(a), g], N, M, 2)
    assert_sum_parity(got, ref, scale)


def test_out_argument_and_errors():
    from keops_amd.torch import Genred

    M, N = 100, 50
    x, y, b, g = _gauss_inputs(M, N, 1, 23)
    xd, yd, bd, gd = to_dev(x, y, b, g)
    out = torch.empty(M, 1, device="cuda")
    res = _genred_gauss(1)(xd, yd, bd, gd, out=out)
    assert res.data_ptr() == out.data_ptr()
    with pytest.raises(ValueError):
        _genred_gauss(1)(xd, yd, bd)  # wrong number of arguments
    with pytest.raises(ValueError):
        _genred_gauss(1)(xd, yd, bd, gd, backend="TPU")
    with pytest.raises(Exception):
        _genred_gauss(1)(xd, yd[:, :2].contiguous(), bd, gd)  # wrong vector size is caught natively
    with pytest.raises(ValueError):
        Genred("Exp(x", ["x=Vi(3)"])(xd)
    with pytest.raises(ValueError):
        _genred_gauss(1)(xd, yd, bd, gd, backend="CPU")  # there is no CPU implementation behind this API
