"""GPU parity of the matrix-core final-product scheme (keops_final_mfma.h): Sum_j f(x_i,y_j) * v_j with
a high-dimensional v.  The scheme is only a schedule, so the result must equal the plain reduction, cf.
the reference's pykeops/test/test_finalchunks.py (Gaussian kernel times a 500-dimensional variable,
compared with the dense torch formula)."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity, to_dev
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu

FORMULA = "Exp(-g*SqDist(x,y))*b"


def _inputs(M, N, Dv, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, 3)).astype(np.float32)
    y = rng.standard_normal((N, 3)).astype(np.float32)
    b = rng.standard_normal((N, Dv)).astype(np.float32)
    g = np.array([0.75], np.float32)
    return x, y, b, g


def _scheme_used(name):
    from keops_amd import keops_io

    return any(m.meta("scheme") == name for m in keops_io._modules.values())


def _aliases(Dv):
    return ["x=Vi(3)", "y=Vj(3)", f"b=Vj({Dv})", "g=Pm(1)"]


@pytest.mark.parametrize("M,N,Dv,scheme", [
    (1000, 3000, 256, "block_sum"),     # few output rows: slabs over the reduced axis + ordered sum
    (777, 1001, 200, "block_sum"),      # ragged last column block, ragged last tile
    (333, 2500, 300, "direct_sum"),     # more column blocks than one wavefront keeps: two workgroups per row block
    (70, 50, 24, "block_sum"),          # smallest dimension that selects the scheme, less than one tile pair
    (256, 20000, 96, "block_sum"),      # several block-sum periods
])
def test_gaussian_times_highdim_vs_oracle(M, N, Dv, scheme):
    from keops_amd.torch import Genred

    x, y, b, g = _inputs(M, N, Dv, 11)
    conv = Genred(FORMULA, _aliases(Dv), reduction_op="Sum", axis=1, sum_scheme=scheme)
    got = conv(*to_dev(x, y, b, g)).cpu().numpy()
    assert _scheme_used("final")
    assert got.shape == (M, Dv)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv)
    assert_sum_parity(got, ref, scale)
    # independent pin: float64 closed form
    x64, y64, b64 = (torch.from_numpy(t).double() for t in (x, y, b))
    K = torch.exp(-0.75 * torch.cdist(x64, y64) ** 2)
    assert_sum_parity(got, (K @ b64).numpy(), (K @ b64.abs()).numpy())


def test_large_rows_subset_and_exact_linearity():
    # enough rows for one slab; rows are independent, so a random subset is compared with the oracle
    from keops_amd.torch import Genred

    M, N, Dv = 60_000, 4_000, 128
    x, y, b, g = _inputs(M, N, Dv, 12)
    conv = Genred(FORMULA, _aliases(Dv), reduction_op="Sum", axis=1)
    xd, yd, bd, gd = to_dev(x, y, b, g)
    got = conv(xd, yd, bd, gd)
    rows = np.sort(np.random.default_rng(3).choice(M, 256, replace=False)).astype(np.int64)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, Dv, rows=rows)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, Dv, rows=rows)
    assert_sum_parity(got[torch.from_numpy(rows).cuda()].cpu().numpy(), ref, scale)
    assert torch.equal(conv(xd, yd, 2 * bd, gd), 2 * got)  # scaling v by a power of two is exact
    assert torch.equal(conv(xd, yd, bd, gd), got)          # and the result is reproducible bit for bit


def test_long_all_positive_sums_stay_in_the_float32_class():
    # 400 000 reduced rows, every term positive: the accumulation error cannot cancel, and a slab of the reduced
    # axis spans several periods of the fold of the register tiles into the slab's partial sum
    from keops_amd.torch import Genred

    M, N, Dv = 4096, 400_000, 64
    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.rand(M, 3, device="cuda", generator=gen)
    y = torch.rand(N, 3, device="cuda", generator=gen)
    b = torch.rand(N, Dv, device="cuda", generator=gen) + 0.5
    g = torch.tensor([0.5], device="cuda")
    got = Genred(FORMULA, _aliases(Dv), reduction_op="Sum", axis=1)(x, y, b, g)
    assert _scheme_used("final")
    rows = torch.arange(0, M, 16, device="cuda")
    ref = torch.exp(-0.5 * torch.cdist(x[rows].double(), y.double()) ** 2) @ b.double()
    rel = ((got[rows].double() - ref).abs() / ref).max().item()
    assert rel <= 1e-5, rel          # measured 1.1e-6


@pytest.mark.parametrize("kw", [dict(dtype_acc="float64"), dict(sum_scheme="kahan_scheme")])
def test_sums_kept_in_double(kw):
    """dtype_acc = float64 and the Kahan scheme stay on the matrix cores: the register tiles are folded into double
    sums every 1024 reduced rows (sum_schemes.py:44-71 with a double accumulator).  An all-positive sum over 400 000
    rows shows the gain: 1.1e-6 with float32 folds, the float32 class of the pair values themselves here."""
    from keops_amd import keops_io
    from keops_amd.torch import Genred

    M, N, Dv = 2048, 400_000, 64
    gen = torch.Generator(device="cuda").manual_seed(2)
    x = torch.rand(M, 3, device="cuda", generator=gen)
    y = torch.rand(N, 3, device="cuda", generator=gen)
    b = torch.rand(N, Dv, device="cuda", generator=gen) + 0.5
    g = torch.tensor([0.5], device="cuda")
    got = Genred(FORMULA, _aliases(Dv), reduction_op="Sum", axis=1, **kw)(x, y, b, g)
    assert keops_io.last_loader.module.meta("scheme") == "final" and keops_io.last_loader.module.meta("fin_acc64") == "1"
    rows = torch.arange(0, M, 8, device="cuda")
    ref = torch.exp(-0.5 * torch.cdist(x[rows].double(), y.double()) ** 2) @ b.double()
    rel = ((got[rows].double() - ref).abs() / ref).max().item()
    assert rel <= 3e-7, rel
    # signed weights, ragged sizes, against the oracle's double accumulation
    M, N, Dv = 777, 5001, 200
    xs, ys, bs, gs = _inputs(M, N, Dv, 21)
    out = Genred(FORMULA, _aliases(Dv), reduction_op="Sum", axis=1, **kw)(*to_dev(xs, ys, bs, gs)).cpu().numpy()
    ref = cpu_reduc("gauss", [xs, ys, bs, gs], M, N, Dv, acc_double=True)
    scale = cpu_reduc("gauss", [xs, ys, np.abs(bs), gs], M, N, Dv, acc_double=True)
    assert_sum_parity(out, ref, scale, tol=2e-6)


def test_axis0_gpu2d_and_gradient():
    from keops_amd.torch import Genred

    M, N, Dv = 500, 640, 160
    rng = np.random.default_rng(13)
    x = rng.standard_normal((M, 3)).astype(np.float32)
    y = rng.standard_normal((N, 3)).astype(np.float32)
    a = rng.standard_normal((M, Dv)).astype(np.float32)
    g = np.array([0.5], np.float32)
    x64, y64, a64 = (torch.from_numpy(t).double() for t in (x, y, a))
    K = torch.exp(-0.5 * torch.cdist(x64, y64) ** 2)
    # reduction over i: the high-dimensional variable is indexed by i, the output by j
    conv = Genred("a*Exp(-g*SqDist(x,y))", ["x=Vi(3)", "y=Vj(3)", f"a=Vi({Dv})", "g=Pm(1)"], reduction_op="Sum", axis=0)
    xd, yd, ad, gd = to_dev(x, y, a, g)
    got = conv(xd, yd, ad, gd, backend="GPU_2D").cpu().numpy()
    assert_sum_parity(got, (K.T @ a64).numpy(), (K.T @ a64.abs()).numpy())
    # gradient with respect to the high-dimensional variable is again a final product (over the other index)
    b = rng.standard_normal((N, Dv)).astype(np.float32)
    bd = torch.from_numpy(b).cuda().requires_grad_(True)
    conv1 = Genred(FORMULA, _aliases(Dv), reduction_op="Sum", axis=1)
    out = conv1(xd, yd, bd, gd)
    e = torch.from_numpy(rng.standard_normal((M, Dv)).astype(np.float32)).cuda()
    (gb,) = torch.autograd.grad(out, [bd], e)
    e64 = e.cpu().double()
    assert_sum_parity(gb.cpu().numpy(), (K.T @ e64).numpy(), (K.T @ e64.abs()).numpy())


def test_lazytensor_front_end_and_fallbacks():
    from keops_amd.torch import Genred, LazyTensor

    M, N, Dv = 300, 400, 192
    x, y, b, g = _inputs(M, N, Dv, 14)
    xd, yd, bd, gd = to_dev(x, y, b, g)
    x_i, y_j, b_j = LazyTensor(xd[:, None, :]), LazyTensor(yd[None, :, :]), LazyTensor(bd[None, :, :])
    got = ((-0.75 * ((x_i - y_j) ** 2).sum(-1)).exp() * b_j).sum(dim=1)
    x64, y64, b64 = (torch.from_numpy(t).double() for t in (x, y, b))
    K = torch.exp(-0.75 * torch.cdist(x64, y64) ** 2)
    assert_sum_parity(got.cpu().numpy(), (K @ b64).numpy(), (K @ b64.abs()).numpy())
    # float64 data are served by the generic kernel, Kahan summation by double sums on the matrix cores: same function
    conv64 = Genred(FORMULA, _aliases(Dv), reduction_op="Sum", axis=1)
    got64 = conv64(xd.double(), yd.double(), bd.double(), gd.double()).cpu().numpy()
    assert np.max(np.abs(got64 - (torch.exp(-0.75 * torch.cdist(xd.double().cpu(), yd.double().cpu()) ** 2) @ b64).numpy())) < 1e-10
    kahan = Genred(FORMULA, _aliases(Dv), reduction_op="Sum", axis=1, sum_scheme="kahan_scheme")(xd, yd, bd, gd)
    assert_sum_parity(kahan.cpu().numpy(), (K @ b64).numpy(), (K @ b64.abs()).numpy())


def test_batches_and_ranges_that_start_inside_a_tile_of_the_split_copy():
    """The staged tiles are cut along the array v from multiples of 32 rows on; a batch of 333 rows or a range
    [77, 1201) starts and ends inside such a tile, and a broadcast batch dimension of v moves the tiles of a batch
    without moving its rows of y."""
    from keops_amd.torch import LazyTensor

    gen = torch.Generator().manual_seed(31)
    B, H, M, N, Dv = 2, 3, 210, 333, 40
    x = torch.randn(B, H, M, 3, generator=gen)
    y = torch.randn(B, H, N, 3, generator=gen)
    v = torch.randn(B, 1, N, Dv, generator=gen)                      # shared by the second batch dimension
    x_i, y_j = LazyTensor(x.cuda()[:, :, :, None, :]), LazyTensor(y.cuda()[:, :, None, :, :])
    v_j = LazyTensor(v.cuda()[:, :, None, :, :])
    got = ((-((x_i - y_j) ** 2).sum(-1)).exp() * v_j).sum(dim=3).cpu()
    assert _scheme_used("final")
    K = torch.exp(-torch.cdist(x.double(), y.double()) ** 2)
    assert_sum_parity(got.numpy(), (K @ v.double()).numpy(), (K @ v.double().abs()).numpy())
    # block-sparse: three row ranges, reduced ranges with odd ends, some of them adjacent
    from keops_amd.torch import Genred

    M, N, Dv = 700, 1500, 72
    xs, ys, bs, gs = _inputs(M, N, Dv, 32)
    ranges_i = torch.tensor([[0, 130], [130, 450], [450, 700]], dtype=torch.int32)
    slices_i = torch.tensor([2, 3, 5], dtype=torch.int32)
    ranges_j = torch.tensor([[77, 500], [500, 1201], [3, 29], [1000, 1033], [1299, 1500]], dtype=torch.int32)
    ranges = (ranges_i, slices_i, ranges_j, ranges_j, torch.tensor([1, 2, 3, 4, 5], dtype=torch.int32),
              torch.tensor([[0, 130], [0, 130], [130, 450], [450, 700], [450, 700]], dtype=torch.int32))
    out = Genred(FORMULA, _aliases(Dv), reduction_op="Sum", axis=1)(*to_dev(xs, ys, bs, gs), ranges=ranges).cpu().numpy()
    mask = torch.zeros(M, N, dtype=torch.float64)
    mask[0:130, 77:1201] = 1
    mask[130:450, 3:29] = 1
    mask[450:700, 1000:1033] = 1
    mask[450:700, 1299:1500] = 1
    x64, y64, b64 = (torch.from_numpy(t).double() for t in (xs, ys, bs))
    K = torch.exp(-0.75 * torch.cdist(x64, y64) ** 2) * mask
    assert_sum_parity(out, (K @ b64).numpy(), (K @ b64.abs()).numpy())
