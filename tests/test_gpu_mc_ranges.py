"""GPU parity of the block-sparse and batched variants of the matrix-core schemes (keops_chk_main,
keops_chk_final, keops_chk_softmax, keops_fin_main built with KEOPS_MC_RANGES), the counterparts of the
reference's GpuReduc1D_ranges_chunks.py and GpuReduc1D_ranges_finalchunks.py.  References are dense float64
torch computations with the same block mask / batch broadcasting."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity, to_dev

pytestmark = pytest.mark.gpu


def _used(**want):
    from keops_amd import keops_io

    return any(all(m.meta(k) == v for k, v in want.items()) for m in keops_io._modules.values())


def _block_ranges(M, N, seed):
    """Irregular row ranges (one longer than a workgroup's 256 rows, one of 5 rows, an uncovered gap) with one to
    three reduced-index ranges each, some adjacent (merged by the kernel); returns the 6-tuple and the dense mask."""
    rng = np.random.default_rng(seed)
    ranges_i = np.array([[0, 5], [5, 400], [400, 1000], [M - 300, M]], np.int64)
    red, slices = [], []
    jcuts = np.sort(rng.choice(np.arange(1, N), 7, replace=False))
    segs = [(0, int(jcuts[0]))] + [(int(jcuts[k]), int(jcuts[k + 1])) for k in range(6)] + [(int(jcuts[6]), N)]
    pick = [[0, 1], [3], [2, 3, 6], [7]]                    # [0,1] and [2,3] are adjacent pairs
    for p in pick:
        red += [segs[k] for k in p]
        slices.append(len(red))
    mask = np.zeros((M, N), bool)
    for (a, b), p in zip(ranges_i, pick):
        for k in p:
            mask[a:b, segs[k][0]:segs[k][1]] = True
    dummy = np.zeros((1, 2), np.int64)
    tup = (ranges_i, np.array(slices, np.int64), np.array(red, np.int64), dummy, np.array([0], np.int64), dummy)
    return tuple(torch.from_numpy(t).cuda() for t in tup), torch.from_numpy(mask)


def test_block_sparse_chunked_sum_final_and_softmax():
    from keops_amd.torch import Genred

    M, N, D, Dv = 1500, 2300, 64, 40
    rng = np.random.default_rng(41)
    x = (rng.standard_normal((M, D)) / D ** 0.25).astype(np.float32)
    y = (rng.standard_normal((N, D)) / D ** 0.25).astype(np.float32)
    b = rng.standard_normal((N, Dv)).astype(np.float32)
    xd, yd, bd = to_dev(x, y, b)
    ranges, mask = _block_ranges(M, N, 7)
    x64, y64, b64 = (torch.from_numpy(t).double() for t in (x, y, b))
    K = torch.exp(-torch.cdist(x64, y64)) * mask
    uncovered = ~mask.any(1)
    assert uncovered.any()

    # post-chunk formula g(s) * v: weighted sum on the matrix cores
    conv = Genred("Exp(-Norm2(x-y))*b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"], reduction_op="Sum", axis=1)
    got = conv(xd, yd, bd, ranges=ranges).cpu()
    assert _used(scheme="chunk", chk_final="1", ranges="1")
    assert_sum_parity(got.numpy(), (K @ b64).numpy(), (K @ b64.abs()).numpy() + 1e-30)
    assert torch.all(got[uncovered] == 0)

    # generic post-chunk formula, per-lane accumulation
    conv2 = Genred("Exp(-Norm2(x-y))*b+b", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})"], reduction_op="Sum", axis=1)
    got2 = conv2(xd, yd, bd, ranges=ranges).cpu()
    assert _used(scheme="chunk", chk_final="0", chk_softmax="0", ranges="1")
    m64 = mask.double()
    assert_sum_parity(got2.numpy(), (K @ b64 + m64 @ b64).numpy(), (K @ b64.abs() + m64 @ b64.abs()).numpy() + 1e-30)

    # log-sum-exp of a scaled inner product over the kept blocks; rows without any block give -inf
    lse = Genred("p*(x|y)", [f"x=Vi({D})", f"y=Vj({D})", "p=Pm(1)"], reduction_op="LogSumExp", axis=1)
    p = torch.tensor([0.7], device="cuda")
    gl = lse(xd, yd, p, ranges=ranges).cpu().double()[:, 0]
    S = (0.7 * x64 @ y64.T).masked_fill(~mask, -float("inf"))
    refl = torch.logsumexp(S, dim=1)
    assert torch.all(torch.isneginf(gl[uncovered]))
    assert float((gl[~uncovered] - refl[~uncovered]).abs().max()) <= 2e-5 * float(refl[~uncovered].abs().max())

    # softmax-weighted sum (attention restricted to the kept blocks)
    att = Genred("p*(x|y)", [f"x=Vi({D})", f"y=Vj({D})", f"b=Vj({Dv})", "p=Pm(1)"], reduction_op="SumSoftMaxWeight", axis=1,
                 formula2="b")
    ga = att(xd, yd, bd, p, ranges=ranges).cpu().double()
    assert _used(scheme="chunk", chk_softmax="1", ranges="1")
    refa = torch.softmax(S[~uncovered], dim=1) @ b64
    assert float((ga[~uncovered] - refa).abs().max()) <= 2e-5 * float(refa.abs().max())


def test_block_sparse_final_product_scheme():
    from keops_amd.torch import Genred

    M, N, Dv = 1500, 2300, 96
    rng = np.random.default_rng(42)
    x = rng.standard_normal((M, 3)).astype(np.float32)
    y = rng.standard_normal((N, 3)).astype(np.float32)
    b = rng.standard_normal((N, Dv)).astype(np.float32)
    g = np.array([0.75], np.float32)
    ranges, mask = _block_ranges(M, N, 8)
    conv = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", f"b=Vj({Dv})", "g=Pm(1)"], reduction_op="Sum", axis=1)
    got = conv(*to_dev(x, y, b, g), ranges=ranges).cpu()
    assert _used(scheme="final", ranges="1")
    x64, y64, b64 = (torch.from_numpy(t).double() for t in (x, y, b))
    K = torch.exp(-0.75 * torch.cdist(x64, y64) ** 2) * mask
    assert_sum_parity(got.numpy(), (K @ b64).numpy(), (K @ b64.abs()).numpy() + 1e-30)
    assert torch.all(got[~mask.any(1)] == 0)


@pytest.mark.parametrize("axis", [1, 0])
def test_batched_attention_with_broadcast_batch_dimensions(axis):
    """(B, H, M, D) queries against keys shared by the heads ((B, 1, N, D)) and per-head values: softmax-weighted
    sum, the plain Gaussian-like final product and a log-sum-exp, all with two batch dimensions."""
    from keops_amd.torch import LazyTensor

    B, H, M, N, D, Dv = 2, 3, 300, 420, 64, 32
    gen = torch.Generator().manual_seed(5)
    q = torch.randn(B, H, M, D, generator=gen) / D ** 0.25
    k = torch.randn(B, 1, N, D, generator=gen) / D ** 0.25
    v = torch.randn(B, H, (N if axis == 1 else M), Dv, generator=gen)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    q_i, k_j = LazyTensor(qd[:, :, :, None, :]), LazyTensor(kd[:, :, None, :, :])
    v_l = LazyTensor(vd[:, :, None, :, :] if axis == 1 else vd[:, :, :, None, :])
    S_ij = (q_i * k_j).sum(-1)
    got = S_ij.sumsoftmaxweight(v_l, dim=3 if axis == 1 else 2).cpu().double()
    assert _used(scheme="chunk", chk_softmax="1", ranges="1")
    S = q.double() @ k.double().transpose(-1, -2)           # (B, H, M, N)
    if axis == 0:
        S = S.transpose(-1, -2)
    ref = torch.softmax(S, dim=-1) @ v.double()
    assert got.shape == ref.shape
    assert float((got - ref).abs().max()) <= 2e-5 * float(ref.abs().max())
    # weighted kernel sum exp(S) v on the same operands (final-product variant of the chunked scheme)
    got2 = (S_ij.exp() * v_l).sum(dim=3 if axis == 1 else 2).cpu().double()
    assert _used(scheme="chunk", chk_final="1", ranges="1")
    E = torch.exp(S)
    assert_sum_parity(got2.numpy(), (E @ v.double()).numpy(), (E @ v.double().abs()).numpy())
    # log-sum-exp (per-lane accumulation variant)
    got3 = S_ij.logsumexp(dim=3 if axis == 1 else 2).cpu().double()[..., 0]
    ref3 = torch.logsumexp(S, dim=-1)
    assert float((got3 - ref3).abs().max()) <= 2e-5 * float(ref3.abs().max())


def test_batched_gaussian_times_highdim_variable():
    from keops_amd.torch import LazyTensor

    B, M, N, Dv = 5, 700, 333, 128
    gen = torch.Generator().manual_seed(6)
    x, y, b = torch.randn(B, M, 3, generator=gen), torch.randn(1, N, 3, generator=gen), torch.randn(B, N, Dv, generator=gen)
    xd, yd, bd = x.cuda(), y.cuda(), b.cuda()
    K_ij = (-0.75 * ((LazyTensor(xd[:, :, None, :]) - LazyTensor(yd[:, None, :, :])) ** 2).sum(-1)).exp()
    got = (K_ij * LazyTensor(bd[:, None, :, :])).sum(dim=2).cpu()
    assert _used(scheme="final", ranges="1")
    K = torch.exp(-0.75 * torch.cdist(x.double(), y.double().expand(B, N, 3)) ** 2)
    assert_sum_parity(got.numpy(), (K @ b.double()).numpy(), (K @ b.double().abs()).numpy())
    # gradient with respect to the batched high-dimensional variable: final product over the other index
    bd.requires_grad_(True)
    out = (K_ij * LazyTensor(bd[:, None, :, :])).sum(dim=2)
    e = torch.randn(B, M, Dv, generator=gen)
    (gb,) = torch.autograd.grad(out, [bd], e.cuda())
    assert_sum_parity(gb.cpu().numpy(), (K.transpose(1, 2) @ e.double()).numpy(), (K.transpose(1, 2) @ e.double().abs()).numpy())
