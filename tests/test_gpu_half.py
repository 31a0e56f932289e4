"""Half-precision data (use_half of the C ABI; pykeops/pykeops/torch/half2_convert.py in the reference): arguments and
result are float16 tensors, the kernels compute in float32 on converted copies and round the result once.  The
expected value is therefore the float32 result of the same call on the (exactly representable) upcast data, rounded
to half: bit-exact; the CPU oracle is the checker for that float32 result."""
import numpy as np
import pytest
import torch

from common import assert_sum_parity
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu


def test_gaussian_sum_in_half_precision_vs_oracle():
    from keops_amd.torch import Genred

    rng = np.random.default_rng(0)
    M, N = 3000, 4000
    x = rng.standard_normal((M, 3)).astype(np.float16)
    y = rng.standard_normal((N, 3)).astype(np.float16)
    b = rng.standard_normal((N, 2)).astype(np.float16)
    g = np.array([0.5], np.float16)
    conv = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)", "g=Pm(1)"], reduction_op="Sum", axis=1)
    dev = [torch.from_numpy(a).cuda() for a in (x, y, b, g)]
    got = conv(*dev)
    assert got.dtype == torch.float16 and got.shape == (M, 2)
    up = [a.astype(np.float32) for a in (x, y, b, g)]
    ref = cpu_reduc("gauss", up, M, N, 2)
    scale = cpu_reduc("gauss", [up[0], up[1], np.abs(up[2]), up[3]], M, N, 2)
    # the float32 result behind the rounding meets the usual bar; the rounding to half adds 2^-11 relative
    f32 = conv(*[d.float() for d in dev])
    assert_sum_parity(f32.cpu().numpy(), ref, scale)
    assert torch.equal(got, f32.half())
    # host tensors and numpy arrays are staged through the device
    assert torch.equal(conv(*[d.cpu() for d in dev]), got.cpu())
    from keops_amd.numpy import Genred as NpGenred

    npconv = NpGenred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)", "g=Pm(1)"], reduction_op="Sum", axis=1)
    assert np.array_equal(npconv(x, y, b, g), got.cpu().numpy())


def test_half_precision_other_schemes_and_gradients():
    from keops_amd import keops_io
    from keops_amd.torch import Genred, LazyTensor

    gen = torch.Generator(device="cuda").manual_seed(1)
    r = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    # chunked matrix-core scheme (D = 64), log-sum-exp, K nearest neighbours, batch dimensions
    x, y, b = (r(2000, 64) / 8).half(), (r(2500, 64) / 8).half(), r(2500, 4).half()
    lap = Genred("Exp(-Norm2(x-y))*b", ["x=Vi(64)", "y=Vj(64)", "b=Vj(4)"], reduction_op="Sum", axis=1)
    got = lap(x, y, b)
    assert keops_io.last_loader.module.meta("scheme") == "chunk"
    # half-precision numbers multiply exactly in float32: the contraction keeps one term per component (one matrix
    # instruction per block instead of three, no centring); the float32 result behind the final rounding is as
    # good as the two-term one of float32 data
    assert keops_io.last_loader.module.meta("chk_single") == "1"
    K = torch.exp(-torch.cdist(x.double(), y.double()))
    ref, scale = K @ b.double(), K @ b.double().abs()
    assert float(((got.double() - ref).abs() / scale).max()) < 6e-4          # the rounding of the result to half
    f32 = lap(x.float(), y.float(), b.float())
    assert keops_io.last_loader.module.meta("chk_single") == "0"
    assert float(((f32.double() - ref).abs() / scale).max()) < 1e-5
    # scalar products of half data, and data far from the origin (uncentred norms, near-pair recomputation)
    lin = Genred("(x|y)*b", ["x=Vi(64)", "y=Vj(64)", "b=Vj(4)"], reduction_op="Sum", axis=1)
    refl, scl = (x.double() @ y.double().T) @ b.double(), (x.double() @ y.double().T).abs() @ b.double().abs()
    assert float(((lin(x, y, b).double() - refl).abs() / scl).max()) < 6e-4
    xo, yo = (x.float() + 3.0).half(), (y.float() + 3.0).half()
    Ko = torch.exp(-torch.cdist(xo.double(), yo.double()))
    assert float(((lap(xo, yo, b).double() - Ko @ b.double()).abs() / (Ko @ b.double().abs())).max()) < 6e-4
    lse = Genred("-SqDist(x,y)", ["x=Vi(64)", "y=Vj(64)"], reduction_op="LogSumExp", axis=1)
    # (the kernel returns the pair (max, sum of shifted exponentials), which is rounded to half before the layer above
    # takes the logarithm, as in the reference: close, not bit-equal)
    assert float((lse(x, y).float() - lse(x.float(), y.float())).abs().max()) < 8e-3
    knn = Genred("SqDist(x,y)", ["x=Vi(64)", "y=Vj(64)"], reduction_op="ArgKMin", axis=1, opt_arg=5)
    # (indices come back as half-precision numbers, exact up to 2048 only: as in the reference)
    assert torch.equal(knn(x, y[:2000].contiguous()), knn(x.float(), y[:2000].float().contiguous()))
    xb, yb, bb = r(3, 500, 3).half(), r(3, 700, 3).half(), r(3, 700, 1).half()
    d = ((LazyTensor(xb[:, :, None, :]) - LazyTensor(yb[:, None, :, :])) ** 2).sum(-1)
    out = ((-d).exp() * LazyTensor(bb[:, None, :, :])).sum(2)
    K = torch.exp(-torch.cdist(xb.double(), yb.double()) ** 2)
    assert out.dtype == torch.float16
    assert float((out.double() - K @ bb.double()).abs().max() / (K @ bb.double()).abs().max()) < 2e-3
    # autograd: gradients are half tensors, equal to the rounded float32 gradients
    xs = (r(300, 3)).half().requires_grad_(True)
    ys, bs = r(400, 3).half(), r(400, 1).half()
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(1)"], reduction_op="Sum", axis=1)
    e = r(300, 1).half()
    (gx,) = torch.autograd.grad(conv(xs, ys, bs), xs, e)
    xf = xs.detach().float().requires_grad_(True)
    (gf,) = torch.autograd.grad(conv(xf, ys.float(), bs.float()), xf, e.float())
    assert gx.dtype == torch.float16
    assert float((gx.float() - gf).abs().max()) <= 2e-3 * float(gf.abs().max())


def test_use_half_through_the_abi_refuses_what_it_cannot_serve():
    from keops_amd import binder, keops_io
    from keops_amd.torch import Genred

    x = torch.randn(100, 3, device="cuda", dtype=torch.float64)
    y = torch.randn(120, 3, device="cuda", dtype=torch.float64)
    conv = Genred("Exp(-SqDist(x,y))", ["x=Vi(3)", "y=Vj(3)"], reduction_op="Sum", axis=1)
    conv(x, y)
    ld = keops_io.last_loader
    p = ld.params
    out = torch.empty(100, 1, device="cuda", dtype=torch.float16)
    with pytest.raises(binder.KeOpsHipError, match="compiled for float"):
        ld.module(1, p.dimy, 100, 120, p.tagI, 0, 1, p.tag1D2D, p.dimred, p.cuda_block_size, p.use_chunk_mode, p.indsi,
                  p.indsj, p.indsp, p.dim, p.dimsx, p.dimsy, p.dimsp, ld.empty_ranges, (100, 1), out.data_ptr(),
                  (x.data_ptr(), y.data_ptr()), ((100, 3), (120, 3)))


def test_half_precision_launch_under_graph_capture():
    """After an eager call that sizes the staging buffer, the conversions and the launch record into a HIP graph; replays
    follow new input values bit for bit."""
    from keops_amd.torch import Genred

    gen = torch.Generator(device="cuda").manual_seed(3)
    x, y, b = (torch.randn(n, d, device="cuda", generator=gen).half() for n, d in ((3000, 3), (4000, 3), (4000, 2)))
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)"], reduction_op="Sum", axis=1)

    def replays_like_eager(fn, inputs, replays=3):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                fn(*inputs)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = fn(*inputs)
        for _ in range(replays):
            for t in inputs:
                t.copy_(torch.randn(t.shape, device="cuda", generator=gen).half())
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = out.clone()
            if not torch.equal(got, fn(*inputs)):
                return False
        return True

    assert replays_like_eager(conv, [x, y, b])


def test_module_compiled_for_half_data_refuses_float32_operands():
    """A chunked module built for half-precision data keeps one half-precision term per component: exact for data that
    is half precision, an 11-bit truncation for float32 data.  The ABI ties the two together: such a module only runs
    with use_half = 1 (and a float32 module only with use_half = 0)."""
    from keops_amd import binder, keops_io
    from keops_amd.torch import Genred

    gen = torch.Generator(device="cuda").manual_seed(3)
    r = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    x, y, b = (r(600, 64) / 8).half(), (r(700, 64) / 8).half(), r(700, 4).half()
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(64)", "y=Vj(64)", "b=Vj(4)"], reduction_op="Sum", axis=1)
    conv(x, y, b)
    ld = keops_io.last_loader
    assert ld.module.meta("chk_single") == "1"
    p = ld.params
    xf, yf, bf = x.float(), y.float(), b.float()
    out = torch.empty(600, 4, device="cuda")
    with pytest.raises(binder.KeOpsHipError, match="compiled for half-precision data"):
        ld.module(1, p.dimy, 600, 700, p.tagI, 0, 0, p.tag1D2D, p.dimred, p.cuda_block_size, p.use_chunk_mode, p.indsi,
                  p.indsj, p.indsp, p.dim, p.dimsx, p.dimsy, p.dimsp, ld.empty_ranges, (600, 4), out.data_ptr(),
                  (xf.data_ptr(), yf.data_ptr(), bf.data_ptr()), ((600, 64), (700, 64), (700, 4)))
    # and the other way round: the float32 module of the same formula does not take use_half = 1
    conv(xf, yf, bf)
    ld32 = keops_io.last_loader
    assert ld32.module.meta("chk_single") == "0"
    outh = torch.empty(600, 4, device="cuda", dtype=torch.float16)
    with pytest.raises(binder.KeOpsHipError, match="compiled for float32 data"):
        ld32.module(1, p.dimy, 600, 700, p.tagI, 0, 1, p.tag1D2D, p.dimred, p.cuda_block_size, p.use_chunk_mode, p.indsi,
                    p.indsj, p.indsp, p.dim, p.dimsx, p.dimsy, p.dimsp, ld32.empty_ranges, (600, 4), outh.data_ptr(),
                    (x.data_ptr(), y.data_ptr(), b.data_ptr()), ((600, 64), (700, 64), (700, 4)))
