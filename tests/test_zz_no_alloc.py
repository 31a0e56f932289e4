"""The entry point that allocates nothing (keops_hip_launch_noalloc): same kernels as keops_hip_launch, workspaces
taken from the library's static device buffer.  Two calls in a row, the second on a smaller input, must reproduce
keops_hip_launch bit for bit; a workspace beyond the buffer is refused with a clear error."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _loader(formula, aliases, nx, ny, red="Sum"):
    from keops_amd.common.operations import preprocess
    from keops_amd.common.parse_type import axis2cat, get_optional_flags
    from keops_amd.keops_io import load_keops_hip

    red_int, f2 = preprocess(red, None)
    flags = get_optional_flags(red_int, "auto", False, "auto", True, True)
    full = f"{red_int}_Reduction({formula},{axis2cat(1)}{',' + f2 if f2 else ''})"
    return load_keops_hip(1, 0, 1, False, 0, full, aliases, len(aliases), "float32", "torch", flags, nx=nx, ny=ny)


def _both(ld, args, M, N):
    p = ld.params
    ref = ld.genred_pytorch(args[0].device, None, M, N, 0, None, *args)
    out = torch.full_like(ref, float("nan"))
    stream = torch.cuda.current_stream().cuda_stream
    ld.module.call_noalloc(M, N, p.tagI, p.tag1D2D, p.dimred, p.indsi, p.indsj, p.indsp, p.dim, p.dimsx, p.dimsy, p.dimsp,
                           tuple(out.shape), out.data_ptr(), tuple(a.data_ptr() for a in args), tuple(tuple(a.shape) for a in args),
                           stream=stream)
    torch.cuda.synchronize()
    return ref, out


def test_noalloc_matches_the_allocating_entry_point_twice_in_a_row():
    from keops_amd import binder

    assert binder.noalloc_scratch_bytes() == 128 << 20
    gen = torch.Generator(device="cuda").manual_seed(0)
    r = lambda *s: torch.randn(*s, device="cuda", generator=gen)
    al = ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)", "g=Pm(1)"]
    g = torch.tensor([0.5], device="cuda")
    # few rows, long reduced axis: column slabs, whose partial accumulators live in the scratch buffer
    M, N = 600, 300_000
    ld = _loader("Exp(-g*SqDist(x,y))*b", al, M, N)
    x, y, b = r(M, 3), r(N, 3), r(N, 2)
    ref, out = _both(ld, [x, y, b, g], M, N)
    assert torch.equal(ref, out)
    # second call, smaller input, same module: the buffer still holds the first call's partials
    M2, N2 = 250, 70_000
    ref2, out2 = _both(ld, [x[:M2].contiguous(), y[:N2].contiguous(), b[:N2].contiguous(), g], M2, N2)
    assert torch.equal(ref2, out2)
    # matrix-core chunked scheme: operand copies, norms and column sums come from the scratch buffer too
    M3, N3 = 3000, 5000
    ldc = _loader("Exp(-Norm2(x-y))*b", ["x=Vi(64)", "y=Vj(64)", "b=Vj(8)"], M3, N3)
    assert ldc.module.meta("scheme") == "chunk"
    xc, yc, bc = r(M3, 64) / 8, r(N3, 64) / 8, r(N3, 8)
    ref3, out3 = _both(ldc, [xc, yc, bc], M3, N3)
    assert torch.equal(ref3, out3)
    ref4, out4 = _both(ldc, [xc[:1000].contiguous(), yc[:777].contiguous(), bc[:777].contiguous()], 1000, 777)
    assert torch.equal(ref4, out4)


def test_noalloc_refuses_what_it_cannot_serve():
    from keops_amd import binder

    gen = torch.Generator(device="cuda").manual_seed(1)
    # 2e6 rows x 17+ slabs of float partials would need more than 128 MiB: clear error, no launch
    M, N = 2_000_000, 200_000
    ld = _loader("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(8)", "g=Pm(1)"], M, N)
    x, y, b = (torch.randn(n, d, device="cuda", generator=gen) for n, d in ((M, 3), (N, 3), (N, 8)))
    g = torch.tensor([0.5], device="cuda")
    p = ld.params
    out = torch.empty(M, 8, device="cuda")
    args = [x, y, b, g]
    call = lambda: ld.module.call_noalloc(M, N, p.tagI, 1, p.dimred, p.indsi, p.indsj, p.indsp, p.dim, p.dimsx, p.dimsy, p.dimsp,
                                          tuple(out.shape), out.data_ptr(), tuple(a.data_ptr() for a in args),
                                          tuple(tuple(a.shape) for a in args), stream=torch.cuda.current_stream().cuda_stream)
    with pytest.raises(binder.KeOpsHipError, match="static scratch buffer"):
        call()
    torch.cuda.synchronize()
    # the allocating entry point serves the same call
    ref = ld.genred_pytorch(x.device, None, M, N, 0, None, *args)
    assert torch.isfinite(ref).all()
