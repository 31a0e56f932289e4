"""Host-resident arguments (tagHostDevice = 0 of the C ABI, the reference's load_args_FromHost /
range_preprocess_from_host, keopscore/keopscore/include/utils_pe.h:66-99): NumPy pointers go straight through ctypes,
the library stages them in one pooled device allocation and returns with `out` in host memory."""
import ctypes

import numpy as np
import pytest
import torch

from common import assert_sum_parity
from oracle.cpu_oracle import cpu_reduc

pytestmark = pytest.mark.gpu

NO_RANGES = np.array([-1], np.int64)


def _module(formula, aliases, red="Sum", axis=1, ranges=False, nx=None, ny=None):
    from keops_amd.keops_io import load_keops_hip
    from keops_amd.common.operations import preprocess
    from keops_amd.common.parse_type import axis2cat, get_optional_flags

    red_int, f2 = preprocess(red, None)
    flags = get_optional_flags(red_int, "auto", False, "auto", True, True)
    full = f"{red_int}_Reduction({formula},{axis2cat(axis)}{',' + f2 if f2 else ''})"
    return load_keops_hip(1, 0, 0, ranges, 0, full, aliases, len(aliases), "float32", "torch", flags, nx=nx, ny=ny)


def test_abi_takes_numpy_pointers_directly():
    M, N = 3000, 4100
    rng = np.random.default_rng(0)
    x, y = rng.standard_normal((M, 3)).astype(np.float32), rng.standard_normal((N, 3)).astype(np.float32)
    b, g = rng.standard_normal((N, 2)).astype(np.float32), np.array([0.7], np.float32)
    ld = _module("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)", "g=Pm(1)"], nx=M, ny=N)
    p = ld.params
    out = np.full((M, 2), np.nan, np.float32)
    args = [x, y, b, g]
    ld.module(0, p.dimy, M, N, p.tagI, 0, 0, p.tag1D2D, p.dimred, p.cuda_block_size, p.use_chunk_mode, p.indsi, p.indsj,
              p.indsp, p.dim, p.dimsx, p.dimsy, p.dimsp, tuple([NO_RANGES.ctypes.data] * 7), out.shape, out.ctypes.data,
              tuple(a.ctypes.data for a in args), tuple(a.shape for a in args), stream=0, sync=False)
    # no synchronisation here: the call returns with out in host memory
    ref = cpu_reduc("gauss", args, M, N, 2)
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 2)
    assert_sum_parity(out, ref, scale)
    # same bits as the device-pointer path
    from keops_amd.torch import Genred

    dev = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)", "g=Pm(1)"], reduction_op="Sum", axis=1)(
        *[torch.from_numpy(a).cuda() for a in args])
    assert np.array_equal(dev.cpu().numpy(), out)


def test_host_ranges_and_numpy_front_end():
    from keops_amd.numpy import Genred as NpGenred

    M, N = 5000, 6000
    rng = np.random.default_rng(5)
    x, y = rng.standard_normal((M, 3)).astype(np.float32), rng.standard_normal((N, 3)).astype(np.float32)
    b, g = rng.standard_normal((N, 1)).astype(np.float32), np.array([0.5], np.float32)
    ranges_i = np.array([[0, 1200], [2000, 4500]], np.int64)
    slices_i = np.array([2, 3], np.int64)
    redranges_j = np.array([[0, 1000], [1000, 2500], [4000, 6000]], np.int64)
    dummy = np.zeros((1, 2), np.int64)
    ranges = (ranges_i, slices_i, redranges_j, dummy, np.array([0], np.int64), dummy)
    conv = NpGenred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(1)", "g=Pm(1)"], reduction_op="Sum", axis=1)
    got = conv(x, y, b, g, ranges=ranges)
    assert isinstance(got, np.ndarray)
    ref = cpu_reduc("gauss", [x, y, b, g], M, N, 1, ranges=ranges[:3])
    scale = cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 1, ranges=ranges[:3]) + 1e-30
    assert_sum_parity(got, ref, scale)
    assert np.all(got[1200:2000] == 0) and np.all(got[4500:] == 0)
    # dense call, K nearest neighbours (indices come back as integers), host torch tensors through the torch front end
    idx = NpGenred("SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], reduction_op="ArgKMin", axis=1, opt_arg=3)(x, y)
    refk = cpu_reduc("sqdist", [x, y], M, N, 1, reduction="ArgKMin", K=3, scheme="direct_sum")
    assert np.array_equal(idx.astype(np.int64), refk.astype(np.int64))
    from keops_amd.torch import Genred

    xt, yt, bt, gt = (torch.from_numpy(a) for a in (x, y, b, g))
    host = Genred("Exp(-g*SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(1)", "g=Pm(1)"], reduction_op="Sum", axis=1)(xt, yt, bt, gt)
    assert not host.is_cuda
    full = cpu_reduc("gauss", [x, y, b, g], M, N, 1)
    assert_sum_parity(host.numpy(), full, cpu_reduc("gauss", [x, y, np.abs(b), g], M, N, 1))


def test_malformed_ranges_are_an_error_not_a_fault():
    """A reduced-index range past the end of the reduced axis, or fewer slices than row ranges, must come back as an
    error code before any kernel runs."""
    from keops_amd import binder
    from keops_amd.torch import Genred

    x, y, b = (torch.randn(n, d, device="cuda") for n, d in ((1000, 3), (1200, 3), (1200, 1)))
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(1)"], reduction_op="Sum", axis=1)
    good = (i64([[0, 500], [500, 1000]]), i64([1, 2]), i64([[0, 600], [600, 1200]]),
            i64([[0, 600], [600, 1200]]), i64([1, 2]), i64([[0, 500], [500, 1000]]))
    ref = conv(x, y, b, ranges=good)
    bad_end = (good[0], good[1], i64([[0, 600], [600, 1300]])) + good[3:]
    with pytest.raises(binder.KeOpsHipError, match="out of bounds"):
        conv(x, y, b, ranges=bad_end)
    few_slices = (good[0], i64([2]), good[2]) + good[3:]
    with pytest.raises(binder.KeOpsHipError, match="slices"):
        conv(x, y, b, ranges=few_slices)
    negative = (good[0], good[1], i64([[-5, 600], [600, 1200]])) + good[3:]
    with pytest.raises(binder.KeOpsHipError, match="out of bounds"):
        conv(x, y, b, ranges=negative)
    assert torch.equal(conv(x, y, b, ranges=good), ref)


def test_host_ranges_are_validated_at_every_call():
    """Host-pointer launches copy their ranges into the same staging addresses call after call: the second call with
    an out-of-bounds range must fail like the first (validation on the host every time, never the device-built
    tables that clamp)."""
    from keops_amd import binder
    from keops_amd.torch import Genred

    x, y, b = (torch.randn(n, d) for n, d in ((1000, 3), (1200, 3), (1200, 1)))
    i64 = lambda v: torch.tensor(v, dtype=torch.int64)
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(1)"], reduction_op="Sum", axis=1)
    good = (i64([[0, 500], [500, 1000]]), i64([1, 2]), i64([[0, 600], [600, 1200]]),
            i64([[0, 600], [600, 1200]]), i64([1, 2]), i64([[0, 500], [500, 1000]]))
    bad = (good[0], good[1], i64([[0, 600], [600, 1300]])) + good[3:]
    ref = conv(x, y, b, ranges=good)
    assert torch.equal(conv(x, y, b, ranges=good), ref)
    for _ in range(2):
        with pytest.raises(binder.KeOpsHipError, match="out of bounds"):
            conv(x, y, b, ranges=bad)
    assert torch.equal(conv(x, y, b, ranges=good), ref)


def test_ranges_clamped_by_the_device_built_tables_fail_the_next_launch():
    """Device tensors that an earlier call has validated are not read back again: the tables are built on the device
    and out-of-bounds indices are clamped.  That never passes silently: unless the caller reads the status
    (keops_hip_ranges_status), the module's next block-sparse launch fails and says why."""
    from keops_amd import binder, keops_io
    from keops_amd.torch import Genred

    x, y, b = (torch.randn(n, d, device="cuda") for n, d in ((1000, 3), (1200, 3), (1200, 2)))
    i64 = lambda v: torch.tensor(v, dtype=torch.int64, device="cuda")
    conv = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(2)"], reduction_op="Sum", axis=1)
    rg = (i64([[0, 500], [500, 1000]]), i64([1, 2]), i64([[0, 600], [600, 1200]]),
          i64([[0, 600], [600, 1200]]), i64([1, 2]), i64([[0, 500], [500, 1000]]))
    ref = conv(x, y, b, ranges=rg)               # validated on the host
    assert torch.equal(conv(x, y, b, ranges=rg), ref)   # tables built on the device
    rg[2][1, 1] = 10 ** 9                        # edited in place: same tensors, now out of bounds
    clamped = conv(x, y, b, ranges=rg)           # clamped to the axis, flagged
    torch.cuda.synchronize()
    assert torch.equal(clamped, ref)
    with pytest.raises(binder.KeOpsHipError, match="clamped"):
        conv(x, y, b, ranges=rg)
    rg[2][1, 1] = 1200
    assert torch.equal(conv(x, y, b, ranges=rg), ref)
    assert keops_io.last_loader.module.ranges_status() == 0
