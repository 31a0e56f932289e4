"""NumPy front end: the same Genred / KernelSolve call signatures on host arrays.

Counterpart of pykeops/pykeops/numpy (generic/generic_red.py, operations.py).  As in the reference, Genred hands
host pointers to the GPU engine, which stages them itself (tagHostDevice = 0, keops_nvrtc.cpp load_args_FromHost):
the arrays are wrapped as host torch tensors without a copy and the result comes back in host memory.  KernelSolve
and LazyTensor, which launch many reductions on the same data, copy their arrays to the current HIP device once.
There is no CPU computation path.
"""
import numpy as np
import torch

from ..torch import Genred as _TorchGenred
from ..torch import KernelSolve as _TorchKernelSolve


def _device(device_id):
    if not torch.cuda.is_available():
        raise RuntimeError("[KeOps] the HIP backend needs a GPU; there is no CPU computation path")
    return torch.device("cuda", torch.cuda.current_device() if device_id in (-1, None) else device_id)


def _to_device(args, dev):
    out = []
    for a in args:
        a = np.ascontiguousarray(a)
        if a.dtype not in (np.float16, np.float32, np.float64):
            raise ValueError("[KeOps] only float16, float32 and float64 arrays are supported")
        out.append(torch.from_numpy(a).to(dev))
    return out


def _ranges_to_device(ranges, dev):
    if ranges is None:
        return None
    return tuple(torch.from_numpy(np.ascontiguousarray(r).astype(np.int64)).to(dev) for r in ranges)


class Genred:
    """``Genred(formula, aliases, reduction_op, axis, ...)(*numpy_arrays) -> numpy array``
    (pykeops/pykeops/numpy/generic/generic_red.py)."""

    def __init__(self, formula, aliases, reduction_op="Sum", axis=0, dtype=None, opt_arg=None, formula2=None,
                 cuda_type=None, dtype_acc="auto", use_double_acc=False, sum_scheme="auto", enable_chunks=True,
                 rec_multVar_highdim=False, use_fast_math=True):
        self._fn = _TorchGenred(formula, aliases, reduction_op=reduction_op, axis=axis, opt_arg=opt_arg,
                                formula2=formula2, dtype_acc=dtype_acc, use_double_acc=use_double_acc,
                                sum_scheme=sum_scheme, enable_chunks=enable_chunks,
                                rec_multVar_highdim=rec_multVar_highdim, use_fast_math=use_fast_math)

    def __call__(self, *args, backend="auto", device_id=-1, ranges=None, out=None):
        if backend == "CPU":
            raise ValueError("[KeOps] backend 'CPU' is not available in the HIP build")
        dev = _device(device_id)
        host = []
        for a in args:
            a = np.ascontiguousarray(a)
            if a.dtype not in (np.float16, np.float32, np.float64):
                raise ValueError("[KeOps] only float16, float32 and float64 arrays are supported")
            host.append(torch.from_numpy(a))
        if ranges is not None:
            ranges = tuple(torch.from_numpy(np.ascontiguousarray(r).astype(np.int64)) for r in ranges)
        res = self._fn(*host, backend=backend.replace("_Host", "").replace("_Device", "").replace("_host", "").replace("_device", ""),
                       device_id=dev.index, ranges=ranges)
        res = res.cpu().numpy()
        if out is not None:
            out[...] = res
            return out
        return res


class KernelSolve:
    """``KernelSolve(formula, aliases, varinvalias, axis)(*numpy_arrays, alpha=..., eps=...)``
    (pykeops/pykeops/numpy/operations.py)."""

    def __init__(self, formula, aliases, varinvalias, axis=0, dtype=None, opt_arg=None, dtype_acc="auto",
                 use_double_acc=False, sum_scheme="auto", enable_chunks=True, rec_multVar_highdim=None,
                 use_fast_math=True):
        self._fn = _TorchKernelSolve(formula, aliases, varinvalias, axis=axis, dtype_acc=dtype_acc,
                                     use_double_acc=use_double_acc, sum_scheme=sum_scheme, enable_chunks=enable_chunks,
                                     rec_multVar_highdim=rec_multVar_highdim, use_fast_math=use_fast_math)

    def __call__(self, *args, backend="auto", device_id=-1, alpha=1e-10, eps=1e-6, ranges=None):
        dev = _device(device_id)
        res = self._fn(*_to_device(args, dev), backend=backend, alpha=alpha, eps=eps,
                       ranges=_ranges_to_device(ranges, dev))
        return res.cpu().numpy()


def _split(output, aliases):
    from ..common.parse_type import get_type

    _, cat, dim, _ = get_type(output)
    return list(aliases), (cat + 1) % 2, dim  # reduce over the other index


def generic_sum(formula, output, *aliases, **kwargs):
    """The first alias names the output and fixes the reduction axis
    (pykeops/pykeops/numpy/generic/generic_ops.py)."""
    al, axis, _ = _split(output, aliases)
    return Genred(formula, al, reduction_op="Sum", axis=axis, **kwargs)


def generic_logsumexp(formula, output, *aliases, **kwargs):
    al, axis, _ = _split(output, aliases)
    return Genred(formula, al, reduction_op="LogSumExp", axis=axis, **kwargs)


def generic_argmin(formula, output, *aliases, **kwargs):
    al, axis, _ = _split(output, aliases)
    return Genred(formula, al, reduction_op="ArgMin", axis=axis, **kwargs)


def generic_argkmin(formula, output, *aliases, **kwargs):
    al, axis, dim = _split(output, aliases)
    return Genred(formula, al, reduction_op="ArgKMin", axis=axis, opt_arg=dim, **kwargs)


# ---- LazyTensor on NumPy arrays (pykeops/pykeops/numpy/lazytensor/LazyTensor.py) ---------------------------

from ..torch.lazytensor import LazyTensor as _TorchLazyTensor  # noqa: E402


def _np_out(res):
    if isinstance(res, torch.Tensor):
        return res.cpu().numpy()
    if isinstance(res, tuple):
        return tuple(_np_out(r) for r in res)
    return res


class LazyTensor(_TorchLazyTensor):
    """The symbolic LazyTensor of the torch layer on NumPy arrays: arrays are moved to the current device when the
    LazyTensor is built and reductions return NumPy arrays."""

    def __init__(self, x=None, axis=None):
        if isinstance(x, np.ndarray):
            if x.dtype not in (np.float16, np.float32, np.float64):
                raise ValueError("[KeOps] only float16, float32 and float64 arrays are supported")
            x = torch.from_numpy(np.ascontiguousarray(x)).to(_device(-1))
        elif isinstance(x, (np.floating, np.integer)):
            x = x.item()
        super().__init__(x, axis)

    def reduction(self, *args, call=True, **kwargs):
        if isinstance(kwargs.get("ranges"), tuple) and isinstance(kwargs["ranges"][0], np.ndarray):
            kwargs["ranges"] = _ranges_to_device(kwargs["ranges"], _device(-1))
        res = super().reduction(*args, call=call, **kwargs)
        if callable(res) and not isinstance(res, torch.Tensor):
            return lambda *a, **k: _np_out(res(*[torch.from_numpy(np.ascontiguousarray(t)).to(_device(-1))
                                                 if isinstance(t, np.ndarray) else t for t in a], **k))
        return _np_out(res)


def Vi(x_or_ind, dim=None):
    return LazyTensor(x_or_ind, axis=0) if dim is None else LazyTensor((x_or_ind, dim, 0))


def Vj(x_or_ind, dim=None):
    return LazyTensor(x_or_ind, axis=1) if dim is None else LazyTensor((x_or_ind, dim, 1))


def Pm(x_or_ind, dim=None):
    return LazyTensor(x_or_ind, axis=2) if dim is None else LazyTensor((x_or_ind, dim, 2))
