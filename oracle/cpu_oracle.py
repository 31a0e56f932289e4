"""TEST INFRASTRUCTURE ONLY: ctypes front door to ``liboracle_cpu.so`` (oracle/cpu_reduc.c).

The library is the CPU restatement of the reference's CpuReduc loops
(keopscore/keopscore/mapreduce/cpu/CpuReduc.py:43-64, CpuReduc_ranges.py:102-230).  Nothing in the
product package imports this module; it serves the test-suite, the smoke test and the benchmark's
cpu_baseline leg as the checker.
"""
import ctypes
import hashlib
import os
import shutil
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

FORMULAS = dict(dense=0, gauss=1, gauss_gradx=2, sqdist=3, lse_gauss=4, laplace=5, l1dist=6, exp_l1=7, scalprod=8,
                gauss_gradx_abs=9)
REDUCTIONS = dict(
    Sum=0, Max_SumShiftExpWeight=1, Max_SumShiftExp=1, Min_ArgMin=2, Max_ArgMax=3, KMin_ArgKMin=4,
    Min=5, ArgMin=6, Max=7, ArgMax=8, KMin=9, ArgKMin=10,
)
SCHEMES = dict(direct_sum=0, block_sum=1, kahan_scheme=2)


def _source_digest():
    h = hashlib.sha256()
    for name in ("cpu_reduc.c", "Makefile"):
        with open(os.path.join(_HERE, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def build(force=False):
    """Compile oracle/cpu_reduc.c into oracle/liboracle_cpu.so (make; gcc only).  A failing compilation is an error.
    Only a machine without make or without a C compiler uses the library that travelled with the tree, and only if
    the digest written when it was built matches the sources beside it."""
    target = os.path.join(_HERE, "liboracle_cpu.so")
    stamp = os.path.join(_HERE, "liboracle_cpu.digest")
    have_tools = shutil.which("make") and (shutil.which(os.environ.get("CC", "cc")) or shutil.which("gcc"))
    if not have_tools:
        if not os.path.exists(target) or not os.path.exists(stamp) or open(stamp).read().strip() != _source_digest():
            raise RuntimeError("oracle: no make / C compiler here and no liboracle_cpu.so built from these sources")
        return target
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, stdout=subprocess.DEVNULL)
    # make is incremental: a library older than cpu_reduc.c is rebuilt, an up-to-date one is left alone
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)
    with open(stamp, "w") as f:
        f.write(_source_digest())
    return target


def lib():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(build())
    return _LIB


def _prep(args, dtype):
    arrs = [np.ascontiguousarray(a, dtype=dtype) for a in args]
    ptrs = (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
    dims = (ctypes.c_int * len(arrs))(*[int(a.shape[-1]) if a.ndim else 1 for a in arrs])
    return arrs, ptrs, dims


def cpu_reduc(formula, args, nx, ny, dimfout, reduction="Sum", K=1, scheme="block_sum",
              acc_double=False, rows=None, ranges=None, dtype=np.float32):
    """Run the oracle.

    formula   : key of FORMULAS ("dense": args = [F table of shape (nx, ny, dimfout)])
    args      : list of numpy arrays, row-major (rows, dim); parameters are (dim,)
    rows      : optional int64 array of output rows to evaluate (exact: rows are independent)
    ranges    : optional (ranges_x (R,2), slices_x (R,), ranges_y (S,2)) int64 triple
    returns   : array (len(rows) or nx, dimout) of dtype
    """
    dtype = np.dtype(dtype)
    suffix = "f32" if dtype == np.float32 else "f64"
    L = lib()
    arrs, ptrs, dims = _prep(args, dtype)
    red = REDUCTIONS[reduction]
    dimout = getattr(L, "oracle_dimout_" + suffix)(red, int(K), int(dimfout))
    if rows is not None:
        rows = np.ascontiguousarray(rows, dtype=np.int64)
        n, rows_p = len(rows), rows.ctypes.data_as(ctypes.c_void_p)
    else:
        n, rows_p = nx, ctypes.c_void_p(0)
    out = np.empty((n, dimout), dtype=dtype)
    common = [FORMULAS[formula], red, int(K), SCHEMES[scheme], int(bool(acc_double)),
              ctypes.c_long(nx), ctypes.c_long(ny), int(dimfout), len(arrs), ptrs, dims]
    if ranges is None:
        rc = getattr(L, "oracle_cpu_reduc_" + suffix)(
            *common, rows_p, ctypes.c_long(n), out.ctypes.data_as(ctypes.c_void_p))
    else:
        rx, sx, ry = [np.ascontiguousarray(r, dtype=np.int64) for r in ranges]
        rc = getattr(L, "oracle_cpu_reduc_ranges_" + suffix)(
            *common, ctypes.c_long(rx.shape[0]), rx.ctypes.data_as(ctypes.c_void_p),
            sx.ctypes.data_as(ctypes.c_void_p), ry.ctypes.data_as(ctypes.c_void_p),
            rows_p, ctypes.c_long(n), out.ctypes.data_as(ctypes.c_void_p))
    if rc != 0:
        raise ValueError("oracle: unsupported sizes (dimred > 512)")
    return out
