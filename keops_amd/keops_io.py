"""Binding layer between the user-level Genred and the native library.

Counterpart of pykeops/pykeops/common/keops_io/LoadKeOps.py:33-243 (alias -> Var rewrite, dtype
map, scheme id, output allocation, pointer/shape tuples) and LoadKeOps_nvrtc.py:18-72 (module
object + call).  The native side is libkeops_hip through ctypes (keops_amd/binder.py).
"""
from __future__ import annotations

import numpy as np
import torch

from . import binder, config
from .common.parse_type import parse_dtype_acc
from .formulas.parse import parse_alias, parse_reduction
from .get_keops_dll import get_keops_dll, plan_row_col_product

_NULL_RANGE = np.array([-1], dtype=np.int64)
_modules = {}


class LoadKeOps_hip:
    empty_ranges = tuple([_NULL_RANGE.ctypes.data] * 7)

    def __init__(self, tagCPUGPU, tag1D2D, tagHostDevice, use_ranges, device_id_request, formula, aliases, nargs,
                 dtype, lang, optional_flags, nx=None, batch_loop=0, pairs=0, batch_total=0):
        if lang not in ("torch", "pytorch"):
            raise ValueError("[KeOps] the HIP backend binds torch tensors only")
        if tagCPUGPU != 1 or tagHostDevice not in (0, 1):
            raise ValueError("[KeOps] the HIP backend computes on the GPU only (backend 'CPU' is not available)")
        aliases_new = []
        for k, alias in enumerate(aliases):
            name, var = parse_alias(alias, k)
            if name is not None:
                aliases_new.append(f"{name}=Var({var.ind},{var.dim},{var.cat})")
        p = self.params = type("Params", (), {})()
        p.aliases_old, p.aliases = list(aliases), aliases_new
        p.red_formula_string = formula
        p.dtype = dtype
        # half-precision data is computed in float32: the library converts the arguments and rounds the result once
        # (use_half of keops_hip_launch; pykeops/pykeops/torch/half2_convert.py computes in half2 arithmetic)
        self.half = dtype == "float16"
        p.c_dtype = dict(float16="float", float32="float", float64="double").get(dtype)
        if p.c_dtype is None:
            raise ValueError(f"[KeOps] data of type {dtype} is not supported (float16, float32, float64 are)")
        p.c_dtype_acc = parse_dtype_acc(optional_flags["dtype_acc"], dtype)
        p.sum_scheme = optional_flags["sum_scheme"]
        p.enable_chunks = optional_flags["enable_chunks"]
        p.mult_var_highdim = optional_flags.get("multVar_highdim", 0)
        p.tagHostDevice, p.tagCPUGPU = tagHostDevice, tagCPUGPU
        # what a twin of this object without the matrix-core schemes is built from (see genred_pytorch)
        self._ctor = (tagCPUGPU, tag1D2D, tagHostDevice, use_ranges, device_id_request, formula, list(aliases), nargs,
                      dtype, lang, dict(optional_flags), nx)
        self._exact = None
        self.plan = None
        if tag1D2D == 0 and p.c_dtype == "float" and p.c_dtype_acc == "float":
            red = parse_reduction(formula, p.aliases)
            self.plan = plan_row_col_product(red, p.c_dtype, optional_flags["use_fast_math"], p.enable_chunks)
        if self.plan is not None:
            # sum_j g_ij (a x_i + c y_j) as a x_i sum_j g_ij + c sum_j g_ij y_j: one scalar reduction and weighted
            # sums of column slices of y, each a module of the chunked scheme (get_keops_dll.plan_row_col_product)
            plan, tagI = self.plan, red.tagI
            D = plan["row"].dim
            width = 64 if D > 128 else 128
            sub_flags = dict(optional_flags, dtype_acc="auto") if self.half else optional_flags
            sub = lambda f, extra: LoadKeOps_hip(tagCPUGPU, tag1D2D, tagHostDevice, use_ranges, device_id_request, f,
                                                 list(aliases) + extra, nargs + len(extra),
                                                 "float32" if self.half else dtype, lang, sub_flags,
                                                 nx=nx, batch_loop=batch_loop, pairs=pairs, batch_total=batch_total)
            self.sub_slices, self.ones_column = [], False
            if plan["c"]:
                for c0 in range(0, D, width):
                    w = min(width, D - c0)
                    # when the last slice has room, a column of ones rides along: its sum is sum_j g_ij
                    if plan["a"] and c0 + w == D and w < width:
                        self.ones_column, w = True, w + 1
                    v = f"Var({nargs},{w},{plan['col'].cat})"
                    self.sub_slices.append((c0, min(D, c0 + w), sub(f"Sum_Reduction(Mult({plan['G']!r},{v}),{tagI})", [v])))
            self.sub_scalar = sub(f"Sum_Reduction({plan['G']!r},{tagI})", []) if (plan["a"] and not self.ones_column) else None
            p.tagI, p.tagZero, p.dim, p.dimred = tagI, 0, D, D
            p.device_id_request, p.nargs = device_id_request, nargs
            p.reduction_op, p.axis = "Sum_Reduction", 1 - tagI
            self.dimout, self.tagIJ, self.module = D, tagI, None
            return
        map_reduce_id = "GpuReduc" + ("1D" if tag1D2D == 0 else "2D") + ("_ranges" if use_ranges else "")
        (p.tag, p.source_name, p.low_level_code_file, p.tagI, p.tagZero, p.use_half, p.use_fast_math,
         p.cuda_block_size, p.use_chunk_mode, p.tag1D2D, p.dimred, p.dim, p.dimy, indsi, indsj, indsp, dimsx,
         dimsy, dimsp) = get_keops_dll(
            map_reduce_id, formula, p.enable_chunks, -1, p.mult_var_highdim, p.aliases, nargs, p.c_dtype,
            p.c_dtype_acc, p.sum_scheme, tagHostDevice, tagCPUGPU, tag1D2D, self.half, optional_flags["use_fast_math"],
            device_id_request, nx=nx, batch_loop=batch_loop, pairs=pairs, batch_total=batch_total,
        )
        # the engine reports (output-indexed, reduced) variable lists; the ABI takes (i, j) lists
        if p.tagI == 1:
            indsi, indsj, dimsx, dimsy = indsj, indsi, dimsy, dimsx
        p.indsi, p.indsj, p.indsp, p.dimsx, p.dimsy, p.dimsp = indsi, indsj, indsp, dimsx, dimsy, dimsp
        p.device_id_request, p.nargs = device_id_request, nargs
        p.reduction_op = formula.split("(")[0]
        p.axis = 1 - p.tagI
        self.dimout, self.tagIJ = p.dim, p.tagI
        self.module = None
        if not p.tagZero:
            key = (p.low_level_code_file, device_id_request, nargs)
            self.module = _modules.get(key)
            if self.module is None:
                self.module = _modules[key] = binder.Module(max(0, device_id_request), nargs, p.low_level_code_file)

    def _row_col_product(self, device_args, ranges, nx, ny, nbatchdims, out, *args):
        plan = self.plan
        row, col = args[plan["row"].ind], args[plan["col"].ind]
        if plan["a"] == -plan["c"]:
            # g (x - y) = g ((x - m) - (y - m)): with m the mean of y the two sums that are subtracted are as small
            # as the cloud allows, which limits the cancellation when the pairs that matter are close
            m = col.mean(dim=-2, keepdim=True)
            row, col = row - m, col - m
        res = total = None
        if self.sub_slices:
            parts = []
            for k, (c0, c1, ld) in enumerate(self.sub_slices):
                v = col[..., c0:c1]
                if self.ones_column and k == len(self.sub_slices) - 1:
                    v = torch.cat([v, torch.ones_like(v[..., :1])], dim=-1)
                parts.append(ld.genred_pytorch(device_args, ranges, nx, ny, nbatchdims, None, *args, v.contiguous()))
            if self.ones_column:
                total, parts[-1] = parts[-1][..., -1:], parts[-1][..., :-1]
            res = parts[0] if len(parts) == 1 else torch.cat(parts, dim=-1)
            if plan["sign"] * plan["c"] < 0:
                res = -res
        if self.sub_scalar is not None:
            total = self.sub_scalar.genred_pytorch(device_args, ranges, nx, ny, nbatchdims, None, *args)
        if total is not None:
            if plan["sign"] * plan["a"] < 0:
                total = -total
            res = row * total if res is None else torch.addcmul(res, row, total)
        if out is None:
            return res
        if tuple(out.shape) != tuple(res.shape) or not out.is_contiguous():
            raise ValueError(f"[KeOps] 'out' must be a contiguous tensor of shape {tuple(res.shape)}")
        return out.copy_(res)

    def genred_pytorch(self, device_args, ranges, nx, ny, nbatchdims, out, *args):
        if self.plan is not None:
            if self.half:
                # several float32 launches combined with torch operations: the conversions happen here
                res = self._row_col_product(device_args, ranges, nx, ny, nbatchdims, None, *[a.float() for a in args]).half()
                if out is None:
                    return res
                if tuple(out.shape) != tuple(res.shape) or not out.is_contiguous():
                    raise ValueError(f"[KeOps] 'out' must be a contiguous tensor of shape {tuple(res.shape)}")
                return out.copy_(res)
            return self._row_col_product(device_args, ranges, nx, ny, nbatchdims, out, *args)
        p = self.params
        if not ranges:
            ranges_ptr, keep = self.empty_ranges, None
        else:
            shapes = np.array([r.shape[0] for r in ranges], dtype=np.int64)
            keep = (ranges, shapes)
            ranges_ptr = tuple(int(r.data_ptr()) for r in ranges) + (shapes.ctypes.data,)
        args_ptr = tuple(int(a.data_ptr()) for a in args)
        argshapes = tuple(tuple(a.shape) for a in args)
        M = nx if p.tagI == 0 else ny
        if nbatchdims:
            # (an argument with fewer leading dimensions, e.g. a parameter given as (dim,), is broadcast over them)
            bshape = np.maximum.reduce([list(a.shape[:nbatchdims]) if a.dim() > nbatchdims else [1] * nbatchdims for a in args])
            shapeout = tuple(int(b) for b in bshape) + (M, p.dim)
        else:
            shapeout = (M, p.dim)
        if out is None:
            out = torch.empty(shapeout, dtype=args[0].dtype, device=device_args)
        elif tuple(out.shape) != shapeout or not out.is_contiguous():
            raise ValueError(f"[KeOps] 'out' must be a contiguous tensor of shape {shapeout}")
        if p.tagZero:
            out.zero_()
            return out
        # host tensors (tagHostDevice = 0): the library stages them itself and returns when out is back on the host
        dev = out.device if out.is_cuda else torch.device("cuda", max(0, p.device_id_request))
        stream = torch.cuda.current_stream(dev).cuda_stream
        try:
            self.module(
                p.tagHostDevice, p.dimy, nx, ny, p.tagI, p.tagZero, int(self.half), p.tag1D2D, p.dimred, p.cuda_block_size,
                p.use_chunk_mode, p.indsi, p.indsj, p.indsp, p.dim, p.dimsx, p.dimsy, p.dimsp, ranges_ptr,
                tuple(out.shape), int(out.data_ptr()), args_ptr, argshapes, stream=stream, sync=False,
            )
        except binder.KeOpsNotCertified:
            # high-dimensional K nearest neighbours with ties at the K-th distance: same call on the exact kernel
            if self._exact is None:
                c = self._ctor
                self._exact = LoadKeOps_hip(*c[:10], dict(c[10], enable_chunks=-1), nx=c[11])
            return self._exact.genred_pytorch(device_args, ranges, nx, ny, nbatchdims, out, *args)
        del keep
        return out

    genred = genred_pytorch

    def import_module(self):
        return self


_loaders = {}
last_loader = None  # the object the most recent call resolved to (diagnostics, tests)


def load_keops_hip(tagCPUGPU, tag1D2D, tagHostDevice, use_ranges, device_id_request, formula, aliases, nargs, dtype,
                   lang, optional_flags, nx=None, ny=None, batch=None):
    """Cached constructor (the reference keeps one LoadKeOps object per parameter set as well,
    pykeops/pykeops/common/keops_io/LoadKeOps.py:23-31): parsing the formula and resolving the
    module happen once, later calls only launch.  ``nx`` / ``ny``: output and reduced rows of the call (of each
    batch); ``batch``: (number of batches, M, N[, full]) of a call with batch dimensions and no block-sparse ranges: a
    few large batches may be served one at a time by a dense module, many batches as row ranges by a block-sparse one
    (``full``: every tensor variable carries every batch dimension, nothing is broadcast)."""
    from .get_keops_dll import _rows_bucket
    from . import config

    rows_hint = nx if (nx is not None and nx < 64 * 256 * config.block_size) else None
    if (nx is not None and nx == 0) or (ny is not None and ny == 0):
        # no pair at all: the general-purpose module writes the reduction's neutral element (the other schemes assume
        # at least one tile of work)
        optional_flags = dict(optional_flags, enable_chunks=0)
    # log2 bucket of the pairs per batch when there are few batches: the engine weighs it against the formula
    batch_loop = int(batch[1] * batch[2]).bit_length() if (batch and 0 < batch[0] <= config.knn_batch_max) else 0
    if batch and batch[0] == 0:
        batch_loop = -1  # block-sparse ranges without batch dimensions
    # log2 bucket of the pairs of all batches together when nothing is broadcast, else 0
    batch_total = int(batch[0] * batch[1] * batch[2]).bit_length() if (batch and batch[0] > 0 and len(batch) > 3 and batch[3]) else 0
    if batch_total > 44:
        batch_total = 44
    # log2 bucket of the pairs of the call (of each batch), 0: unknown or beyond every threshold of the engine
    pairs = int(nx * ny).bit_length() if (nx is not None and ny is not None) else 0
    if pairs > 40:
        pairs = 0
    key = (tagCPUGPU, tag1D2D, tagHostDevice, bool(use_ranges), device_id_request, formula, tuple(aliases), nargs,
           dtype, lang, tuple(sorted(optional_flags.items())), _rows_bucket(rows_hint), batch_loop, pairs, batch_total,
           config.radial_min_pairs_log2, config.radial_ranges_min_pairs_log2)
    global last_loader
    obj = _loaders.get(key)
    if obj is None:
        obj = _loaders[key] = LoadKeOps_hip(tagCPUGPU, tag1D2D, tagHostDevice, use_ranges, device_id_request, formula,
                                            aliases, nargs, dtype, lang, optional_flags, nx=nx, batch_loop=batch_loop, pairs=pairs,
                                            batch_total=batch_total)
    last_loader = obj
    return obj


keops_binder = {"hip": load_keops_hip}
