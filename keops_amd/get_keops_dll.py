"""Engine entry: formula string -> compiled kernel module + launch metadata.

Counterpart of keopscore/keopscore/get_keops_dll.py:78-159 (scheme selection, zero-formula
bypass, metadata tuple) and keopscore/keopscore/binders/LinkCompile.py:19-125 (sha256 tag,
compile-if-absent).  Instead of emitting a whole CUDA kernel as text, the engine emits a short
"plug-in" - the straight-line formula body plus geometry macros - that is prepended to one of
the hand-written HIP templates embedded in libkeops_hip.
"""
from __future__ import annotations

import hashlib
import os
import threading

from . import binder, config
from .formulas import Lir, lower, parse_reduction
from .formulas.ops import Zero
from .formulas.reductions import KIND_KMIN, KIND_MAX, KIND_MIN, Reduction, Sum_Reduction, Zero_Reduction

SUM_SCHEMES = dict(direct_sum=0, block_sum=1, kahan_scheme=2)

_cache = {}
_lock = threading.Lock()


class VarLayout:
    """Which argument goes where in the packed x_i / y_j / p arrays of the kernels
    (code_gen_utils.py:531-564 Var_loader).  "row" variables are indexed like the output."""

    def __init__(self, red: Reduction):
        tagI = red.tagI
        vs = red.formula.variables
        self.rowvars = [v for v in vs if v.cat == tagI]
        self.colvars = [v for v in vs if v.cat == 1 - tagI]
        self.parvars = [v for v in vs if v.cat == 2]
        self.dimx = sum(v.dim for v in self.rowvars)
        self.dimy = sum(v.dim for v in self.colvars)
        self.dimp = sum(v.dim for v in self.parvars)
        self.names = {}
        for group, arr in ((self.rowvars, "xi"), (self.colvars, "yj"), (self.parvars, "p")):
            off = 0
            for v in group:
                for k in range(v.dim):
                    self.names[(v.cat, v.ind, k)] = f"{arr}[{off + k}]"
                off += v.dim

    @staticmethod
    def table(group):
        args = [v.ind for v in group] or [0]
        dims = [v.dim for v in group] or [0]
        offs, o = [], 0
        for v in group:
            offs.append(o)
            o += v.dim
        offs = offs or [0]
        return args, dims, offs


def _c_list(xs):
    return "{" + ", ".join(str(int(x)) for x in xs) + "}"


def choose_geometry(red, layout, nops, sizeof_t, nx=None, irregular=False):
    """Rows per lane / tile length: register budget first, then enough workgroups for the chip
    (``irregular``: block-sparse / batched launches, whose workgroups do unequal amounts of work and
    need many more of them to balance over the compute units)."""
    block = config.block_size
    dimy_pad = 0 if layout.dimy == 0 else -(-layout.dimy // (16 // sizeof_t)) * (16 // sizeof_t)
    per_row = layout.dimx + 2 * red.dimred * (2 if sizeof_t == 8 else 1) + min(nops, 32)
    rows = config.max_rows_per_lane
    while rows > 1 and rows * per_row + 2 * dimy_pad + 24 > 128:
        rows //= 2
    if nx is not None:
        # keep at least ~2 workgroups per compute unit when the row count allows it
        while rows > 1 and nx < (config.irregular_wg_per_cu if irregular else 2) * 256 * block * rows:
            rows //= 2
    tile_j = config.lds_tile_bytes // max(1, dimy_pad * sizeof_t)
    tile_j = max(64, min(1024, 1 << (tile_j.bit_length() - 1)))
    # very wide reduced-index rows: shorter tiles so that the staged tile still fits the LDS of a compute unit
    while tile_j > 16 and tile_j * dimy_pad * sizeof_t > 96 * 1024:
        tile_j //= 2
    unroll = 2 if nops * rows <= 128 else 1
    return dict(block=block, rows=rows, tile_j=tile_j, dimy_pad=dimy_pad, unroll=unroll)


def _lse_group(red, geo, nops):
    """Columns folded per running-maximum update of the log-sum-exp (KEOPS_LSE_GROUP).  A group inlines that many
    evaluations of the formula per output row of a lane: worth it while the update (17.7 against 12.5 instructions
    per pair) weighs against the formula, and a burden on the compiler when the formula is long (D = 100:
    6 minutes of compilation with groups of 8, seconds with 1)."""
    work = nops * geo["rows"]
    if work > 640:
        return 1
    if work > 160:
        return min(2, config.lse_group)
    return config.lse_group if (red.formula.dim <= 2 and geo["rows"] <= 2) else min(4, config.lse_group)


def generate_plugin(red, dtype, dtypeacc, sum_scheme, use_fast_math, nargs, nx=None, geometry=None, irregular=False):
    """HIP source of the kernel module for a reduction; returns (source, meta dict)."""
    sizeof_t = 8 if dtype == "double" else 4
    layout = VarLayout(red)
    # reductions that return indices are compared bit for bit: their pair values keep the
    # reference's operation order, without fused multiply-add contraction
    exact = red.kind in (KIND_MIN, KIND_MAX, KIND_KMIN)
    L = Lir(row_cat=red.tagI, fast_math=use_fast_math, dtype=dtype, exact_order=exact)
    outs = lower(red.formula, L)
    pragma = ["    #pragma clang fp contract(off)"] if exact else []
    lines, exprs = L.emit(outs, layout.names, indent="    ", segment=config.segment_statements, segment_prefix=pragma,
                          segment_min=config.segment_threshold)
    lines = pragma + lines
    nops = L.count_ops(outs)
    geo = choose_geometry(red, layout, nops, sizeof_t, nx, irregular)
    if geometry:
        geo.update(geometry)
    ra, rd, ro = VarLayout.table(layout.rowvars)
    ca, cd, co = VarLayout.table(layout.colvars)
    pa, pd, po = VarLayout.table(layout.parvars)
    meta = dict(
        scheme="conv", block=geo["block"], rows=geo["rows"], tile_j=geo["tile_j"], dimred=red.dimred, dimout=red.dim,
        sizeof_t=sizeof_t, sizeof_acc=8 if dtypeacc == "double" else 4, nrowvars=len(layout.rowvars),
        ncolvars=len(layout.colvars), nparvars=len(layout.parvars), nops=nops, red_kind=red.kind,
    )
    src = []
    src.append("//@keops " + " ".join(f"{k}={v}" for k, v in meta.items()))
    src.append(f"// reduction: {red!r}")
    src.append(f"typedef {dtype} T;\ntypedef {dtypeacc} TACC;")
    src.append('#include "keops_common.h"')
    defs = dict(
        KEOPS_NARGS=nargs, KEOPS_DIMX=layout.dimx, KEOPS_DIMY=layout.dimy, KEOPS_DIMY_PAD=geo["dimy_pad"],
        KEOPS_DIMP=layout.dimp, KEOPS_DIMFOUT=red.formula.dim, KEOPS_DIMRED=red.dimred, KEOPS_DIMOUT=red.dim,
        KEOPS_RED_KIND=red.kind, KEOPS_RED_KEEP=red.keep, KEOPS_RED_K=red.K, KEOPS_SUM_SCHEME=SUM_SCHEMES[sum_scheme],
        KEOPS_BLOCK=geo["block"], KEOPS_ROWS=geo["rows"], KEOPS_TILE_J=geo["tile_j"], KEOPS_UNROLL_J=geo["unroll"],
        KEOPS_LSE_GROUP=_lse_group(red, geo, nops),
        KEOPS_NROWVARS=len(layout.rowvars), KEOPS_NCOLVARS=len(layout.colvars), KEOPS_NPARVARS=len(layout.parvars),
    )
    src += [f"#define {k} {v}" for k, v in defs.items()]
    for name, vals in (("row_arg", ra), ("row_dim", rd), ("row_off", ro), ("col_arg", ca), ("col_dim", cd),
                       ("col_off", co), ("par_arg", pa), ("par_dim", pd), ("par_off", po)):
        src.append(f"static __device__ constexpr int keops_{name}[] = {_c_list(vals)};")
    dx, dy, dp = max(1, layout.dimx), max(1, geo["dimy_pad"]), max(1, layout.dimp)
    src += L.prelude
    src.append("struct KeopsFormula {")
    src.append(
        f"  static __device__ __forceinline__ void eval(const T (&xi)[{dx}], const T (&yj)[{dy}], "
        f"const T (&p)[{dp}], T (&fout)[{red.formula.dim}]) {{"
    )
    src += lines
    src += [f"    fout[{k}] = {e};" for k, e in enumerate(exprs)]
    src.append("  }\n};")
    src.append('#include "keops_conv.h"')
    return "\n".join(src) + "\n", meta


def match_knn_sqdist(red, dtype, map_reduce_id, batch_loop=0, pairs=0):
    """(row variable, column variable) when ``red`` is a K-min family reduction of SqDist between an
    output-indexed and a reduced-index variable of dimension config.knn_min_dim..256 in float32, on the dense
    scheme or (``batch_loop``) on batch dimensions served one batch at a time; None otherwise.  Such reductions
    run on the matrix-core filter + exact re-rank kernels.  ``pairs``: when not 0, the call holds less than
    2**pairs pairs; small problems stay on the general-purpose kernel, whose fixed cost is lower."""
    from .formulas import ops as O

    # batch_loop: 0 none; > 0: few large batches served one at a time (log2 bucket of the pairs per batch);
    # -1: block-sparse ranges without batch dimensions (the adaptive kernel with a range cursor)
    if red.kind != KIND_KMIN or dtype != "float" or ("_ranges" in map_reduce_id and not batch_loop) or red.K > 64:
        return None
    if batch_loop == -1 and not config.knn_ranges:
        return None
    f = red.formula
    if f.name != "Sum" or f.children[0].name != "Square" or f.children[0].children[0].name != "Subtract":
        return None
    a, b = f.children[0].children[0].children
    if not (isinstance(a, O.Var) and isinstance(b, O.Var)) or a.dim != b.dim or not config.knn_min_dim <= a.dim <= 256:
        return None
    if {a.cat, b.cat} != {0, 1}:
        return None
    if pairs and (1 << (int(pairs) - 1)) * max(a.dim, 16) < config.knn_min_work:
        # the pre-pass, the warm-up of the adaptive lists and the merge cost about 0.3 ms whatever the size
        return None
    if "_ranges" in map_reduce_id and batch_loop > 0 and (1 << (int(batch_loop) - 1)) * max(a.dim, 8) < config.knn_batch_min_work:
        # one pass per batch costs about 0.3 ms of launches: below this the batched general-purpose kernel wins
        return None
    return (a, b) if a.cat == red.tagI else (b, a)


def generate_knn_plugin(red, rowvar, colvar, nargs, block_sparse=False):
    """Module source for the matrix-core K-nearest-neighbour scheme (kernels/keops_knn_mfma.h); ``block_sparse``: the
    variant for launches with a ``ranges`` tuple (adaptive kernel only, GpuReduc1D_ranges.py:127-165)."""
    D = rowvar.dim
    dpad = -(-D // 16) * 16
    # low dimensions: neighbours are close compared with the norms, the operands are split as hi + lo
    split = int(D < 32)
    qsets, tj = config.knn_qsets, config.knn_tile_j
    if not (1 <= config.knn_filter_qsets <= 4 and 1 <= config.knn_sample_qsets <= 2 and 1 <= qsets <= 2):
        raise ValueError("[KeOps] the KNN kernels take one or two 32-query operand sets per wavefront (the filter: up to four)")
    # as many wavefronts as the LDS budget allows share one staged reference tile: the K-lists of the
    # 32*qsets queries of every wavefront live in LDS (8 bytes per entry)
    fixed = tj * (dpad * 2 * (1 + split) + 16) + tj * 4
    waves = config.knn_max_waves
    while waves > 1 and fixed + waves * (32 * qsets * (red.K * 8 + 4) + 512) > config.knn_lds_budget:
        waves //= 2
    # sampling pass (threshold estimate): the K-list of a query lives in the registers of one lane, so the
    # geometry of the filter (four wavefronts per SIMD, 128 registers each) holds for small K only
    swaves, sqsets = config.knn_sample_waves, config.knn_sample_qsets
    if red.K > 16 or dpad * (1 + split) > 64:
        swaves = min(swaves, 8)
    # the filter's workgroup is a whole compute unit that drains at every tile change: longer tiles there
    ftj = max(tj, min(config.knn_filter_tile_j, 64 * config.knn_filter_waves))
    while ftj > tj and ftj * (dpad * 2 * (1 + split) + 16) > 96 * 1024:
        ftj //= 2
    # dense launches in 32 dimensions and more: the fixed-threshold filter also exists on signed bytes
    i8 = int(config.knn_i8 and not split and not block_sparse and D >= 32)
    meta = dict(scheme="knn", knn_i8=i8, block=64 * waves, rows=1, tile_j=tj, dimred=red.dimred, dimout=red.dim, sizeof_t=4,
                sizeof_acc=4, nrowvars=1, ncolvars=1, nparvars=0, knn_d=D, knn_dpad=dpad, knn_k=red.K,
                knn_qb=waves * 32 * qsets, knn_fwaves=config.knn_filter_waves, knn_fqsets=config.knn_filter_qsets,
                knn_sample=config.knn_sample, knn_split=split, knn_ftj=ftj, knn_sqb=swaves * 32 * sqsets, knn_sblock=64 * swaves,
                rowarg=rowvar.ind, colarg=colvar.ind, ranges=int(block_sparse))
    src = ["//@keops " + " ".join(f"{k}={v}" for k, v in meta.items()), f"// reduction: {red!r}", "typedef float T;"]
    if block_sparse:
        src += ["#define KEOPS_MC_RANGES 1", "#define KNN_RANGES 1"]
    defs = dict(KEOPS_NARGS=nargs, KNN_D=D, KNN_DPAD=dpad, KNN_K=red.K, KEOPS_RED_KEEP=red.keep, KEOPS_DIMOUT=red.dim,
                KNN_QSETS=qsets, KNN_TJ=tj, KNN_WAVES=waves, KNN_FWAVES=config.knn_filter_waves,
                KNN_FQSETS=config.knn_filter_qsets, KNN_FTJ=ftj, KNN_SWAVES=swaves, KNN_SQSETS=sqsets, KNN_SPLIT=split, KNN_I8=i8)
    src += [f"#define {k} {v}" for k, v in defs.items()]
    src.append('#include "keops_knn_mfma.h"')
    return "\n".join(src) + "\n", meta


def match_vchunk(red):
    """(node, E, long variables) when the formula contains exactly one Sum(E) over an elementwise expression E of
    more than config.vchunk_min_dim components whose long operands are plain i- or j-indexed variables that appear
    nowhere else (the reference's chunkable operations and its rule against mixing chunked and post-chunk
    variables, Chunkable_Op.py:20-41, Chunk_Mode_Constants.py:56-60); None otherwise."""
    from .formulas import ops as O

    def elementwise(node, D):
        if isinstance(node, O.Var):
            return node.dim == 1 or (node.dim == D and node.cat in (0, 1))
        if not node.children:
            return node.dim == 1  # constants
        return isinstance(node, O.Elementwise) and node.dim in (1, D) and all(elementwise(c, D) for c in node.children)

    found = []
    exact = red.kind in (KIND_MIN, KIND_MAX, KIND_KMIN)
    for node in red.formula.walk():
        if node.children and node.children[0].dim > config.vchunk_min_dim and node not in [f[0] for f in found]:
            E, pair = None, None
            if node.name == "Sum":
                E = node.children[0]
            elif node.name == "Scalprod":
                # (a|b) = Sum(a*b); index-carrying reductions keep the reference's fused multiply-add chain
                # (Scalprod.py:32-36): the two factors are then evaluated separately and folded with an explicit fma
                E = O.Mult(node.children[0], node.children[1])
                if exact:
                    pair = (node.children[0], node.children[1])
                    if not all(elementwise(c, c.dim) and c.dim == node.children[0].dim for c in pair):
                        E = None
            if E is not None and E.dim == node.children[0].dim and elementwise(E, E.dim):
                found.append((node, E, pair))
    if len(found) != 1:
        return None
    node, E, pair = found[0]
    longs = [v for v in E.variables if v.dim == E.dim and v.dim > 1]
    if not longs or any(v.cat not in (0, 1) for v in longs):
        return None
    post = red.formula.replace(node, O.Var(1 << 30, 1, 3))
    if any(v in longs for v in post.variables) or any(v.dim > config.vchunk_min_dim for v in post.variables):
        return None
    return node, E, longs, pair


def generate_vchunk_plugin(red, match, dtype, dtypeacc, sum_scheme, use_fast_math, nargs, irregular=False):
    """Module source for formulas with one long elementwise sum (GpuReduc1D_chunks.py:19-118 without matrix-core
    form: L1 distances, weighted or transformed sums, float64 contractions): the general-purpose kernels of
    kernels/keops_conv.h built with KEOPS_VCHUNK, where the long rows stay in memory (the reduced-index ones staged in
    LDS tile by tile, the output-indexed ones streamed through the cache) and only the running sums of a tile of
    columns live in registers."""
    from .formulas import ops as O

    node, E, longs, pair = match
    D = E.dim
    sizeof_t = 8 if dtype == "double" else 4
    vec = 16 // sizeof_t
    dpad = -(-D // vec) * vec
    svar = O.Var(1 << 30, 1, 3)
    post = red.formula.replace(node, svar)
    exact = red.kind in (KIND_MIN, KIND_MAX, KIND_KMIN)
    full = VarLayout(red)
    row_long = [v for v in full.rowvars if v in longs]
    col_long = [v for v in full.colvars if v in longs]

    # short variables of E: collect them through a copy of E whose long variables are replaced by scalars
    Es, stand_in = E, {}
    for n, v in enumerate(longs):
        stand_in[v] = O.Var((1 << 20) + n, 1, v.cat)
        Es = Es.replace(v, stand_in[v])
    if Es.dim != 1:
        return None, None

    class _All:
        tagI = red.tagI
        formula = O.Concat(post, Es)

    small = VarLayout(_All)
    small_rows = [v for v in small.rowvars if v not in stand_in.values()]
    small_cols = [v for v in small.colvars if v not in stand_in.values()]
    names, dimx, dimy = {}, 0, 0
    for group, arr in ((small_rows, "xi"), (small_cols, "yj"), (small.parvars, "p")):
        off = 0
        for v in group:
            for k in range(v.dim):
                names[(v.cat, v.ind, k)] = f"{arr}[{off + k}]"
            off += v.dim
        if arr == "xi":
            dimx = off
        elif arr == "yj":
            dimy = off
    dimp = small.dimp
    for n, v in enumerate(row_long):
        names[(v.cat, stand_in[v].ind, 0)] = f"xl[{n}]"
    for n, v in enumerate(col_long):
        names[(v.cat, stand_in[v].ind, 0)] = f"yl[{n}]"
    names[(3, svar.ind, 0)] = "s"
    pragma = ["    #pragma clang fp contract(off)"] if exact else []
    Le = Lir(row_cat=red.tagI, fast_math=use_fast_math, dtype=dtype, exact_order=exact)
    if pair is None:
        e_lines, e_exprs = Le.emit(lower(Es, Le), names, indent="    ")
    else:
        # the two factors of the scalar product, one component each
        factors = []
        for f in pair:
            for v in longs:
                f = f.replace(v, stand_in[v])
            factors.append(f)
        e_lines, e_exprs = Le.emit(lower(factors[0], Le) + lower(factors[1], Le), names, indent="    ")
    Lp = Lir(row_cat=red.tagI, fast_math=use_fast_math, dtype=dtype, exact_order=exact)
    p_outs = lower(post, Lp)
    p_lines, p_exprs = Lp.emit(p_outs, names, indent="    ")
    uses_yj = any(v.cat == 1 - red.tagI for v in Es.variables if v not in stand_in.values())
    dimy_pad = 0 if dimy == 0 else -(-dimy // vec) * vec
    # columns per tile: their running sums live in registers, their long rows in LDS
    per_col = (len(col_long) * dpad + dimy_pad) * sizeof_t
    tile_j = 32
    while tile_j > 4 and tile_j * per_col > 64 * 1024:
        tile_j //= 2
    if tile_j * per_col > 96 * 1024:
        return None, None
    # tables in the order of the full variable lists (the launcher's offsets follow it); long variables are flagged
    def table(group, shorts):
        args, dims, offs, flag, o = [], [], [], [], 0
        for v in group:
            args.append(v.ind)
            dims.append(v.dim)
            flag.append(int(v not in shorts))
            offs.append(0 if v not in shorts else o)
            o += v.dim if v in shorts else 0
        return (args or [0]), (dims or [0]), (offs or [0]), (flag or [0])

    ra, rd, ro, rl = table(full.rowvars, small_rows)
    ca, cd, co, cl = table(full.colvars, small_cols)
    pa, pd, po = VarLayout.table(full.parvars)
    if [v for v in full.parvars] != [v for v in small.parvars]:
        return None, None
    meta = dict(scheme="conv", block=config.block_size, rows=1, tile_j=tile_j, dimred=red.dimred, dimout=red.dim,
                sizeof_t=sizeof_t, sizeof_acc=8 if dtypeacc == "double" else 4, nrowvars=len(full.rowvars),
                ncolvars=len(full.colvars), nparvars=len(full.parvars), nops=Lp.count_ops(p_outs), red_kind=red.kind,
                vchunk=D)
    src = ["//@keops " + " ".join(f"{k}={v}" for k, v in meta.items()), f"// reduction: {red!r}",
           f"typedef {dtype} T;\ntypedef {dtypeacc} TACC;", '#include "keops_common.h"']
    defs = dict(
        KEOPS_NARGS=nargs, KEOPS_DIMX=dimx, KEOPS_DIMY=dimy, KEOPS_DIMY_PAD=dimy_pad, KEOPS_DIMP=dimp,
        KEOPS_DIMFOUT=post.dim, KEOPS_DIMRED=red.dimred, KEOPS_DIMOUT=red.dim, KEOPS_RED_KIND=red.kind,
        KEOPS_RED_KEEP=red.keep, KEOPS_RED_K=red.K, KEOPS_SUM_SCHEME=SUM_SCHEMES[sum_scheme],
        KEOPS_BLOCK=config.block_size, KEOPS_ROWS=1, KEOPS_TILE_J=tile_j, KEOPS_UNROLL_J=1, KEOPS_LSE_GROUP=1,
        KEOPS_NROWVARS=len(full.rowvars), KEOPS_NCOLVARS=len(full.colvars), KEOPS_NPARVARS=len(full.parvars),
        KEOPS_VCHUNK=1, VCH_D=D, VCH_DPAD=dpad, VCH_NROW=len(row_long), VCH_NCOL=len(col_long), VCH_USES_YJ=int(uses_yj), VCH_FMA=int(pair is not None),
    )
    src += [f"#define {k} {v}" for k, v in defs.items()]
    for name, vals in (("row_arg", ra), ("row_dim", rd), ("row_off", ro), ("row_long", rl), ("col_arg", ca), ("col_dim", cd),
                       ("col_off", co), ("col_long", cl), ("par_arg", pa), ("par_dim", pd), ("par_off", po),
                       ("vch_row", [full.rowvars.index(v) for v in row_long] or [0]),
                       ("vch_col", [full.colvars.index(v) for v in col_long] or [0])):
        src.append(f"static __device__ constexpr int keops_{name}[] = {_c_list(vals)};")
    dx, dy, dp = max(1, dimx), max(1, dimy_pad), max(1, dimp)
    nr, nc = max(1, len(row_long)), max(1, len(col_long))
    src.append("// one component of the long sum: xl / yl hold that component of the long variables")
    src.append("struct KeopsChunkFormula {")
    src.append(f"  static __device__ __forceinline__ T eval(const T (&xl)[{nr}], const T (&yl)[{nc}], const T (&xi)[{dx}], "
               f"const T (&yj)[{dy}], const T (&p)[{dp}]{'' if pair is None else ', T& fb'}) {{")
    src += pragma + e_lines
    src.append(f"    return {e_exprs[0]};" if pair is None else f"    fb = {e_exprs[1]};\n    return {e_exprs[0]};")
    src.append("  }\n};")
    src.append("// post-chunk formula: s is the value of the long sum")
    src.append("struct KeopsFormula {")
    src.append(f"  static __device__ __forceinline__ void eval(const T (&xi)[{dx}], const T (&yj)[{dy}], "
               f"const T (&p)[{dp}], const T s, T (&fout)[{post.dim}]) {{")
    src += pragma + p_lines
    src += [f"    fout[{k}] = {e};" for k, e in enumerate(p_exprs)]
    src.append("  }\n};")
    src.append('#include "keops_conv.h"')
    return "\n".join(src) + "\n", meta


def match_knn_highdim(red, dtype, map_reduce_id, use_fast_math):
    """(mode, node, row variable, column variable) in match_chunk's format when ``red`` is a K-min family reduction
    of SqDist between an output-indexed and a reduced-index variable of more than 256 (the limit of the KNN
    scheme) and at most config.chunk_max_dim components, float32, dense: the chunked sweep keeps K +
    config.knn_highdim_margin approximate candidates per row and a second kernel re-ranks them exactly."""
    from .formulas import ops as O

    if (red.kind != KIND_KMIN or dtype != "float" or not use_fast_math or "_ranges" in map_reduce_id
            or red.K + config.knn_highdim_margin > 40 or red.formula.dim != 1):
        return None
    f = red.formula
    if f.name != "Sum" or f.children[0].name != "Square" or f.children[0].children[0].name != "Subtract":
        return None
    a, b = f.children[0].children[0].children
    if not (isinstance(a, O.Var) and isinstance(b, O.Var)) or a.dim != b.dim or not 256 < a.dim <= config.chunk_max_dim:
        return None
    if {a.cat, b.cat} != {0, 1}:
        return None
    return (0, f) + ((a, b) if a.cat == red.tagI else (b, a))


def generate_knn_highdim_plugin(red, match, nargs):
    """Chunked module whose sweep runs a KMin_ArgKMin reduction with K + margin entries on the approximate
    distances, plus the exact re-rank kernels (kernels/keops_chunk_mfma.h, CHK_KNN_K)."""
    from .formulas.reductions import KMin_ArgKMin_Reduction

    inner = KMin_ArgKMin_Reduction(red.formula, red.K + config.knn_highdim_margin, red.tagI)
    source, meta = generate_chunk_plugin(inner, match, "float", "direct_sum", nargs)
    if source is None:
        return None, None
    meta.update(dimred=red.dimred, dimout=red.dim, chk_knn=red.K, chk_knn_inner=inner.K)
    head, body = source.split("\n", 1)
    head = "//@keops " + " ".join(f"{k}={v}" for k, v in meta.items())
    defs = f"#define CHK_KNN_K {red.K}\n#define CHK_KNN_KEEP {red.keep}\n#define CHK_KNN_DIMOUT {red.dim}\n"
    marker = '#include "keops_common.h"\n'
    assert marker in body
    return head + "\n" + body.replace(marker, marker + defs, 1), meta


def match_chunk(red, dtype, map_reduce_id, use_fast_math, want="float"):
    """(mode, node, row variable, column variable) when the formula of a Sum / log-sum-exp reduction
    contains exactly one high-dimensional contraction SqDist(x_i, y_j) (mode 0) or <x_i, y_j> (mode 1)
    between plain variables of dimension config.chunk_min_dim..config.chunk_max_dim (24..1024) that appear nowhere else in the formula (the
    reference's conditions, Chunkable_Op.py:20-41 and Chunk_Mode_Constants.py:56-60, with the
    matrix-core dimension range instead of its >= 146 threshold).  None otherwise."""
    from .formulas import ops as O
    from .formulas.reductions import KIND_LSE, KIND_SUM

    if red.kind not in (KIND_SUM, KIND_LSE) or dtype != want or not use_fast_math:
        return None
    dmin, dmax = (config.chunk_min_dim, config.chunk_max_dim) if want == "float" else (config.chunk64_min_dim, config.chunk64_max_dim)
    found = []
    for node in red.formula.walk():
        mode = pair = None
        if node.name == "Sum" and node.children[0].name == "Square" and node.children[0].children[0].name == "Subtract":
            mode, pair = 0, node.children[0].children[0].children
        elif node.name == "Scalprod":
            mode, pair = 1, node.children
        if mode is None:
            continue
        a, b = pair
        if isinstance(a, O.Var) and isinstance(b, O.Var) and a.dim == b.dim and dmin <= a.dim <= dmax and {a.cat, b.cat} == {0, 1}:
            if node not in [f[1] for f in found]:
                found.append((mode, node, a, b))
    if len(found) != 1:
        return None
    mode, node, a, b = found[0]
    post = red.formula.replace(node, O.Var(1 << 30, 1, 3))
    if any(v == a or v == b for v in post.variables):
        return None  # the chunked variables also appear outside the contraction
    return (mode, node) + ((a, b) if a.cat == red.tagI else (b, a))


def plan_row_col_product(red, dtype, use_fast_math, enable_chunks):
    """Sum reductions of g_ij * w_ij where g is a scalar function of one high-dimensional contraction between an
    output-indexed variable x_i and a reduced-index variable y_j, and w is x_i, y_j, x_i - y_j or y_j - x_i: the
    gradients of radial and scalar-product kernels with respect to their points (Grad of Exp(-g*SqDist(x,y))*b with
    respect to x is -2 g <e_i, b_j> K_ij (x_i - y_j)).  The long vectors outside the contraction keep such formulas
    off the chunked scheme (Chunk_Mode_Constants.py:56-60) and on a kernel that holds whole rows per lane, but

        sum_j g_ij (a x_i + c y_j) = a x_i sum_j g_ij + c sum_j g_ij y_j

    is one scalar chunked reduction and matrix-core weighted sums of column slices of y.  Returns None or a dict
    with sign, G (the scalar formula), row / col (the variables) and their coefficients a, c."""
    from .formulas import ops as O

    if not enable_chunks or enable_chunks < 0 or not isinstance(red, Sum_Reduction) or dtype != "float" or not use_fast_math:
        return None
    F, sign = red.formula, 1
    while F.name == "Minus":
        F, sign = F.children[0], -sign
    if F.name != "Mult" or len(F.children) != 2:
        return None
    for G, W in (F.children, F.children[::-1]):
        if G.dim != 1 or W.dim < config.chunk_min_dim:
            continue
        wsign = 1
        while W.name == "Minus":
            W, wsign = W.children[0], -wsign
        if isinstance(W, O.Var):
            terms = [(1, W)]
        elif W.name in ("Subtract", "Add") and all(isinstance(c, O.Var) for c in W.children):
            terms = [(1, W.children[0]), (-1 if W.name == "Subtract" else 1, W.children[1])]
        else:
            continue
        m = match_chunk(Sum_Reduction(G, red.tagI), dtype, "GpuReduc1D", use_fast_math)
        if m is None:
            continue
        _, _, row, col = m
        if any(v != row and v != col for _, v in terms) or len({v for _, v in terms}) != len(terms):
            continue
        coef = {v: c for c, v in terms}
        return dict(sign=sign * wsign, G=G, row=row, col=col, a=coef.get(row, 0), c=coef.get(col, 0))
    return None


def generate_chunk_plugin(red, match, dtypeacc, sum_scheme, nargs, irregular=False, half_data=False):
    """Module source for the matrix-core chunked scheme (kernels/keops_chunk_mfma.h); ``irregular``: the
    block-sparse / batched variant (GpuReduc1D_ranges_chunks.py:21-183)."""
    from .formulas import ops as O
    from .formulas.reductions import Reduction

    from .formulas.reductions import KIND_SUM

    mode, node, xvar, yvar = match
    svar = O.Var(1 << 30, 1, 3)
    post = red.formula.replace(node, svar)
    # beyond 256 components the split operands of 32 output rows no longer fit the registers of one wavefront:
    # nc wavefronts share the rows, each contracts 1/nc of the components, partial tiles meet in LDS
    nc = 1 if xvar.dim <= 256 else (2 if xvar.dim <= 512 else 4)
    # post-chunk formula g(s, ...) * v_j of a float32 Sum: the product with v also runs on the matrix cores
    final = None
    if (nc == 1 and red.kind == KIND_SUM and dtypeacc == "float" and sum_scheme in ("block_sum", "direct_sum")
            and post.name == "Mult" and len(post.children) == 2):
        for g, v in (post.children, post.children[::-1]):
            if (g.dim == 1 and isinstance(v, O.Var) and v.cat == 1 - red.tagI and v.dim == post.dim
                    and v.dim <= (64 if xvar.dim > 128 else 128)):
                final = (g, v)
                break
    # post-chunk formulas [F'(s, ...), v_j] or [F', 1, v_j] of a float32 log-sum-exp family reduction: online softmax
    # with the weighted sum on the matrix cores
    from .formulas.reductions import KIND_LSE

    softmax = None
    if nc == 1 and red.kind == KIND_LSE and dtypeacc == "float" and sum_scheme != "kahan_scheme" and post.name == "Concat":
        Fp, G = post.children
        one = 0
        if G.name == "Concat" and isinstance(G.children[0], O.IntCst) and G.children[0].val == 1:
            one, G = 1, G.children[1]
        if Fp.dim == 1 and isinstance(G, O.Var) and G.cat == 1 - red.tagI and G.dim <= (64 if xvar.dim > 128 else 128):
            softmax = (Fp, G, one)
    full_post = post
    if final is not None:
        post = final[0]
    elif softmax is not None:
        post = softmax[0]
    wvar = final[1] if final is not None else (softmax[1] if softmax is not None else None)

    class _Post:  # what VarLayout needs: the post-chunk formula with the reduction's orientation
        formula, tagI = post, red.tagI

    layout = VarLayout(_Post)
    layout.names[(3, svar.ind, 0)] = "s"
    L = Lir(row_cat=red.tagI, fast_math=True, dtype="float")
    outs = lower(post, L)
    lines, exprs = L.emit(outs, layout.names, indent="    ")
    D = xvar.dim
    dpad = -(-D // (16 * nc)) * 16 * nc
    dimy_pad = 0 if layout.dimy == 0 else -(-layout.dimy // 4) * 4
    waves = config.chunk_waves
    split3 = int(wvar is not None and config.final_split3)
    # LDS of the kernel: staged tile (hi|lo rows), the other reduced-index variables, and either the v tile
    # (final-product variant) or the accumulator exchange of the two lanes of a row
    def lds_bytes(w):
        tile = 32 * (dpad * 4 + 16)
        fixed = 128 + 32 * max(1, dimy_pad) * 4
        if wvar is not None:
            vtile = 3 * (-(-wvar.dim // 32)) * 32 * 40 * 2 if split3 else 32 * (-(-wvar.dim // 32)) * 32 * 4
            return tile + fixed + vtile + 128 * w
        # the accumulator exchange reuses the memory of the staged tile
        merge = (32 * w // nc) * (2 * nc - 1) * red.dimred * (8 if dtypeacc == "double" else 4)
        return max(tile, merge) + fixed + (w * 16 * 64 * 4 if nc > 1 else 0)
    while waves > nc and lds_bytes(waves) > config.knn_lds_budget:
        waves //= 2
    if waves < nc or lds_bytes(waves) > config.knn_lds_budget:
        return None, None
    ra, rd, ro = VarLayout.table(layout.rowvars)
    ca, cd, co = VarLayout.table(layout.colvars)
    pa, pd, po = VarLayout.table(layout.parvars)
    ncol_extra = 1 + (1 if wvar is not None and wvar not in layout.colvars else 0)
    meta = dict(scheme="chunk", block=64 * waves, rows=1, tile_j=32, dimred=red.dimred, dimout=red.dim, sizeof_t=4,
                sizeof_acc=8 if dtypeacc == "double" else 4, nrowvars=len(layout.rowvars) + 1,
                ncolvars=len(layout.colvars) + ncol_extra, nparvars=len(layout.parvars), chk_d=D, chk_dpad=dpad,
                chk_mode=mode, chk_qb=32 * waves // nc, chk_final=int(final is not None), chk_softmax=int(softmax is not None),
                chk_xarg=xvar.ind, chk_yarg=yvar.ind, ranges=int(irregular), chk_split3=int(split3 and config.chunk_presplit),
                chk_vcols=0 if wvar is None else -(-wvar.dim // 32) * 32, nops=L.count_ops(outs),
                chk_single=int(bool(half_data)), chk_robust=int(config.chunk_robust and not half_data))
    src = ["//@keops " + " ".join(f"{k}={v}" for k, v in meta.items()), f"// reduction: {red!r}",
           f"typedef float T;\ntypedef {dtypeacc} TACC;", f"#define KEOPS_MC_RANGES {int(irregular)}",
           '#include "keops_common.h"']
    defs = dict(
        KEOPS_NARGS=nargs, CHK_D=D, CHK_DPAD=dpad, CHK_MODE=mode, CHK_XARG=xvar.ind, CHK_YARG=yvar.ind, CHK_WAVES=waves, CHK_NC=nc,
        CHK_ROBUST=int(config.chunk_robust),
        KEOPS_DIMX=layout.dimx, KEOPS_DIMY=layout.dimy, KEOPS_DIMY_PAD=dimy_pad, KEOPS_DIMP=layout.dimp,
        KEOPS_DIMFOUT=post.dim, KEOPS_DIMRED=red.dimred, KEOPS_DIMOUT=red.dim, KEOPS_RED_KIND=red.kind,
        KEOPS_RED_KEEP=red.keep, KEOPS_RED_K=red.K, KEOPS_SUM_SCHEME=SUM_SCHEMES[sum_scheme],
        KEOPS_NROWVARS=len(layout.rowvars), KEOPS_NCOLVARS=len(layout.colvars), KEOPS_NPARVARS=len(layout.parvars),
    )
    if final is not None:
        defs.update(KEOPS_DIMFOUT=full_post.dim, CHK_FINAL=1, CHK_FV_ARG=final[1].ind, CHK_FV_DIM=final[1].dim,
                    CHK_FNB=-(-final[1].dim // 32), CHK_PERIOD=config.final_period,
                    CHK_BLOCKSUM=int(sum_scheme == "block_sum"))
    elif softmax is not None:
        defs.update(KEOPS_DIMFOUT=full_post.dim, CHK_SOFTMAX=1, CHK_SM_ONE=softmax[2], CHK_FV_ARG=softmax[1].ind,
                    CHK_FV_DIM=softmax[1].dim, CHK_FNB=-(-softmax[1].dim // 32))
    near = (0.125 if D < 32 else 0.25) if config.chunk_near == "auto" else float(config.chunk_near)
    if half_data:
        # half-precision data: exact products of single terms, no centring; the expansion of a squared distance is off
        # by 2^-24 of the norms only, so far fewer values need the recomputation (and uncentred norms are large)
        near = min(near, 1.0 / 256)
        defs["CHK_SINGLE"] = 1
    defs["CHK_NEAR"] = f"{near!r}f"
    defs["CHK_SPLIT3"] = split3
    defs["CHK_WTERMS"] = int(config.final_weight_terms)
    defs["CHK_PRESPLIT"] = int(config.chunk_presplit)
    src += [f"#define {k} {v}" for k, v in defs.items()]
    for name, vals in (("row_arg", ra), ("row_dim", rd), ("row_off", ro), ("col_arg", ca), ("col_dim", cd),
                       ("col_off", co), ("par_arg", pa), ("par_dim", pd), ("par_off", po)):
        src.append(f"static __device__ constexpr int keops_{name}[] = {_c_list(vals)};")
    dx, dy, dp = max(1, layout.dimx), max(1, dimy_pad), max(1, layout.dimp)
    src.append("struct KeopsFormula {")
    src.append(f"  static __device__ __forceinline__ void eval(const T (&xi)[{dx}], const T (&yj)[{dy}], "
               f"const T (&p)[{dp}], const T s, T (&fout)[{post.dim}]) {{")
    src += lines + [f"    fout[{k}] = {e};" for k, e in enumerate(exprs)]
    src.append("  }\n};")
    src.append('#include "keops_chunk_mfma.h"')
    return "\n".join(src) + "\n", meta


def generate_chunk64_plugin(red, match, sum_scheme, nargs, irregular=False):
    """Module source for the float64 matrix-core chunked scheme (kernels/keops_chunk_f64.h): the contraction on
    v_mfma_f64_16x16x4_f64, the post-chunk formula in double precision on the vector ALU; ``irregular``: the
    block-sparse / batched variant."""
    from .formulas import ops as O

    mode, node, xvar, yvar = match
    svar = O.Var(1 << 30, 1, 3)
    post = red.formula.replace(node, svar)

    class _Post:  # what VarLayout needs: the post-chunk formula with the reduction's orientation
        formula, tagI = post, red.tagI

    layout = VarLayout(_Post)
    layout.names[(3, svar.ind, 0)] = "s"
    L = Lir(row_cat=red.tagI, fast_math=True, dtype="double")
    outs = lower(post, L)
    lines, exprs = L.emit(outs, layout.names, indent="    ")
    D = xvar.dim
    dpad = -(-D // 8) * 8
    dimy_pad = 0 if layout.dimy == 0 else -(-layout.dimy // 2) * 2
    waves = 8
    rb = 2 if dpad <= 128 else 1   # 16-row blocks per wavefront: the operands of 2 x 128 or 1 x 256 components take 128 registers
    lds = 32 * (dpad * 8 + 16) + 32 * 8 + 32 * max(1, dimy_pad) * 8
    if max(lds, 8 * 16 * rb * waves * 3 * red.dimred) > config.knn_lds_budget:
        return None, None
    ra, rd, ro = VarLayout.table(layout.rowvars)
    ca, cd, co = VarLayout.table(layout.colvars)
    pa, pd, po = VarLayout.table(layout.parvars)
    meta = dict(scheme="chunk64", block=64 * waves, rows=1, tile_j=32, dimred=red.dimred, dimout=red.dim, sizeof_t=8,
                sizeof_acc=8, nrowvars=len(layout.rowvars) + 1, ncolvars=len(layout.colvars) + 1,
                nparvars=len(layout.parvars), chk_d=D, chk_dpad=dpad, chk_mode=mode, chk_qb=16 * rb * waves,
                chk_xarg=xvar.ind, chk_yarg=yvar.ind, ranges=int(irregular), nops=L.count_ops(outs))
    src = ["//@keops " + " ".join(f"{k}={v}" for k, v in meta.items()), f"// reduction: {red!r}",
           "typedef double T;\ntypedef double TACC;", f"#define KEOPS_MC_RANGES {int(irregular)}",
           '#include "keops_common.h"']
    defs = dict(
        KEOPS_NARGS=nargs, CHK_D=D, CHK_DPAD=dpad, CHK_MODE=mode, CHK_XARG=xvar.ind, CHK_YARG=yvar.ind, CHK_WAVES=waves, CHK_RB=rb,
        KEOPS_DIMX=layout.dimx, KEOPS_DIMY=layout.dimy, KEOPS_DIMY_PAD=dimy_pad, KEOPS_DIMP=layout.dimp,
        KEOPS_DIMFOUT=post.dim, KEOPS_DIMRED=red.dimred, KEOPS_DIMOUT=red.dim, KEOPS_RED_KIND=red.kind,
        KEOPS_RED_KEEP=red.keep, KEOPS_RED_K=red.K, KEOPS_SUM_SCHEME=SUM_SCHEMES[sum_scheme],
        KEOPS_NROWVARS=len(layout.rowvars), KEOPS_NCOLVARS=len(layout.colvars), KEOPS_NPARVARS=len(layout.parvars),
    )
    src += [f"#define {k} {v}" for k, v in defs.items()]
    for name, vals in (("row_arg", ra), ("row_dim", rd), ("row_off", ro), ("col_arg", ca), ("col_dim", cd),
                       ("col_off", co), ("par_arg", pa), ("par_dim", pd), ("par_off", po)):
        src.append(f"static __device__ constexpr int keops_{name}[] = {_c_list(vals)};")
    dx, dy, dp = max(1, layout.dimx), max(1, dimy_pad), max(1, layout.dimp)
    src.append("struct KeopsFormula {")
    src.append(f"  static __device__ __forceinline__ void eval(const T (&xi)[{dx}], const T (&yj)[{dy}], "
               f"const T (&p)[{dp}], const T s, T (&fout)[{post.dim}]) {{")
    src += lines + [f"    fout[{k}] = {e};" for k, e in enumerate(exprs)]
    src.append("  }\n};")
    src.append('#include "keops_chunk_f64.h"')
    return "\n".join(src) + "\n", meta


def match_final(red, dtype, dtypeacc, sum_scheme, map_reduce_id, use_fast_math=True):
    """(scalar kernel f, variable v) when ``red`` is Sum_Reduction(f * v) with f of dimension 1 and v a
    plain reduced-index variable of dimension >= config.final_chunk_min_dim (24), in float32 on the dense
    scheme (the shape GpuReduc1D_finalchunks.py:100-106 expects); None otherwise.  The scheme evaluates f with the
    hardware's fast exp / sqrt / reciprocal and forms the product from bfloat16 terms: use_fast_math=False keeps
    such formulas on the exact vector kernel."""
    from .formulas import ops as O
    from .formulas.reductions import KIND_SUM

    if red.kind != KIND_SUM or dtype != "float" or dtypeacc not in ("float", "double") or not use_fast_math:
        return None
    if sum_scheme not in ("block_sum", "direct_sum", "kahan_scheme"):
        return None
    # sums kept in double (dtype_acc = float64; the Kahan scheme is served the same way): dense launches only
    if (dtypeacc == "double" or sum_scheme == "kahan_scheme") and "_ranges" in map_reduce_id:
        return None
    F = red.formula
    if F.name != "Mult" or len(F.children) != 2:
        return None
    for f, v in (F.children, F.children[::-1]):
        if f.dim == 1 and isinstance(v, O.Var) and v.cat == 1 - red.tagI and v.dim == F.dim and v.dim >= config.final_chunk_min_dim:
            # a 32-column matrix tile costs as much as ~22 vector multiply-adds per pair: just above a
            # multiple of 32 the vector kernel is still the faster one
            if v.dim > 32 and v.dim % 32 != 0 and v.dim % 32 < 8 and v.dim < 128:
                return None
            return f, v
    return None


def generate_final_plugin(red, match, sum_scheme, nargs, irregular=False, acc64=False):
    """Module source for the matrix-core final-product scheme (kernels/keops_final_mfma.h); ``irregular``: the
    block-sparse / batched variant (GpuReduc1D_ranges_finalchunks.py:20-91); ``acc64``: the register tiles are folded
    into double sums every ``config.final_period_acc64`` reduced rows."""
    f, vvar = match
    acc64 = bool(acc64) and not irregular

    class _Inner:  # what VarLayout needs: the scalar kernel with the reduction's orientation
        formula, tagI = f, red.tagI

    layout = VarLayout(_Inner)
    L = Lir(row_cat=red.tagI, fast_math=True, dtype="float")
    outs = lower(f, L)
    lines, exprs = L.emit(outs, layout.names, indent="    ")
    dimy_pad = 0 if layout.dimy == 0 else -(-layout.dimy // 4) * 4
    nbtot = -(-vvar.dim // 32)
    nb = min(nbtot, config.final_max_blocks)
    # balance the column blocks over the workgroups that share a row block
    nz = -(-nbtot // nb)
    nb = -(-nbtot // nz)
    waves, tj = config.final_waves, config.final_tile_j
    ra, rd, ro = VarLayout.table(layout.rowvars)
    ca, cd, co = VarLayout.table(layout.colvars)
    pa, pd, po = VarLayout.table(layout.parvars)
    meta = dict(scheme="final", block=64 * waves, rows=1, tile_j=tj, dimred=red.dimred, dimout=red.dim, sizeof_t=4,
                sizeof_acc=8 if acc64 else 4, nrowvars=len(layout.rowvars), ncolvars=len(layout.colvars) + (0 if vvar in layout.colvars else 1),
                nparvars=len(layout.parvars), fin_dv=vvar.dim, fin_varg=vvar.ind, fin_nb=nb, fin_nz=nz, fin_qb=32 * waves, ranges=int(irregular),
                fin_acc64=int(acc64),
                fin_split3=int(config.final_split3 and tj % 16 == 0),
                nops=L.count_ops(outs))
    src = ["//@keops " + " ".join(f"{k}={v}" for k, v in meta.items()), f"// reduction: {red!r}",
           f"typedef float T;\ntypedef {'double' if acc64 else 'float'} TACC;", f"#define KEOPS_MC_RANGES {int(irregular)}",
           '#include "keops_common.h"']
    defs = dict(
        KEOPS_NARGS=nargs, FIN_DV=vvar.dim, FIN_VARG=vvar.ind, FIN_NB=nb, FIN_WAVES=waves, FIN_TJ=tj,
        FIN_PERIOD=config.final_period_acc64 if acc64 else config.final_period,
        FIN_BLOCKSUM=int(sum_scheme == "block_sum" or acc64), FIN_ACC64=int(acc64),
        FIN_SPLIT3=int(config.final_split3 and tj % 16 == 0),
        KEOPS_DIMX=layout.dimx, KEOPS_DIMY=layout.dimy, KEOPS_DIMY_PAD=dimy_pad, KEOPS_DIMP=layout.dimp,
        KEOPS_NROWVARS=len(layout.rowvars), KEOPS_NCOLVARS=len(layout.colvars), KEOPS_NPARVARS=len(layout.parvars),
    )
    src += [f"#define {k} {v}" for k, v in defs.items()]
    for name, vals in (("row_arg", ra), ("row_dim", rd), ("row_off", ro), ("col_arg", ca), ("col_dim", cd),
                       ("col_off", co), ("par_arg", pa), ("par_dim", pd), ("par_off", po)):
        src.append(f"static __device__ constexpr int keops_{name}[] = {_c_list(vals)};")
    dx, dy, dp = max(1, layout.dimx), max(1, dimy_pad), max(1, layout.dimp)
    src.append("struct KeopsFormula {")
    src.append(f"  static __device__ __forceinline__ void eval(const T (&xi)[{dx}], const T (&yj)[{dy}], "
               f"const T (&p)[{dp}], T (&fout)[1]) {{")
    src += lines + [f"    fout[{k}] = {e};" for k, e in enumerate(exprs)]
    src.append("  }\n};")
    src.append('#include "keops_final_mfma.h"')
    return "\n".join(src) + "\n", meta


def _linear_coef(E, svar):
    """Uniform (parameter-only) formula C with E = C * svar, or None when E is not of that form."""
    from .formulas import ops as O

    def uniform(f):
        return all(v.cat == 2 for v in f.variables)

    if E == svar:
        return O.IntCst(1)
    if E.name == "Minus":
        c = _linear_coef(E.children[0], svar)
        return None if c is None else O.Minus(c)
    if E.name == "Mult" and len(E.children) == 2:
        for a, b in (E.children, E.children[::-1]):
            if uniform(a) and a.dim == 1:
                c = _linear_coef(b, svar)
                if c is not None:
                    return O.Mult(a, c)
    if E.name == "Divide" and len(E.children) == 2:
        a, b = E.children
        if uniform(b) and b.dim == 1:
            c = _linear_coef(a, svar)
            if c is not None:
                return O.Divide(c, b)
    return None


def match_radial(red, dtype, dtypeacc, sum_scheme, use_fast_math, map_reduce_id, pairs=0, block_sparse=False, batch_total=0):
    """dict(x, y, coef, A, W, diff) when the formula of a float32 Sum reduction on the dense scheme is a product

        [+-]  A(i-variables)  *  Exp(C * SqDist(x, y))  *  W(j-variables)  [ * (x - y) | (y - x) ]

    with x an output-indexed and y a reduced-index variable of at most config.radial_max_dim (8) components, C a scalar
    formula of the parameters, A scalar, W of at most config.radial_max_dv (8) components (scalar when the difference
    factor is present): the Gaussian kernel sums and their gradients with respect to the points and the weights.  Here
    "i" means indexed like the output.  One factor may be a scalar product <u_i, v_j> of an output-indexed and a
    reduced-index vector: the sums are then accumulated per component of v_j and contracted with u_i once per output
    row.  Such sums take their exponents from the matrix cores
    (kernels/keops_radial_mfma.h) when the data allow it; with the difference factor, the kernel accumulates
    sum_j K_ij w_j [y^_j, 1] and the last pass forms A_i (x^_i S - sum_j K_ij w_j y^_j) for the points centred on the
    mean of y.  ``pairs``: when not 0, the call holds less than 2**pairs pairs; small calls stay on the
    general-purpose kernel alone, whose fixed cost is lower."""
    from .formulas import ops as O
    from .formulas.reductions import KIND_SUM

    if (not config.radial or red.kind != KIND_SUM or dtype != "float" or dtypeacc != "float" or not use_fast_math
            or sum_scheme == "kahan_scheme"):
        return None
    # launches with ranges: block-sparse patterns without batch dimensions, where every row range gets its own centre,
    # and batches that no variable is broadcast over (``batch_total``: log2 bucket of their pairs together), which
    # are row ranges with one reduced range each
    if "_ranges" in map_reduce_id:
        if not config.radial_ranges or not (block_sparse or batch_total):
            return None
        if not block_sparse:
            pairs = batch_total
    if pairs and int(pairs) < (config.radial_ranges_min_pairs_log2 if "_ranges" in map_reduce_id else config.radial_min_pairs_log2):
        return None
    row_cat, col_cat = red.tagI, 1 - red.tagI
    # the factors of the product, signs and scalar constants pulled out
    sign, factors, stack = 1, [], [red.formula]
    while stack:
        f = stack.pop()
        if f.name == "Minus":
            sign = -sign
            stack.append(f.children[0])
        elif f.name == "Mult" and len(f.children) == 2:
            stack.extend(f.children[::-1])
        else:
            factors.append(f)
    exps = [f for f in factors if f.name == "Exp" and f.depends_on_cat(0) and f.depends_on_cat(1)]
    if len(exps) != 1 or exps[0].dim != 1:
        return None
    E = exps[0].children[0]
    found = []
    for node in E.walk():
        if node.name == "Sum" and node.children[0].name == "Square" and node.children[0].children[0].name == "Subtract":
            a, b = node.children[0].children[0].children
            if (isinstance(a, O.Var) and isinstance(b, O.Var) and a.dim == b.dim and 1 <= a.dim <= config.radial_max_dim
                    and {a.cat, b.cat} == {0, 1} and node not in [f[0] for f in found]):
                found.append((node, a, b))
    if len(found) != 1:
        return None
    node, a, b = found[0]
    svar = O.Var(1 << 30, 1, 3)
    coef = _linear_coef(E.replace(node, svar), svar)
    if coef is None:
        return None
    x, y = (a, b) if a.cat == row_cat else (b, a)
    A, Wf, diff, U = [], [], 0, None
    for f in factors:
        if f is exps[0]:
            continue
        if f.name == "Subtract" and set(f.children) == {x, y} and f.dim == x.dim and x.dim > 1:
            if diff:
                return None
            diff = 1 if f.children[0] == x else -1
        elif (f.name == "Scalprod" and len(f.children) == 2 and U is None and f.children[0].dim == f.children[1].dim > 1
              and any(not c.depends_on_cat(col_cat) and c.depends_on_cat(row_cat) for c in f.children)
              and any(not c.depends_on_cat(row_cat) and c.depends_on_cat(col_cat) for c in f.children)):
            # <u_i, v_j>: the sums are accumulated per component of v_j, u_i contracts them once per output row
            u, v = f.children if f.children[0].depends_on_cat(row_cat) else f.children[::-1]
            U = u
            Wf.append(v)
        elif not f.depends_on_cat(col_cat) and f.depends_on_cat(row_cat):
            if f.dim != 1:
                return None
            A.append(f)
        elif not f.depends_on_cat(row_cat):
            Wf.append(f)
        else:
            return None  # a factor of both indices other than the exponential
    vec = [f for f in Wf if f.dim != 1]
    if len(vec) > 1 or (diff and vec and U is None):
        return None
    dimw = vec[0].dim if vec else 1

    def fits(n):  # accumulated components per pair
        return 1 <= n <= max(config.radial_max_dv, config.radial_mm_max_dv if config.radial_mm_min_dv <= n else 0)

    if diff:
        # (with vector weights the general-purpose kernel contracts <u_i, v_j> first and keeps D sums per pair, while
        # this family keeps dim(v) (D + 1): measured, it only wins while the fused-multiply-add variant holds them)
        # beyond 8 sums the sweep forms <u_i, v_j> per pair itself and keeps D + 1 sums (u_i of its rows in registers)
        if red.formula.dim != x.dim or x.dim + 1 > config.radial_max_dv:
            return None
        if U is not None and dimw * (x.dim + 1) > config.radial_max_dv and dimw > max(config.radial_upair_max_dw,
                                                                                         config.radial_bilinear_max_dw if config.radial_bilinear else 0):
            return None
        if U is None and not fits(x.dim + 1):
            return None
    elif U is not None:
        if red.formula.dim != 1 or not fits(dimw):
            return None
    elif dimw != red.formula.dim or not fits(dimw):
        return None

    def product(fs):
        out = None
        for f in sorted(fs, key=lambda f: f.dim):  # scalars first: one multiplication per component at the end
            out = f if out is None else O.Mult(out, f)
        return out

    return dict(x=x, y=y, coef=coef, A=product(A), W=product(Wf), diff=diff, sign=sign, U=U)


def generate_radial_section(red, match, nargs, rows_per_block=0):
    """Source text appended to a general-purpose module: tables, the straight-line bodies of struct
    KeopsRadFormula and the template kernels/keops_radial_mfma.h; returns (text, meta entries).
    ``rows_per_block`` > 0: block-sparse variant (kernels/keops_radial_ranges.h), whose workgroups own that many rows,
    like the general-purpose kernel of the same module: both read one lookup table."""
    from .formulas import ops as O
    from .formulas.lir import LOG2E

    x, y, coef, A, W, diff, sign = (match[k] for k in ("x", "y", "coef", "A", "W", "diff", "sign"))
    U = match.get("U")                 # row factor u_i of a scalar product <u_i, v_j> (v_j is then the vector in W)
    D = x.dim
    dimw = 1 if W is None else W.dim
    du = 0 if U is None else U.dim
    # a factor <u_i, v_j>: out of the matrix cores like the exponent when its term products fit the slot vectors
    # (decided below, once the exponent's slots are counted), else expanded per component of v_j or formed per pair
    bil = 0
    upair = int(bool(diff and U is not None and dimw * (D + 1) > config.radial_max_dv))  # <u_i, v_j> formed per pair
    Dv = (D + 1 if upair else dimw * (D + 1)) if diff else dimw   # components accumulated per pair
    dout = D if diff else (1 if U is not None else dimw)          # components of the output
    # slots of the scalar product, by decreasing magnitude: (row term, column term) of every component, the terms
    # of the two squared norms against 1.  kind 0: zero, 1: one, 2: component term (comp, term), 3: norm term
    H, Mi, Lo = 0, 1, 2
    rows, cols = [], []

    def prod(tr, tc):
        for k in range(D):
            rows.append((2, k, tr))
            cols.append((2, k, tc))

    def norm(n):
        rows.append((3, 0, n)); cols.append((1, 0, 0))
        rows.append((1, 0, 0)); cols.append((3, 0, n))

    def pad(mult):
        while len(rows) % mult:
            rows.append((0, 0, 0)); cols.append((0, 0, 0))

    prod(H, H); norm(0)
    if D + 2 <= 8:
        pad(8)  # the big terms, which cancel, share one 8-slot group: the hardware adds a group exactly
    prod(H, Mi); prod(Mi, H); norm(1)
    prod(Mi, Mi); prod(H, Lo); prod(Lo, H); norm(2)
    prod(Mi, Lo); norm(3)
    pad(16)
    nkb = nke = len(rows) // 16
    if nkb > 4:
        return None, None
    # (with the difference factor only: a plain sum over <u_i, v_j> is cheaper expanded per component of v_j, 15.0
    # against 16.8 ms at three components)
    if U is not None and diff and config.radial_bilinear and dimw <= config.radial_bilinear_max_dw and nke + -(-6 * dimw // 16) <= config.radial_bilinear_max_nkb:
        # slot kind 4: term of a component of u_i (rows) / v_j (columns); six term products per component
        bil, upair = 1, 0
        for tr, tc in ((H, H), (H, Mi), (Mi, H), (Mi, Mi), (H, Lo), (Lo, H)):
            for k in range(dimw):
                rows.append((4, k, tr))
                cols.append((4, k, tc))
        pad(16)
        nkb = len(rows) // 16
        Dv = D + 1 if diff else 1
    # output rows per wavefront (32-row blocks) and wavefronts per workgroup: the accumulators (16 per block and
    # accumulated component) live in registers
    # from config.radial_mm_min_dv accumulated components on, the weighted sum runs on the matrix cores too (the three
    # bfloat16 terms of the weights side by side in the 32 operand columns): 16 accumulators per block of 32 rows
    if upair and dimw > config.radial_upair_max_dw:
        return None, None  # too wide for the per-pair form, and the slot vectors had no room
    mm = int(config.radial_mm_min_dv <= Dv <= config.radial_mm_max_dv and not upair and not bil)
    if Dv > config.radial_max_dv and not mm:
        return None, None  # the accumulators of that many components do not fit the registers
    rb = (config.radial_mm_rb if mm else 2) if (mm or Dv <= config.radial_rb2_max_dv) else 1
    if upair:
        rb = 1  # 16 x dim(u) registers per 32-row block hold the row factors
    tj = ((256 if mm else 512) if config.radial_tile_j == "auto" else int(config.radial_tile_j))
    if tj % 32 or not 32 <= tj <= 1024:
        raise ValueError("[KeOps] KEOPS_AMD_RADIAL_TJ must be a multiple of 32 between 32 and 1024")
    waves = 8
    if rows_per_block:
        if rows_per_block % (32 * rb) or not 2 <= rows_per_block // (32 * rb) <= 16:
            return None, None
        waves = rows_per_block // (32 * rb)
    one = O.IntCst(1)

    class _W:
        formula, tagI = (W if W is not None else one), red.tagI

    class _A:
        formula, tagI = (A if A is not None else one), red.tagI

    class _AU:  # the variables of both row factors share one table
        formula, tagI = (_A.formula if U is None else O.Mult(_A.formula, O.Sum(U))), red.tagI

    wl, al = VarLayout(_W), VarLayout(_AU)
    if wl.rowvars or al.colvars:
        return None, None
    # the parameter table serves every body: the one of the whole reduction (as the general-purpose kernel's)
    full = VarLayout(red)
    pnames = {key: name for key, name in full.names.items() if key[0] == 2}

    def body(formula, names):
        L = Lir(row_cat=red.tagI, fast_math=True, dtype="float")
        nm = dict(names)
        nm.update(pnames)
        lines, exprs = L.emit(lower(formula, L), nm, indent="    ")
        return list(L.prelude), lines, exprs

    w_pre, w_lines, w_exprs = body(_W.formula, wl.names)
    a_pre, a_lines, a_exprs = body(_A.formula, al.names)
    u_pre, u_lines, u_exprs = body(U, al.names) if U is not None else ([], [], [])
    k_pre, k_lines, k_exprs = body(coef, {})
    ca, cd, co = VarLayout.table(wl.colvars)
    ra, rd, ro = VarLayout.table(al.rowvars)
    meta = dict(radial=1, rad_ranges=int(bool(rows_per_block)), rad_mm=mm, rad_mm_nb=-(-3 * Dv // 32), rad_ws=(dimw + D + 1 if upair else Dv), rad_bil=bil, rad_d=D, rad_dv=Dv, rad_dout=dout, rad_nkb=nkb, rad_rb=rb, rad_waves=waves, rad_xarg=x.ind,
                rad_yarg=y.ind, rad_tj=tj,
                rad_exact_xw=-(-D // 4) * 4 * (2 if diff else 1) + -(-dimw // 4) * 4)
    src = ["", "// ---- exponents of the radial kernel on the matrix cores (kernels/keops_radial_mfma.h) ----"]
    defs = dict(RAD_RANGES=int(bool(rows_per_block)), RAD_MM=mm, RAD_MM_TERMS=int(config.radial_mm_terms), RAD_TJ=tj, RAD_D=D, RAD_DV=Dv, RAD_DW=dimw, RAD_DU=du, RAD_UPAIR=upair, RAD_BIL=bil, RAD_NKE=nke, RAD_DOUT=dout, RAD_DIFF=diff, RAD_SIGN=f"{float(sign)!r}f", RAD_NKB=nkb,
                RAD_RB=rb, RAD_WAVES=waves, RAD_XARG=x.ind, RAD_YARG=y.ind, RAD_LIMIT=f"{float(config.radial_limit if not rows_per_block else config.radial_ranges_limit)!r}f", RAD_EXACT_FRAC=f"{float(config.radial_exact_frac)!r}f",
                RAD_NCOLVARS=len(wl.colvars), RAD_DIMY=wl.dimy, RAD_NROWVARS=len(al.rowvars), RAD_DIMX=al.dimx)
    src += [f"#define {k} {v}" for k, v in defs.items()]
    for name, vals in (("row_kind", [r[0] for r in rows]), ("row_comp", [r[1] for r in rows]), ("row_term", [r[2] for r in rows]),
                       ("col_kind", [c[0] for c in cols]), ("col_comp", [c[1] for c in cols]), ("col_term", [c[2] for c in cols]),
                       ("col_arg", ca), ("col_dim", cd), ("col_off", co), ("row_arg", ra), ("row_dim", rd), ("row_off", ro)):
        src.append(f"static __device__ constexpr int rad_{name}[] = {_c_list(vals)};")
    dy, dx, dp = max(1, wl.dimy), max(1, al.dimx), max(1, full.dimp)
    src += w_pre + a_pre + u_pre + k_pre
    src.append("struct KeopsRadFormula {")
    src.append("  // the coefficient of the squared distance in the exponent")
    src.append(f"  static __device__ __forceinline__ T coef(const T (&p)[{dp}]) {{")
    src += k_lines
    src.append(f"    return {k_exprs[0]};")
    src.append("  }")
    src.append("  // log2(e) times that coefficient")
    src.append(f"  static __device__ __forceinline__ T kappa(const T (&p)[{dp}]) {{")
    src += k_lines
    src.append(f"    return ({k_exprs[0]}) * {LOG2E!r}f;")
    src.append("  }")
    src.append("  // factors that depend on the reduced index: the weights of a column")
    src.append(f"  static __device__ __forceinline__ void weights(const T (&yj)[{dy}], const T (&p)[{dp}], T (&w)[{dimw}]) {{")
    src += w_lines + [f"    w[{k}] = {e};" for k, e in enumerate(w_exprs)]
    src.append("  }")
    src.append("  // factors that depend on the output index: applied once per output row")
    src.append(f"  static __device__ __forceinline__ T rowscale(const T (&xi)[{dx}], const T (&p)[{dp}]) {{")
    src += a_lines
    src.append(f"    return {a_exprs[0]};")
    src.append("  }")
    if U is not None:
        src.append("  // row factor of a scalar product with the weights: contracts the accumulated sums once per output row")
        src.append(f"  static __device__ __forceinline__ void rowvec(const T (&xi)[{dx}], const T (&p)[{dp}], T (&u)[{du}]) {{")
        src += u_lines + [f"    u[{k}] = {e};" for k, e in enumerate(u_exprs)]
        src.append("  }")
    src.append("};")
    src.append('#include "keops_radial_mfma.h"')
    return "\n".join(src) + "\n", meta


def get_keops_dll(
    map_reduce_id, red_formula_string, enable_chunks, enable_finalchunks, mul_var_highdim, aliases, nargs, dtype,
    dtypeacc, sum_scheme_string, tagHostDevice, tagCPUGPU, tag1D2D, use_half, use_fast_math, device_id, nx=None,
    batch_loop=0, pairs=0, batch_total=0,
):
    """Same arguments and same 19-tuple as the reference's get_keops_dll (get_keops_dll.py:78-159),
    plus ``nx``: the number of output rows of the call being prepared, used to pick the number of
    rows per lane, and ``batch_loop``: when not 0, the "_ranges" of the scheme id stand for a few batches
    of less than 2**batch_loop pairs each without block-sparse ranges, which a dense module may serve one batch
    at a time; ``pairs``: when not 0, the call (each batch of it) holds less than 2**pairs pairs; ``batch_total``: when
    not 0, all batches together hold less than 2**batch_total pairs and no variable is broadcast over a batch dimension.  ``dtype`` / ``dtypeacc`` are C
    type names ("float" | "double").  ``use_half``: the data are half-precision numbers (converted to float32 copies by
    the library before the launch): modules are compiled for float, and the chunked matrix-core scheme keeps one
    half-precision term per component instead of two."""
    if dtype not in ("float", "double") or (use_half and dtype != "float"):
        raise ValueError("[KeOps] the HIP backend computes in float32 (also for half-precision data) or float64")
    if "Gpu" not in map_reduce_id:
        raise ValueError("[KeOps] the HIP engine only builds Gpu map-reduce schemes")
    red = parse_reduction(red_formula_string, aliases)
    layout = VarLayout(red)
    sizeof_t = 8 if dtype == "double" else 4
    rows_hint = None
    if nx is not None:
        # only the bucket matters for the cache key
        rows_hint = nx if nx < 64 * 256 * config.block_size else None
    key = (map_reduce_id, repr(red), tuple(aliases), nargs, dtype, dtypeacc, sum_scheme_string, tag1D2D,
           use_fast_math, _rows_bucket(rows_hint), int(enable_chunks), bool(enable_finalchunks), int(batch_loop), int(pairs), int(batch_total),
           binder.templates_digest(), bool(config.radial), int(config.radial_min_pairs_log2), int(config.radial_ranges_min_pairs_log2), float(config.radial_limit), float(config.radial_exact_frac), bool(config.radial_ranges), int(config.radial_mm_min_dv),
           int(config.radial_mm_rb), int(config.radial_mm_terms), bool(config.radial_bilinear), bool(config.knn_i8), bool(use_half))
    with _lock:
        hit = _cache.get(key)
    if hit is not None:
        return hit

    tagZero = int(isinstance(red, Zero_Reduction) or (isinstance(red.formula, Zero) and isinstance(red, Sum_Reduction)))
    use_chunk_mode = 0
    if tagZero:
        target, tag, src_file = "", "zero", ""
    else:
        irregular = "_ranges" in map_reduce_id
        # Min / ArgMin / Min_ArgMin of a scalar formula are the K = 1 members of the K-min family (same accumulator
        # and output layout, same "first index wins" rule): they share its matrix-core schemes
        red_k = red
        if red.kind == KIND_MIN and red.formula.dim == 1 and config.min_as_kmin:
            from .formulas.reductions import KEEP_BOTH, KEEP_VAL, ArgKMin_Reduction, KMin_ArgKMin_Reduction, KMin_Reduction

            cls = KMin_ArgKMin_Reduction if red.keep == KEEP_BOTH else (KMin_Reduction if red.keep == KEEP_VAL else ArgKMin_Reduction)
            red_k = cls(red.formula, 1, red.tagI)
        # enable_chunks: 1 every scheme, 0 the general-purpose kernel only, -1 no matrix-core scheme (exact float32
        # arithmetic in the reference's order) but the vector-ALU chunked variant for long sums
        mc = int(enable_chunks) > 0
        knn = match_knn_sqdist(red_k, dtype, map_reduce_id, batch_loop, pairs) if mc else None
        knn_batches = False
        if knn is None and mc and irregular and batch_loop >= 0 and batch_total and config.knn_ranges:
            # many batches, none of them large enough to be served on its own: every batch becomes a row range of the
            # block-sparse variant (queries and references carry every batch dimension in full)
            knn = match_knn_sqdist(red_k, dtype, map_reduce_id, -1, batch_total)
            knn_batches = knn is not None
        knn_hd = match_knn_highdim(red_k, dtype, map_reduce_id, use_fast_math) if (mc and knn is None) else None
        chk = match_chunk(red, dtype, map_reduce_id, use_fast_math) if (mc and knn is None) else None
        # double precision: the contraction on the float64 matrix instruction, when there are enough output rows to
        # fill the chip without column slabs (the vector-ALU chunked kernel has them)
        chk64 = None
        if mc and dtype == "double" and dtypeacc == "double" and config.chunk64 and (rows_hint is None or rows_hint >= config.chunk64_min_rows):
            chk64 = match_chunk(red, dtype, map_reduce_id, use_fast_math, want="double")
        fin = None
        if enable_finalchunks and mc and knn is None and chk is None:
            fin = match_final(red, dtype, dtypeacc, sum_scheme_string, map_reduce_id, use_fast_math)
        if knn is not None:
            source, meta = generate_knn_plugin(red_k, knn[0], knn[1], nargs, block_sparse=(irregular and (batch_loop == -1 or knn_batches)))
            use_chunk_mode = 3  # matrix-core filter scheme (no counterpart among the reference's chunk modes)
        elif fin is not None:
            source, meta = generate_final_plugin(red, fin, sum_scheme_string, nargs, irregular=irregular,
                                                 acc64=(dtypeacc == "double" or sum_scheme_string == "kahan_scheme"))
            use_chunk_mode = 2  # as the reference's final-chunk mode (get_keops_dll.py:101-108)
        elif chk is not None:
            source, meta = generate_chunk_plugin(red, chk, dtypeacc, sum_scheme_string, nargs, irregular=irregular,
                                                 half_data=bool(use_half))
            use_chunk_mode = 1 if source is not None else 0
        elif knn_hd is not None:
            source, meta = generate_knn_highdim_plugin(red_k, knn_hd, nargs)
            use_chunk_mode = 1 if source is not None else 0
        elif chk64 is not None:
            source, meta = generate_chunk64_plugin(red, chk64, sum_scheme_string, nargs, irregular=irregular)
            use_chunk_mode = 1 if source is not None else 0
        else:
            source = None
        if source is None and enable_chunks:
            vch = match_vchunk(red)
            if vch is not None:
                source, meta = generate_vchunk_plugin(red, vch, dtype, dtypeacc, sum_scheme_string, use_fast_math, nargs,
                                                      irregular=irregular)
                use_chunk_mode = 1 if source is not None else 0
        if source is None:
            source, meta = generate_plugin(red, dtype, dtypeacc, sum_scheme_string, use_fast_math, nargs, nx=rows_hint,
                                           irregular=irregular)
            block_sparse = irregular and batch_loop == -1
            batched = irregular and batch_loop >= 0 and batch_total > 0
            rad = match_radial(red, dtype, dtypeacc, sum_scheme_string, use_fast_math, map_reduce_id, pairs, block_sparse,
                               batch_total if batched else 0) if mc else None
            if rad is not None:
                section, rmeta = generate_radial_section(red, rad, nargs,
                                                         int(meta["block"]) * int(meta["rows"]) if (block_sparse or batched) else 0)
                if section is not None:
                    meta.update(rmeta)
                    head, body = source.split("\n", 1)
                    source = "//@keops " + " ".join(f"{k}={v}" for k, v in meta.items()) + "\n" + body + section
        tag = hashlib.sha256((source + binder.templates_digest() + str(use_fast_math)).encode()).hexdigest()[:16]
        folder = config.get_build_folder()
        target = os.path.join(folder, f"hsaco_{tag}")
        src_file = os.path.join(folder, f"{tag}.hip")
        if not os.path.exists(target):
            config.message(f"Compiling formula {red_formula_string} ... ", end="", flush=True)
            with open(src_file, "w") as f:
                f.write(source)
            binder.compile_module(target, source, use_fast_math, max(0, device_id))
            config.message("OK", flush=True)
    res = (
        tag, src_file, target, red.tagI, tagZero, int(bool(use_half)), int(bool(use_fast_math)), config.block_size, use_chunk_mode,
        0 if tagZero else tag1D2D, red.dimred, red.dim, layout.dimy,
        tuple(v.ind for v in layout.rowvars), tuple(v.ind for v in layout.colvars), tuple(v.ind for v in layout.parvars),
        tuple(v.dim for v in layout.rowvars), tuple(v.dim for v in layout.colvars), tuple(v.dim for v in layout.parvars),
    )
    with _lock:
        _cache[key] = res
    return res


def _rows_bucket(nx):
    if nx is None:
        return -1
    b = 0
    while (2 * 256 * config.block_size) << b <= nx:
        b += 1
    return b
