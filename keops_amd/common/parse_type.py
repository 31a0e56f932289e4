"""Alias / option parsing shared by the user-level classes.

Same behaviour as pykeops/pykeops/common/parse_type.py (get_type :71-131, get_sizes :48-68,
complete_aliases :9-45, get_optional_flags :134-207, parse_dtype_acc :210-240) and
pykeops/pykeops/common/utils.py:11-35 (axis2cat / cat2axis).
"""
import functools
import re

from ..formulas.parse import parse_alias

SUM_LIKE = ("Sum", "Max_SumShiftExp", "Max_SumShiftExpWeight")


def axis2cat(axis):
    """axis = dimension that is reduced (0: over i, 1: over j); cat = index that remains."""
    if axis in (0, 1):
        return (axis + 1) % 2
    raise ValueError("Axis should be 0 or 1.")


def cat2axis(cat):
    if cat in (0, 1):
        return (cat + 1) % 2
    raise ValueError("Category should be Vi or Vj.")


@functools.lru_cache(maxsize=4096)
def get_type(type_str, position_in_list=None):
    """'x = Vi(3)' -> ('x', 0, 3, position); 'Var(2,5,1)' -> (None, 1, 5, 2).  Pure function of its arguments,
    called for every alias of every reduction call: memoised."""
    s = type_str.replace("Vx", "Vi").replace("Vy", "Vj")
    name, var = parse_alias(s, position_in_list if position_in_list is not None else 0)
    pos = var.ind
    bare = s.replace(" ", "").split("=")[-1]
    if position_in_list is None and re.fullmatch(r"(Vi|Vj|Pm)\(\d+\)", bare):
        pos = None
    return name, var.cat, var.dim, pos


def complete_aliases(formula, aliases):
    """Append the Var(pos,dim,cat) terms of ``formula`` whose position lies beyond the alias list."""
    found = set(re.findall(r"Var\(\d+,\d+,\d+\)", formula.replace(" ", "")))
    extra = {}
    for var in found:
        pos = int(re.search(r"\d+", var).group(0))
        if pos >= len(aliases):
            extra[pos] = var
    aliases = list(aliases) + [None] * len(extra)
    for pos, var in extra.items():
        if pos >= len(aliases):
            raise ValueError(f"[KeOps] variable {var} leaves a gap in the argument list")
        aliases[pos] = var
    return aliases


def get_sizes(aliases, *args):
    nx = ny = None
    for k, sig in enumerate(aliases):
        _, cat, _, pos = get_type(sig, position_in_list=k)
        if cat == 0 and nx is None:
            nx = args[pos].shape[-2]
        elif cat == 1 and ny is None:
            ny = args[pos].shape[-2]
    return (1 if nx is None else nx), (1 if ny is None else ny)


def get_optional_flags(reduction_op_internal, dtype_acc, use_double_acc, sum_scheme, enable_chunks, use_fast_math=True):
    if dtype_acc != "auto" and use_double_acc:
        raise ValueError("[KeOps] you cannot set both options use_double_acc and dtype_acc.")
    if use_double_acc:
        dtype_acc = "float64"
    sum_like = reduction_op_internal in SUM_LIKE
    if dtype_acc != "auto" and not sum_like:
        raise ValueError(
            "[KeOps] parameter dtype_acc should be set to 'auto' for no-sum type reductions (Min, Max, ArgMin, etc.)"
        )
    if sum_scheme == "auto":
        sum_scheme = "block_sum" if sum_like else "direct_sum"
    if sum_scheme in ("block_sum", "kahan_scheme"):
        if not sum_like:
            raise ValueError(f'[KeOps] sum_scheme="{sum_scheme}" is only valid for sum type reductions.')
    elif sum_scheme != "direct_sum":
        raise ValueError(
            '[KeOps] invalid value for option sum_scheme : should be one of "auto", "direct_sum", "block_sum" or "kahan_scheme".'
        )
    return dict(
        dtype_acc=dtype_acc, sum_scheme=sum_scheme, use_fast_math=1 if use_fast_math else 0,
        # False: no matrix-core scheme (exact float32 / float64 arithmetic); long sums still keep their rows in memory
        enable_chunks=1 if enable_chunks else -1,
    )


def parse_dtype_acc(dtype_acc, dtype):
    """User-level accumulator dtype -> C type name."""
    if dtype_acc == "auto":
        dtype_acc = dtype
    if dtype == "float32" and dtype_acc not in ("float32", "float64"):
        raise ValueError("[KeOps] invalid parameter dtype_acc : should be either 'float32' or 'float64' when dtype is 'float32'")
    if dtype == "float64" and dtype_acc != "float64":
        raise ValueError("[KeOps] invalid parameter dtype_acc : should be 'float64' when dtype is 'float64'")
    if dtype == "float16":
        # half-precision data is computed and accumulated in float32 by the HIP backend, whatever is asked for
        if dtype_acc not in ("float16", "float32"):
            raise ValueError("[KeOps] invalid parameter dtype_acc : should be either 'float16' or 'float32' when dtype is 'float16'")
        return "float"
    return dict(float32="float", float64="double")[dtype_acc]
