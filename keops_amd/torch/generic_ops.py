"""Alias-driven shortcuts around Genred (pykeops/pykeops/torch/generic/generic_ops.py:8-201):
``generic_sum("Exp(-SqDist(X,Y))*B", "A = Vi(1)", "X = Vi(3)", "Y = Vj(3)", "B = Vj(1)")``:
the first alias names the output and fixes the reduction axis."""
from ..common.parse_type import get_type
from .generic_red import Genred


def _split(aliases):
    out, *rest = aliases
    _, cat, _, _ = get_type(out)
    return rest, (cat + 1) % 2  # reduce over the other index


def generic_sum(formula, output, *aliases, **kwargs):
    al, axis = _split((output,) + aliases)
    return Genred(formula, al, reduction_op="Sum", axis=axis, **kwargs)


def generic_logsumexp(formula, output, *aliases, **kwargs):
    al, axis = _split((output,) + aliases)
    return Genred(formula, al, reduction_op="LogSumExp", axis=axis, **kwargs)


def generic_argmin(formula, output, *aliases, **kwargs):
    al, axis = _split((output,) + aliases)
    return Genred(formula, al, reduction_op="ArgMin", axis=axis, **kwargs)


def generic_argkmin(formula, output, *aliases, **kwargs):
    al, axis = _split((output,) + aliases)
    _, _, dimout, _ = get_type(output)
    return Genred(formula, al, reduction_op="ArgKMin", axis=axis, opt_arg=dimout, **kwargs)
