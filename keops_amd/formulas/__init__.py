"""Symbolic formulas: tree (ops), reductions, string parser and scalar lowering."""
from .ops import FormulaError, Op, Var, Grad  # noqa: F401
from .parse import parse, parse_alias, parse_reduction  # noqa: F401
from .reductions import Reduction  # noqa: F401
from .lir import Lir, lower  # noqa: F401
