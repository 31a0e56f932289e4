"""Formula-string front end.

Turns ``"Sum_Reduction(Exp(-g*SqDist(x,y))*b,0)"`` plus aliases such as ``"x=Vi(3)"`` /
``"x=Var(0,3,0)"`` into a reduction descriptor.  The grammar is the reference's
(keopscore/keopscore/formulas/GetReduction.py:19-39 evaluates the string with Python's ``eval``;
pykeops/pykeops/common/keops_io/LoadKeOps.py:47-64 rewrites ``Vi/Vj/Pm`` aliases to ``Var``):
function-call syntax for operations, infix ``+ - * / ** |``, unary minus, comparisons, integer
literals.  Here the string is walked through Python's ``ast`` module instead of being evaluated.
"""
from __future__ import annotations

import ast
import re

from . import ops, reductions
from .ops import FormulaError, Op, Var, as_op

_CATS = dict(Vi=0, Vj=1, Pm=2, Vx=0, Vy=1)


def parse_alias(alias, position):
    """'x=Vi(3)' | 'x=Vi(0,3)' | 'x=Var(0,3,0)' | 'Vi(3)' | 'Var(0,3,0)' -> (name or None, Var)."""
    s = alias.replace(" ", "")
    name = None
    if "=" in s:
        name, s = s.split("=", 1)
    m = re.fullmatch(r"(Vi|Vj|Pm|Vx|Vy)\((\d+)(?:,(\d+))?\)", s)
    if m:
        a, b = int(m.group(2)), m.group(3)
        ind, dim = (position, a) if b is None else (a, int(b))
        return name, Var(ind, dim, _CATS[m.group(1)])
    m = re.fullmatch(r"Var\((\d+),(\d+),(\d+)\)", s)
    if m:
        return name, Var(int(m.group(1)), int(m.group(2)), int(m.group(3)))
    raise FormulaError(
        f"{alias} does not match the 'var = [Vi|Vj|Pm](dim)', 'var = [Vi|Vj|Pm](pos,dim)', "
        "'[Vi|Vj|Pm](pos,dim)' or 'Var(pos,dim,cat)' format"
    )


class _Builder(ast.NodeVisitor):
    def __init__(self, names):
        self.names = names

    def generic_visit(self, node):
        raise FormulaError(f"unsupported syntax in formula: {ast.dump(node)}")

    def visit_Expression(self, node):
        return self.visit(node.body)

    def visit_Constant(self, node):
        if isinstance(node.value, (int, float)) and not isinstance(node.value, bool):
            return node.value
        raise FormulaError(f"unsupported literal {node.value!r}")

    def visit_Tuple(self, node):
        # index lists of TensorDot / Kron, e.g. (2, 3)
        return tuple(self.visit(e) for e in node.elts)

    visit_List = visit_Tuple

    def visit_Name(self, node):
        if node.id in self.names:
            return self.names[node.id]
        raise FormulaError(f"unknown variable '{node.id}' in formula")

    def visit_UnaryOp(self, node):
        v = self.visit(node.operand)
        if isinstance(node.op, ast.USub):
            return -v
        if isinstance(node.op, ast.UAdd):
            return v
        raise FormulaError("unsupported unary operator")

    def visit_BinOp(self, node):
        a, b = self.visit(node.left), self.visit(node.right)
        if not isinstance(a, Op) and not isinstance(b, Op):
            # plain Python arithmetic on literals, e.g. the 1/2 in IntCst-free user strings
            a = as_op(a)
        op = node.op
        if isinstance(op, ast.Add):
            return a + b
        if isinstance(op, ast.Sub):
            return a - b
        if isinstance(op, ast.Mult):
            return a * b
        if isinstance(op, ast.Div):
            return a / b
        if isinstance(op, ast.Pow):
            return as_op(a) ** b
        if isinstance(op, ast.BitOr):
            return as_op(a) | b
        raise FormulaError("unsupported binary operator")

    def visit_Compare(self, node):
        if len(node.ops) != 1:
            raise FormulaError("chained comparisons are not supported")
        a, b = as_op(self.visit(node.left)), as_op(self.visit(node.comparators[0]))
        op = node.ops[0]
        if isinstance(op, ast.Lt):
            return a < b
        if isinstance(op, ast.LtE):
            return a <= b
        if isinstance(op, ast.Gt):
            return a > b
        if isinstance(op, ast.GtE):
            return a >= b
        raise FormulaError("unsupported comparison")

    def visit_Call(self, node):
        if not isinstance(node.func, ast.Name) or node.keywords:
            raise FormulaError("unsupported call syntax in formula")
        fn = node.func.id
        args = [self.visit(a) for a in node.args]
        if fn in reductions.REDUCTIONS:
            return reductions.REDUCTIONS[fn](*args)
        if fn in ops.FUNCTIONS:
            try:
                return ops.FUNCTIONS[fn](*args)
            except TypeError as e:
                raise FormulaError(f"bad arguments for {fn}: {e}") from None
        raise FormulaError(f"unknown operation '{fn}' in formula")


def parse(string, aliases=()):
    """Parse a formula or reduction string.  Returns an Op or a Reduction."""
    names = {}
    for k, alias in enumerate(aliases):
        if alias is None:
            continue
        name, var = parse_alias(alias, k)
        if name is not None:
            names[name] = var
    try:
        tree = ast.parse(string.strip(), mode="eval")
    except SyntaxError as e:
        raise FormulaError(f"cannot parse formula '{string}': {e}") from None
    return _Builder(names).visit(tree)


def parse_reduction(string, aliases=()):
    red = parse(string, aliases)
    if not isinstance(red, reductions.Reduction):
        raise FormulaError(f"'{string}' is not a reduction")
    return red
