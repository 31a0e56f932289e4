"""Symbolic formula tree for the map-reduce engine.

A formula F(x_i, y_j, p) is an immutable tree of :class:`Op` nodes.  Every node knows its output
dimension, how to lower itself to scalar SSA code (``lower``) and how to back-propagate a
gradient through itself (``diff_t``, the transposed differential).  The grammar, the operator
names, their argument meaning and their constructor-time simplifications mirror the reference's
formula layer (keopscore/keopscore/formulas/Operation.py:11-260, formulas/maths/*.py,
formulas/variables/*.py); the implementation is a single table-driven module whose lowering
target is straight-line scalar code for the hand-written HIP kernel templates, not C++ loop text.
"""
from __future__ import annotations

import math

from .lir import Lir


import copy as _copy

class FormulaError(ValueError):
    """Raised for ill-formed formulas (mirrors KeOps_Error -> ValueError in the reference)."""


# ----------------------------------------------------------------------------- base class


class Op:
    """Immutable formula node.  ``children`` are Ops, ``params`` are plain Python values."""

    name = "Op"
    __slots__ = ("children", "params", "dim", "_hash", "_vars")

    def __init__(self, children=(), params=(), dim=1):
        self.children = tuple(children)
        self.params = tuple(params)
        self.dim = int(dim)
        self._hash = None
        self._vars = None

    # -- structure ----------------------------------------------------------------------
    def _key(self):
        return (self.name, self.children, self.params, self.dim)

    def __eq__(self, other):
        return isinstance(other, Op) and self is other or (
            isinstance(other, Op) and hash(self) == hash(other) and self._key() == other._key()
        )

    def __hash__(self):
        if self._hash is None:
            self._hash = hash(self._key())
        return self._hash

    def __repr__(self):
        parts = [repr(c) for c in self.children] + [repr(p) for p in self.params]
        return f"{self.name}({','.join(parts)})"

    @property
    def variables(self):
        """Sorted tuple of the distinct :class:`Var` leaves below this node."""
        if self._vars is None:
            acc = set()
            for c in self.children:
                acc.update(c.variables)
            self._vars = tuple(sorted(acc, key=lambda v: (v.ind, v.cat, v.dim)))
        return self._vars

    def depends_on_cat(self, cat):
        return any(v.cat == cat for v in self.variables)

    def replace(self, old, new):
        if self == old:
            return new
        if not self.children:
            return self
        kids = [c.replace(old, new) for c in self.children]
        return self.rebuild(kids)

    def substitute(self, mapping, memo=None):
        """Replace several sub-formulas at once (``mapping``: old -> new) in one traversal; shared sub-trees are
        rebuilt once."""
        if memo is None:
            memo = {}
        r = mapping.get(self)
        if r is not None:
            return r
        if not self.children:
            return self
        r = memo.get(id(self))
        if r is None:
            kids = [c.substitute(mapping, memo) for c in self.children]
            r = self if all(k is c for k, c in zip(kids, self.children)) else self.rebuild(kids)
            memo[id(self)] = r
        return r

    def rename_vars(self, mapping, memo=None):
        """Copy of this tree with variables renamed (``mapping``: Var -> Var of the same dimension and category,
        injective).  A pure renaming cannot enable or undo a simplification, so nodes are cloned without going
        through the simplifying constructors."""
        if memo is None:
            memo = {}
        if not self.children:
            return mapping.get(self, self)
        r = memo.get(id(self))
        if r is None:
            kids = tuple(c.rename_vars(mapping, memo) for c in self.children)
            if all(k is c for k, c in zip(kids, self.children)):
                r = self
            else:
                r = _copy.copy(self)
                r.children, r._hash, r._vars = kids, None, None
            memo[id(self)] = r
        return r

    def rebuild(self, kids):
        """Re-create this node over new children through the simplifying constructor."""
        return BUILDERS[self.name](*kids, *self.params)

    def walk(self):
        yield self
        for c in self.children:
            yield from c.walk()

    # -- semantics ----------------------------------------------------------------------
    def lower(self, L: Lir, kids):
        raise NotImplementedError(self.name)

    def diff_t(self, v, gradin):
        raise NotImplementedError(f"gradient of {self.name} is not implemented")

    # -- operator sugar (same redirections as the reference's Operation.__mul__ & co) -----
    def __add__(self, o):
        return Add(self, as_op(o))

    def __radd__(self, o):
        return Add(as_op(o), self)

    def __sub__(self, o):
        return Subtract(self, as_op(o))

    def __rsub__(self, o):
        return Subtract(as_op(o), self)

    def __mul__(self, o):
        return Mult(self, as_op(o))

    def __rmul__(self, o):
        return Mult(as_op(o), self)

    def __truediv__(self, o):
        return Divide(self, as_op(o))

    def __rtruediv__(self, o):
        if o == 1:
            return Inv(self)
        return Divide(as_op(o), self)

    def __neg__(self):
        return Minus(self)

    def __pow__(self, m):
        if m == 2:
            return Square(self)
        if isinstance(m, int):
            return Pow(self, m)
        return Powf(self, as_op(m))

    def __or__(self, o):
        return Scalprod(self, as_op(o))

    def __lt__(self, o):
        return LessThan(self, as_op(o))

    def __gt__(self, o):
        return LessThan(as_op(o), self)

    def __le__(self, o):
        return LessOrEqual(self, as_op(o))

    def __ge__(self, o):
        return LessOrEqual(as_op(o), self)


def as_op(x):
    if isinstance(x, Op):
        return x
    if isinstance(x, bool):
        raise FormulaError("booleans are not formula operands")
    if isinstance(x, int):
        return IntCst(x)
    if isinstance(x, float):
        if x == int(x) and abs(x) < 2**24:
            return IntCst(int(x))
        return FloatCst(x)
    raise FormulaError(f"invalid operand type {type(x)}")


def _bdim(*dims):
    """Broadcast rule of VectApply (code_gen_utils.py:390-431): all dims equal, or 1."""
    d = max(dims)
    for k in dims:
        if k not in (1, d):
            raise FormulaError(f"incompatible dimensions {dims}")
    return d


def _bcast(ids, d):
    return ids if len(ids) == d else ids * d


# ----------------------------------------------------------------------------- leaves


class Var(Op):
    """Var(ind, dim, cat): cat 0 = indexed by i, 1 = indexed by j, 2 = parameter."""

    name = "Var"
    __slots__ = ("ind", "cat")

    def __init__(self, ind, dim, cat):
        super().__init__((), (int(ind), int(dim), int(cat)), dim)
        self.ind, self.cat = int(ind), int(cat)
        if self.cat not in (0, 1, 2, 3):
            raise FormulaError("Var category must be 0 (i), 1 (j) or 2 (parameter)")

    def __repr__(self):
        return f"Var({self.ind},{self.dim},{self.cat})"

    @property
    def variables(self):
        return (self,)

    def replace(self, old, new):
        return new if self == old else self

    def lower(self, L, kids):
        return [L.load(self.cat, self.ind, k) for k in range(self.dim)]

    def diff_t(self, v, gradin):
        return gradin if self == v else Zero(v.dim)


def Vi(ind, dim):
    return Var(ind, dim, 0)


def Vj(ind, dim):
    return Var(ind, dim, 1)


def Pm(ind, dim):
    return Var(ind, dim, 2)


class Zero(Op):
    name = "Zero"

    def __init__(self, dim):
        super().__init__((), (int(dim),), dim)

    def lower(self, L, kids):
        z = L.const(0.0)
        return [z] * self.dim

    def diff_t(self, v, gradin):
        return Zero(v.dim)


class IntCst(Op):
    name = "IntCst"

    def __init__(self, val):
        super().__init__((), (int(val),), 1)

    @property
    def val(self):
        return self.params[0]

    def lower(self, L, kids):
        return [L.const(float(self.val))]

    def diff_t(self, v, gradin):
        return Zero(v.dim)


class RatCstNode(Op):
    name = "RatCst"

    def __init__(self, p, q):
        super().__init__((), (int(p), int(q)), 1)

    @property
    def p(self):
        return self.params[0]

    @property
    def q(self):
        return self.params[1]

    def lower(self, L, kids):
        return [L.const(self.p / self.q)]

    def diff_t(self, v, gradin):
        return Zero(v.dim)


def RatCst(p, q):
    if q == 0:
        raise FormulaError("RatCst with zero denominator")
    g = math.gcd(int(p), int(q))
    p, q = int(p) // g, int(q) // g
    if q < 0:
        p, q = -p, -q
    if q == 1:
        return IntCst(p)
    return RatCstNode(p, q)


def IntInv(n):
    return RatCst(1, n)


class FloatCst(Op):
    """Literal floating-point constant (an extension: the reference only has Int/RatCst)."""

    name = "FloatCst"

    def __init__(self, val):
        super().__init__((), (float(val),), 1)

    def lower(self, L, kids):
        return [L.const(self.params[0])]

    def diff_t(self, v, gradin):
        return Zero(v.dim)


def _is_const(f):
    return isinstance(f, (IntCst, RatCstNode, FloatCst))


def _const_value(f):
    if isinstance(f, IntCst):
        return f.val
    if isinstance(f, RatCstNode):
        return f.p / f.q
    return f.params[0]


# ----------------------------------------------------------------------------- elementwise


class Elementwise(Op):
    """Vectorised scalar operation with the broadcasting rule of VectorizedScalarOp.py:8-57."""

    def __init__(self, *children, params=()):
        super().__init__(children, params, _bdim(*[c.dim for c in children]))

    def scalar(self, L, *a):
        raise NotImplementedError

    def derivatives(self):
        """d out / d child_k as formulas of the children (same dims, broadcastable)."""
        raise NotImplementedError(f"gradient of {self.name} is not implemented")

    def lower(self, L, kids):
        kids = [_bcast(k, self.dim) for k in kids]
        return [self.scalar(L, *[k[i] for k in kids]) for i in range(self.dim)]

    def diff_t(self, v, gradin):
        # VectorizedScalarOp.DiffT (VectorizedScalarOp.py:33-40): sum_k child_k.DiffT(v, d_k * gradin),
        # where a child of dim 1 under a vector output receives the summed gradient.
        ders = self.derivatives()
        out = Zero(v.dim)
        for c, d in zip(self.children, ders):
            if not any(w == v for w in c.variables):
                continue
            g = Mult(d, gradin)
            if c.dim == 1 and g.dim > 1:
                g = Sum(g)
            out = Add(out, c.diff_t(v, g))
        return out


def _unary(name, scalar, deriv=None):
    def _scalar(self, L, a):
        return scalar(L, a)

    def _derivs(self):
        if deriv is None:
            raise NotImplementedError(f"gradient of {name} is not implemented")
        return (deriv(self.children[0], self),)

    cls = type(name + "Node", (Elementwise,), dict(name=name, scalar=_scalar, derivatives=_derivs, __slots__=()))
    return cls


# scalar bodies follow keopscore/keopscore/utils/math_functions.py:73-178 (cpu_code column)
MinusNode = _unary("Minus", lambda L, a: L.neg(a), lambda f, s: IntCst(-1))
ExpNode = _unary("Exp", lambda L, a: L.exp(a), lambda f, s: s)
LogNode = _unary("Log", lambda L, a: L.log(a), lambda f, s: Inv(f))
SqrtNode = _unary("Sqrt", lambda L, a: L.sqrt(a), lambda f, s: Mult(IntInv(2), Rsqrt(f)))
RsqrtNode = _unary("Rsqrt", lambda L, a: L.rsqrt0(a), lambda f, s: Mult(RatCst(-1, 2), Pow(s, 3)))
InvNode = _unary("Inv", lambda L, a: L.rcp(a), lambda f, s: Minus(Square(s)))
SquareNode = _unary("Square", lambda L, a: L.mul(a, a), lambda f, s: Mult(IntCst(2), f))
AbsNode = _unary("Abs", lambda L, a: L.abs(a), lambda f, s: Sign(f))
SignNode = _unary("Sign", lambda L, a: L.sign(a), lambda f, s: Zero(1))
StepNode = _unary("Step", lambda L, a: L.select(L.lt(a, L.const(0.0)), L.const(0.0), L.const(1.0)), lambda f, s: Zero(1))
ReLUNode = _unary("ReLU", lambda L, a: L.select(L.lt(a, L.const(0.0)), L.const(0.0), a), lambda f, s: Step(f))
SinNode = _unary("Sin", lambda L, a: L.call("sin", a), lambda f, s: Cos(f))
CosNode = _unary("Cos", lambda L, a: L.call("cos", a), lambda f, s: Minus(Sin(f)))
AsinNode = _unary("Asin", lambda L, a: L.call("asin", a), lambda f, s: Rsqrt(Subtract(IntCst(1), Square(f))))
AcosNode = _unary("Acos", lambda L, a: L.call("acos", a), lambda f, s: Minus(Rsqrt(Subtract(IntCst(1), Square(f)))))
AtanNode = _unary("Atan", lambda L, a: L.call("atan", a), lambda f, s: Inv(Add(IntCst(1), Square(f))))
FloorNode = _unary("Floor", lambda L, a: L.call("floor", a), lambda f, s: Zero(1))
XLogXNode = _unary(
    "XLogX",
    lambda L, a: L.select(L.ne(a, L.const(0.0)), L.mul(a, L.log(a)), L.const(0.0)),
    lambda f, s: Add(Log(f), IntCst(1)),
)
SinXDivXNode = _unary(
    "SinXDivX",
    lambda L, a: L.select(L.ne(a, L.const(0.0)), L.div(L.call("sin", a), a), L.const(1.0)),
    lambda f, s: Subtract(Divide(Cos(f), f), Divide(Sin(f), Square(f))),
)


def _simple(cls):
    def build(f):
        f = as_op(f)
        if isinstance(f, Zero) and cls in (SinNode, AsinNode, AtanNode, AbsNode, SignNode, ReLUNode, FloorNode, XLogXNode, SqrtNode):
            return f
        return cls(f)

    build.__name__ = cls.name
    return build


Log, Rsqrt, Inv, Abs, Sign, Step, ReLU = map(_simple, (LogNode, RsqrtNode, InvNode, AbsNode, SignNode, StepNode, ReLUNode))
Sin, Cos, Asin, Acos, Atan, Floor, XLogX, SinXDivX = map(
    _simple, (SinNode, CosNode, AsinNode, AcosNode, AtanNode, FloorNode, XLogXNode, SinXDivXNode)
)
Sqrt = _simple(SqrtNode)


def Exp(f):
    return ExpNode(as_op(f))


def Minus(f):
    # Minus.py:42-62: -0 -> 0, -(-f) -> f, -(n) -> (-n), -(p/q) -> (-p)/q
    f = as_op(f)
    if isinstance(f, Zero):
        return f
    if isinstance(f, MinusNode):
        return f.children[0]
    if isinstance(f, IntCst):
        return IntCst(-f.val)
    if isinstance(f, RatCstNode):
        return RatCst(-f.p, f.q)
    if isinstance(f, FloatCst):
        return FloatCst(-f.params[0])
    return MinusNode(f)


def Square(f):
    f = as_op(f)
    if isinstance(f, Zero):
        return f
    if isinstance(f, MinusNode):
        return SquareNode(f.children[0])
    if isinstance(f, IntCst):
        return IntCst(f.val * f.val)
    return SquareNode(f)


class PowNode(Elementwise):
    name = "Pow"
    __slots__ = ()

    def __init__(self, f, m):
        Op.__init__(self, (f,), (int(m),), f.dim)

    def scalar(self, L, a):
        return L.powi(a, self.params[0])

    def derivatives(self):
        m = self.params[0]
        return (Mult(IntCst(m), Pow(self.children[0], m - 1)),)


def Pow(f, m):
    f = as_op(f)
    m = int(m)
    if m == 1:
        return f
    if m == 0:
        return IntCst(1) if f.dim == 1 else SumT(IntCst(1), f.dim)
    if m == 2:
        return Square(f)
    return PowNode(f, m)


class RoundNode(Elementwise):
    name = "Round"
    __slots__ = ()

    def __init__(self, f, d):
        Op.__init__(self, (f,), (int(d),), f.dim)

    def scalar(self, L, a):
        d = self.params[0]
        if d == 0:
            return L.call("round", a)
        s = L.const(float(10**d))
        return L.div(L.call("round", L.mul(a, s)), s)

    def derivatives(self):
        return (Zero(1),)


def Round(f, d=0):
    return RoundNode(as_op(f), d)


# -- binary / ternary elementwise -------------------------------------------------------


class AddNode(Elementwise):
    name = "Add"
    __slots__ = ()

    def scalar(self, L, a, b):
        return L.add(a, b)

    def diff_t(self, v, gradin):
        a, b = self.children
        return Add(a.diff_t(v, _adj_bcast(gradin, a.dim)), b.diff_t(v, _adj_bcast(gradin, b.dim)))


class SubtractNode(Elementwise):
    name = "Subtract"
    __slots__ = ()

    def scalar(self, L, a, b):
        return L.sub(a, b)

    def diff_t(self, v, gradin):
        a, b = self.children
        return Subtract(a.diff_t(v, _adj_bcast(gradin, a.dim)), b.diff_t(v, _adj_bcast(gradin, b.dim)))


class MultNode(Elementwise):
    name = "Mult"
    __slots__ = ()

    def scalar(self, L, a, b):
        return L.mul(a, b)

    def diff_t(self, v, gradin):
        # Mult.py:28-38
        fa, fb = self.children
        if isinstance(fb, ExpNode) and fb.dim == 1 and fa.dim >= gradin.dim:
            # d(a*exp(u)) = (da + a du) * exp(u): keeps a single exponential in the gradient
            (u,) = fb.children
            return Mult(Add(fa.diff_t(v, _adj_bcast(gradin, fa.dim)), u.diff_t(v, _sp(gradin, fa))), fb)
        if fa.dim == 1 and fb.dim > 1:
            return Add(fa.diff_t(v, _sp(gradin, fb)), fb.diff_t(v, Mult(fa, gradin)))
        if fb.dim == 1 and fa.dim > 1:
            return Add(fa.diff_t(v, Mult(fb, gradin)), fb.diff_t(v, _sp(gradin, fa)))
        return Add(fa.diff_t(v, _adj_bcast(Mult(fb, gradin), fa.dim)), fb.diff_t(v, _adj_bcast(Mult(fa, gradin), fb.dim)))


class DivideNode(Elementwise):
    name = "Divide"
    __slots__ = ()

    def scalar(self, L, a, b):
        return L.div(a, b)

    def diff_t(self, v, gradin):
        # d(a/b) = da/b - a db / b^2
        fa, fb = self.children
        ga = Divide(gradin, fb)
        gb = Minus(Divide(Mult(gradin, fa), Square(fb)))
        return Add(fa.diff_t(v, _adj_bcast(ga, fa.dim)), fb.diff_t(v, _adj_bcast(gb, fb.dim)))


def _adj_bcast(g, dim):
    """Adjoint of broadcasting a dim-1 operand to the gradient's dimension."""
    if g.dim == dim:
        return g
    if dim == 1:
        return Sum(g)
    if g.dim == 1:
        return SumT(g, dim)
    raise FormulaError("incompatible dimensions in gradient broadcast")


def _sp(g, f):
    """Scalprod that tolerates a scalar gradient against a vector (or vice versa)."""
    if g.dim == f.dim:
        return Scalprod(g, f) if g.dim > 1 else Mult(g, f)
    if g.dim == 1:
        return Mult(g, Sum(f))
    if f.dim == 1:
        return Mult(Sum(g), f)
    raise FormulaError("incompatible dimensions in Scalprod")


def Broadcast(f, dim):
    if f.dim == dim or dim == 1:
        return f
    if f.dim == 1:
        return SumT(f, dim)
    raise FormulaError("dimensions are not compatible for Broadcast operation")


def Add(a, b):
    # Add.py:50-134: 0+f, f+0, cst folding, f+f -> 2f, f+(-g) -> f-g, n*f+f -> (n+1)*f ...
    a, b = as_op(a), as_op(b)
    _bdim(a.dim, b.dim)
    if isinstance(a, Zero):
        return Broadcast(b, a.dim)
    if isinstance(b, Zero):
        return Broadcast(a, b.dim)
    if isinstance(a, IntCst) and isinstance(b, IntCst):
        return IntCst(a.val + b.val)
    if _is_rat(a) and _is_rat(b):
        pa, qa = _rat(a)
        pb, qb = _rat(b)
        return RatCst(pa * qb + pb * qa, qa * qb)
    if a == b:
        return Mult(IntCst(2), a)
    if isinstance(b, MinusNode):
        return Subtract(a, b.children[0])
    if isinstance(a, MinusNode):
        return Subtract(b, a.children[0])
    if isinstance(a, MultNode) and isinstance(a.children[0], IntCst) and a.children[1] == b:
        return Mult(IntCst(a.children[0].val + 1), b)
    if isinstance(b, MultNode) and isinstance(b.children[0], IntCst) and b.children[1] == a:
        return Mult(IntCst(b.children[0].val + 1), a)
    if (
        isinstance(a, MultNode)
        and isinstance(b, MultNode)
        and isinstance(a.children[0], IntCst)
        and isinstance(b.children[0], IntCst)
        and a.children[1] == b.children[1]
    ):
        return Mult(IntCst(a.children[0].val + b.children[0].val), a.children[1])
    return AddNode(a, b)


def Subtract(a, b):
    # Subtract.py:48-128
    a, b = as_op(a), as_op(b)
    _bdim(a.dim, b.dim)
    if isinstance(a, Zero):
        return Minus(Broadcast(b, a.dim))
    if isinstance(b, Zero):
        return Broadcast(a, b.dim)
    if isinstance(a, IntCst) and isinstance(b, IntCst):
        return IntCst(a.val - b.val)
    if _is_rat(a) and _is_rat(b):
        pa, qa = _rat(a)
        pb, qb = _rat(b)
        return RatCst(pa * qb - pb * qa, qa * qb)
    if a == b:
        return Zero(a.dim)
    if isinstance(b, MinusNode):
        return Add(a, b.children[0])
    if isinstance(a, MultNode) and isinstance(a.children[0], IntCst) and a.children[1] == b:
        return Mult(IntCst(a.children[0].val - 1), b)
    if isinstance(b, MultNode) and isinstance(b.children[0], IntCst) and b.children[1] == a:
        return Mult(IntCst(1 - b.children[0].val), a)
    return SubtractNode(a, b)


def _is_rat(f):
    return isinstance(f, (IntCst, RatCstNode))


def _rat(f):
    return (f.val, 1) if isinstance(f, IntCst) else (f.p, f.q)


def Mult(a, b):
    # Mult.py:53-157, same normal form: constants to the left, exponentials to the right,
    # minus signs pulled out, f*f -> f^2, SumT broadcast folded.
    a, b = as_op(a), as_op(b)
    _bdim(a.dim, b.dim)
    if isinstance(a, Zero):
        return Broadcast(a, b.dim) if a.dim >= b.dim else Zero(b.dim)
    if isinstance(b, Zero):
        return Broadcast(b, a.dim) if b.dim >= a.dim else Zero(a.dim)
    if _is_rat(a) and _is_rat(b):
        pa, qa = _rat(a)
        pb, qb = _rat(b)
        return RatCst(pa * pb, qa * qb)
    if isinstance(a, IntCst):
        if a.val == 1:
            return b
        if a.val == -1:
            return Minus(b)
    if isinstance(b, IntCst) or (isinstance(b, RatCstNode) and not _is_rat(a)):
        return Mult(b, a)
    if _is_rat(a) and isinstance(b, MultNode) and _is_rat(b.children[0]):
        return Mult(Mult(a, b.children[0]), b.children[1])
    if isinstance(b, MultNode) and _is_rat(b.children[0]) and not _is_rat(a):
        return Mult(b.children[0], Mult(a, b.children[1]))
    if (
        isinstance(a, MultNode)
        and _is_rat(a.children[0])
        and not isinstance(b, ExpNode)
        and not (a.children[1].dim == 1 and b.dim > 1)
    ):
        return Mult(a.children[0], Mult(a.children[1], b))
    if isinstance(a, MinusNode) and isinstance(b, MinusNode):
        return Mult(a.children[0], b.children[0])
    if isinstance(a, MinusNode):
        return Minus(Mult(a.children[0], b))
    if isinstance(b, MinusNode):
        return Minus(Mult(a, b.children[0]))
    if a == b:
        return Square(a)
    # keep scalar factors together and to the left of vector factors, so that a product of a
    # vector with several scalars costs one multiply per component
    if a.dim > 1 and b.dim == 1 and not isinstance(b, ExpNode):
        return Mult(b, a)
    if a.dim == 1 and b.dim > 1 and isinstance(b, MultNode) and b.children[0].dim == 1:
        return Mult(Mult(a, b.children[0]), b.children[1])
    if b.dim == 1 and a.dim > 1 and isinstance(a, MultNode) and a.children[0].dim == 1:
        return Mult(Mult(a.children[0], b), a.children[1])
    if isinstance(b, SumTNode):
        if isinstance(a, SumTNode):
            return SumT(Mult(a.children[0], b.children[0]), a.dim)
        if a.dim == 1:
            return SumT(Mult(a, b.children[0]), b.dim)
        if a.dim == b.dim:
            return Mult(a, b.children[0])
    elif isinstance(a, SumTNode):
        return Mult(b, a)
    if isinstance(a, ExpNode) and isinstance(b, ExpNode) and a.dim == b.dim:
        return Exp(Add(a.children[0], b.children[0]))
    if isinstance(a, ExpNode) and a.dim >= b.dim and not isinstance(b, ExpNode):
        return Mult(b, a)
    if isinstance(a, MultNode) and isinstance(a.children[1], ExpNode):
        u, e = a.children
        if isinstance(b, ExpNode) and b.dim == e.dim:
            return Mult(u, Exp(Add(e.children[0], b.children[0])))
        if b.dim <= e.dim and not isinstance(b, ExpNode):
            return Mult(Mult(u, b), e)
    if isinstance(b, MultNode) and isinstance(b.children[1], ExpNode) and not _is_rat(a) and not isinstance(a, ExpNode):
        if a.dim <= b.children[1].dim or b.children[0].dim >= a.dim:
            return Mult(Mult(a, b.children[0]), b.children[1])
    return MultNode(a, b)


def Divide(a, b):
    # Divide.py:52-62
    a, b = as_op(a), as_op(b)
    _bdim(a.dim, b.dim)
    if isinstance(a, Zero):
        return Broadcast(a, b.dim) if a.dim >= b.dim else Zero(b.dim)
    if isinstance(b, Zero):
        raise FormulaError("division by zero")
    if isinstance(b, IntCst):
        return Mult(IntInv(b.val), a)
    if isinstance(b, RatCstNode):
        return Mult(RatCst(b.q, b.p), a)
    if a == b:
        return IntCst(1) if a.dim == 1 else SumT(IntCst(1), a.dim)
    return DivideNode(a, b)


def _binary(name, scalar, derivs=None):
    def _scalar(self, L, a, b):
        return scalar(L, a, b)

    def _derivs(self):
        if derivs is None:
            return (Zero(1), Zero(1))
        return derivs(*self.children, self)

    return type(name + "Node", (Elementwise,), dict(name=name, scalar=_scalar, derivatives=_derivs, __slots__=()))


PowfNode = _binary(
    "Powf",
    lambda L, a, b: L.call("pow", a, b),
    lambda a, b, s: (Mult(b, Powf(a, Subtract(b, IntCst(1)))), Mult(Log(a), s)),
)
Atan2Node = _binary(
    "Atan2",
    lambda L, a, b: L.call("atan2", a, b),
    lambda a, b, s: (Divide(b, Add(Square(a), Square(b))), Minus(Divide(a, Add(Square(a), Square(b))))),
)
EqualNode = _binary("Equal", lambda L, a, b: L.select(L.eq(a, b), L.const(1.0), L.const(0.0)))
NotEqualNode = _binary("NotEqual", lambda L, a, b: L.select(L.ne(a, b), L.const(1.0), L.const(0.0)))
LessThanNode = _binary("LessThan", lambda L, a, b: L.select(L.lt(a, b), L.const(1.0), L.const(0.0)))
LessOrEqualNode = _binary("LessOrEqual", lambda L, a, b: L.select(L.le(a, b), L.const(1.0), L.const(0.0)))


def _mk2(cls):
    def build(a, b):
        return cls(as_op(a), as_op(b))

    build.__name__ = cls.name
    return build


Powf, Atan2, Equal, NotEqual, LessThan, LessOrEqual = map(
    _mk2, (PowfNode, Atan2Node, EqualNode, NotEqualNode, LessThanNode, LessOrEqualNode)
)


class IfElseNode(Elementwise):
    """IfElse(f,a,b) = a where f >= 0, b elsewhere (math_functions.py:139-141)."""

    name = "IfElse"
    __slots__ = ()

    def scalar(self, L, f, a, b):
        return L.select(L.le(L.const(0.0), f), a, b)

    def diff_t(self, v, gradin):
        f, a, b = self.children
        if f.dim == 1:
            return IfElse(f, a.diff_t(v, _adj_bcast(gradin, a.dim)), b.diff_t(v, _adj_bcast(gradin, b.dim)))
        return _ifelse_grad(self, v, gradin)


def _ifelse_grad(node, v, gradin):
    f, a, b = node.children
    mask = Broadcast(Step(f), node.dim)
    ga = Mult(mask, gradin)
    gb = Mult(Subtract(IntCst(1), mask), gradin)
    return Add(a.diff_t(v, _adj_bcast(ga, a.dim)), b.diff_t(v, _adj_bcast(gb, b.dim)))


def IfElse(f, a, b):
    return IfElseNode(as_op(f), as_op(a), as_op(b))


class ClampNode(Elementwise):
    """Clamp(x,a,b) = a if x<a, b if x>b, else x (math_functions.py:143-146)."""

    name = "Clamp"
    __slots__ = ()

    def scalar(self, L, x, a, b):
        return L.select(L.lt(x, a), a, L.select(L.lt(b, x), b, x))

    def diff_t(self, v, gradin):
        x, a, b = self.children
        inside = Mult(LessOrEqual(a, x), LessOrEqual(x, b))  # 1 on [a,b]
        below = LessThan(x, a)
        above = LessThan(b, x)
        out = x.diff_t(v, _adj_bcast(Mult(inside, gradin), x.dim))
        out = Add(out, a.diff_t(v, _adj_bcast(Mult(below, gradin), a.dim)))
        return Add(out, b.diff_t(v, _adj_bcast(Mult(above, gradin), b.dim)))


def Clamp(x, a, b):
    return ClampNode(as_op(x), as_op(a), as_op(b))


class ClampIntNode(Elementwise):
    name = "ClampInt"
    __slots__ = ()

    def __init__(self, x, a, b):
        Op.__init__(self, (x,), (int(a), int(b)), x.dim)

    def scalar(self, L, x):
        a, b = L.const(float(self.params[0])), L.const(float(self.params[1]))
        return L.select(L.lt(x, a), a, L.select(L.lt(b, x), b, x))

    def derivatives(self):
        return (DiffClampInt(self.children[0], *self.params),)


def ClampInt(x, a, b):
    return ClampIntNode(as_op(x), a, b)


class DiffClampIntNode(Elementwise):
    name = "DiffClampInt"
    __slots__ = ()

    def __init__(self, x, a, b):
        Op.__init__(self, (x,), (int(a), int(b)), x.dim)

    def scalar(self, L, x):
        a, b = L.const(float(self.params[0])), L.const(float(self.params[1]))
        return L.select(L.lt(x, a), L.const(0.0), L.select(L.lt(b, x), L.const(0.0), L.const(1.0)))

    def derivatives(self):
        return (Zero(1),)


def DiffClampInt(x, a, b):
    return DiffClampIntNode(as_op(x), a, b)


class ModNode(Elementwise):
    """Mod(x,n,d) = x - n*floor((x-d)/n) (math_functions.py:155-158)."""

    name = "Mod"
    __slots__ = ()

    def scalar(self, L, x, n, d):
        return L.sub(x, L.mul(n, L.call("floor", L.div(L.sub(x, d), n))))

    def derivatives(self):
        return (IntCst(1), Zero(1), Zero(1))


def Mod(x, n, d=0):
    return ModNode(as_op(x), as_op(n), as_op(d))


# ----------------------------------------------------------------------------- vector ops


class SumNode(Op):
    name = "Sum"
    __slots__ = ()

    def __init__(self, f):
        super().__init__((f,), (), 1)

    def lower(self, L, kids):
        # Sum.py:20-24: out = 0; out += arg[k] in order
        (a,) = kids
        acc = a[0]
        for t in a[1:]:
            acc = L.add(acc, t)
        return [acc]

    def diff_t(self, v, gradin):
        f = self.children[0]
        return f.diff_t(v, SumT(gradin, f.dim))


def Sum(f):
    # Sum.py:48-66
    f = as_op(f)
    if f.dim == 1:
        return f
    if isinstance(f, Zero):
        return Zero(1)
    if isinstance(f, SumTNode):
        return Mult(IntCst(f.dim), f.children[0])
    if isinstance(f, MinusNode):
        return Minus(Sum(f.children[0]))
    if isinstance(f, MultNode):
        a, b = f.children
        if a.dim == 1:
            return Mult(a, Sum(b))
        if b.dim == 1:
            return Mult(Sum(a), b)
        return Scalprod(a, b)
    return SumNode(f)


class SumTNode(Op):
    """SumT(f, dim): broadcast a scalar to a vector (adjoint of Sum)."""

    name = "SumT"
    __slots__ = ()

    def __init__(self, f, dim):
        super().__init__((f,), (int(dim),), dim)

    def lower(self, L, kids):
        return kids[0] * self.dim

    def diff_t(self, v, gradin):
        return self.children[0].diff_t(v, Sum(gradin))


def SumT(f, dim):
    f = as_op(f)
    if f.dim != 1:
        if f.dim == dim:
            return f
        raise FormulaError("SumT expects a scalar formula")
    if dim == 1:
        return f
    if isinstance(f, Zero):
        return Zero(dim)
    return SumTNode(f, dim)


class ScalprodNode(Op):
    name = "Scalprod"
    __slots__ = ()

    def __init__(self, a, b):
        if a.dim != b.dim:
            raise FormulaError("Dimensions must be the same for Scalprod")
        super().__init__((a, b), (), 1)

    def lower(self, L, kids):
        a, b = kids
        acc = L.mul(a[0], b[0])
        for s, t in zip(a[1:], b[1:]):
            acc = L.fma(s, t, acc)  # Scalprod.py:32-36 uses fma
        return [acc]

    def diff_t(self, v, gradin):
        a, b = self.children
        return Add(a.diff_t(v, Mult(gradin, b)), b.diff_t(v, Mult(gradin, a)))


def Scalprod(a, b):
    # Scalprod.py:49-70
    a, b = as_op(a), as_op(b)
    if isinstance(a, Zero) or isinstance(b, Zero):
        return Zero(1)
    if a.dim == 1:
        return Mult(a, Sum(b))
    if b.dim == 1:
        return Mult(Sum(a), b)
    if a == b:
        return Sum(Square(a))
    if isinstance(a, MinusNode):
        return Minus(Scalprod(a.children[0], b))
    if isinstance(b, MinusNode):
        return Minus(Scalprod(a, b.children[0]))
    for f, g in ((a, b), (b, a)):
        if isinstance(f, MultNode):
            u, w = f.children
            if u.dim == 1:
                return Mult(u, Scalprod(w, g))
            if w.dim == 1:
                return Mult(w, Scalprod(u, g))
        if isinstance(f, SumTNode):
            return Mult(f.children[0], Sum(g))
    return ScalprodNode(a, b)


def SqNorm2(f):
    return Sum(Square(as_op(f)))


def Norm2(f):
    f = as_op(f)
    return Sqrt(Scalprod(f, f))


def SqDist(a, b):
    return SqNorm2(Subtract(as_op(a), as_op(b)))


def Normalize(f):
    f = as_op(f)
    return Mult(Rsqrt(SqNorm2(f)), f)


def WeightedSqNorm(a, x):
    # WeightedSqNorm.py: scalar weight -> a*|x|^2, diagonal -> <a, x^2>, full matrix -> x^T A x
    a, x = as_op(a), as_op(x)
    if a.dim == 1:
        return Mult(a, SqNorm2(x))
    if a.dim == x.dim:
        return Scalprod(a, Square(x))
    if a.dim == x.dim * x.dim:
        return Scalprod(x, MatVecMult(a, x))
    raise FormulaError("incompatible dimensions in WeightedSqNorm")


def WeightedSqDist(s, a, b):
    return WeightedSqNorm(s, Subtract(as_op(a), as_op(b)))


class ConcatNode(Op):
    name = "Concat"
    __slots__ = ()

    def __init__(self, a, b):
        super().__init__((a, b), (), a.dim + b.dim)

    def lower(self, L, kids):
        return kids[0] + kids[1]

    def diff_t(self, v, gradin):
        a, b = self.children
        return Add(a.diff_t(v, Extract(gradin, 0, a.dim)), b.diff_t(v, Extract(gradin, a.dim, b.dim)))


def Concat(a, b):
    return ConcatNode(as_op(a), as_op(b))


class ExtractNode(Op):
    name = "Extract"
    __slots__ = ()

    def __init__(self, f, start, dim):
        if start < 0 or start + dim > f.dim:
            raise FormulaError("Index out of bound in Extract")
        super().__init__((f,), (int(start), int(dim)), dim)

    def lower(self, L, kids):
        s, d = self.params
        return kids[0][s : s + d]

    def diff_t(self, v, gradin):
        f = self.children[0]
        return f.diff_t(v, ExtractT(gradin, self.params[0], f.dim))


def Extract(f, start, dim):
    f = as_op(f)
    if start == 0 and dim == f.dim:
        return f
    if isinstance(f, Zero):
        return Zero(dim)
    if isinstance(f, ConcatNode):
        a, b = f.children
        if start + dim <= a.dim:
            return Extract(a, start, dim)
        if start >= a.dim:
            return Extract(b, start - a.dim, dim)
    if isinstance(f, SumTNode):
        return SumT(f.children[0], dim)
    return ExtractNode(f, start, dim)


class ExtractTNode(Op):
    """ExtractT(f, start, dim): embed f into a zero vector of size dim at offset start."""

    name = "ExtractT"
    __slots__ = ()

    def __init__(self, f, start, dim):
        if start < 0 or start + f.dim > dim:
            raise FormulaError("Index out of bound in ExtractT")
        super().__init__((f,), (int(start), int(dim)), dim)

    def lower(self, L, kids):
        s, d = self.params
        z = L.const(0.0)
        return [z] * s + kids[0] + [z] * (d - s - len(kids[0]))

    def diff_t(self, v, gradin):
        f = self.children[0]
        return f.diff_t(v, Extract(gradin, self.params[0], f.dim))


def ExtractT(f, start, dim):
    f = as_op(f)
    if start == 0 and dim == f.dim:
        return f
    if isinstance(f, Zero):
        return Zero(dim)
    return ExtractTNode(f, start, dim)


def Elem(f, m):
    return Extract(as_op(f), m, 1)


def ElemT(f, n, m):
    return ExtractT(as_op(f), m, n)


class OneHotNode(Op):
    name = "OneHot"
    __slots__ = ()

    def __init__(self, f, dim):
        if f.dim != 1:
            raise FormulaError("One-hot representation is only supported for scalar formulas.")
        super().__init__((f,), (int(dim),), dim)

    def lower(self, L, kids):
        r = L.call("floor", L.add(kids[0][0], L.const(0.5)))  # (int)(x + .5), OneHot.py
        return [L.select(L.eq(r, L.const(float(k))), L.const(1.0), L.const(0.0)) for k in range(self.dim)]

    def diff_t(self, v, gradin):
        return Zero(v.dim)


def OneHot(f, dim):
    return OneHotNode(as_op(f), dim)


class BSplineImplNode(Op):
    """All B-spline functions of order ``order`` on the knot vector ``knots``, sampled at the scalar ``x``, by
    De Boor's recursion in place (maths/BSpline.py:19-95): n_knots - 1 values, of which the first
    n_knots - order - 1 are the splines (the others are intermediate storage)."""

    name = "BSpline_Impl"
    __slots__ = ()

    def __init__(self, knots, x, order):
        order = int(order)
        if order < 0:
            raise FormulaError(f"The order of a BSpline must be >= 0, but received {order}.")
        if x.dim != 1:
            raise FormulaError(f"BSplines must be sampled at scalar values, but received a vector of size {x.dim}.")
        if knots.dim < order + 2:
            raise FormulaError(f"BSplines of order {order} require at least {order + 2} knots, but only received "
                               f"a vector of size {knots.dim}.")
        super().__init__((knots, x), (order,), knots.dim - 1)

    def lower(self, L, kids):
        t, (x,) = kids
        one, zero = L.const(1.0), L.const(0.0)
        # order 0: indicator of t[j] <= x < t[j+1]
        out = [L.select(L.le(t[j], x), L.select(L.lt(x, t[j + 1]), one, zero), zero) for j in range(self.dim)]

        def ratio(lo, hi):  # (x - t_lo) / (t_hi - t_lo), 0 on an empty knot span
            return L.select(L.lt(t[lo], t[hi]), L.div(L.sub(x, t[lo]), L.sub(t[hi], t[lo])), zero)

        for k in range(1, self.params[0] + 1):
            r1 = ratio(0, k)
            for i in range(self.dim - k):
                r2 = ratio(i + 1, i + 1 + k)
                out[i] = L.add(L.mul(r1, out[i]), L.mul(L.sub(one, r2), out[i + 1]))
                r1 = r2
        return out

    def diff_t(self, v, gradin):
        raise NotImplementedError("KeOps BSplines are not yet differentiable. Please consider disabling autograd "
                                  "for the relevant variables with 'x.detach()'.")


def BSpline(knots, x, order):
    """Vector of the n_knots - order - 1 B-spline functions of order ``order`` at x (maths/BSpline.py:112-115)."""
    knots, x = as_op(knots), as_op(x)
    return Extract(BSplineImplNode(knots, x, order), 0, knots.dim - int(order) - 1)


def _softdtw_table(L, x, y, gamma):
    """r[j][i] of the soft dynamic time warping recursion on squared differences (maths/SoftDTW_SqDist.py:31-69):
    r = (x_i - y_j)^2 + softmin_gamma(r[j-1][i-1], r[j-1][i], r[j][i-1])."""
    n, m = len(x), len(y)
    r = [[None] * n for _ in range(m)]

    def d2(i, j):
        d = L.sub(x[i], y[j])
        return L.mul(d, d)

    def fmin(a, b):
        return L.select(L.lt(b, a), b, a)

    r[0][0] = d2(0, 0)
    for i in range(1, n):
        r[0][i] = L.add(d2(i, 0), r[0][i - 1])
    for j in range(1, m):
        r[j][0] = L.add(d2(0, j), r[j - 1][0])
        for i in range(1, n):
            a, b, c = r[j - 1][i - 1], r[j - 1][i], r[j][i - 1]
            mn = fmin(fmin(a, b), c)
            e = L.add(L.add(L.exp(L.div(L.sub(mn, a), gamma)), L.exp(L.div(L.sub(mn, c), gamma))),
                      L.exp(L.div(L.sub(mn, b), gamma)))
            r[j][i] = L.add(d2(i, j), L.sub(mn, L.mul(gamma, L.log(e))))
    return r


class SoftDTWSqDistNode(Op):
    """Soft-DTW discrepancy between the series x (size n) and y (size m) with smoothing gamma, on squared
    differences (maths/SoftDTW_SqDist.py:21-83)."""

    name = "SoftDTW_SqDist"
    __slots__ = ()

    def __init__(self, x, y, gamma):
        if gamma.dim != 1:
            raise FormulaError("input gamma should be scalar")
        super().__init__((x, y, gamma), (), 1)

    def lower(self, L, kids):
        x, y, (gamma,) = kids
        return [_softdtw_table(L, x, y, gamma)[-1][-1]]

    def diff_t(self, v, gradin):
        x, y, gamma = self.children
        if v in gamma.variables:
            raise FormulaError("autograd wrt gamma in SoftDTW_SqDist operation not implemented.")
        grad = Mult(GradSoftDTWSqDistNode(x, y, gamma), gradin)
        return Add(x.diff_t(v, Extract(grad, 0, x.dim)), y.diff_t(v, Extract(grad, x.dim, y.dim)))


class GradSoftDTWSqDistNode(Op):
    """Gradient of SoftDTW_SqDist with respect to (x, y), size n + m: forward table, then the backward recursion
    on the alignment weights e[j][i] (maths/SoftDTW_SqDist.py:86-213)."""

    name = "GradSoftDTW_SqDist"
    __slots__ = ()

    def __init__(self, x, y, gamma):
        if gamma.dim != 1:
            raise FormulaError("input gamma should be scalar")
        super().__init__((x, y, gamma), (), x.dim + y.dim)

    def lower(self, L, kids):
        x, y, (gamma,) = kids
        n, m = len(x), len(y)
        r = _softdtw_table(L, x, y, gamma)
        two = L.const(2.0)

        def diff(i, j):
            return L.sub(x[i], y[j])

        def w(r_to, r_from, d):  # exp((r_to - r_from - d^2) / gamma): share of cell `to` that came through `from`
            return L.exp(L.div(L.sub(L.sub(r_to, r_from), L.mul(d, d)), gamma))

        e = [[None] * n for _ in range(m)]
        e[m - 1][n - 1] = L.const(1.0)
        for i in range(n - 2, -1, -1):
            e[m - 1][i] = L.mul(w(r[m - 1][i + 1], r[m - 1][i], diff(i + 1, m - 1)), e[m - 1][i + 1])
        for j in range(m - 2, -1, -1):
            e[j][n - 1] = L.mul(w(r[j + 1][n - 1], r[j][n - 1], diff(n - 1, j + 1)), e[j + 1][n - 1])
            for i in range(n - 2, -1, -1):
                a = w(r[j][i + 1], r[j][i], diff(i + 1, j))
                b = w(r[j + 1][i], r[j][i], diff(i, j + 1))
                c = w(r[j + 1][i + 1], r[j][i], diff(i + 1, j + 1))
                e[j][i] = L.add(L.add(L.mul(a, e[j][i + 1]), L.mul(b, e[j + 1][i])), L.mul(c, e[j + 1][i + 1]))
        gx, gy = [L.const(0.0)] * n, [L.const(0.0)] * m
        for j in range(m):
            for i in range(n):
                t = L.mul(L.mul(two, diff(i, j)), e[j][i])
                gx[i] = L.add(gx[i], t)
                gy[j] = L.sub(gy[j], t)
        return gx + gy

    def diff_t(self, v, gradin):
        raise FormulaError("autograd for GradSoftDTW_SqDist operation not implemented.")


def SoftDTW_SqDist(x, y, gamma):
    return SoftDTWSqDistNode(as_op(x), as_op(y), as_op(gamma))


class VecReduceNode(Op):
    """Max / Min / ArgMax / ArgMin over the components of a vector formula."""

    __slots__ = ()

    def __init__(self, f):
        super().__init__((f,), (), 1)

    def lower(self, L, kids):
        (a,) = kids
        is_max = self.name in ("Max", "ArgMax")
        best, idx = a[0], L.const(0.0)
        for k, t in enumerate(a[1:], 1):
            c = L.lt(best, t) if is_max else L.lt(t, best)
            idx = L.select(c, L.const(float(k)), idx)
            best = L.select(c, t, best)
        return [idx if self.name.startswith("Arg") else best]

    def diff_t(self, v, gradin):
        f = self.children[0]
        if self.name.startswith("Arg"):
            return Zero(v.dim)
        arg = ArgMax(f) if self.name == "Max" else ArgMin(f)
        return f.diff_t(v, Mult(OneHot(arg, f.dim), gradin))


MaxNode = type("MaxNode", (VecReduceNode,), dict(name="Max", __slots__=()))
MinNode = type("MinNode", (VecReduceNode,), dict(name="Min", __slots__=()))
ArgMaxNode = type("ArgMaxNode", (VecReduceNode,), dict(name="ArgMax", __slots__=()))
ArgMinNode = type("ArgMinNode", (VecReduceNode,), dict(name="ArgMin", __slots__=()))


def Max(f):
    return MaxNode(as_op(f))


def Min(f):
    return MinNode(as_op(f))


def ArgMax(f):
    return ArgMaxNode(as_op(f))


def ArgMin(f):
    return ArgMinNode(as_op(f))


class MatVecMultNode(Op):
    """MatVecMult(A, x): A is (n x m) stored column-major, out_i = sum_k A[k*n+i] x_k (MatVecMult.py)."""

    name = "MatVecMult"
    __slots__ = ()

    def __init__(self, a, x):
        if a.dim % x.dim:
            raise FormulaError("Dimensions of A and B are not compatible for matrix-vector product")
        super().__init__((a, x), (), a.dim // x.dim)

    def lower(self, L, kids):
        a, x = kids
        n = self.dim
        out = []
        for i in range(n):
            acc = L.mul(a[i], x[0])
            for k in range(1, len(x)):
                acc = L.fma(a[k * n + i], x[k], acc)
            out.append(acc)
        return out

    def diff_t(self, v, gradin):
        a, x = self.children
        return Add(a.diff_t(v, TensorProd(x, gradin)), x.diff_t(v, VecMatMult(gradin, a)))


def MatVecMult(a, x):
    return MatVecMultNode(as_op(a), as_op(x))


class VecMatMultNode(Op):
    """VecMatMult(x, A): out_k = sum_i x_i A[k*n+i] with n = dim(x) (VecMatMult.py)."""

    name = "VecMatMult"
    __slots__ = ()

    def __init__(self, x, a):
        if a.dim % x.dim:
            raise FormulaError("Dimensions of A and B are not compatible for vector-matrix product")
        super().__init__((x, a), (), a.dim // x.dim)

    def lower(self, L, kids):
        x, a = kids
        n = len(x)
        out = []
        for k in range(self.dim):
            acc = L.mul(x[0], a[k * n])
            for i in range(1, n):
                acc = L.fma(x[i], a[k * n + i], acc)
            out.append(acc)
        return out

    def diff_t(self, v, gradin):
        x, a = self.children
        return Add(x.diff_t(v, MatVecMult(a, gradin)), a.diff_t(v, TensorProd(gradin, x)))


def VecMatMult(x, a):
    return VecMatMultNode(as_op(x), as_op(a))


class TensorProdNode(Op):
    """TensorProd(a, b): out[i*dim(b)+j] = a_i b_j (TensorProd.py)."""

    name = "TensorProd"
    __slots__ = ()

    def __init__(self, a, b):
        super().__init__((a, b), (), a.dim * b.dim)

    def lower(self, L, kids):
        a, b = kids
        return [L.mul(s, t) for s in a for t in b]

    def diff_t(self, v, gradin):
        a, b = self.children
        # out viewed as a (dim(a) x dim(b)) row-major matrix G: da = G b, db = G^T a
        return Add(a.diff_t(v, VecMatMult(b, gradin)), b.diff_t(v, MatVecMult(gradin, a)))


def TensorProd(a, b):
    return TensorProdNode(as_op(a), as_op(b))


class DifferenceMatrixNode(Op):
    """DifferenceMatrix(x, y): out[j*dim(x)+i] = x_i - y_j, the table of differences that
    LazyTensor.difference_matrix asks for (pykeops/common/lazy_tensor.py:1591-1597; the reference's formula layer holds
    no such operation, its definition is the one of pykeops/sandbox/test_soft_dtw_kernel_dissmatrix.py:238-267)."""

    name = "DifferenceMatrix"
    __slots__ = ()

    def __init__(self, x, y):
        super().__init__((x, y), (), x.dim * y.dim)

    def lower(self, L, kids):
        x, y = kids
        return [L.sub(s, t) for t in y for s in x]

    def diff_t(self, v, gradin):
        x, y = self.children
        n, m = x.dim, y.dim
        # gradin viewed as an (m x n) row-major table G: dx_i = sum_j G[j][i], dy_j = -sum_i G[j][i]
        rows = [Extract(gradin, j * n, n) for j in range(m)]
        gx, gy = rows[0], Sum(rows[0])
        for r in rows[1:]:
            gx, gy = Add(gx, r), Concat(gy, Sum(r))
        return Add(x.diff_t(v, gx), y.diff_t(v, Minus(gy)))


def DifferenceMatrix(x, y):
    return DifferenceMatrixNode(as_op(x), as_op(y))


def _ints(t, what):
    try:
        return tuple(int(x) for x in t)
    except TypeError:
        raise FormulaError(f"TensorDot: {what} must be a list of integers") from None


class TensorDotNode(Op):
    """TensorDot(a, b, dimsfa, dimsfb, contfa, contfb[, permute]) (maths/TensorDot.py:51-140): a and b are
    row-major tensors of shapes dimsfa / dimsfb; axes contfa of a are contracted with axes contfb of b
    (paired in order); the result carries the kept axes of a, then those of b, and source axis k of
    that result ends at position permute[k]."""

    name = "TensorDot"
    __slots__ = ()

    def __init__(self, a, b, dimsfa, dimsfb, contfa, contfb, permute=None):
        dimsfa, dimsfb = _ints(dimsfa, "dimsfa"), _ints(dimsfb, "dimsfb")
        contfa, contfb = _ints(contfa, "contfa"), _ints(contfb, "contfb")
        if math.prod(dimsfa) != a.dim or math.prod(dimsfb) != b.dim:
            raise FormulaError("TensorDot: tensor shapes do not match the operand dimensions")
        if len(contfa) != len(contfb) or [dimsfa[k] for k in contfa] != [dimsfb[k] for k in contfb]:
            raise FormulaError("TensorDot: contracted axes do not match")
        if len(set(contfa)) != len(contfa) or len(set(contfb)) != len(contfb):
            raise FormulaError("TensorDot: repeated contraction axis")
        keep_a = [k for k in range(len(dimsfa)) if k not in contfa]
        keep_b = [k for k in range(len(dimsfb)) if k not in contfb]
        nkeep = len(keep_a) + len(keep_b)
        permute = tuple(range(nkeep)) if permute is None else _ints(permute, "permute")
        if sorted(permute) != list(range(nkeep)):
            raise FormulaError("TensorDot: permute must be a permutation of the kept axes")
        dim = math.prod([dimsfa[k] for k in keep_a]) * math.prod([dimsfb[k] for k in keep_b])
        super().__init__((a, b), (dimsfa, dimsfb, contfa, contfb, permute), dim)

    def _layout(self):
        dimsfa, dimsfb, contfa, contfb, permute = self.params
        keep_a = [k for k in range(len(dimsfa)) if k not in contfa]
        keep_b = [k for k in range(len(dimsfb)) if k not in contfb]
        return dimsfa, dimsfb, list(contfa), list(contfb), list(permute), keep_a, keep_b

    def out_shape(self):
        dimsfa, dimsfb, _, _, permute, keep_a, keep_b = self._layout()
        keep = [dimsfa[k] for k in keep_a] + [dimsfb[k] for k in keep_b]
        shape = [0] * len(keep)
        for k, dst in enumerate(permute):
            shape[dst] = keep[k]
        return tuple(shape)

    def lower(self, L, kids):
        import numpy as np

        a, b = kids
        dimsfa, dimsfb, contfa, contfb, permute, keep_a, keep_b = self._layout()
        C = math.prod([dimsfa[k] for k in contfa])
        ia = np.arange(len(a)).reshape(dimsfa or (1,)).transpose(keep_a + contfa).reshape(-1, C) if dimsfa else np.zeros((1, 1), int)
        ib = np.arange(len(b)).reshape(dimsfb or (1,)).transpose(keep_b + contfb).reshape(-1, C) if dimsfb else np.zeros((1, 1), int)
        res = np.empty((ia.shape[0], ib.shape[0]), dtype=object)
        for r in range(ia.shape[0]):
            for c in range(ib.shape[0]):
                acc = None
                for k in range(C):
                    t = L.mul(a[int(ia[r, k])], b[int(ib[c, k])])
                    acc = t if acc is None else L.add(acc, t)
                res[r, c] = acc
        keep = [dimsfa[k] for k in keep_a] + [dimsfb[k] for k in keep_b]
        if keep:
            axes = sorted(range(len(permute)), key=permute.__getitem__)  # destination axis i <- source axis axes[i]
            res = res.reshape(keep).transpose(axes)
        return [x for x in res.ravel()]

    def diff_t(self, v, gradin):
        a, b = self.children
        dimsfa, dimsfb, contfa, contfb, permute, keep_a, keep_b = self._layout()
        gshape = self.out_shape()
        na = len(keep_a)

        def part(wrt_a):
            # d(first operand) = TensorDot(gradin, other): contract the gradient axes that came from the
            # other operand with that operand's kept axes, then order the result like the operand itself
            if wrt_a:
                other, odims, okeep, ocont = b, dimsfb, keep_b, contfb
                gcont = [permute[na + t] for t in range(len(keep_b))]
                mine_keep, mine_cont, src0 = keep_a, contfa, 0
            else:
                other, odims, okeep, ocont = a, dimsfa, keep_a, contfa
                gcont = [permute[t] for t in range(na)]
                mine_keep, mine_cont, src0 = keep_b, contfb, na
            gkeep = [p for p in range(len(gshape)) if p not in gcont]   # ascending positions of the gradient
            orest = [k for k in range(len(odims)) if k not in okeep]     # = sorted(ocont)
            perm = []
            for p in gkeep:
                s = permute.index(p) - src0    # which kept axis of my operand sits at gradient position p
                perm.append(mine_keep[s])
            for beta in orest:
                perm.append(mine_cont[ocont.index(beta)])
            return TensorDot(gradin, other, gshape, odims, gcont, okeep, perm)

        return Add(a.diff_t(v, part(True)), b.diff_t(v, part(False)))


def TensorDot(a, b, dimsfa, dimsfb, contfa, contfb, permute=None):
    return TensorDotNode(as_op(a), as_op(b), dimsfa, dimsfb, contfa, contfb, permute)


def Kron(a, b, dimsfa, dimsfb):
    """Kronecker product as np.kron (maths/Kron.py): einsum('ij..,lm..->iljm..')."""
    dimsfa, dimsfb = _ints(dimsfa, "dimsfa"), _ints(dimsfb, "dimsfb")
    if len(dimsfa) != len(dimsfb):
        raise FormulaError("Kron: both tensors must have the same number of axes")
    n = len(dimsfa)
    return TensorDot(a, b, dimsfa, dimsfb, (), (), tuple(range(0, 2 * n, 2)) + tuple(range(1, 2 * n, 2)))


def SqNormIso(s, x):
    """s |x|^2 (maths/SqNormIso.py)."""
    return Mult(as_op(s), SqNorm2(x))


def SqNormDiag(s, x):
    """sum_k s_k x_k^2 (maths/SqNormDiag.py)."""
    return Sum(Mult(as_op(s), Square(x)))


def SymSqNorm(a, x):
    """sum_ij a_ij x_i x_j (maths/SymSqNorm.py)."""
    x = as_op(x)
    return Sum(Mult(as_op(a), TensorProd(x, x)))


def Ind(*k):
    """Index list literal of the formula grammar, e.g. TensorDot(a, b, Ind(2,3), Ind(3,2), Ind(1), Ind(0))."""
    return tuple(int(x) for x in k)


# ----------------------------------------------------------------------------- registry

BUILDERS = dict(
    Var=Var, Zero=Zero, IntCst=IntCst, RatCst=RatCst, FloatCst=FloatCst,
    Minus=Minus, Exp=Exp, Log=Log, Sqrt=Sqrt, Rsqrt=Rsqrt, Inv=Inv, Square=Square, Abs=Abs, Sign=Sign,
    Step=Step, ReLU=ReLU, Sin=Sin, Cos=Cos, Asin=Asin, Acos=Acos, Atan=Atan, Floor=Floor, XLogX=XLogX,
    SinXDivX=SinXDivX, Pow=Pow, Round=Round, Add=Add, Subtract=Subtract, Mult=Mult, Divide=Divide,
    Powf=Powf, Atan2=Atan2, Equal=Equal, NotEqual=NotEqual, LessThan=LessThan, LessOrEqual=LessOrEqual,
    IfElse=IfElse, Clamp=Clamp, ClampInt=ClampInt, DiffClampInt=DiffClampInt, Mod=Mod, Sum=Sum, SumT=SumT,
    Scalprod=Scalprod, Concat=Concat, Extract=Extract, ExtractT=ExtractT, OneHot=OneHot, Max=Max, Min=Min,
    ArgMax=ArgMax, ArgMin=ArgMin, MatVecMult=MatVecMult, VecMatMult=VecMatMult, TensorProd=TensorProd,
    TensorDot=TensorDot, SoftDTW_SqDist=SoftDTW_SqDist, DifferenceMatrix=DifferenceMatrix,
    GradSoftDTW_SqDist=lambda x, y, g: GradSoftDTWSqDistNode(as_op(x), as_op(y), as_op(g)),
    BSpline_Impl=lambda knots, x, order: BSplineImplNode(as_op(knots), as_op(x), order),
)

# names that only exist as constructors (they expand into the nodes above)
FUNCTIONS = dict(
    BUILDERS,
    Vi=Vi, Vj=Vj, Pm=Pm, IntInv=IntInv, SqNorm2=SqNorm2, Norm2=Norm2, SqDist=SqDist, Normalize=Normalize,
    WeightedSqNorm=WeightedSqNorm, WeightedSqDist=WeightedSqDist, Elem=Elem, ElemT=ElemT,
    Kron=Kron, SqNormIso=SqNormIso, SqNormDiag=SqNormDiag, SymSqNorm=SymSqNorm, Ind=Ind, BSpline=BSpline,
)


def Grad(formula, v, gradin=None):
    """[d_v F]^T . gradin (autodiff/Grad.py:14-27)."""
    if gradin is None:
        if v.cat == 2:
            raise FormulaError("Grad without gradin is not implemented for parameters")
        inds = [w.ind for w in formula.variables]
        gradin = Var(1 + max(inds) if inds else 0, formula.dim, 1 - v.cat)
    return formula.diff_t(v, gradin)


FUNCTIONS["Grad"] = Grad


def GradMatrix(f, v):
    """Matrix of the gradient operator of f with respect to v (transpose of the Jacobian), row by row: the
    concatenation over the standard basis e_k of the output space of [d_v f]^T e_k (maths/GradMatrix.py:22-34)."""
    f, v = as_op(f), as_op(v)
    if not isinstance(v, Var):
        raise FormulaError("GradMatrix(F, v): v must be a variable")
    res = None
    for k in range(f.dim):
        g = f.diff_t(v, ElemT(IntCst(1), f.dim, k))
        res = g if res is None else Concat(res, g)
    return res


FUNCTIONS["GradMatrix"] = GradMatrix


def _fresh_probe(dim, *formulas):
    """A variable no formula contains, used as a symbolic cotangent that must vanish from the result."""
    inds = [w.ind for f in formulas for w in f.variables]
    return Var(1 + (max(inds) if inds else 0) + (1 << 20), dim, 3)


def Diff(formula, v, u):
    """Forward-mode differential D_v F . u (autodiff/Diff.py:14-34: the adjoint of the gradient map).
    The gradient G(g) = [d_v F]^T g is linear in its cotangent g, so its adjoint applied to u is the gradient
    of <G(g), u> with respect to g: reverse mode twice, and g drops out."""
    formula, v, u = as_op(formula), as_op(v), as_op(u)
    if not isinstance(v, Var) or u.dim != v.dim:
        raise FormulaError("Diff(F, v, u): v must be a variable and u must have its dimension")
    g = _fresh_probe(formula.dim, formula, v, u)
    inner = Scalprod(formula.diff_t(v, g), u) if v.dim > 1 else Mult(formula.diff_t(v, g), u)
    res = inner.diff_t(g, IntCst(1))
    if g in res.variables:
        raise FormulaError("Diff: the formula contains an operation whose gradient is not linear in its cotangent")
    return res


def Divergence(formula, v):
    """Trace of the Jacobian of F with respect to v (autodiff/Divergence.py:15-37); dim(F) = dim(v)."""
    formula, v = as_op(formula), as_op(v)
    if formula.dim != v.dim:
        raise FormulaError("Divergence requires formula and variable to have the same dimension.")
    acc = Zero(1)
    for k in range(v.dim):
        acc = Add(acc, Elem(Diff(formula, v, ElemT(IntCst(1), v.dim, k)), k))
    return acc


def TraceOperator(formula, v):
    """Trace of a formula that is linear in the variable v (LinearOperators/TraceOperator.py:27-101 with w = 1):
    dim(F) = dim(v): sum_k M_kk of the matrix M of F; dim(F) = 1: sum_k M_k.  The Jacobian of a linear formula does not
    depend on v, so v is absent from the result (a formula that still contains it was not linear)."""
    formula, v = as_op(formula), as_op(v)
    if not isinstance(v, Var):
        raise FormulaError("TraceOperator(F, v): v must be a variable")
    if formula.dim == v.dim:
        res = Divergence(formula, v)
    elif formula.dim == 1:
        res = Diff(formula, v, SumT(IntCst(1), v.dim))
    else:
        raise FormulaError(f"TraceOperator: output dimension should be 1 or {v.dim} (got {formula.dim}).")
    if v in res.variables:
        raise FormulaError("TraceOperator: the formula must be a linear function of the variable")
    return res


def Laplacian(formula, v):
    """Divergence of the gradient of a scalar formula (autodiff/Laplacian.py:16-23)."""
    formula, v = as_op(formula), as_op(v)
    if formula.dim != 1:
        raise FormulaError("Laplacian is only implemented for scalar formula.")
    return Divergence(formula.diff_t(v, IntCst(1)), v)


FUNCTIONS.update(Diff=Diff, Divergence=Divergence, Laplacian=Laplacian, TraceOperator=TraceOperator)
