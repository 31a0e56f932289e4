"""LazyTensor: symbolic (M,N,D) tensors that are reduced without ever being stored.

User-level counterpart of pykeops/pykeops/common/lazy_tensor.py:30-2823 and
pykeops/pykeops/torch/lazytensor/LazyTensor.py:1-87 for torch tensors: same constructor rules
((M,1,D) -> i-variable, (1,N,D) -> j-variable, (D,) / float -> parameter, int -> constant,
leading batch dimensions with broadcasting), same operator / method names and the same reduction
entry points, which build a formula and call :class:`keops_amd.torch.Genred`.

Unlike the reference, which edits formula *strings*, a LazyTensor here wraps the formula tree of
keops_amd.formulas directly; every data tensor is a placeholder variable that receives its final
position (Var(k,dim,cat)) when a reduction is requested.
"""
from __future__ import annotations

import itertools
import math

import torch

from ..formulas import ops as O
from .generic_red import Genred

_ids = itertools.count(1 << 20)  # placeholder variable indices, far above any user-chosen position


def _broadcast_batch(a, b):
    if a is None:
        return b
    if b is None:
        return a
    if len(a) != len(b):
        raise ValueError(f"Incompatible batch dimensions: {a} and {b}.")
    out = []
    for x, y in zip(a, b):
        if x != y and 1 not in (x, y):
            raise ValueError(f"Incompatible batch dimensions: {a} and {b}.")
        out.append(max(x, y))
    return tuple(out)


_genred_cache = {}
_constants = {}


def _constant_tensor(value, dtype, device):
    """Device tensor of a Python number or list of numbers used as a parameter; the same constants recur on every
    pass of an iterative algorithm, and building one costs a host-to-device copy."""
    key = (tuple(value) if isinstance(value, (list, tuple)) else value, dtype, device)
    try:
        t = _constants.get(key)
    except TypeError:  # nested lists and the like
        return torch.tensor(value, dtype=dtype, device=device)
    if t is None:
        if len(_constants) >= 256:
            _constants.clear()
        t = _constants[key] = torch.tensor(value, dtype=dtype, device=device)
    return t




class LazyTensor:
    """Symbolic wrapper for torch tensors (see the module docstring)."""

    def __init__(self, x=None, axis=None):
        self.formula = None       # Op
        self.variables = {}       # placeholder index -> tensor (or list of floats)
        self.symbolic = set()     # indices of user-positioned Var(ind,dim,cat) with no data attached
        self.batchdims = None
        self.ni = self.nj = None
        self.ranges = None
        self.backend = None
        self._dtype = None
        if x is None:
            return
        if isinstance(x, tuple):
            if len(x) != 3 or not all(isinstance(t, int) for t in x):
                raise ValueError("LazyTensors(tuple) is only valid if tuple = (ind,dim,cat) is a triplet of integers.")
            if axis is not None:
                raise ValueError("'axis' parameter should not be given when 'x' is of the form (ind,dim,cat).")
            self.formula = O.Var(*x)
            self.symbolic.add(x[0])
            return
        if isinstance(x, bool):
            raise TypeError("LazyTensors cannot be built from booleans")
        if isinstance(x, int):
            self.formula = O.IntCst(x)
            return
        if isinstance(x, float):
            x = [x]
        if isinstance(x, list):
            if axis not in (None, 2):
                raise ValueError("Lists of numbers are handled as Parameter variables, with an optional 'axis' argument that is equal to 2.")
            self._attach(x, len(x), 2)
            return
        if not isinstance(x, torch.Tensor):
            raise TypeError(
                "LazyTensors should be built from torch tensors, float/integer numbers, lists of floats "
                f"or 3-uples of integers. Received: {type(x)}"
            )
        self._dtype = x.dtype
        if x.dim() == 0:
            x = x.view(1)
        if x.dim() >= 3:
            if axis is not None:
                raise ValueError("'axis' parameter should not be given when 'x' is a 3D tensor.")
            if x.dim() > 3:
                self.batchdims = tuple(x.shape[:-3])
            if x.shape[-3] == 1 and x.shape[-2] == 1:
                x, axis = x.squeeze(-2).squeeze(-2), 2
            elif x.shape[-3] == 1:
                x, axis = x.squeeze(-3), 1
            elif x.shape[-2] == 1:
                x, axis = x.squeeze(-2), 0
            else:
                raise ValueError("If 'x' is a 3D+ tensor, its shape should be one of (..,M,1,D), (..,1,N,D) or (..,1,1,D).")
        if x.dim() >= 2 and axis != 2:
            if axis not in (0, 1):
                raise ValueError("When 'x' is encoded as a 2D array, LazyTensor expects an explicit 'axis' value in {0,1}.")
            if axis == 0:
                self.ni = x.shape[-2]
            else:
                self.nj = x.shape[-2]
            self._attach(x, x.shape[-1], axis)
        elif x.dim() == 1 or axis == 2:
            if axis not in (None, 2):
                raise ValueError("When 'x' is encoded as a 1D or 0D array, 'axis' must be None or 2 (= Parameter variable).")
            self._attach(x, x.shape[-1], 2)
        else:
            raise ValueError(f"LazyTensors can be built from 0D, 1D, 2D or 3D+ tensors. Received x of shape: {x.shape}.")

    def _attach(self, data, dim, cat):
        k = next(_ids)
        self.variables[k] = data
        self.formula = O.Var(k, dim, cat)

    # ------------------------------------------------------------------ bookkeeping
    @property
    def ndim(self):
        return self.formula.dim

    @property
    def nbatchdims(self):
        return 0 if self.batchdims is None else len(self.batchdims)

    @property
    def shape(self):
        b = () if self.batchdims is None else self.batchdims
        return b + (1 if self.ni is None else self.ni, 1 if self.nj is None else self.nj, self.ndim)

    def dim(self):
        return len(self.shape)

    def __str__(self):
        """Verbose identifier: formula, symbolic variables and shape (lazy_tensor.py:959-996)."""
        out = f"KeOps LazyTensor\n    formula: {self.formula!r}"
        if self.symbolic:
            out += "\n    symbolic variables: " + ", ".join(f"Var{v}" for v in sorted(self.symbolic))
        return out + f"\n    shape: {self.shape}"

    @property
    def dtype(self):
        return self._dtype

    def _like(self, formula, *others):
        res = type(self)()
        res.formula = formula
        srcs = (self,) + others
        for s in srcs:
            res.variables.update(s.variables)
            res.symbolic |= s.symbolic
            res.batchdims = _broadcast_batch(res.batchdims, s.batchdims)
            for prop in ("ni", "nj", "backend", "_dtype"):
                a, b = getattr(res, prop), getattr(s, prop)
                if a is not None and b is not None and a != b:
                    raise ValueError(f"Incompatible values for attribute {prop}: {a} and {b}.")
                if a is None:
                    setattr(res, prop, b)
            if s.ranges is not None:
                if res.ranges is not None and res.ranges is not s.ranges and not all(
                    torch.equal(p, q) for p, q in zip(res.ranges, s.ranges)
                ):
                    raise ValueError("Incompatible values for attribute ranges.")
                res.ranges = s.ranges
        return res

    def _lift(self, other):
        return other if isinstance(other, LazyTensor) else type(self)(other)

    def unary(self, fn, *params):
        return self._like(fn(self.formula, *params))

    def binary(self, other, fn):
        other = self._lift(other)
        return self._like(fn(self.formula, other.formula), other)

    def ternary(self, a, b, fn):
        a, b = self._lift(a), self._lift(b)
        return self._like(fn(self.formula, a.formula, b.formula), a, b)

    # ------------------------------------------------------------------ arithmetic
    def __add__(self, o):
        return self.binary(o, O.Add)

    def __radd__(self, o):
        return self if (isinstance(o, int) and o == 0) else self._lift(o).binary(self, O.Add)

    def __sub__(self, o):
        return self.binary(o, O.Subtract)

    def __rsub__(self, o):
        return self._lift(o).binary(self, O.Subtract)

    def __mul__(self, o):
        return self.binary(o, O.Mult)

    def __rmul__(self, o):
        return self._lift(o).binary(self, O.Mult)

    def __truediv__(self, o):
        return self.binary(o, O.Divide)

    def __rtruediv__(self, o):
        return self._lift(o).binary(self, O.Divide)

    def __or__(self, o):
        return self.binary(o, O.Scalprod)

    def __ror__(self, o):
        return self._lift(o).binary(self, O.Scalprod)

    def __neg__(self):
        return self.unary(O.Minus)

    def __abs__(self):
        return self.unary(O.Abs)

    def __pow__(self, p):
        if isinstance(p, int):
            return self.unary(O.Pow, p)
        if isinstance(p, float) and p == 0.5:
            return self.sqrt()
        if isinstance(p, float) and p == -0.5:
            return self.rsqrt()
        return self.binary(p, O.Powf)

    def __lt__(self, o):
        return self.binary(o, O.LessThan)

    def __le__(self, o):
        return self.binary(o, O.LessOrEqual)

    def __gt__(self, o):
        return self._lift(o).binary(self, O.LessThan)

    def __ge__(self, o):
        return self._lift(o).binary(self, O.LessOrEqual)

    def __eq__(self, o):
        return self.binary(o, O.Equal)

    def __ne__(self, o):
        return self.binary(o, O.NotEqual)

    __hash__ = object.__hash__

    def __matmul__(self, v, **kwargs):
        """K @ v: sum_j K_ij v_j with v a (N,) vector or a (..,N,D) tensor, K of trailing dimension 1; keyword
        arguments (sum_scheme, out, backend, ...) go to the reduction (lazy_tensor.py:2490-2527)."""
        if isinstance(v, LazyTensor):
            return (self * v).sum(self.nbatchdims + 1, **kwargs)
        if self.ndim != 1:
            raise ValueError("The 'K @ v' syntax is only supported for LazyTensors 'K' whose trailing dimension "
                             f"is equal to 1. Here, K.shape = {self.shape}.")
        if v.ndim == 1:
            return (self * type(self)(v.reshape(1, -1, 1))).sum(self.nbatchdims + 1, **kwargs).reshape(-1)
        return (self * type(self)(v.reshape(v.shape[:-2] + (1,) + v.shape[-2:]))).sum(self.nbatchdims + 1, **kwargs)

    def __getitem__(self, key):
        if isinstance(key, int):
            return self.unary(O.Elem, key)
        if isinstance(key, slice) and key.step in (None, 1):
            start = 0 if key.start is None else key.start
            stop = self.ndim if key.stop is None else key.stop
            return self.unary(O.Extract, start, stop - start)
        raise ValueError("LazyTensors only support indexing of the last dimension with an int or a unit-step slice")

    # ------------------------------------------------------------------ maths
    def exp(self):
        return self.unary(O.Exp)

    def log(self):
        return self.unary(O.Log)

    def xlogx(self):
        return self.unary(O.XLogX)

    def sqrt(self):
        return self.unary(O.Sqrt)

    def rsqrt(self):
        return self.unary(O.Rsqrt)

    def square(self):
        return self.unary(O.Square)

    def abs(self):
        return self.unary(O.Abs)

    def sign(self):
        return self.unary(O.Sign)

    def step(self):
        return self.unary(O.Step)

    def relu(self):
        return self.unary(O.ReLU)

    def sin(self):
        return self.unary(O.Sin)

    def cos(self):
        return self.unary(O.Cos)

    def asin(self):
        return self.unary(O.Asin)

    def acos(self):
        return self.unary(O.Acos)

    def atan(self):
        return self.unary(O.Atan)

    def atan2(self, other):
        return self.binary(other, O.Atan2)

    def floor(self):
        return self.unary(O.Floor)

    def round(self, d=0):
        return self.unary(O.Round, d)

    def sinxdivx(self):
        return self.unary(O.SinXDivX)

    def sinc(self):
        """sin(pi x) / (pi x), as torch.sinc (lazy_tensor.py:1267-1274)."""
        return (math.pi * self).sinxdivx()

    def power(self, other):
        return self ** other

    def mod(self, modulus, offset=0):
        return self.ternary(modulus, offset, O.Mod)

    def clamp(self, a, b):
        if isinstance(a, int) and isinstance(b, int):
            return self.unary(O.ClampInt, a, b)
        return self.ternary(a, b, O.Clamp)

    def ifelse(self, a, b):
        return self.ternary(a, b, O.IfElse)

    def sqnorm2(self):
        return self.unary(O.SqNorm2)

    def norm2(self):
        return self.unary(O.Norm2)

    def norm(self, dim):
        if dim not in (-1, len(self.shape) - 1):
            raise ValueError("KeOps only supports norms over the last dimension.")
        return self.norm2()

    def normalize(self):
        return self.unary(O.Normalize)

    def sqdist(self, other):
        return self.binary(other, O.SqDist)

    def weightedsqnorm(self, other):
        return self.binary(other, lambda f, s: O.WeightedSqNorm(s, f))

    def weightedsqdist(self, g, s):
        return self.ternary(g, s, lambda f, gg, ss: O.WeightedSqDist(ss, f, gg))

    def elem(self, i):
        return self.unary(O.Elem, i)

    def extract(self, i, d):
        return self.unary(O.Extract, i, d)

    def extract_t(self, i, d):
        return self.unary(O.ExtractT, i, d)

    def concat(self, other):
        return self.binary(other, O.Concat)

    @staticmethod
    def concatenate(tuple_of_lt, axis=-1):
        """``LazyTensor.concatenate((x_1, ..., x_n), -1)``: concatenation along the last dimension, the only
        one that supports it (lazy_tensor.py:1728-1760)."""
        if not isinstance(tuple_of_lt, tuple) or len(tuple_of_lt) == 0 or not isinstance(tuple_of_lt[0], LazyTensor):
            raise ValueError("LazyTensor.concatenate is implemented on non-empty tuples of LazyTensors.")
        if axis not in (-1, len(tuple_of_lt[0].shape) - 1):
            raise ValueError("LazyTensor only supports concatenation along the last axis.")
        res = tuple_of_lt[0]
        for o in tuple_of_lt[1:]:
            res = res.concat(o)
        return res

    @staticmethod
    def cat(tuple_of_lt, dim):
        """torch-style alias of :meth:`concatenate`."""
        return LazyTensor.concatenate(tuple_of_lt, dim)

    def softdtw_sqdist(self, other, gamma):
        """Soft-DTW discrepancy (squared differences) between the series self and other, smoothing gamma."""
        return self.ternary(other, gamma, O.SoftDTW_SqDist)

    def grad_matrix(self, other):
        """Matrix of the gradient operator of self with respect to the variable other, flattened row by row."""
        other = self._lift(other)
        return self._like(O.GradMatrix(self.formula, other.formula), other)

    def bspline(self, x, k=0):
        """Vector of B-spline functions of order k for the knots ``self``, evaluated at the scalar x."""
        return self.binary(x, lambda knots, t: O.BSpline(knots, t, k))

    def one_hot(self, D):
        return self.unary(O.OneHot, D)

    def matvecmult(self, other):
        return self.binary(other, O.MatVecMult)

    def vecmatmult(self, other):
        return self.binary(other, O.VecMatMult)

    def tensorprod(self, other):
        return self.binary(other, O.TensorProd)

    def difference_matrix(self, other):
        """Table of differences x_i - y_j of two vectors, of size dim(self) * dim(other), entry (j, i) at j*dim(self)+i
        (lazy_tensor.py "difference_matrix")."""
        return self.binary(other, O.DifferenceMatrix)

    def diff(self, other, diffin):
        """Symbolic forward-mode differential [d_other self] . diffin (lazy_tensor.py "diff")."""
        other, diffin = self._lift(other), self._lift(diffin)
        if not isinstance(other.formula, O.Var):
            raise ValueError("LazyTensor.diff expects a variable as its first argument")
        return self._like(O.Diff(self.formula, other.formula, diffin.formula), other, diffin)

    def divergence(self, other):
        """Symbolic divergence with respect to the variable ``other`` (lazy_tensor.py "divergence")."""
        other = self._lift(other)
        return self._like(O.Divergence(self.formula, other.formula), other)

    def trace_operator(self, var):
        """Trace of self with respect to the variable ``var``, of which self must be a linear function
        (lazy_tensor.py "trace_operator").  The variable leaves the formula: it needs no data when the result is reduced."""
        var = self._lift(var)
        if not isinstance(var.formula, O.Var):
            raise ValueError("LazyTensor.trace_operator expects a variable")
        res = self._like(O.TraceOperator(self.formula, var.formula), var)
        res.variables.pop(var.formula.ind, None)
        res.symbolic.discard(var.formula.ind)
        return res

    def laplacian(self, other):
        """Symbolic Laplacian of a scalar formula with respect to ``other`` (lazy_tensor.py "laplacian")."""
        other = self._lift(other)
        return self._like(O.Laplacian(self.formula, other.formula), other)

    def keops_tensordot(self, other, dimfa, dimfb, contfa, contfb, *args):
        """Tensor contraction of the vectors of self and other viewed as tensors of shapes dimfa / dimfb,
        like np.tensordot, with an optional final axis permutation (lazy_tensor.py "keops_tensordot")."""
        permute = tuple(args[0]) if args else None
        return self.binary(other, lambda a, b: O.TensorDot(a, b, tuple(dimfa), tuple(dimfb), tuple(contfa), tuple(contfb), permute))

    def keops_kron(self, other, dimfself, dimfother):
        """Kronecker product, as np.kron on tensors of shapes dimfself / dimfother (lazy_tensor.py "keops_kron")."""
        return self.binary(other, lambda a, b: O.Kron(a, b, tuple(dimfself), tuple(dimfother)))

    def grad(self, other, gradin):
        """Symbolic gradient [d_other self]^T gradin (lazy_tensor.py "grad")."""
        other, gradin = self._lift(other), self._lift(gradin)
        if not isinstance(other.formula, O.Var):
            raise ValueError("LazyTensor.grad expects a variable as its first argument")
        return self._like(O.Grad(self.formula, other.formula, gradin.formula), other, gradin)

    def t(self):
        """Exchange the roles of the i and j axes."""
        res = self._like(self.formula)
        mapping = {}
        for v in self.formula.variables:
            if v.cat in (0, 1):
                mapping[v] = O.Var(v.ind, v.dim, 1 - v.cat)
        f = self.formula
        for old, new in mapping.items():
            tmp = O.Var(-1 - old.ind, old.dim, 3)
            f = f.replace(old, tmp)
        for old, new in mapping.items():
            f = f.replace(O.Var(-1 - old.ind, old.dim, 3), new)
        res.formula = f
        res.ni, res.nj = self.nj, self.ni
        if self.ranges is not None:
            res.ranges = (*self.ranges[3:6], *self.ranges[0:3])
        return res

    @property
    def T(self):
        return self.t()

    # ------------------------------------------------------------------ reductions
    def _axis(self, axis, dim):
        if axis is None:
            axis = dim
        if axis is None:
            raise ValueError("Reductions must be called with an 'axis' (or 'dim') argument.")
        if axis < 0:
            axis += len(self.shape)
        axis -= self.nbatchdims
        return axis

    def reduction(self, reduction_op, other=None, opt_arg=None, axis=None, dim=None, call=True, _solve_pid=None, **kwargs):
        """Apply a reduction over axis 0 (i) or 1 (j) (lazy_tensor.py:648-777)."""
        axis = self._axis(axis, dim)
        if axis not in (0, 1):
            raise ValueError("Reductions must be performed along axis 0 (= i) or 1 (= j), after the batch dimensions.")
        whole = self if other is None else self._like(self.formula, other)
        # final positions: user-positioned symbolic variables keep theirs, data tensors fill the rest
        taken = sorted(whole.symbolic)
        order = sorted(whole.variables)
        pos, k = {}, 0
        for pid in order:
            while k in taken:
                k += 1
            pos[pid] = k
            k += 1

        def settle(f):
            moved = {v: O.Var(pos[v.ind], v.dim, v.cat) for v in f.variables if v.ind in pos and pos[v.ind] != v.ind}
            return f.rename_vars(moved) if moved else f

        formula = settle(self.formula)
        formula2 = None if other is None else settle(other.formula)
        nvars = (max(list(pos.values()) + taken) + 1) if (pos or taken) else 0
        aliases = [None] * nvars
        for f in (formula,) + (() if formula2 is None else (formula2,)):
            for v in f.variables:
                aliases[v.ind] = f"Var({v.ind},{v.dim},{v.cat})"
        if any(a is None for a in aliases):
            raise ValueError("the variables of the formula must occupy positions 0..n-1 without gaps")
        init_kw = {k: kwargs.pop(k) for k in list(kwargs) if k in
                   ("dtype_acc", "use_double_acc", "sum_scheme", "enable_chunks", "use_fast_math", "rec_multVar_highdim")}
        if reduction_op == "Solve":
            from .operations import KernelSolve

            solve_kw = {k: kwargs.pop(k) for k in list(kwargs) if k in ("alpha", "eps")}
            svar = next(v for v in formula.variables if v.ind == pos[_solve_pid])
            solver = KernelSolve(repr(formula), aliases, f"Var({svar.ind},{svar.dim},{svar.cat})", axis=axis, **init_kw)

            def fn(*args, **kw):
                return solver(*args, **solve_kw, **kw)
        else:
            # one Genred object per (formula, options): iterative algorithms rebuild the same LazyTensor every pass
            f1, f2 = repr(formula), None if formula2 is None else repr(formula2)
            key = (f1, f2, tuple(aliases), reduction_op, axis, opt_arg, tuple(sorted(init_kw.items())))
            try:
                fn = _genred_cache.get(key)
            except TypeError:  # unhashable option value
                key, fn = None, None
            if fn is None:
                fn = Genred(f1, aliases, reduction_op=reduction_op, axis=axis, opt_arg=opt_arg, formula2=f2, **init_kw)
                if key is not None:
                    if len(_genred_cache) >= 512:
                        _genred_cache.clear()
                    _genred_cache[key] = fn
        data = [None] * nvars
        cats = {v.ind: v.cat for f in (formula,) + (() if formula2 is None else (formula2,)) for v in f.variables}
        dev = next((t.device for t in whole.variables.values() if isinstance(t, torch.Tensor)), None)
        dtype = whole._dtype or torch.float32
        nb = whole.nbatchdims
        for pid, t in whole.variables.items():
            if pos[pid] not in cats:
                continue
            if not isinstance(t, torch.Tensor):
                t = _constant_tensor(t, dtype, dev)
            want = nb + (1 if cats[pos[pid]] == 2 else 2)
            if t.dim() < want:
                t = t.view((1,) * (want - t.dim()) + tuple(t.shape))
            data[pos[pid]] = t
        call_kw = dict(kwargs)
        if whole.ranges is not None and "ranges" not in call_kw:
            call_kw["ranges"] = whole.ranges
        if whole.backend is not None and "backend" not in call_kw:
            call_kw["backend"] = whole.backend

        def run(*extra):
            args, it = list(data), iter(extra)
            for k2 in range(nvars):
                if args[k2] is None:
                    args[k2] = next(it)
            return fn(*args, **call_kw)

        if call and all(d is not None for d in data):
            return run()
        return run

    def solve(self, other, var=None, call=True, **kwargs):
        """Solution ``a`` of ``sum_j self_ij a_j = other_i`` (plus ``alpha * a``) by conjugate gradient, for a
        symmetric positive definite ``self`` (lazy_tensor.py:779-897; keyword arguments alpha, eps, backend,
        ranges and the Genred options).  ``other`` is a 2D tensor (one row per index i) or an i-indexed
        LazyTensor holding one."""
        if var is not None:
            raise NotImplementedError("solve(var=...) with a symbolic unknown is not available")
        if isinstance(other, LazyTensor):
            if len(other.variables) != 1 or not isinstance(other.formula, O.Var) or other.formula.cat != 0:
                raise ValueError("'other' must be a plain i-indexed variable")
            other = next(iter(other.variables.values()))
        if not isinstance(other, torch.Tensor) or other.dim() < 2:
            raise ValueError("'other' must be a 2D tensor, one row per index i")
        unknown = LazyTensor(other, axis=1)  # the unknown is indexed like the reduced axis; 'other' is its start value
        pid = next(iter(unknown.variables))
        return (self * unknown).reduction("Solve", axis=self.nbatchdims + 1, call=call, _solve_pid=pid, **kwargs)

    def matvec(self, v):
        """Matrix-vector product with a 1D tensor, for scipy-style linear operator code (lazy_tensor.py matvec)."""
        return self @ v

    def rmatvec(self, v):
        return self.T @ v

    def sum(self, axis=None, dim=None, **kwargs):
        ax = axis if axis is not None else dim
        if ax in (-1, len(self.shape) - 1):
            return self.unary(O.Sum)
        return self.reduction("Sum", axis=axis, dim=dim, **kwargs)

    def sum_reduction(self, axis=None, dim=None, **kwargs):
        return self.reduction("Sum", axis=axis, dim=dim, **kwargs)

    def logsumexp(self, axis=None, dim=None, weight=None, **kwargs):
        if weight is None:
            return self.reduction("LogSumExp", axis=axis, dim=dim, **kwargs)
        return self.reduction("LogSumExp", other=self._lift(weight), axis=axis, dim=dim, **kwargs)

    def logsumexp_reduction(self, **kwargs):
        return self.logsumexp(**kwargs)

    def sumsoftmaxweight(self, weight, axis=None, dim=None, **kwargs):
        return self.reduction("SumSoftMaxWeight", other=self._lift(weight), axis=axis, dim=dim, **kwargs)

    def min(self, axis=None, dim=None, **kwargs):
        ax = axis if axis is not None else dim
        if ax in (-1, len(self.shape) - 1):
            return self.unary(O.Min)
        return self.reduction("Min", axis=axis, dim=dim, **kwargs)

    def argmin(self, axis=None, dim=None, **kwargs):
        ax = axis if axis is not None else dim
        if ax in (-1, len(self.shape) - 1):
            return self.unary(O.ArgMin)
        return self.reduction("ArgMin", axis=axis, dim=dim, **kwargs)

    def min_argmin(self, axis=None, dim=None, **kwargs):
        return self.reduction("Min_ArgMin", axis=axis, dim=dim, **kwargs)

    def max(self, axis=None, dim=None, **kwargs):
        ax = axis if axis is not None else dim
        if ax in (-1, len(self.shape) - 1):
            return self.unary(O.Max)
        return self.reduction("Max", axis=axis, dim=dim, **kwargs)

    def argmax(self, axis=None, dim=None, **kwargs):
        ax = axis if axis is not None else dim
        if ax in (-1, len(self.shape) - 1):
            return self.unary(O.ArgMax)
        return self.reduction("ArgMax", axis=axis, dim=dim, **kwargs)

    def max_argmax(self, axis=None, dim=None, **kwargs):
        return self.reduction("Max_ArgMax", axis=axis, dim=dim, **kwargs)

    def Kmin(self, K, axis=None, dim=None, **kwargs):
        return self.reduction("KMin", opt_arg=K, axis=axis, dim=dim, **kwargs)

    def argKmin(self, K, axis=None, dim=None, **kwargs):
        return self.reduction("ArgKMin", opt_arg=K, axis=axis, dim=dim, **kwargs)

    def Kmin_argKmin(self, K, axis=None, dim=None, **kwargs):
        return self.reduction("KMin_ArgKMin", opt_arg=K, axis=axis, dim=dim, **kwargs)


# the reference also exposes every reduction under a "<name>_reduction" alias (lazy_tensor.py)
for _name in ("min", "argmin", "min_argmin", "max", "argmax", "max_argmax", "Kmin", "argKmin", "Kmin_argKmin",
              "sumsoftmaxweight"):
    setattr(LazyTensor, _name + "_reduction", getattr(LazyTensor, _name))


def Vi(x_or_ind, dim=None):
    """Vi(x): x (M,D) as an i-variable; Vi(ind, dim): symbolic i-variable (lazy_tensor.py Vi)."""
    if dim is None:
        return LazyTensor(x_or_ind, axis=0)
    return LazyTensor((x_or_ind, dim, 0))


def Vj(x_or_ind, dim=None):
    if dim is None:
        return LazyTensor(x_or_ind, axis=1)
    return LazyTensor((x_or_ind, dim, 1))


def Pm(x_or_ind, dim=None):
    if dim is None:
        return LazyTensor(x_or_ind, axis=2)
    return LazyTensor((x_or_ind, dim, 2))
