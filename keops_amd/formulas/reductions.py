"""Reduction descriptors: what is folded over the reduced index, and its gradient.

Mirrors keopscore/keopscore/formulas/reductions/*.py: each class fixes the dimension of the
running accumulator (``dimred``), the dimension of the stored output (``dim``), the numeric
policy id the HIP templates switch on (``kind``) and ``diff_t`` (DiffT in the reference).
``tagI`` is the category of the *output* index (0: output indexed by i, reduction over j).
"""
from __future__ import annotations

from . import ops
from .ops import Concat, Exp, Extract, FormulaError, Grad, IntCst, Op, Subtract, Zero

# policy ids shared with keops_amd/csrc/kernels/reductions.h
KIND_SUM, KIND_LSE, KIND_MIN, KIND_MAX, KIND_KMIN, KIND_ZERO = 0, 1, 2, 3, 4, 5
# what FinalizeOutput keeps of a (value, index) accumulator
KEEP_BOTH, KEEP_VAL, KEEP_IDX = 0, 1, 2


class Reduction:
    string_id = "Reduction"
    kind = KIND_SUM
    keep = KEEP_BOTH
    K = 1

    def __init__(self, formula: Op, tagI: int):
        if tagI not in (0, 1):
            raise FormulaError("the reduction axis tag must be 0 or 1")
        self.formula = formula
        self.tagI = int(tagI)
        self.tagJ = 1 - self.tagI

    @property
    def variables(self):
        return self.formula.variables

    def __repr__(self):
        return f"{self.string_id}({self.formula!r},{self.tagI})"

    def diff_t(self, v, gradin, f0=None):
        raise NotImplementedError(f"autodiff through {self.string_id} is not supported")


class Sum_Reduction(Reduction):
    string_id = "Sum_Reduction"
    kind = KIND_SUM

    def __init__(self, formula, tagI):
        super().__init__(formula, tagI)
        self.dim = self.dimred = formula.dim

    def diff_t(self, v, gradin, f0=None):
        # Sum_Reduction.py:42-45
        g = Grad(self.formula, v, gradin)
        if isinstance(g, Zero):
            return Zero_Reduction(v.dim, v.cat % 2)
        return Sum_Reduction(g, v.cat % 2)


class Zero_Reduction(Reduction):
    string_id = "Zero_Reduction"
    kind = KIND_ZERO

    def __init__(self, dim, tagI):
        super().__init__(Zero(dim), tagI)
        self.dim = self.dimred = dim

    def __repr__(self):
        return f"Zero_Reduction({self.dim},{self.tagI})"

    def diff_t(self, v, gradin, f0=None):
        return Zero_Reduction(v.dim, v.cat % 2)


class Max_SumShiftExpWeight_Reduction(Reduction):
    """(m_i, s_i) with m = max_j f_ij and s = sum_j exp(f_ij - m_i) g_ij; the Python layer
    turns it into log-sum-exp / softmax (Max_SumShiftExpWeight_Reduction.py:17-33)."""

    string_id = "Max_SumShiftExpWeight_Reduction"
    kind = KIND_LSE

    def __init__(self, formulaF, tagI, formulaG=None):
        if formulaG is None:
            formulaG = IntCst(1)
        if formulaF.dim != 1:
            raise FormulaError("Max_SumShiftExpWeight_Reduction requires first formula of dimension 1.")
        super().__init__(Concat(formulaF, formulaG), tagI)
        self.formulaF, self.formulaG = formulaF, formulaG
        self.dim = self.dimred = formulaF.dim + formulaG.dim

    def __repr__(self):
        return f"{self.string_id}({self.formulaF!r},{self.tagI},{self.formulaG!r})"

    def diff_t(self, v, gradin, MS=None):
        # Only valid once (m, s) has been flattened to m + log(s) (or a weighted softmax) and
        # gradin = [dL, dL / s] has been back-propagated (same caveat as the reference, :89-103).
        F, G = self.formulaF, self.formulaG
        M = Extract(MS, 0, F.dim)
        gradin_S = Extract(gradin, F.dim, G.dim)
        return Sum_Reduction(ops.Mult(Exp(Subtract(F, M)), G), self.tagI).diff_t(v, gradin_S)


Max_SumShiftExp_Reduction = Max_SumShiftExpWeight_Reduction


class _ValIdx(Reduction):
    def __init__(self, formula, tagI):
        super().__init__(formula, tagI)
        self.dimred = 2 * formula.dim
        self.dim = self.dimred if self.keep == KEEP_BOTH else formula.dim

    def diff_t(self, v, gradin, f0=None):
        if self.keep == KEEP_IDX:
            return Zero_Reduction(v.dim, v.cat % 2)
        raise NotImplementedError(f"autodiff through {self.string_id} is not supported")


def _mk_validx(name, kind, keep):
    return type(name, (_ValIdx,), dict(string_id=name, kind=kind, keep=keep))


Min_ArgMin_Reduction = _mk_validx("Min_ArgMin_Reduction", KIND_MIN, KEEP_BOTH)
Min_Reduction = _mk_validx("Min_Reduction", KIND_MIN, KEEP_VAL)
ArgMin_Reduction = _mk_validx("ArgMin_Reduction", KIND_MIN, KEEP_IDX)
Max_ArgMax_Reduction = _mk_validx("Max_ArgMax_Reduction", KIND_MAX, KEEP_BOTH)
Max_Reduction = _mk_validx("Max_Reduction", KIND_MAX, KEEP_VAL)
ArgMax_Reduction = _mk_validx("ArgMax_Reduction", KIND_MAX, KEEP_IDX)


class _KMin(Reduction):
    kind = KIND_KMIN

    def __init__(self, formula, K, tagI):
        super().__init__(formula, tagI)
        self.K = int(K)
        if self.K < 1:
            raise FormulaError("K must be a positive integer")
        self.dimred = 2 * self.K * formula.dim
        self.dim = self.dimred if self.keep == KEEP_BOTH else self.K * formula.dim

    def __repr__(self):
        return f"{self.string_id}({self.formula!r},{self.K},{self.tagI})"

    def diff_t(self, v, gradin, f0=None):
        if self.keep == KEEP_IDX:
            return Zero_Reduction(v.dim, v.cat % 2)
        raise NotImplementedError(f"autodiff through {self.string_id} is not supported")


KMin_ArgKMin_Reduction = type("KMin_ArgKMin_Reduction", (_KMin,), dict(string_id="KMin_ArgKMin_Reduction", keep=KEEP_BOTH))
KMin_Reduction = type("KMin_Reduction", (_KMin,), dict(string_id="KMin_Reduction", keep=KEEP_VAL))
ArgKMin_Reduction = type("ArgKMin_Reduction", (_KMin,), dict(string_id="ArgKMin_Reduction", keep=KEEP_IDX))


def Grad_WithSavedForward(red, v, gradin, f0):
    """autodiff/Grad_WithSavedForward.py:4-5."""
    return red.diff_t(v, gradin, f0)


def Diff_WithSavedForward(red, v, u, f0):
    """Forward-mode differential of a reduction (autodiff/Diff_WithSavedForward.py): the differential
    of a sum is the sum of the differentials, indexed like the original output."""
    if isinstance(red, Zero_Reduction):
        return Zero_Reduction(red.dim, red.tagI)
    if isinstance(red, Max_SumShiftExpWeight_Reduction):
        # Valid once (m, s) is flattened to m + log(s) or a weighted softmax by the Python layer: the tangent of
        # the output is [0, d(sum_j exp(F - m) G)] with the saved maximum m held fixed, whose image through the
        # flattening is the tangent of the flattened result (Max_SumShiftExpWeight_Reduction.py:105-121).
        F, G = red.formulaF, red.formulaG
        M = Extract(f0, 0, F.dim)
        d = ops.Diff(ops.Mult(Exp(Subtract(F, M)), G), v, u)
        if isinstance(d, Zero):
            return Zero_Reduction(red.dim, red.tagI)
        return Sum_Reduction(Concat(Zero(F.dim), d), red.tagI)
    if not isinstance(red, Sum_Reduction):
        raise NotImplementedError(f"forward-mode differentiation through {red.string_id} is not supported")
    d = ops.Diff(red.formula, v, u)
    if isinstance(d, Zero):
        return Zero_Reduction(red.dim, red.tagI)
    return Sum_Reduction(d, red.tagI)


REDUCTIONS = dict(
    Sum_Reduction=Sum_Reduction, Zero_Reduction=Zero_Reduction,
    Max_SumShiftExp_Reduction=Max_SumShiftExp_Reduction,
    Max_SumShiftExpWeight_Reduction=Max_SumShiftExpWeight_Reduction,
    Min_ArgMin_Reduction=Min_ArgMin_Reduction, Min_Reduction=Min_Reduction, ArgMin_Reduction=ArgMin_Reduction,
    Max_ArgMax_Reduction=Max_ArgMax_Reduction, Max_Reduction=Max_Reduction, ArgMax_Reduction=ArgMax_Reduction,
    KMin_ArgKMin_Reduction=KMin_ArgKMin_Reduction, KMin_Reduction=KMin_Reduction,
    ArgKMin_Reduction=ArgKMin_Reduction, Grad_WithSavedForward=Grad_WithSavedForward,
    Diff_WithSavedForward=Diff_WithSavedForward,
)
