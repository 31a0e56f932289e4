"""Scalar SSA program ("low-level IR") that a formula tree lowers to.

Every value is one scalar; vector-valued formula nodes become Python lists of value ids.  Values
are hash-consed (common sub-expressions are shared), constants are folded, and a few algebraic
peepholes keep the per-pair instruction count of the generated HIP code minimal:

* ``exp(u)`` is emitted as the hardware base-2 exponential ``exp2(u * log2(e))``.  The argument ``u`` itself is
  computed the way the reference computes it -- its operations in the reference's order, every product and sum
  rounded on its own (no fused multiply-adds), the factor ``log2(e)`` applied to the rounded ``u`` and not merged into
  a factor of it: an exponential magnifies a relative error of its argument by ``|u|``, so a kernel value deep in the
  tail (``u = -80``) is only as good as ``u`` is bit for bit, and rows whose every term lies there exist (a kernel much
  narrower than the spacing of the points).  On this GPU a product and a sum issue in the time of one fused
  multiply-add, so the only cost is the separate ``log2(e)`` multiplication.
* negations are pushed outwards (they are free source modifiers on the VALU).

The program is printed as straight-line C++ (``const T t7 = t3 * t5;``): with every index a
compile-time constant the compiler keeps all values in VGPRs.
"""
from __future__ import annotations

import math

LOG2E = 1.4426950408889634
LN2 = 0.6931471805599453

# value "levels": how often a value changes in the map-reduce loop nest
UNIFORM, PER_ROW, PER_PAIR = 0, 1, 2


class Lir:
    def __init__(self, row_cat=0, fast_math=True, dtype="float", exact_order=False):
        self.row_cat = row_cat  # category (0 = i, 1 = j) of the variables indexed like the output
        # exact_order: keep the reference's operation order and roundings (explicit fused
        # multiply-adds only where the reference calls fma, no re-association); used when the
        # reduction returns indices, whose parity is bit-exact
        self.exact = bool(exact_order)
        self.fast = bool(fast_math) and not self.exact
        self.fast_fn = bool(fast_math)  # hardware exp2/log2/rcp/sqrt approximations allowed
        self.dtype = dtype
        self.nodes = []  # (op, args...) tuples
        self.level = []
        self.index = {}
        self.loads = {}  # (cat, ind) -> set of component indices actually read
        self.rounded = set()  # values whose operation must not be contracted with a neighbour (arguments of exp)

    # ------------------------------------------------------------------ construction
    def _mk(self, key, level):
        i = self.index.get(key)
        if i is None:
            i = len(self.nodes)
            self.nodes.append(key)
            self.level.append(level)
            self.index[key] = i
        return i

    def _lvl(self, *ids):
        return max(self.level[i] for i in ids)

    def const(self, v):
        v = float(v)
        if v == 0.0:
            v = 0.0  # merge -0.0
        return self._mk(("const", v), UNIFORM)

    def is_const(self, i, v=None):
        n = self.nodes[i]
        return n[0] == "const" and (v is None or n[1] == v)

    def cval(self, i):
        return self.nodes[i][1]

    def load(self, cat, ind, k):
        self.loads.setdefault((cat, ind), set()).add(k)
        if cat == 2:
            lvl = UNIFORM
        elif cat == 3:
            lvl = PER_PAIR  # chunk accumulator input (value computed by the kernel per pair)
        else:
            lvl = PER_ROW if cat == self.row_cat else PER_PAIR
        return self._mk(("load", cat, ind, k), lvl)

    def neg(self, a):
        n = self.nodes[a]
        if n[0] == "const":
            return self.const(-n[1])
        if n[0] == "neg":
            return n[1]
        if n[0] == "sub":
            return self.sub(n[2], n[1])
        return self._mk(("neg", a), self.level[a])

    def add(self, a, b):
        if self.is_const(a) and self.is_const(b):
            return self.const(self.cval(a) + self.cval(b))
        if self.is_const(a, 0.0):
            return b
        if self.is_const(b, 0.0):
            return a
        if self.nodes[b][0] == "neg":
            return self.sub(a, self.nodes[b][1])
        if self.nodes[a][0] == "neg":
            return self.sub(b, self.nodes[a][1])
        return self._mk(("add", a, b), self._lvl(a, b))

    def sub(self, a, b):
        if self.is_const(a) and self.is_const(b):
            return self.const(self.cval(a) - self.cval(b))
        if self.is_const(b, 0.0):
            return a
        if self.is_const(a, 0.0):
            return self.neg(b)
        if self.nodes[b][0] == "neg":
            return self.add(a, self.nodes[b][1])
        if a == b and self.fast:
            return self.const(0.0)
        return self._mk(("sub", a, b), self._lvl(a, b))

    def mul(self, a, b):
        na, nb = self.nodes[a], self.nodes[b]
        if na[0] == "const" and nb[0] == "const":
            return self.const(na[1] * nb[1])
        for p, q in ((a, b), (b, a)):
            if self.is_const(p, 1.0):
                return q
            if self.is_const(p, -1.0):
                return self.neg(q)
            if self.is_const(p, 0.0) and self.fast:
                return self.const(0.0)
        if na[0] == "neg" and nb[0] == "neg":
            return self.mul(na[1], nb[1])
        if na[0] == "neg":
            return self.neg(self.mul(na[1], b))
        if nb[0] == "neg":
            return self.neg(self.mul(a, nb[1]))
        if self.fast:
            # hoisting: a factor that changes less often than its partner joins the partner's own
            # slow-changing sub-factor, (u * (v * w)) -> ((u * v) * w) when level(u), level(v) < level(w),
            # so that the slow product is computed outside the pair loop.
            for p, q in ((a, b), (b, a)):
                nq = self.nodes[q]
                if nq[0] == "mul" and self.level[p] < self.level[q]:
                    for lo, hi in ((nq[1], nq[2]), (nq[2], nq[1])):
                        if self.level[lo] < self.level[q] and self.level[hi] == self.level[q]:
                            return self.mul(self.mul(p, lo), hi)
        if a > b:
            a, b = b, a
        return self._mk(("mul", a, b), self._lvl(a, b))

    def fma(self, a, b, c):
        """a*b + c; printed as a plain multiply-add (the compiler contracts it) unless the exact
        operation order is requested, where it is a genuine single-rounding fma."""
        if self.exact:
            return self._mk(("fma", a, b, c), self._lvl(a, b, c))
        return self.add(self.mul(a, b), c)

    def div(self, a, b):
        if self.is_const(a) and self.is_const(b) and self.cval(b) != 0.0:
            return self.const(self.cval(a) / self.cval(b))
        if self.is_const(b, 1.0):
            return a
        if self.fast_fn and not self.exact:
            return self.mul(a, self.rcp(b))
        return self._mk(("div", a, b), self._lvl(a, b))

    def rcp(self, a):
        if self.is_const(a) and self.cval(a) != 0.0:
            return self.const(1.0 / self.cval(a))
        return self._mk(("rcp", a), self.level[a])

    def exp(self, a):
        if self.is_const(a):
            return self.const(math.exp(self.cval(a)))
        if self.dtype == "float" and self.fast_fn:
            if self.exact:
                return self._mk(("exp2", self.mul(a, self.const(LOG2E))), self.level[a])
            # u as the reference rounds it, then one product with log2(e): see the head of this file
            neg = self.nodes[a][0] == "neg"
            u = self.nodes[a][1] if neg else a
            self._keep_rounded(u)
            c = self.const(LOG2E)
            t = self._mk(("mul", min(u, c), max(u, c)), self.level[a])
            self.rounded.add(t)
            return self._mk(("exp2", self._mk(("neg", t), self.level[a]) if neg else t), self.level[a])
        return self._mk(("exp", a), self.level[a])

    def _keep_rounded(self, a):
        """Marks the sums and products below ``a`` that change with the pair or the output row."""
        stack = [a]
        while stack:
            i = stack.pop()
            n = self.nodes[i]
            if i in self.rounded or n[0] in ("const", "load") or self.level[i] == UNIFORM:
                continue
            if n[0] in ("add", "sub", "mul"):
                self.rounded.add(i)
            stack.extend(n[2:] if n[0] == "call" else n[1:])

    def log(self, a):
        if self.is_const(a) and self.cval(a) > 0:
            return self.const(math.log(self.cval(a)))
        if self.dtype == "float" and self.fast_fn:
            return self.mul(self._mk(("log2", a), self.level[a]), self.const(LN2))
        return self._mk(("log", a), self.level[a])

    def sqrt(self, a):
        if self.is_const(a) and self.cval(a) >= 0:
            return self.const(math.sqrt(self.cval(a)))
        return self._mk(("sqrt", a), self.level[a])

    def rsqrt0(self, a):
        """x == 0 ? 0 : 1/sqrt(x)  (keops_rsqrt, math_functions.py:104-108)."""
        if self.is_const(a):
            v = self.cval(a)
            return self.const(0.0 if v == 0 else 1.0 / math.sqrt(v))
        return self._mk(("rsqrt0", a), self.level[a])

    def abs(self, a):
        if self.is_const(a):
            return self.const(abs(self.cval(a)))
        if self.nodes[a][0] == "neg":
            return self.abs(self.nodes[a][1])
        return self._mk(("abs", a), self.level[a])

    def sign(self, a):
        return self._mk(("sign", a), self.level[a])

    def powi(self, a, m):
        if m < 0:
            return self.rcp(self.powi(a, -m))
        if m == 0:
            return self.const(1.0)
        # square-and-multiply
        result, base = None, a
        while m:
            if m & 1:
                result = base if result is None else self.mul(result, base)
            m >>= 1
            if m:
                base = self.mul(base, base)
        return result

    def call(self, fn, *args):
        return self._mk(("call", fn) + tuple(args), self._lvl(*args))

    # comparisons produce boolean values, only usable as the first argument of select
    def lt(self, a, b):
        return self._mk(("lt", a, b), self._lvl(a, b))

    def le(self, a, b):
        return self._mk(("le", a, b), self._lvl(a, b))

    def eq(self, a, b):
        return self._mk(("eq", a, b), self._lvl(a, b))

    def ne(self, a, b):
        return self._mk(("ne", a, b), self._lvl(a, b))

    def select(self, c, a, b):
        if a == b:
            return a
        return self._mk(("select", c, a, b), self._lvl(c, a, b))

    # ------------------------------------------------------------------ printing
    def live(self, outputs):
        seen = set()
        stack = list(outputs)
        while stack:
            i = stack.pop()
            if i in seen:
                continue
            seen.add(i)
            n = self.nodes[i]
            if n[0] == "const" or n[0] == "load":
                continue
            start = 2 if n[0] == "call" else 1
            stack.extend(n[start:])
        return seen

    def count_ops(self, outputs, level=PER_PAIR):
        """Number of arithmetic values at a given level (a proxy for VALU work per pair)."""
        live = self.live(outputs)
        return sum(1 for i in live if self.level[i] == level and self.nodes[i][0] not in ("const", "load", "neg"))

    def _lit(self, v):
        if v != v:
            return "(T)NAN"
        if v in (float("inf"), float("-inf")):
            return "(T)INFINITY" if v > 0 else "-(T)INFINITY"
        return f"(T){v!r}" if self.dtype == "double" else f"{float(v)!r}f".replace("e+", "e")

    def emit(self, outputs, names, indent="    ", segment=0, segment_prefix=(), segment_min=0):
        """C++ statements computing ``outputs`` (value ids).

        ``names`` maps a load key (cat, ind, k) to the C++ expression that reads it.
        Returns (lines, exprs) where exprs[k] is the C++ expression of outputs[k].

        ``segment`` > 0: a body of more than ``segment_min`` statements (formulas on vectors of hundreds of components)
        is cut into non-inlined device functions ``keops_seg_<k>(xi, yj, p, keops_live)`` of at most that many
        statements each, whose definitions are left in ``self.prelude`` (to be placed before the caller); values
        that cross a cut travel through the array ``keops_live``.  The compiler's time grows much faster than
        linearly with the length of one straight-line function; that of a sequence of bounded functions does not.
        ``segment_prefix``: lines repeated at the top of every such function (pragmas).
        """
        self.prelude = []
        live = self.live(outputs)
        f32 = self.dtype == "float"
        ref = {}
        lines = []
        stmts = []  # (value id, is boolean, expression, ids of the operands)
        for i in sorted(live):
            n = self.nodes[i]
            op = n[0]
            if op == "const":
                ref[i] = self._lit(n[1])
                continue
            if op == "load":
                ref[i] = names[(n[1], n[2], n[3])]
                continue
            a = [ref[j] for j in (n[2:] if op == "call" else n[1:])]
            boolean = False
            if op == "neg":
                e = f"-{a[0]}"
            elif op in ("add", "sub", "mul") and i in self.rounded:
                e = f"keops_{op}_rounded({a[0]}, {a[1]})"
            elif op in ("add", "sub", "mul", "div"):
                e = f"{a[0]} {dict(add='+', sub='-', mul='*', div='/')[op]} {a[1]}"
            elif op == "fma":
                e = f"keops_fma({a[0]}, {a[1]}, {a[2]})"
            elif op == "rcp":
                e = f"__builtin_amdgcn_rcpf({a[0]})" if f32 and self.fast_fn else f"(T)1 / {a[0]}"
            elif op == "exp2":
                e = f"__builtin_amdgcn_exp2f({a[0]})"
            elif op == "exp":
                e = f"keops_exp({a[0]})"
            elif op == "log2":
                e = f"__builtin_amdgcn_logf({a[0]})"
            elif op == "log":
                e = f"keops_log({a[0]})"
            elif op == "sqrt":
                e = f"__builtin_amdgcn_sqrtf({a[0]})" if f32 and self.fast_fn and not self.exact else f"keops_sqrt({a[0]})"
            elif op == "rsqrt0":
                r = f"__builtin_amdgcn_rsqf({a[0]})" if f32 and self.fast_fn and not self.exact else f"(T)1 / keops_sqrt({a[0]})"
                e = f"({a[0]} == (T)0) ? (T)0 : {r}"
            elif op == "abs":
                e = f"keops_abs({a[0]})"
            elif op == "sign":
                e = f"({a[0]} > (T)0) ? (T)1 : (({a[0]} < (T)0) ? -(T)1 : (T)0)"
            elif op == "call":
                e = f"keops_{n[1]}({', '.join(a)})"
            elif op in ("lt", "le", "eq", "ne"):
                e = f"{a[0]} {dict(lt='<', le='<=', eq='==', ne='!=')[op]} {a[1]}"
                boolean = True
            elif op == "select":
                e = f"{a[0]} ? {a[1]} : {a[2]}"
            else:
                raise AssertionError(op)
            ref[i] = f"t{i}"
            lines.append(f"{indent}const {'bool' if boolean else 'T'} t{i} = {e};")
            stmts.append((i, boolean, e, [j for j in (n[2:] if op == "call" else n[1:])]))
        if not segment or len(stmts) <= max(segment, segment_min):
            return lines, [ref[o] for o in outputs]

        # ---- long bodies: bounded, non-inlined functions ----
        seg_of = {st[0]: k // segment for k, st in enumerate(stmts)}
        nseg = (len(stmts) + segment - 1) // segment
        is_bool = {st[0]: st[1] for st in stmts}
        crossing = {}  # value id -> slot of keops_live
        for i, _, _, deps in stmts:
            for j in deps:
                if j in seg_of and seg_of[j] != seg_of[i] and j not in crossing:
                    crossing[j] = len(crossing)
        for o in outputs:
            if o in seg_of and o not in crossing:
                crossing[o] = len(crossing)
        for k in range(nseg):
            body = [st for st in stmts if seg_of[st[0]] == k]
            fn = [f"static __device__ __attribute__((noinline)) void keops_seg_{k}(const T* __restrict__ xi, "
                  f"const T* __restrict__ yj, const T* __restrict__ p, T* __restrict__ keops_live) {{"]
            fn += list(segment_prefix)
            ins = sorted({j for st in body for j in st[3] if j in seg_of and seg_of[j] != k})
            for j in ins:
                if is_bool[j]:
                    fn.append(f"  const bool t{j} = keops_live[{crossing[j]}] != (T)0;")
                else:
                    fn.append(f"  const T t{j} = keops_live[{crossing[j]}];")
            for i, boolean, e, _ in body:
                fn.append(f"  const {'bool' if boolean else 'T'} t{i} = {e};")
                if i in crossing:
                    fn.append(f"  keops_live[{crossing[i]}] = {'(T)' if boolean else ''}t{i};")
            fn.append("}")
            self.prelude += fn
        calls = [f"{indent}T keops_live[{max(1, len(crossing))}];"]
        calls += [f"{indent}keops_seg_{k}(xi, yj, p, keops_live);" for k in range(nseg)]
        exprs = [f"keops_live[{crossing[o]}]" if o in crossing else ref[o] for o in outputs]
        return calls, exprs


def lower(formula, L: Lir):
    """Lower a formula tree into ``L``; returns the list of output value ids (memoised per node)."""
    memo = {}

    def rec(node):
        r = memo.get(node)
        if r is None:
            kids = [rec(c) for c in node.children]
            r = node.lower(L, kids)
            assert len(r) == node.dim, (node.name, len(r), node.dim)
            memo[node] = r
        return r

    return rec(formula)
