"""Host-logic tests of the formula layer: grammar, simplification, autodiff and scalar lowering,
checked against dense torch expressions (the reference's own test style, keopscore/keopscore/
test/test_op.py:18-188: M=300, N=500-like random inputs, forward and gradient vs torch)."""
import numpy as np
import pytest
import torch

from keops_amd.formulas import FormulaError, Lir, lower, parse, parse_reduction
from keops_amd.formulas import ops as O

from host_eval import dense_eval

M, N = 7, 9
torch.manual_seed(0)


def _t(*shape, lo=-1.0, hi=1.0):
    return (torch.rand(*shape, dtype=torch.float64) * (hi - lo) + lo)


def _check(formula, aliases, targs, torch_fn, grad_wrt=(), tol=1e-10):
    """targs: torch tensors shaped (M,d)/(N,d)/(d,); torch_fn gets broadcastable views."""
    views = []
    for a, al in zip(targs, aliases):
        cat = parse(al.split("=")[1] if "=" in al else al, []).cat
        views.append(a[:, None, :] if cat == 0 else (a[None, :, :] if cat == 1 else a[None, None, :]))
    leaves = [v.detach().clone().requires_grad_(True) for v in views]
    ref = torch_fn(*leaves)
    got = dense_eval(formula, aliases, [a.numpy() for a in targs], M, N)
    ref_b = torch.broadcast_to(ref, (M, N, ref.shape[-1])).detach().numpy()
    assert got.shape == ref_b.shape, (got.shape, ref_b.shape)
    assert np.allclose(got, ref_b, rtol=tol, atol=tol), formula
    op = parse(formula, aliases)
    for k in grad_wrt:
        v = op.variables[[w.ind for w in op.variables].index(k)]
        eta = O.Var(len(targs), op.dim, 1 - v.cat if v.cat < 2 else 0)
        gop = O.Grad(op, v, eta)
        E = _t(M if eta.cat == 0 else N, op.dim)
        gdense = dense_eval(gop, None, [a.numpy() for a in targs] + [E.numpy()], M, N)
        Ev = E[:, None, :] if eta.cat == 0 else E[None, :, :]
        (gref,) = torch.autograd.grad((torch.broadcast_to(ref, (M, N, ref.shape[-1])) * Ev).sum(), leaves[k], retain_graph=True)
        # dense pairwise gradient summed over the axis the variable does not depend on
        if v.cat == 0:
            g = gdense.sum(1)
            gr = gref.reshape(M, -1).numpy()
        elif v.cat == 1:
            g = gdense.sum(0)
            gr = gref.reshape(N, -1).numpy()
        else:
            g = gdense.sum((0, 1))
            gr = gref.reshape(-1).numpy()
        assert np.allclose(g, gr, rtol=1e-8, atol=1e-8), (formula, k)


AL = ["x=Vi(0,3)", "y=Vj(1,3)", "p=Pm(2,1)", "b=Vj(3,2)"]


def _args():
    return [_t(M, 3), _t(N, 3), _t(1, lo=0.5, hi=1.5), _t(N, 2)]


UNARY = {
    "Exp": (torch.exp, (-1, 1)), "Log": (torch.log, (0.5, 2)), "Sqrt": (torch.sqrt, (0.5, 2)),
    "Rsqrt": (torch.rsqrt, (0.5, 2)), "Inv": (lambda t: 1 / t, (0.5, 2)), "Square": (lambda t: t * t, (-1, 1)),
    "Abs": (torch.abs, (-1, 1)), "Sign": (torch.sign, (-1, 1)), "Step": (lambda t: (t >= 0).double(), (-1, 1)),
    "ReLU": (torch.relu, (-1, 1)), "Sin": (torch.sin, (-1, 1)), "Cos": (torch.cos, (-1, 1)),
    "Asin": (torch.asin, (-0.9, 0.9)), "Acos": (torch.acos, (-0.9, 0.9)), "Atan": (torch.atan, (-1, 1)),
    "Floor": (torch.floor, (-3, 3)), "XLogX": (lambda t: t * torch.log(t), (0.5, 2)),
    "SinXDivX": (lambda t: torch.sin(t) / t, (0.2, 2)), "Minus": (lambda t: -t, (-1, 1)),
}


@pytest.mark.parametrize("name", sorted(UNARY))
def test_unary_ops(name):
    fn, (lo, hi) = UNARY[name]
    targs = [_t(M, 3, lo=lo, hi=hi), _t(N, 3, lo=lo, hi=hi)]
    al = ["x=Vi(0,3)", "y=Vj(1,3)"]
    grad = () if name in ("Sign", "Step", "Floor") else (0, 1)
    # x*y keeps products inside the op's domain for positive ranges; use a sum for signed ones
    if lo > 0:
        _check(f"{name}(x*y)", al, targs, lambda x, y: fn(x * y), grad)
    else:
        _check(f"{name}((x+y)/2)", al, targs, lambda x, y: fn((x + y) / 2), grad)


def test_binary_and_broadcast_ops():
    a = _args()
    _check("(x-y)*p + y/(p+2)", AL, a, lambda x, y, p, b: (x - y) * p + y / (p + 2), (0, 1, 2))
    _check("(x|y)*b", AL, a, lambda x, y, p, b: (x * y).sum(-1, keepdim=True) * b, (0, 1, 3))
    _check("Powf(Abs(x)+1, y)", AL, a, lambda x, y, p, b: torch.pow(x.abs() + 1, y), (0, 1))
    _check("Pow(x,3)+Pow(y,-2)", AL, [_t(M, 3), _t(N, 3, lo=0.5, hi=1.5), a[2], a[3]],
           lambda x, y, p, b: x**3 + y**-2.0, (0, 1))
    _check("Atan2(x,y+3)", AL, a, lambda x, y, p, b: torch.atan2(x, y + 3), (0, 1))
    _check("x/SumT(p+Sum(y*y),3)", AL, a, lambda x, y, p, b: x / (p + (y * y).sum(-1, keepdim=True)), (0, 1, 2))
    _check("IfElse(x-y, x*2, y*p)", AL, a, lambda x, y, p, b: torch.where(x - y >= 0, x * 2, y * p), (0, 1, 2))
    _check("Clamp(x, y-1, y+1)", AL, a, lambda x, y, p, b: torch.minimum(torch.maximum(x, y - 1), y + 1), (0, 1))
    _check("ClampInt(3*x, -1, 1)", AL, a, lambda x, y, p, b: torch.clamp(3 * x, -1, 1), (0,))
    _check("Mod(5*x, 2, 0)", AL, a, lambda x, y, p, b: 5 * x - 2 * torch.floor(5 * x / 2))
    _check("Round(3*x, 1)", AL, a, lambda x, y, p, b: torch.round(30 * x) / 10)
    _check("(x<y) + (x<=y)*2 + Equal(x,x) + NotEqual(x,y)", AL, a,
           lambda x, y, p, b: (x < y).double() + 2 * (x <= y).double() + 1 + (x != y).double())


def test_vector_ops():
    a = _args()
    _check("SqDist(x,y)", AL, a, lambda x, y, p, b: ((x - y) ** 2).sum(-1, keepdim=True), (0, 1))
    _check("Norm2(x-y)", AL, a, lambda x, y, p, b: (x - y).norm(dim=-1, keepdim=True), (0, 1))
    _check("Normalize(x+y)", AL, a, lambda x, y, p, b: (x + y) / (x + y).norm(dim=-1, keepdim=True), (0, 1))
    _check("SqNorm2(x)*y", AL, a, lambda x, y, p, b: (x * x).sum(-1, keepdim=True) * y, (0, 1))
    _check("Concat(x, b)", AL, a, lambda x, y, p, b: torch.cat([x.expand(M, N, 3), b.expand(M, N, 2)], -1), (0, 3))
    _check("Extract(Concat(x*y, b), 2, 3)", AL, a,
           lambda x, y, p, b: torch.cat([(x * y).expand(M, N, 3), b.expand(M, N, 2)], -1)[..., 2:5], (0, 1, 3))
    _check("ExtractT(b*p, 1, 4)", AL, a,
           lambda x, y, p, b: torch.cat([0 * b[..., :1], b * p, 0 * b[..., :1]], -1), (2, 3))
    _check("Elem(x,1)*ElemT(Elem(y,2), 3, 0)", AL, a,
           lambda x, y, p, b: x[..., 1:2] * torch.cat([y[..., 2:3], 0 * y[..., :2]], -1), (0, 1))
    _check("Max(x*y)+Min(x-y)", AL, a,
           lambda x, y, p, b: (x * y).max(-1, keepdim=True)[0] + (x - y).min(-1, keepdim=True)[0], (0, 1))
    _check("ArgMax(x*y)+2*ArgMin(x*y)", AL, a,
           lambda x, y, p, b: ((x * y).argmax(-1, keepdim=True) + 2 * (x * y).argmin(-1, keepdim=True)).double())
    _check("OneHot(Floor(Abs(2*Elem(x,0))), 3)", AL, a,
           lambda x, y, p, b: torch.nn.functional.one_hot(torch.floor((2 * x[..., 0]).abs()).long(), 3).double())
    _check("WeightedSqDist(p, x, y)", AL, a, lambda x, y, p, b: p * ((x - y) ** 2).sum(-1, keepdim=True), (0, 1, 2))
    _check("WeightedSqNorm(y, x)", AL, a, lambda x, y, p, b: (y * x * x).sum(-1, keepdim=True), (0, 1))
    al2 = ["A=Vi(0,6)", "v=Vj(1,2)", "w=Vj(2,3)"]
    t2 = [_t(M, 6), _t(N, 2), _t(N, 3)]
    # A is a (3 x 2) matrix stored column-major: out_i = sum_k A[k*3+i] v_k
    _check("MatVecMult(A, v)", al2, t2,
           lambda A, v, w: (A.expand(M, N, 6).reshape(M, N, 2, 3) * v.expand(M, N, 2)[..., None]).sum(-2), (0, 1))
    _check("VecMatMult(w, A)", al2, t2,
           lambda A, v, w: (A.expand(M, N, 6).reshape(M, N, 2, 3) * w.expand(M, N, 3)[..., None, :]).sum(-1), (0, 2))
    _check("TensorProd(v, w)", al2, t2,
           lambda A, v, w: (v.expand(M, N, 2)[..., :, None] * w.expand(M, N, 3)[..., None, :]).reshape(M, N, 6), (1, 2))
    # entry (j, i) of the table of differences v_i - w_j sits at j*dim(v)+i
    _check("DifferenceMatrix(v, w)*A", al2, t2,
           lambda A, v, w: (v.expand(M, N, 2)[..., None, :] - w.expand(M, N, 3)[..., :, None]).reshape(M, N, 6) * A, (0, 1, 2))
    _check("SqNorm2(MatVecMult(A, v))", al2, t2,
           lambda A, v, w: ((A.expand(M, N, 6).reshape(M, N, 2, 3) * v.expand(M, N, 2)[..., None]).sum(-2) ** 2).sum(-1, keepdim=True), (0, 1))


def test_gaussian_and_its_gradients():
    al = ["x=Vi(0,3)", "y=Vj(1,3)", "b=Vj(2,2)", "g=Pm(3,1)"]
    a = [_t(M, 3), _t(N, 3), _t(N, 2), _t(1, lo=0.5, hi=1.5)]
    _check("Exp(-g*SqDist(x,y))*b", al, a, lambda x, y, b, g: torch.exp(-g * ((x - y) ** 2).sum(-1, keepdim=True)) * b,
           (0, 1, 2, 3), tol=1e-12)
    _check("Exp(-Norm2(x-y))*b", al, a, lambda x, y, b, g: torch.exp(-(x - y).norm(dim=-1, keepdim=True)) * b, (0, 1, 2))
    # second order: gradient of the gradient formula (cf. pykeops/test/test_lazytensor_gaussian_cpu.py)
    op = parse("Exp(-g*SqDist(x,y))*b", al)
    x, y, b, g = op.variables
    e = O.Var(4, 2, 0)
    g1 = O.Grad(op, x, e)          # dim 3, depends on x,y,b,g,e
    e2 = O.Var(5, 3, 0)
    g2 = O.Grad(g1, x, e2)
    E, E2 = _t(M, 2), _t(M, 3)
    dense = dense_eval(g2, None, [t.numpy() for t in a] + [E.numpy(), E2.numpy()], M, N).sum(1)
    xt = a[0].clone().requires_grad_(True)
    K = torch.exp(-a[3] * ((xt[:, None] - a[1][None]) ** 2).sum(-1, keepdim=True)) * a[2][None]
    (gx,) = torch.autograd.grad((K * E[:, None]).sum(), xt, create_graph=True)
    (ggx,) = torch.autograd.grad((gx * E2).sum(), xt)
    assert np.allclose(dense, ggx.numpy(), rtol=1e-8, atol=1e-10)


def test_simplifications():
    al = ["x=Vi(0,3)", "y=Vj(1,3)", "s=Pm(2,1)"]
    x, y, s = parse("x", al), parse("y", al), parse("s", al)
    assert isinstance(x - x, O.Zero) and (x - x).dim == 3
    assert x * 1 == x and 1 * x == x and x + O.Zero(3) == x
    assert repr(-(-x)) == repr(x)
    assert repr(x * x) == repr(O.Square(x))
    assert isinstance(O.Grad(parse("Exp(s)*y", al), x, O.Var(3, 3, 1)), O.Zero)
    assert repr(parse("SqDist(x,y)", al)) == "Sum(Square(Subtract(Var(0,3,0),Var(1,3,1))))"
    assert repr(parse("2*(3*x)", al)) == repr(parse("6*x", al))
    assert repr(parse("IntInv(2)*IntCst(4)", al)) == "IntCst(2)"
    assert parse("Sum(s*x)", al) == parse("s*Sum(x)", al)
    # Exp(a)*Exp(b) -> Exp(a+b): one exponential per pair
    e = parse("Exp(-s*SqNorm2(x))*Exp(-SqNorm2(y))", al)
    assert sum(1 for n in e.walk() if n.name == "Exp") == 1


def test_gaussian_lowering_is_minimal():
    """The Gaussian kernel costs 3 sub + 3 mul + 2 add (the squared distance in the reference's order, nothing fused:
    a product and a sum issue in the time of one fused multiply-add), the product with g, the product with log2(e),
    exp2 and the weight per pair.  The argument of the exponential is the reference's own, rounding for rounding, and
    log2(e) multiplies the rounded argument: a coefficient merged with log2(e) would shift every exponent by up to
    2^-24 of its size, which a kernel value in the far tail (exponent -80) shows as 1e-5."""
    al = ["x=Var(0,3,0)", "y=Var(1,3,1)", "b=Var(2,1,1)", "g=Var(3,1,2)"]
    red = parse_reduction("Sum_Reduction(Exp(-g*SqDist(x,y))*b,0)", al)
    L = Lir(row_cat=0, fast_math=True)
    outs = lower(red.formula, L)
    assert L.count_ops(outs) == 12  # sub x3, mul x3, add x2, g, log2(e), exp2, weight
    names = {(v.cat, v.ind, k): f"a{v.ind}[{k}]" for v in red.formula.variables for k in range(v.dim)}
    lines, _ = L.emit(outs, names)
    text = "\n".join(lines)
    # the reference's operation order (Subtract.py:21-24, Square.py:17-18, Sum.py:20-24, Mult.py:25), every operation
    # of the argument rounded on its own, then one product with log2(e)
    assert text.count("keops_sub_rounded") == 3 and text.count("keops_mul_rounded") == 5 and text.count("keops_add_rounded") == 2
    assert "keops_mul_rounded(a3[0], " in text and "1.4426950408889634f" in text
    g = parse_reduction("Grad_WithSavedForward(Sum_Reduction(Exp(-g*SqDist(x,y))*b,0),Var(0,3,0),Var(4,1,0),Var(5,1,0))", al)
    L = Lir(row_cat=0, fast_math=True)
    assert L.count_ops(lower(g.formula, L)) <= 19


def test_parser_errors_and_aliases():
    with pytest.raises(FormulaError):
        parse("Foo(x)", ["x=Vi(3)"])
    with pytest.raises(FormulaError):
        parse("x+z", ["x=Vi(3)"])
    with pytest.raises(FormulaError):
        parse("x+y", ["x=Vi(3)", "y=Vj(2)"])
    with pytest.raises(FormulaError):
        parse("__import__('os')", [])
    with pytest.raises(FormulaError):
        parse_reduction("Exp(x)", ["x=Vi(3)"])
    assert repr(parse("Vi(0,3)+Vj(1,3)*Pm(2,1)", [])) == "Add(Var(0,3,0),Mult(Var(2,1,2),Var(1,3,1)))"
    r = parse_reduction("KMin_ArgKMin_Reduction(SqDist(x,y),10,0)", ["x=Vi(64)", "y=Vj(64)"])
    assert (r.K, r.dim, r.dimred, r.tagI) == (10, 20, 20, 0)
    r = parse_reduction("Max_SumShiftExp_Reduction(l-SqDist(x,y)*e,0)", ["x=Vi(3)", "y=Vj(3)", "l=Vj(1)", "e=Pm(1)"])
    assert (r.dim, r.dimred) == (2, 2)
    r = parse_reduction("Max_SumShiftExpWeight_Reduction(SqDist(x,y),1,Concat(IntCst(1),x))", ["x=Vi(3)", "y=Vj(3)"])
    assert (r.dim, r.tagI) == (5, 1)


def test_tensordot_kron_and_quadratic_forms():
    """TensorDot against torch.tensordot / einsum (values and gradients with respect to both operands,
    cf. the reference's pykeops/test/test_lazytensor_tensordot.py cases), Kron against torch.kron."""
    al = ["a=Vi(0,12)", "b=Vj(1,24)", "c=Vj(2,6)", "s=Vj(3,9)", "u=Vi(4,3)"]
    t = [_t(M, 12), _t(N, 24), _t(N, 6), _t(N, 9), _t(M, 3)]

    def A(a):
        return a.expand(M, N, 12).reshape(M, N, 2, 2, 3)

    def B(b):
        return b.expand(M, N, 24).reshape(M, N, 2, 3, 4)

    # contract the last two axes of a (2,2,3) with the first two of b (2,3,4): result (2,4)
    _check("TensorDot(a, b, Ind(2,2,3), Ind(2,3,4), Ind(1,2), Ind(0,1))", al, t,
           lambda a, b, c, s, u: torch.einsum("mnijk,mnjkl->mnil", A(a), B(b)).reshape(M, N, 8), (0, 1))
    # crossed pairing (axis 0 of a with axis 0 of b, axis 2 with axis 1) and a permuted result (4,2) instead of (2,4)
    _check("TensorDot(a, b, Ind(2,2,3), Ind(2,3,4), Ind(0,2), Ind(0,1), Ind(1,0))", al, t,
           lambda a, b, c, s, u: torch.einsum("mnijk,mnikl->mnlj", A(a), B(b)).reshape(M, N, 8), (0, 1))
    # no contraction: outer product with interleaved axes = Kronecker product of a (2,6) and c (2,3) matrix
    _check("Kron(a, c, Ind(2,6), Ind(2,3))", al, t,
           lambda a, b, c, s, u: torch.einsum("mnij,mnkl->mnikjl", a.expand(M, N, 12).reshape(M, N, 2, 6),
                                              c.expand(M, N, 6).reshape(M, N, 2, 3)).reshape(M, N, 72), (0, 2))
    # repr -> parse round trip (the LazyTensor front end passes repr(formula) to Genred)
    op = parse("TensorDot(a, b, Ind(2,2,3), Ind(2,3,4), Ind(0,2), Ind(0,1), Ind(1,0))", al)
    assert parse(repr(op)) == op
    # quadratic forms
    _check("SymSqNorm(s, u)", al, t,
           lambda a, b, c, s, u: torch.einsum("mnij,mni,mnj->mn", s.expand(M, N, 9).reshape(M, N, 3, 3),
                                              u.expand(M, N, 3), u.expand(M, N, 3))[..., None], (3, 4))
    _check("SqNormDiag(Extract(s,0,3), u)+SqNormIso(Elem(s,4), u)", al, t,
           lambda a, b, c, s, u: (s[..., :3] * u * u).sum(-1, keepdim=True) + s[..., 4:5] * (u * u).sum(-1, keepdim=True), (3, 4))
    with pytest.raises(Exception):
        parse("TensorDot(a, b, Ind(2,2,3), Ind(2,3,4), Ind(1), Ind(2))", al)


def test_forward_mode_diff_divergence_laplacian():
    """Diff (forward mode), Divergence and Laplacian against torch.func / closed forms."""
    al = ["x=Vi(0,3)", "y=Vj(1,3)", "u=Vi(2,3)", "g=Pm(3,1)"]
    a = [_t(M, 3), _t(N, 3), _t(M, 3), _t(1, lo=0.5, hi=1.5)]

    def F(x, y, g):
        return torch.exp(-g * ((x - y) ** 2).sum(-1, keepdim=True)) * (x + y)

    def jvp(x, y, u, g):
        xb, yb, ub = (t.expand(M, N, 3) for t in (x, y, u))
        return torch.func.jvp(lambda z: F(z, yb, g), (xb,), (ub,))[1]

    _check("Diff(Exp(-g*SqDist(x,y))*(x+y), x, u)", al, a, jvp)
    # divergence of the vector field z -> exp(-g|z-y|^2)(z+y) at z = x
    def div(x, y, u, g):
        xb, yb = x.expand(M, N, 3).reshape(-1, 3), y.expand(M, N, 3).reshape(-1, 3)
        J = torch.func.vmap(torch.func.jacrev(lambda z, w: F(z, w, g)))(xb, yb)
        return torch.diagonal(J, dim1=-2, dim2=-1).sum(-1).reshape(M, N, 1)

    _check("Divergence(Exp(-g*SqDist(x,y))*(x+y), x)", al, a, div)
    # Laplacian of a Gaussian: (4 g^2 r^2 - 2 g D) exp(-g r^2)
    def lap(x, y, u, g):
        r2 = ((x - y) ** 2).sum(-1, keepdim=True)
        return (4 * g * g * r2 - 6 * g) * torch.exp(-g * r2)

    _check("Laplacian(Exp(-g*SqDist(x,y)), x)", al, a, lap)


def test_trace_operator_of_linear_formulas():
    """TraceOperator(F, v) for F linear in v (keopscore/formulas/LinearOperators/TraceOperator.py:27-101): the trace of
    the matrix of F when dim(F) = dim(v), the sum of its coefficients when dim(F) = 1; v leaves the formula."""
    rng = np.random.default_rng(3)
    A, x, p = rng.random((M, 9)), rng.random((N, 3)), rng.random(1)
    al = ["A=Vi(0,9)", "x=Vj(1,3)", "p=Pm(2,1)", "v=Vj(3,3)"]
    f = parse("TraceOperator(MatVecMult(A,v)*p + 2*v, v)", al)
    assert f.dim == 1 and sorted(w.ind for w in f.variables) == [0, 2]
    got = dense_eval(f, None, [A, x, p], M, N)
    # MatVecMult(A, v)_i = sum_k A[3k + i] v_k: the diagonal is A[0], A[4], A[8]
    assert np.allclose(got[:, :, 0], (A[:, 0] + A[:, 4] + A[:, 8])[:, None] * p + 6, rtol=1e-12)
    g = parse("TraceOperator((A|Concat(Concat(v,v),v))*p + (x|v), v)", al)
    got = dense_eval(g, None, [A, x, p], M, N)
    assert np.allclose(got[:, :, 0], A.sum(1)[:, None] * p + x.sum(1)[None, :], rtol=1e-12)
    with pytest.raises(FormulaError, match="linear"):
        parse("TraceOperator(v*v, v)", al)
    with pytest.raises(FormulaError, match="dimension"):
        parse("TraceOperator(Concat(v,v), v)", al)


def test_forward_mode_through_log_sum_exp_reduction():
    """Diff_WithSavedForward of a Max_SumShiftExpWeight reduction: [0, d(sum_j exp(F - m) G)] with the saved
    maximum m; flattened as the Python layer does (tangent of m + log s is ds / s) it must equal the jvp of a
    dense weighted log-sum-exp (cf. the reference's pykeops/test/test_torch_func_logsumexp.py)."""
    x, y, w, u = _t(M, 3), _t(N, 3), _t(N, 1, lo=0.2, hi=1.0), _t(M, 3)
    al = ["x=Var(0,3,0)", "y=Var(1,3,1)", "w=Var(2,1,1)", "u=Var(3,3,0)", "ms=Var(4,2,0)"]
    red = parse_reduction("Diff_WithSavedForward(Max_SumShiftExpWeight_Reduction(-SqDist(x,y),0,w),x,u,ms)", al)
    assert red.string_id == "Sum_Reduction" and red.dim == 2 and red.tagI == 0

    def lse(x_):
        F = -((x_[:, None, :] - y[None, :, :]) ** 2).sum(-1)
        return torch.log((torch.exp(F) * w[None, :, 0]).sum(1))

    F = -((x[:, None, :] - y[None, :, :]) ** 2).sum(-1)
    m = F.max(1, keepdim=True).values
    s = (torch.exp(F - m) * w[None, :, 0]).sum(1, keepdim=True)
    ms = torch.cat([m, s], 1)
    dense = dense_eval(red.formula, None, [t.numpy() for t in (x, y, w, u, ms)], M, N)   # (M, N, 2)
    dms = dense.sum(1)
    assert np.all(dms[:, 0] == 0)
    _, ref = torch.func.jvp(lse, (x,), (u,))
    assert np.allclose(dms[:, 1] / s[:, 0].numpy(), ref.numpy(), rtol=1e-10, atol=1e-10)
    # a tangent that the formula does not depend on gives the zero reduction
    z = parse_reduction("Diff_WithSavedForward(Max_SumShiftExpWeight_Reduction(-SqDist(x,y),0,w),Var(5,1,2),Var(6,1,2),ms)", al)
    assert z.string_id == "Zero_Reduction"


def test_long_bodies_as_chains_of_functions():
    """The segmented emission (functions of a few statements chained through a value array) computes what the
    single straight-line body computes, including boolean values that cross a cut and outputs that are loads or
    constants."""
    al = ["x=Vi(0,6)", "y=Vj(1,6)", "g=Pm(2,1)"]
    a = [_t(M, 6).numpy(), _t(N, 6).numpy(), _t(1, lo=0.5, hi=1.5).numpy()]
    for formula in (
        "Concat(Exp(-g*SqDist(x,y))*(x+y), IfElse(x-y, Abs(x)*Step(y), Sin(x*y)+Square(y)))",
        "Concat(Concat(x, IntCst(2)), Sum(Sqrt(Abs(x-y)))*Extract(y,1,2))",
    ):
        whole = dense_eval(formula, al, a, M, N)
        for seg in (1, 3, 7):
            assert np.array_equal(dense_eval(formula, al, a, M, N, segment=seg), whole), (formula, seg)


@pytest.mark.parametrize("order", [0, 1, 3])
def test_bspline_against_scipy(order):
    """BSpline(knots, x, order): the n_knots - order - 1 basis functions of De Boor's recursion, against
    scipy.interpolate.BSpline.basis_element on a non-uniform knot vector with a repeated knot."""
    from scipy.interpolate import BSpline as SciBSpline

    knots = np.array([[0.0, 0.5, 0.5, 1.2, 2.0, 2.7, 3.1, 4.0]])
    nk = knots.shape[1]
    P = 57
    x = np.linspace(-0.313, 4.237, P)[:, None]  # no sample on a knot: scipy closes the last span on the right
    al = [f"t=Pm(0,{nk})", "x=Vi(1,1)"]
    got = dense_eval(f"BSpline(t,x,{order})", al, [knots[0], x], P, 1)[:, 0, :]
    assert got.shape == (P, nk - order - 1)
    ref = np.zeros_like(got)
    for i in range(nk - order - 1):
        if knots[0, i] < knots[0, i + order + 1]:
            b = SciBSpline.basis_element(knots[0, i:i + order + 2], extrapolate=False)(x[:, 0])
            ref[:, i] = np.nan_to_num(b)
    inside = (x[:, 0] >= 0.0) & (x[:, 0] < 4.0)
    assert np.allclose(got[inside], ref[inside], atol=1e-12)
    assert np.all(got[~inside] == 0)
    assert np.allclose(got[(x[:, 0] >= knots[0, order]) & (x[:, 0] < knots[0, nk - order - 1])].sum(1), 1.0)  # partition of unity
    with pytest.raises(FormulaError):
        parse("BSpline(t,x,7)", al)
    with pytest.raises(NotImplementedError):
        O.Grad(parse(f"BSpline(t,x,{order})", al), O.Var(1, 1, 0), O.Var(2, nk - order - 1, 0))


def test_softdtw_and_grad_matrix():
    """SoftDTW_SqDist against a plain torch dynamic program (value and gradients through autograd), and
    GradMatrix against torch.func.jacrev."""
    n, m = 5, 4
    x, y, g = _t(M, n), _t(N, m), _t(1, lo=0.3, hi=0.9)

    def softdtw(xv, yv, gam):
        r = [[None] * n for _ in range(m)]
        for j in range(m):
            for i in range(n):
                d2 = (xv[..., i] - yv[..., j]) ** 2
                if i == 0 and j == 0:
                    r[j][i] = d2
                elif j == 0:
                    r[j][i] = d2 + r[j][i - 1]
                elif i == 0:
                    r[j][i] = d2 + r[j - 1][i]
                else:
                    prev = torch.stack([r[j - 1][i - 1], r[j - 1][i], r[j][i - 1]], -1)
                    r[j][i] = d2 - gam * torch.logsumexp(-prev / gam, -1)
        return r[m - 1][n - 1][..., None]

    al = [f"x=Vi(0,{n})", f"y=Vj(1,{m})", "g=Pm(2,1)"]
    _check("SoftDTW_SqDist(x,y,g)", al, [x, y, g], lambda xv, yv, gv: softdtw(xv, yv, gv[..., 0]), grad_wrt=(0, 1), tol=1e-9)

    al2 = ["x=Vi(0,3)", "y=Vj(1,3)"]
    x3, y3 = _t(M, 3), _t(N, 3)

    def F(xv, yv):
        return torch.cat([torch.exp(-((xv - yv) ** 2).sum(-1, keepdim=True)) * yv[..., :1], (xv * yv)[..., 1:]], -1)

    got = dense_eval("GradMatrix(Concat(Exp(-SqDist(x,y))*Elem(y,0), Extract(x*y,1,2)), x)", al2, [x3.numpy(), y3.numpy()], M, N)
    xb, yb = x3[:, None, :].expand(M, N, 3), y3[None, :, :].expand(M, N, 3)
    jac = torch.func.vmap(torch.func.vmap(torch.func.jacrev(F)))(xb, yb)      # (M, N, out 3, in 3)
    assert np.allclose(got, jac.reshape(M, N, 9).numpy(), rtol=1e-10, atol=1e-10)
