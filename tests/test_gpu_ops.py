"""Every operation of the formula layer on the compute device: forward value and gradients of a Sum reduction
through Genred on cuda against dense torch float64, in float32 with and without fast math and in float64.

The reference runs the same matrix on its compute device (keopscore/keopscore/test/test_op.py:18-188: every maths
operation, forward and gradient against torch; pykeops/pykeops/test/test_torch.py).  tests/test_formulas.py checks
the same operations on the host with std:: stand-ins for the device functions; here the device spellings themselves
run (hiprtc has to resolve every __ocml_* symbol and the fast-math variants have to meet the bar)."""
import zlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

M, N = 37, 53
X3, Y3, P1, B2 = ("i", 3), ("j", 3), ("p", 1), ("j", 2)
AL = ["x=Vi(0,3)", "y=Vj(1,3)", "p=Pm(2,1)", "b=Vj(3,2)"]
AL2 = ["x=Vi(0,3)", "y=Vj(1,3)"]
ALM = ["A=Vi(0,6)", "v=Vj(1,2)", "w=Vj(2,3)"]


def _mat(A):
    return A.expand(M, N, 6).reshape(M, N, 2, 3)


def _cat(*ts):
    return torch.cat([t.expand(M, N, t.shape[-1]) for t in ts], -1)


# name: (formula, aliases, [(category, dim, lo, hi)], torch function of broadcastable float64 views, differentiated arguments)
def _unary(name, fn, lo, hi, grad=True):
    if lo > 0:
        return (f"{name}(x*y)", AL2, [("i", 3, lo ** 0.5, hi ** 0.5), ("j", 3, lo ** 0.5, hi ** 0.5)], lambda x, y: fn(x * y), (0, 1) if grad else ())
    return (f"{name}((x+y)/2)", AL2, [("i", 3, lo, hi), ("j", 3, lo, hi)], lambda x, y: fn((x + y) / 2), (0, 1) if grad else ())


STD = [("i", 3, -1, 1), ("j", 3, -1, 1), ("p", 1, 0.5, 1.5), ("j", 2, -1, 1)]
MAT = [("i", 6, -1, 1), ("j", 2, -1, 1), ("j", 3, -1, 1)]
CASES = {
    "Exp": _unary("Exp", torch.exp, -1, 1),
    "Log": _unary("Log", torch.log, 0.5, 2),
    "Sqrt": _unary("Sqrt", torch.sqrt, 0.5, 2),
    "Rsqrt": _unary("Rsqrt", torch.rsqrt, 0.5, 2),
    "Inv": _unary("Inv", lambda t: 1 / t, 0.5, 2),
    "Square": _unary("Square", lambda t: t * t, -1, 1),
    "Abs": _unary("Abs", torch.abs, -1, 1),
    "Sign": _unary("Sign", torch.sign, -1, 1, grad=False),
    "Step": _unary("Step", lambda t: (t >= 0).double(), -1, 1, grad=False),
    "ReLU": _unary("ReLU", torch.relu, -1, 1),
    "Sin": _unary("Sin", torch.sin, -3, 3),
    "Cos": _unary("Cos", torch.cos, -3, 3),
    "Asin": _unary("Asin", torch.asin, -0.9, 0.9),
    "Acos": _unary("Acos", torch.acos, -0.9, 0.9),
    "Atan": _unary("Atan", torch.atan, -2, 2),
    "Floor": _unary("Floor", torch.floor, -3, 3, grad=False),
    "XLogX": _unary("XLogX", lambda t: t * torch.log(t), 0.5, 2),
    "SinXDivX": _unary("SinXDivX", lambda t: torch.sin(t) / t, 0.2, 2),
    "Minus": _unary("Minus", lambda t: -t, -1, 1),
    "AddSubMultDiv": ("(x-y)*p + y/(p+2)", AL, STD, lambda x, y, p, b: (x - y) * p + y / (p + 2), (0, 1, 2)),
    "Scalprod": ("(x|y)*b", AL, STD, lambda x, y, p, b: (x * y).sum(-1, keepdim=True) * b, (0, 1, 3)),
    "Powf": ("Powf(Abs(x)+1, y)", AL, STD, lambda x, y, p, b: torch.pow(x.abs() + 1, y), (0, 1)),
    "Pow": ("Pow(x,3)+Pow(y,-2)", AL, [("i", 3, -1, 1), ("j", 3, 0.5, 1.5), P1 + (0.5, 1.5), B2 + (-1, 1)],
            lambda x, y, p, b: x ** 3 + y ** -2.0, (0, 1)),
    "Atan2": ("Atan2(x,y+3)", AL, STD, lambda x, y, p, b: torch.atan2(x, y + 3), (0, 1)),
    "SumT": ("x/SumT(p+Sum(y*y),3)", AL, STD, lambda x, y, p, b: x / (p + (y * y).sum(-1, keepdim=True)), (0, 1, 2)),
    "IfElse": ("IfElse(x-y, x*2, y*p)", AL, STD, lambda x, y, p, b: torch.where(x - y >= 0, x * 2, y * p), (0, 1, 2)),
    "Clamp": ("Clamp(x, y-1, y+1)", AL, STD, lambda x, y, p, b: torch.minimum(torch.maximum(x, y - 1), y + 1), (0, 1)),
    "ClampInt": ("ClampInt(3*x, -1, 1)+y", AL, STD, lambda x, y, p, b: torch.clamp(3 * x, -1, 1) + y, (0,)),
    "Mod": ("Mod(5*x, 2, 0)+y", AL, STD, lambda x, y, p, b: 5 * x - 2 * torch.floor(5 * x / 2) + y, ()),
    "Round": ("Round(3*x, 1)+y", AL, STD, lambda x, y, p, b: torch.round(30 * x) / 10 + y, ()),
    "Comparisons": ("(x<y) + (x<=y)*2 + Equal(x,x) + NotEqual(x,y)", AL, STD,
                    lambda x, y, p, b: (x < y).double() + 2 * (x <= y).double() + 1 + (x != y).double(), ()),
    "SqDist": ("SqDist(x,y)", AL, STD, lambda x, y, p, b: ((x - y) ** 2).sum(-1, keepdim=True), (0, 1)),
    "Norm2": ("Norm2(x-y)", AL, STD, lambda x, y, p, b: (x - y).norm(dim=-1, keepdim=True), (0, 1)),
    "Normalize": ("Normalize(x+y)", AL, STD, lambda x, y, p, b: (x + y) / (x + y).norm(dim=-1, keepdim=True), (0, 1)),
    "SqNorm2": ("SqNorm2(x)*y", AL, STD, lambda x, y, p, b: (x * x).sum(-1, keepdim=True) * y, (0, 1)),
    "Concat": ("Concat(x, b)", AL, STD, lambda x, y, p, b: _cat(x, b), (0, 3)),
    "Extract": ("Extract(Concat(x*y, b), 2, 3)", AL, STD, lambda x, y, p, b: _cat(x * y, b)[..., 2:5], (0, 1, 3)),
    "ExtractT": ("ExtractT(b*p, 1, 4)+Elem(x,0)", AL, STD,
                 lambda x, y, p, b: _cat(0 * b[..., :1], b * p, 0 * b[..., :1]) + x[..., :1], (2, 3)),
    "ElemElemT": ("Elem(x,1)*ElemT(Elem(y,2), 3, 0)", AL, STD,
                  lambda x, y, p, b: x[..., 1:2] * _cat(y[..., 2:3], 0 * y[..., :2]), (0, 1)),
    "MaxMin": ("Max(x*y)+Min(x-y)", AL, STD,
               lambda x, y, p, b: (x * y).max(-1, keepdim=True)[0] + (x - y).min(-1, keepdim=True)[0], (0, 1)),
    "ArgMaxArgMin": ("ArgMax(x*y)+2*ArgMin(x*y)", AL, STD,
                     lambda x, y, p, b: ((x * y).argmax(-1, keepdim=True) + 2 * (x * y).argmin(-1, keepdim=True)).double(), ()),
    "OneHot": ("OneHot(Floor(Abs(2*Elem(x,0))), 3)+y", AL, STD,
               lambda x, y, p, b: torch.nn.functional.one_hot(torch.floor((2 * x[..., 0]).abs()).long(), 3).double() + y, ()),
    "WeightedSqDist": ("WeightedSqDist(p, x, y)", AL, STD, lambda x, y, p, b: p * ((x - y) ** 2).sum(-1, keepdim=True), (0, 1, 2)),
    "WeightedSqNorm": ("WeightedSqNorm(y, x)", AL, STD, lambda x, y, p, b: (y * x * x).sum(-1, keepdim=True), (0, 1)),
    "MatVecMult": ("MatVecMult(A, v)", ALM, MAT, lambda A, v, w: (_mat(A) * v.expand(M, N, 2)[..., None]).sum(-2), (0, 1)),
    "VecMatMult": ("VecMatMult(w, A)", ALM, MAT, lambda A, v, w: (_mat(A) * w.expand(M, N, 3)[..., None, :]).sum(-1), (0, 2)),
    "TensorProd": ("TensorProd(v, w)+A", ALM, MAT,
                   lambda A, v, w: (v.expand(M, N, 2)[..., :, None] * w.expand(M, N, 3)[..., None, :]).reshape(M, N, 6) + A, (1, 2)),
    "DifferenceMatrix": ("DifferenceMatrix(v, w)*A", ALM, MAT,
                         lambda A, v, w: (v.expand(M, N, 2)[..., None, :] - w.expand(M, N, 3)[..., :, None]).reshape(M, N, 6) * A, (0, 1, 2)),
    "SqNormIsoDiag": ("SqNormIso(p, x-y)+SqNormDiag(y, x)", AL, STD,
                      lambda x, y, p, b: p * ((x - y) ** 2).sum(-1, keepdim=True) + (y * x * x).sum(-1, keepdim=True), (0, 1, 2)),
    "SymSqNorm": ("SymSqNorm(A, v)", ["A=Vi(0,4)", "v=Vj(1,2)"], [("i", 4, -1, 1), ("j", 2, -1, 1)],
                  lambda A, v: (A.expand(M, N, 4).reshape(M, N, 2, 2) * v.expand(M, N, 2)[..., :, None] * v.expand(M, N, 2)[..., None, :]).sum((-1, -2))[..., None],
                  (0, 1)),
    "DiffClampInt": ("DiffClampInt(3*x, -1, 1)*y", AL, STD, lambda x, y, p, b: ((3 * x >= -1) & (3 * x <= 1)).double() * y, (1,)),
    "Constants": ("IntCst(2)*x + RatCst(1,3)*y - IntInv(4)*p + FloatCst(0.75)", AL, STD, lambda x, y, p, b: 2 * x + y / 3 - p / 4 + 0.75, (0, 1, 2)),
    "TensorDot": ("TensorDot(A, w, Ind(2,3), Ind(3), Ind(1), Ind(0))", ALM, MAT,
                  lambda A, v, w: (A.expand(M, N, 6).reshape(M, N, 2, 3) * w.expand(M, N, 3)[..., None, :]).sum(-1), (0, 2)),
    "GaussianOfMatVec": ("Exp(-SqNorm2(MatVecMult(A, v)-w))", ALM, MAT,
                         lambda A, v, w: torch.exp(-(((_mat(A) * v.expand(M, N, 2)[..., None]).sum(-2) - w) ** 2).sum(-1, keepdim=True)),
                         (0, 1, 2)),
}


def _inputs(name, spec):
    gen = torch.Generator().manual_seed(zlib.crc32(name.encode()))
    out = []
    for cat, dim, lo, hi in spec:
        rows = {"i": (M,), "j": (N,), "p": ()}[cat]
        out.append(torch.rand(*rows, dim, dtype=torch.float64, generator=gen) * (hi - lo) + lo)
    return out, gen


def _views(spec, tensors):
    return [t[:, None, :] if c == "i" else (t[None, :, :] if c == "j" else t[None, None, :]) for (c, _, _, _), t in zip(spec, tensors)]


@pytest.mark.parametrize("dtype,fast", [("float32", True), ("float32", False), ("float64", True)])
@pytest.mark.parametrize("name", sorted(CASES))
def test_operation_forward_and_gradients_on_the_device(name, dtype, fast):
    from keops_amd.torch import Genred

    formula, aliases, spec, fn, grad_wrt = CASES[name]
    tdt = getattr(torch, dtype)
    host, gen = _inputs(name, spec)
    # the reference sees the values the device sees: rounded to the data type first
    host = [t.to(tdt).double() for t in host]
    dev = [t.to(tdt).cuda().requires_grad_(k in grad_wrt) for k, t in enumerate(host)]
    leaves = [v.detach().clone().requires_grad_(True) for v in _views(spec, host)]
    dense = fn(*leaves)
    dense = torch.broadcast_to(dense, (M, N, dense.shape[-1]))
    ref = dense.sum(1)
    scale = dense.abs().sum(1) + 1e-300
    conv = Genred(formula, aliases, reduction_op="Sum", axis=1, use_fast_math=fast)
    out = conv(*dev)
    assert out.shape == ref.shape and out.dtype == tdt
    # float32: the bar of the map-reduce sums (1e-5 relative to sum_j |F_ij|; fast math replaces exp / log / sqrt / the
    # division by the hardware approximations, 1-2 ulp each); float64: libm-class
    tol = 1e-5 if dtype == "float32" else 1e-12
    err = float(((out.detach().cpu().double() - ref.detach()).abs() / scale.detach()).max())
    assert err <= tol, f"{name} forward: {err:.3e}"
    if not grad_wrt:
        return
    e = torch.rand(M, ref.shape[-1], dtype=torch.float64, generator=gen).to(tdt).double() - 0.5
    got = torch.autograd.grad((out * e.to(tdt).cuda()).sum(), [dev[k] for k in grad_wrt])
    want = torch.autograd.grad((dense * e[:, None, :]).sum(), [leaves[k] for k in grad_wrt])
    gtol = 2e-5 if dtype == "float32" else 1e-11
    for k, g, w in zip(grad_wrt, got, want):
        w = w.reshape(g.shape)
        assert g.dtype == tdt
        gerr = float((g.detach().cpu().double() - w).norm() / w.norm().clamp_min(1e-300))
        assert gerr <= gtol, f"{name} gradient with respect to argument {k}: {gerr:.3e}"
