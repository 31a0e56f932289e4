"""Scheme selection of the engine (keops_amd/get_keops_dll.py) on the CPU: which formulas the planners and matchers
take, and that the modules they generate compile for gfx950 (hiprtc cross-compiles without a GPU)."""
import pytest

from keops_amd import config
from keops_amd.formulas import parse_reduction
from keops_amd.get_keops_dll import (get_keops_dll, match_chunk, match_knn_highdim, match_knn_sqdist, match_vchunk,
                                     plan_row_col_product)


def _grad(formula, var, D, tag=0):
    al = [f"x=Var(0,{D},0)", f"y=Var(1,{D},1)", "b=Var(2,4,1)", "g=Var(3,1,2)", "e=Var(4,4,0)", "r=Var(5,4,0)"]
    return parse_reduction(f"Grad_WithSavedForward(Sum_Reduction({formula},{tag}),{var},e,r)", al), al


@pytest.mark.parametrize("formula,a,c", [("Exp(-g*SqDist(x,y))*b", 1, -1), ("Exp(-Norm2(x-y))*b", 1, -1), ("Exp(x|y)*b", 0, 1)])
def test_point_gradients_are_planned_as_scalar_and_weighted_sums(formula, a, c):
    D = 96
    red, al = _grad(formula, f"Var(0,{D},0)", D)
    plan = plan_row_col_product(red, "float", True, 1)
    assert plan is not None and (plan["a"], plan["c"]) == (a, c)
    assert plan["row"].ind == 0 and plan["col"].ind == 1
    # the scalar factor survives a round trip through its string form, which is how the sub-reductions are built
    again = parse_reduction(f"Sum_Reduction({plan['G']!r},0)", al)
    assert repr(again.formula) == repr(plan["G"])
    # gradient with respect to y: reduction over i, the roles of the two variables swap
    red_y, _ = _grad(formula, f"Var(1,{D},1)", D)
    plan_y = plan_row_col_product(red_y, "float", True, 1)
    assert plan_y is not None and plan_y["row"].ind == 1 and plan_y["col"].ind == 0
    # not for float64, without fast math, without chunks, or when the long variables appear elsewhere
    assert plan_row_col_product(red, "double", True, 1) is None
    assert plan_row_col_product(red, "float", True, 0) is None
    red_b, _ = _grad(formula, "Var(2,4,1)", D)
    assert plan_row_col_product(red_b, "float", True, 1) is None
    red_m, _ = _grad(formula + "*Sum(x)", f"Var(0,{D},0)", D)
    assert plan_row_col_product(red_m, "float", True, 1) is None


def test_long_sum_matcher_takes_elementwise_sums_only():
    al = ["x=Var(0,300,0)", "y=Var(1,300,1)", "b=Var(2,3,1)", "w=Var(3,1,0)", "z=Var(4,300,1)"]
    ok = ["Sum_Reduction(Exp(-Sum(Abs(x-y)))*b,0)", "ArgKMin_Reduction(Sum(Abs(x-y)),5,0)",
          "Max_SumShiftExp_Reduction(-Sum(Abs(x-y)*w),1)", "Sum_Reduction(Sum(Exp(x*y)*z),0)"]
    for f in ok:
        m = match_vchunk(parse_reduction(f, al))
        assert m is not None and m[1].dim == 300, f
    no = ["Sum_Reduction(Sum(Abs(x-y))*Sum(Abs(x-z)),0)",      # two long sums
          "Sum_Reduction(Sum(Abs(x-y))*z,0)",                   # a long variable outside the sum
          "Sum_Reduction(Exp(-Sum(Abs(x-y)))*b+Sum(x),0)",      # chunked variable outside the sum
          "Sum_Reduction(Max(x-y)*b,0)"]                        # not a sum
    for f in no:
        assert match_vchunk(parse_reduction(f, al)) is None, f
    short = parse_reduction("Sum_Reduction(Exp(-Sum(Abs(x-y)))*b,0)", ["x=Var(0,64,0)", "y=Var(1,64,1)", "b=Var(2,3,1)"])
    assert match_vchunk(short) is None and config.vchunk_min_dim >= 64


def test_nearest_neighbour_schemes_by_dimension_and_size():
    def red(D, K=10, op="ArgKMin_Reduction"):
        return parse_reduction(f"{op}(SqDist(x,y),{K},0)", [f"x=Var(0,{D},0)", f"y=Var(1,{D},1)"])

    assert match_knn_sqdist(red(64), "float", "GpuReduc1D") is not None
    assert match_knn_sqdist(red(64), "double", "GpuReduc1D") is None
    assert match_knn_sqdist(red(300), "float", "GpuReduc1D") is None
    assert match_knn_highdim(red(300), "float", "GpuReduc1D", True) is not None
    assert match_knn_highdim(red(300), "float", "GpuReduc1D_ranges", True) is None
    assert match_knn_highdim(red(300, K=40), "float", "GpuReduc1D", True) is None
    assert match_knn_highdim(red(2000), "float", "GpuReduc1D", True) is None
    assert match_chunk(red(300), "float", "GpuReduc1D", True) is None
    # small calls stay on the general-purpose kernel, a few large batches may use the dense scheme
    small = (1 << 20).bit_length()
    assert match_knn_sqdist(red(64), "float", "GpuReduc1D", pairs=small) is None
    assert match_knn_sqdist(red(64), "float", "GpuReduc1D", pairs=36) is not None
    assert match_knn_sqdist(red(64), "float", "GpuReduc1D_ranges", batch_loop=0) is None
    assert match_knn_sqdist(red(64), "float", "GpuReduc1D_ranges", batch_loop=34) is not None
    assert match_knn_sqdist(red(64), "float", "GpuReduc1D_ranges", batch_loop=20) is None


@pytest.mark.parametrize("formula,dtype,mode,key", [
    ("ArgMin_Reduction(SqDist(x,y),0)", "float", 3, "scheme=knn"),
    ("Min_ArgMin_Reduction(SqDist(u,v),0)", "float", 1, "chk_knn=1"),
    ("KMin_Reduction(Sum(Abs(u-v)),3,1)", "float", 1, "vchunk=500"),
    ("Sum_Reduction(Exp(-SqDist(u,v)),0)", "double", 1, "vchunk=500"),
])
def test_modules_of_the_new_schemes_compile(formula, dtype, mode, key):
    al = ["x=Var(0,20,0)", "y=Var(1,20,1)", "u=Var(2,500,0)", "v=Var(3,500,1)"]
    res = get_keops_dll("GpuReduc1D", formula, 1, -1, 0, al, 4, dtype, dtype, "direct_sum", 1, 1, 0, False, True, 0)
    assert res[8] == mode
    with open(res[1]) as f:
        assert key in f.readline()
    # the same reductions without matrix-core schemes (what a fallback asks for)
    exact = get_keops_dll("GpuReduc1D", formula, -1, -1, 0, al, 4, dtype, dtype, "direct_sum", 1, 1, 0, False, True, 0)
    with open(exact[1]) as f:
        head = f.readline()
    assert "scheme=conv" in head


def test_lazytensor_settles_variables_in_one_pass_and_reuses_the_reduction_object():
    """Data tensors get positions 0..n-1 in order of appearance (a pure renaming of the symbolic tree) and two
    LazyTensors with the same formula and options share one Genred object."""
    import torch

    from keops_amd.formulas.ops import Exp, Sum, Var
    from keops_amd.torch import LazyTensor
    from keops_amd.torch import lazytensor as lt

    f = Exp(-Sum((Var(7, 3, 0) - Var(9, 3, 1)) ** 2)) * Var(12, 2, 1)
    g = f.rename_vars({Var(7, 3, 0): Var(0, 3, 0), Var(9, 3, 1): Var(1, 3, 1), Var(12, 2, 1): Var(2, 2, 1)})
    assert repr(g) == repr(f).replace("Var(7,", "Var(0,").replace("Var(9,", "Var(1,").replace("Var(12,", "Var(2,")
    assert [v.ind for v in g.variables] == [0, 1, 2] and [v.ind for v in f.variables] == [7, 9, 12]
    assert f.rename_vars({}) is f

    def build(x, y, b):
        K = (-((LazyTensor(x[:, None, :]) - LazyTensor(y[None, :, :])) ** 2).sum(-1)).exp() * LazyTensor(b[None, :, :])
        return K.sum(1, call=False)

    lt._genred_cache.clear()
    r1 = build(torch.zeros(5, 3), torch.zeros(7, 3), torch.zeros(7, 2))
    n = len(lt._genred_cache)
    r2 = build(torch.ones(6, 3), torch.ones(4, 3), torch.ones(4, 2))
    assert n == 1 and len(lt._genred_cache) == 1 and callable(r1) and callable(r2)
    (key,) = lt._genred_cache
    assert key[0] == "Mult(Exp(Minus(Sum(Square(Subtract(Var(0,3,0),Var(1,3,1)))))),Var(2,2,1))"


def test_no_fast_math_keeps_every_formula_off_the_matrix_core_schemes():
    """use_fast_math=False means float32 arithmetic with library exp / sqrt on the vector kernel: neither the chunked
    nor the final-product scheme (bfloat16-split products, hardware exp2 / rsq) may be chosen."""
    al = ["x=Var(0,3,0)", "y=Var(1,3,1)", "b=Var(2,32,1)", "u=Var(3,64,0)", "v=Var(4,64,1)", "c=Var(5,2,1)"]
    for formula in ("Sum_Reduction(Exp(-Sqrt(SqDist(x,y)))*b,0)", "Sum_Reduction(Exp(-SqDist(u,v))*c,0)"):
        fast = get_keops_dll("GpuReduc1D", formula, 1, -1, 0, al, 6, "float", "float", "block_sum", 1, 1, 0, False, True, 0)
        exact = get_keops_dll("GpuReduc1D", formula, 1, -1, 0, al, 6, "float", "float", "block_sum", 1, 1, 0, False, False, 0)
        assert fast[8] in (1, 2) and exact[8] == 0
        with open(exact[1]) as f:
            src = f.read()
        assert "scheme=conv" in src.splitlines()[0] and "__builtin_amdgcn_exp2f" not in src
