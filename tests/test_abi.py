"""CPU-side checks of the C ABI: the library loads, exports every symbol include/keops_hip.h declares,
cross-compiles kernel modules for gfx950 through hiprtc without a GPU, and reports errors through return
codes.  No kernel is launched here."""
import ctypes
import os
import re
import struct

import pytest

from keops_amd import binder
from keops_amd.get_keops_dll import get_keops_dll

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "keops_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(keops_hip_\w+)\s*\(", header))
    assert {"keops_hip_compile", "keops_hip_module_create", "keops_hip_module_destroy", "keops_hip_launch",
            "keops_hip_last_error"} <= declared
    lib = ctypes.CDLL(binder.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert binder.lib().keops_hip_abi_version() == 3
    assert re.fullmatch(r"[0-9a-f]{64}", binder.templates_digest())


def test_compile_errors_are_reported_not_raised_across_abi(tmp_path):
    target = str(tmp_path / "bad")
    with pytest.raises(binder.KeOpsHipError) as e:
        binder.compile_module(target, "this is not HIP", True, 0)
    assert "hiprtc" in str(e.value)
    assert not os.path.exists(target)
    lib = binder.lib()
    assert lib.keops_hip_module_create(0, 1, b"/nonexistent/module") is None
    assert b"cannot open" in lib.keops_hip_last_error()


@pytest.mark.parametrize("formula,aliases,expected_scheme", [
    ("Sum_Reduction(Exp(-g*SqDist(x,y))*b,0)", ["x=Var(0,3,0)", "y=Var(1,3,1)", "b=Var(2,1,1)", "g=Var(3,1,2)"], "conv"),
    ("KMin_ArgKMin_Reduction(SqDist(x,y),10,0)", ["x=Var(0,64,0)", "y=Var(1,64,1)"], "knn"),
    ("Sum_Reduction(Exp(-Sqrt(SqDist(x,y)))*b,1)", ["x=Var(0,256,0)", "y=Var(1,256,1)", "b=Var(2,16,0)"], "chunk"),
])
def test_cross_compilation_and_module_file_format(formula, aliases, expected_scheme):
    os.environ.setdefault("KEOPS_HIP_ARCH", "gfx950")
    res = get_keops_dll("GpuReduc1D", formula, 1, -1, 0, aliases, len(aliases), "float", "float",
                        "block_sum" if "Sum_" in formula else "direct_sum", 1, 1, 0, False, True, 0)
    tag, src, target, tagI, tagZero = res[:5]
    assert tagZero == 0 and os.path.exists(target)
    data = open(target, "rb").read()
    (n,) = struct.unpack("<Q", data[:8])
    assert data[8:12] == b"\x7fELF"
    (m,) = struct.unpack("<Q", data[8 + n:16 + n])
    meta = data[16 + n:16 + n + m].decode()
    assert f"scheme={expected_scheme}" in meta and "dimred=" in meta
    assert len(res) == 19 and res[3] == (1 if formula.endswith(",1)") else 0)


def test_metadata_tuple_matches_reference_conventions():
    """dimx/dimy/indices as get_keops_dll.py:139-159 returns them."""
    al = ["x=Var(0,3,0)", "y=Var(1,3,1)", "b=Var(2,8,1)", "g=Var(3,1,2)"]
    r = get_keops_dll("GpuReduc1D", "Sum_Reduction(Exp(-g*SqDist(x,y))*b,0)", 1, -1, 0, al, 4, "float", "float",
                      "block_sum", 1, 1, 0, False, True, 0)
    assert (r[3], r[4], r[10], r[11], r[12]) == (0, 0, 8, 8, 11)          # tagI, tagZero, dimred, dim, dimy
    assert r[13:19] == ((0,), (1, 2), (3,), (3,), (3, 8), (1,))           # indsi, indsj, indsp, dimsx, dimsy, dimsp
    g = get_keops_dll("GpuReduc1D", "Grad_WithSavedForward(Sum_Reduction(Exp(-g*SqDist(x,y))*b,0),Var(1,3,1),"
                      "Var(4,8,0),Var(5,8,0))", 1, -1, 0, al + ["Var(4,8,0)", "Var(5,8,0)"], 6, "float", "float",
                      "block_sum", 1, 1, 0, False, True, 0)
    assert g[3] == 1 and g[11] == 3  # gradient wrt a j-variable: output indexed by j, dimension 3
    z = get_keops_dll("GpuReduc1D", "Grad_WithSavedForward(Sum_Reduction(Exp(-SqDist(x,y)),0),Var(2,8,1),Var(4,1,0),"
                      "Var(5,1,0))", 1, -1, 0, al + ["Var(4,1,0)", "Var(5,1,0)"], 6, "float", "float", "block_sum",
                      1, 1, 0, False, True, 0)
    assert z[4] == 1  # the formula does not depend on b: zero reduction, no kernel


def test_genred_front_end_host_logic():
    from keops_amd.common.operations import preprocess
    from keops_amd.common.parse_type import complete_aliases, get_optional_flags, get_sizes, get_type
    from keops_amd.torch import Genred

    g = Genred("SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], reduction_op="ArgKMin", axis=1, opt_arg=10)
    assert g.formula == "ArgKMin_Reduction(SqDist(x,y),10,0)"
    g = Genred("l-SqDist(x,y)*e", ["x=Vi(3)", "y=Vj(3)", "l=Vj(1)", "e=Pm(1)"], reduction_op="LogSumExp", axis=1)
    assert g.formula == "Max_SumShiftExp_Reduction(l-SqDist(x,y)*e,0)" and g.optional_flags["sum_scheme"] == "block_sum"
    assert preprocess("SumSoftMaxWeight", "w") == ("Max_SumShiftExpWeight", "Concat(IntCst(1),w)")
    assert get_type("x = Vi(3)", 0) == ("x", 0, 3, 0) and get_type("Pm(2,5)") == (None, 2, 5, 2)
    assert get_type("Var(4,7,1)") == (None, 1, 7, 4)
    assert complete_aliases("F(Var(2,1,0),Var(0,3,0))", ["x=Vi(3)", "y=Vj(3)"]) == ["x=Vi(3)", "y=Vj(3)", "Var(2,1,0)"]
    with pytest.raises(ValueError):
        get_optional_flags("Min", "float64", False, "auto", True)
    with pytest.raises(ValueError):
        get_optional_flags("Min", "auto", False, "block_sum", True)
    with pytest.raises(ValueError):
        Genred("SqDist(x,y)", ["x=Vi(3)", "y=Vj(3)"], axis=2)

    class T:  # shape-only stand-in
        def __init__(self, *s):
            self.shape = s

    assert get_sizes(["x=Vi(3)", "y=Vj(3)", "p=Pm(1)"], T(5, 3), T(7, 3), T(1)) == (5, 7)


def test_cache_folder_controls(tmp_path):
    """set_build_folder / clean_keops_amd (pykeops.set_build_folder, clean_pykeops): modules are compiled
    into the chosen folder (cross-compilation needs no GPU) and removed again."""
    import os

    import keops_amd
    from keops_amd.get_keops_dll import get_keops_dll

    os.environ.setdefault("KEOPS_HIP_ARCH", "gfx950")
    default = keops_amd.get_build_folder()
    try:
        folder = keops_amd.set_build_folder(str(tmp_path / "cache"))
        assert folder == keops_amd.get_build_folder() and os.path.isdir(folder)
        al = ["x=Var(0,2,0)", "y=Var(1,2,1)"]
        r = get_keops_dll("GpuReduc1D", "Sum_Reduction(SqDist(x,y),0)", 1, -1, 0, al, 2, "float", "float", "block_sum",
                          1, 1, 0, False, True, 0)
        assert r[2].startswith(folder) and os.path.exists(r[2])
        assert keops_amd.clean_keops_amd() >= 1
        assert not os.path.exists(r[2])
    finally:
        assert keops_amd.set_build_folder(None) == default


def test_reference_named_helpers_exist_and_health_check_runs(capsys):
    """pykeops' top-level helpers (pykeops/__init__.py:20-104) under their own names."""
    import keops_amd

    for name in ("set_verbose", "get_build_folder", "set_build_folder", "clean_pykeops", "check_health",
                 "test_torch_bindings", "test_numpy_bindings"):
        assert callable(getattr(keops_amd, name)), name
    assert keops_amd.check_health() is True
    out = capsys.readouterr().out
    assert "libkeops_hip.so" in out and "cache folder" in out


def test_arguments_in_different_memories_are_rejected():
    """x on a GPU and a parameter on the host (or an output buffer that lives elsewhere than the arguments) is the
    reference's ValueError, not a launch with mismatched pointers (pykeops/pykeops/common/get_options.py)."""
    from keops_amd.common.get_options import get_tag_backend

    class Fake:
        def __init__(self, cuda):
            self.is_cuda = cuda

    with pytest.raises(ValueError, match="different memory locations"):
        get_tag_backend("auto", [Fake(True), Fake(True), Fake(False)])
    assert get_tag_backend("auto", [Fake(True), Fake(True)]) == (1, 0, 1)
    assert get_tag_backend("GPU_2D", [Fake(False), Fake(False)]) == (1, 1, 0)
