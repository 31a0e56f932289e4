"""keops_amd: MI355X-native backend for KeOps-style tiled map-reduce (Genred / LazyTensor API)."""
__version__ = "0.1.0"

from . import config as _config


def set_verbose(val):
    """Print (or not) a line when a formula is compiled (pykeops.set_verbose)."""
    _config.verbose = bool(val)


def get_build_folder():
    """Folder of the on-disk cache of compiled kernel modules (pykeops.get_build_folder)."""
    return _config.get_build_folder()


def set_build_folder(path=None):
    """Use ``path`` for the on-disk cache of compiled kernel modules (pykeops.set_build_folder); modules
    already loaded in this process stay valid."""
    from . import get_keops_dll as _g
    from . import keops_io as _io

    folder = _config.set_build_folder(path)
    _g._cache.clear()
    _io._loaders.clear()
    return folder


def clean_keops_amd(recompile_library=False):
    """Delete the compiled kernel modules of the cache folder (pykeops.clean_pykeops); with
    ``recompile_library`` also rebuild libkeops_hip.so from its sources."""
    import os

    from . import get_keops_dll as _g
    from . import keops_io as _io

    folder = _config.get_build_folder()
    n = 0
    for f in os.listdir(folder):
        if f.startswith("hsaco_") or f.endswith(".hip"):
            os.remove(os.path.join(folder, f))
            n += 1
    _g._cache.clear()
    _io._loaders.clear()
    _io._modules.clear()
    if recompile_library:
        from .csrc import build_lib

        build_lib.build(force=True)
    _config.message(f"{n} cached files removed from {folder}")
    return n


def test_torch_bindings():
    """Small self-test on the current HIP device (pykeops.test_torch_bindings): a Gaussian-weighted sum
    compared with the dense torch formula."""
    import torch

    from .torch import Genred

    x, y, b = (torch.arange(k, k + 12, dtype=torch.float32, device="cuda").reshape(4, 3) / 10 for k in (1, 2, 3))
    out = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(3)"], reduction_op="Sum", axis=1)(x, y, b)
    ref = torch.exp(-torch.cdist(x, y) ** 2) @ b
    ok = bool(torch.allclose(out, ref, rtol=1e-5, atol=1e-6))
    print("keops_amd with torch bindings is working!" if ok else "keops_amd: unexpected result", flush=True)
    return ok


def clean_pykeops(recompile_jit_binaries=True):
    """Name used by the reference (pykeops/__init__.py:47-61): empties the cache folder; the native library is
    rebuilt on request."""
    return clean_keops_amd(recompile_library=bool(recompile_jit_binaries))


def test_numpy_bindings():
    """As test_torch_bindings on NumPy arrays staged through the device (pykeops.test_numpy_bindings)."""
    import numpy as np

    from .numpy import Genred

    x, y, b = (np.arange(k, k + 12, dtype=np.float32).reshape(4, 3) / 10 for k in (1, 2, 3))
    out = Genred("Exp(-SqDist(x,y))*b", ["x=Vi(3)", "y=Vj(3)", "b=Vj(3)"], reduction_op="Sum", axis=1)(x, y, b)
    ref = np.exp(-((x[:, None, :] - y[None, :, :]) ** 2).sum(-1)) @ b
    ok = bool(np.allclose(out, ref, rtol=1e-5, atol=1e-6))
    print("keops_amd with numpy bindings is working!" if ok else "keops_amd: unexpected result", flush=True)
    return ok


def check_health():
    """What a launch depends on, printed (keopscore.check_health, pykeops/__init__.py:64-80): the native library and
    its entry points, the hiprtc compiler behind it, the cache folder and the devices torch sees."""
    import os

    from . import binder

    lib = binder.lib()
    folder = _config.get_build_folder()
    print(f"library        : {binder.LIB_PATH} (templates {binder.templates_digest()[:12]})")
    print(f"cache folder   : {folder} ({'writable' if os.access(folder, os.W_OK) else 'NOT writable'}, "
          f"{sum(f.startswith('hsaco_') for f in os.listdir(folder))} compiled modules)")
    try:
        import torch

        n = torch.cuda.device_count() if torch.cuda.is_available() else 0
        names = ", ".join(torch.cuda.get_device_name(k) for k in range(n)) or "none visible"
        print(f"devices        : {n} ({names})")
    except ImportError:
        print("devices        : torch is not importable")
    return lib is not None
