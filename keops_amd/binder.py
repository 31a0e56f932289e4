"""ctypes binding of libkeops_hip.so (the C ABI of include/keops_hip.h).

Plays the role of the reference's two native bindings: the ctypes call into nvrtc_jit.so
(keopscore/keopscore/binders/nvrtc/Gpu_link_compile.py:78-91) and the pybind11 module
pykeops_nvrtc (pykeops/pykeops/common/keops_io/pykeops_nvrtc.cpp:13-103).  The library is built
in-tree by keops_amd/csrc/build_lib.py; a missing library is an error, there is no fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libkeops_hip.so")
_lib = None


class KeOpsHipError(RuntimeError):
    pass


NOT_CERTIFIED = -7  # KEOPS_HIP_NOT_CERTIFIED of include/keops_hip.h


class KeOpsNotCertified(KeOpsHipError):
    """A high-dimensional K-nearest-neighbour launch could not prove its result exact: run the exact kernel."""


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            from .csrc import build_lib

            build_lib.build()
        L = ctypes.CDLL(LIB_PATH)
        L.keops_hip_last_error.restype = ctypes.c_char_p
        L.keops_hip_templates_digest.restype = ctypes.c_char_p
        L.keops_hip_module_create.restype = ctypes.c_void_p
        L.keops_hip_module_create.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_char_p]
        L.keops_hip_module_destroy.argtypes = [ctypes.c_void_p]
        L.keops_hip_module_meta.restype = ctypes.c_char_p
        L.keops_hip_module_meta.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        L.keops_hip_module_set_timing.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.keops_hip_module_last_kernel_ms.restype = ctypes.c_double
        L.keops_hip_module_last_kernel_ms.argtypes = [ctypes.c_void_p]
        L.keops_hip_compile.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int, ctypes.c_int]
        I64, P = ctypes.c_int64, ctypes.c_void_p
        L.keops_hip_launch.argtypes = [
            P, ctypes.c_int, I64, I64, I64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, I64, I64, ctypes.c_int,
            P, ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int, I64, P, P, P, P, P, ctypes.c_int, P, P, P, P, P,
            ctypes.c_int,
        ]
        L.keops_hip_launch_noalloc.argtypes = [
            P, I64, I64, ctypes.c_int, ctypes.c_int, I64, P, ctypes.c_int, P, ctypes.c_int, P, ctypes.c_int, I64, P, P, P,
            P, ctypes.c_int, P, P, P, P, P,
        ]
        L.keops_hip_noalloc_scratch_bytes.restype = ctypes.c_size_t
        L.keops_hip_ranges_status.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint)]
        L.keops_hip_path_status.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint)]
        _lib = L
    return _lib


def noalloc_scratch_bytes():
    return int(lib().keops_hip_noalloc_scratch_bytes())


_calib = None


def calibrate(kind, chains, blocks, iters, device_id=0):
    """(milliseconds, counted instructions per wavefront) of one loop-only calibration kernel: keops_calibrate of
    csrc/keops_calibrate.h, in the benchmark-only library libkeops_calibrate.so (built by csrc/build_lib.py)."""
    global _calib
    if _calib is None:
        from .csrc import build_lib

        path = build_lib.CALIB_LIB
        if not os.path.exists(path):
            build_lib.build()
        _calib = ctypes.CDLL(path)
        _calib.keops_calibrate.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_double)] * 2
    ms, ipw = ctypes.c_double(0), ctypes.c_double(0)
    rc = _calib.keops_calibrate(int(device_id), int(kind), int(chains), int(blocks), int(iters), ctypes.byref(ms), ctypes.byref(ipw))
    if rc != 0:
        raise KeOpsHipError(f"calibration failed (code {rc}): kind or chains out of range, or no device")
    return ms.value, ipw.value


def mfma_probe(a_bits, b_bits, acc0=0.0, device_id=0):
    """out[32][32] = acc0 + a b^T of one v_mfma_f32_32x32x16_bf16 on bfloat16 bit patterns a_bits[32][16], b_bits[32][16]
    (numpy uint16): keops_calibrate_mfma_probe of csrc/keops_calibrate.h."""
    import numpy as np

    global _calib
    if _calib is None:
        from .csrc import build_lib

        if not os.path.exists(build_lib.CALIB_LIB):
            build_lib.build()
        _calib = ctypes.CDLL(build_lib.CALIB_LIB)
        _calib.keops_calibrate.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_double)] * 2
    a = np.ascontiguousarray(a_bits, dtype=np.uint16).reshape(32, 16)
    b = np.ascontiguousarray(b_bits, dtype=np.uint16).reshape(32, 16)
    out = np.zeros((32, 32), np.float32)
    fn = _calib.keops_calibrate_mfma_probe
    fn.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]
    rc = fn(int(device_id), a.ctypes.data, b.ctypes.data, float(acc0), out.ctypes.data)
    if rc != 0:
        raise KeOpsHipError(f"matrix-core probe failed (code {rc})")
    return out


def last_error():
    return lib().keops_hip_last_error().decode(errors="replace")


def device_count():
    return lib().keops_hip_device_count()


def templates_digest():
    return lib().keops_hip_templates_digest().decode()


def compile_module(target_file, source, use_fast_math=True, device_id=0):
    rc = lib().keops_hip_compile(target_file.encode(), source.encode(), int(bool(use_fast_math)), int(device_id))
    if rc != 0:
        raise KeOpsHipError(f"kernel compilation failed (code {rc}): {last_error()}")


_iarr_cache = {}


def _iarr(ctype, values):
    """ctypes array of ``values``; the small constant tuples of a call (variable indices, dimensions,
    shapes) recur on every launch, so the arrays are kept."""
    key = (ctype, tuple(values))
    arr = _iarr_cache.get(key)
    if arr is None:
        if len(_iarr_cache) > 4096:
            _iarr_cache.clear()
        arr = _iarr_cache[key] = (ctype * max(1, len(key[1])))(*key[1])
    return arr


class Module:
    """A loaded kernel module (KeOps_module_float/double of the reference)."""

    def __init__(self, device_id, nargs, target_file):
        self.handle = lib().keops_hip_module_create(int(device_id), int(nargs), target_file.encode())
        if not self.handle:
            raise KeOpsHipError(f"cannot load kernel module: {last_error()}")
        self.nargs = nargs

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h and _lib is not None:
            _lib.keops_hip_module_destroy(h)

    def meta(self, key):
        v = lib().keops_hip_module_meta(self.handle, key.encode())
        return None if v is None else v.decode()

    def set_timing(self, enabled):
        lib().keops_hip_module_set_timing(self.handle, int(bool(enabled)))

    def ranges_status(self):
        """Status bits of the last block-sparse launch whose table was built on the device
        (keops_hip_ranges_status of include/keops_hip.h); waits for that launch."""
        st = ctypes.c_uint(0)
        if lib().keops_hip_ranges_status(self.handle, ctypes.byref(st)) != 0:
            raise KeOpsHipError(last_error())
        return int(st.value)

    def path_status(self):
        """1 when the first of the module's two kernel families served the last launch (matrix-core exponents of a
        Gaussian-type sum, byte filter of a K-nearest-neighbour search), 0 when the other one did
        (keops_hip_path_status of include/keops_hip.h); waits for that launch."""
        st = ctypes.c_uint(0)
        if lib().keops_hip_path_status(self.handle, ctypes.byref(st)) != 0:
            raise KeOpsHipError(last_error())
        return int(st.value)

    def last_kernel_ms(self):
        return lib().keops_hip_module_last_kernel_ms(self.handle)

    def __call__(self, tagHostDevice, dimy, nx, ny, tagI, tagZero, use_half, tag1D2D, dimred, block_size,
                 use_chunk_mode, indsi, indsj, indsp, dimout, dimsx, dimsy, dimsp, ranges_ptr, shapeout,
                 out_ptr, args_ptr, argshapes, stream=0, sync=False):
        """Same positional arguments as KeOps_module_python::operator() (pykeops_nvrtc.cpp:17-23),
        plus the stream to launch on and whether to wait for completion."""
        ci, cj, cp = _iarr(ctypes.c_int, indsi), _iarr(ctypes.c_int, indsj), _iarr(ctypes.c_int, indsp)
        dx, dy, dp = _iarr(ctypes.c_int64, dimsx), _iarr(ctypes.c_int64, dimsy), _iarr(ctypes.c_int64, dimsp)
        rp = (ctypes.c_void_p * 7)(*ranges_ptr)
        so = _iarr(ctypes.c_int64, shapeout)
        ap = (ctypes.c_void_p * max(1, len(args_ptr)))(*args_ptr)
        flat = [int(d) for shp in argshapes for d in shp]
        sh = _iarr(ctypes.c_int64, flat)
        nd = _iarr(ctypes.c_int, [len(shp) for shp in argshapes])
        rc = lib().keops_hip_launch(
            self.handle, int(tagHostDevice), int(dimy), int(nx), int(ny), int(tagI), int(tagZero), int(bool(use_half)), int(tag1D2D),
            int(dimred), int(block_size), int(use_chunk_mode), ci, len(indsi), cj, len(indsj), cp, len(indsp),
            int(dimout), dx, dy, dp, rp, so, len(shapeout), ctypes.c_void_p(out_ptr), ap, sh, nd,
            ctypes.c_void_p(stream), int(bool(sync)),
        )
        if rc == NOT_CERTIFIED:
            raise KeOpsNotCertified(last_error())
        if rc != 0:
            raise KeOpsHipError(f"kernel launch failed (code {rc}): {last_error()}")
        return 0

    def call_noalloc(self, nx, ny, tagI, tag1D2D, dimred, indsi, indsj, indsp, dimout, dimsx, dimsy, dimsp, shapeout,
                     out_ptr, args_ptr, argshapes, stream=0):
        """keops_hip_launch_noalloc: device pointers, no ranges, no batch dimensions; workspaces come from the
        library's static scratch buffer and nothing is allocated."""
        ci, cj, cp = _iarr(ctypes.c_int, indsi), _iarr(ctypes.c_int, indsj), _iarr(ctypes.c_int, indsp)
        dx, dy, dp = _iarr(ctypes.c_int64, dimsx), _iarr(ctypes.c_int64, dimsy), _iarr(ctypes.c_int64, dimsp)
        so = _iarr(ctypes.c_int64, shapeout)
        ap = (ctypes.c_void_p * max(1, len(args_ptr)))(*args_ptr)
        sh = _iarr(ctypes.c_int64, [int(d) for shp in argshapes for d in shp])
        nd = _iarr(ctypes.c_int, [len(shp) for shp in argshapes])
        rc = lib().keops_hip_launch_noalloc(
            self.handle, int(nx), int(ny), int(tagI), int(tag1D2D), int(dimred), ci, len(indsi), cj, len(indsj), cp,
            len(indsp), int(dimout), dx, dy, dp, so, len(shapeout), ctypes.c_void_p(out_ptr), ap, sh, nd,
            ctypes.c_void_p(stream),
        )
        if rc != 0:
            raise KeOpsHipError(f"kernel launch failed (code {rc}): {last_error()}")
        return 0
