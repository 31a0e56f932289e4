"""Host-side evaluator for generated formula bodies (test helper, CPU only).

Compiles the straight-line code that keops_amd.formulas emits for a formula with g++ and
evaluates it on every (i, j) pair, so that the parser, the simplifier, the autodiff rules and the
scalar lowering can be checked against dense torch expressions without a GPU.
"""
import ctypes
import hashlib
import os
import subprocess
import tempfile

import numpy as np

from keops_amd.formulas import Lir, lower, parse

_PREAMBLE = r"""
#include <cmath>
#include <cstdint>
typedef %(T)s T;
static inline T keops_exp(T x) { return std::exp(x); }
static inline T keops_log(T x) { return std::log(x); }
static inline T keops_sqrt(T x) { return std::sqrt(x); }
static inline T keops_abs(T x) { return std::fabs(x); }
static inline T keops_sin(T x) { return std::sin(x); }
static inline T keops_cos(T x) { return std::cos(x); }
static inline T keops_asin(T x) { return std::asin(x); }
static inline T keops_acos(T x) { return std::acos(x); }
static inline T keops_atan(T x) { return std::atan(x); }
static inline T keops_atan2(T y, T x) { return std::atan2(y, x); }
static inline T keops_pow(T x, T y) { return std::pow(x, y); }
static inline T keops_fma(T a, T b, T c) { return std::fma(a, b, c); }
static inline T keops_add_rounded(T a, T b) { return a + b; }
static inline T keops_sub_rounded(T a, T b) { return a - b; }
static inline T keops_mul_rounded(T a, T b) { return a * b; }
static inline T keops_floor(T x) { return std::floor(x); }
static inline T keops_round(T x) { return std::round(x); }
static inline float __builtin_amdgcn_exp2f(float x) { return std::exp2(x); }
static inline float __builtin_amdgcn_logf(float x) { return std::log2(x); }
static inline float __builtin_amdgcn_sqrtf(float x) { return std::sqrt(x); }
static inline float __builtin_amdgcn_rcpf(float x) { return 1.0f / x; }
static inline float __builtin_amdgcn_rsqf(float x) { return 1.0f / std::sqrt(x); }
"""

_cache = {}


def dense_eval(formula, aliases, args, M, N, dtype=np.float64, fast_math=False, segment=0):
    """Evaluate a formula string (or Op) on all pairs.  args[k] is (M,d) | (N,d) | (d,) following the
    category of variable k.  Returns an array (M, N, dim).  ``segment`` > 0: the body is emitted as a chain of
    functions of that many statements (the form used for very long formulas), on the concatenated xi / yj / p
    arrays of the kernels."""
    op = parse(formula, aliases) if isinstance(formula, str) else formula
    ctype = "double" if np.dtype(dtype) == np.float64 else "float"
    L = Lir(row_cat=0, fast_math=fast_math, dtype=ctype)
    outs = lower(op, L)
    names, decl = {}, []
    if segment:
        off = {0: 0, 1: 0, 2: 0}
        arr = {0: "xi", 1: "yj", 2: "p"}
        copies = []
        for v in op.variables:
            idx = {0: "i", 1: "j", 2: "0"}[v.cat]
            for k in range(v.dim):
                names[(v.cat, v.ind, k)] = f"{arr[v.cat]}[{off[v.cat] + k}]"
            copies.append(f"    for (int k = 0; k < {v.dim}; k++) {arr[v.cat]}[{off[v.cat]} + k] = "
                          f"((const T*)args[{v.ind}] + (int64_t){idx} * {v.dim})[k];")
            off[v.cat] += v.dim
        decl = [f"    T xi[{max(1, off[0])}], yj[{max(1, off[1])}], p[{max(1, off[2])}];"] + copies
        lines, exprs = L.emit(outs, names, segment=segment, segment_min=0)
    else:
        for v in op.variables:
            for k in range(v.dim):
                names[(v.cat, v.ind, k)] = f"a{v.ind}[{k}]"
        lines, exprs = L.emit(outs, names)
        for v in op.variables:
            idx = {0: "i", 1: "j", 2: "0"}[v.cat]
            decl.append(f"    const T* a{v.ind} = (const T*)args[{v.ind}] + (int64_t){idx} * {v.dim};")
    body = "\n".join(decl + lines + [f"    o[{k}] = {e};" for k, e in enumerate(exprs)])
    prelude = "#define __device__\n" + "\n".join(L.prelude) + "\n"
    src = _PREAMBLE % dict(T=ctype) + prelude + f"""
extern "C" void dense(int64_t M, int64_t N, const void* const* args, T* out) {{
  for (int64_t i = 0; i < M; i++) for (int64_t j = 0; j < N; j++) {{
    T* o = out + (i * N + j) * {op.dim};
{body}
  }}
}}
"""
    key = hashlib.sha256(src.encode()).hexdigest()[:16]
    lib = _cache.get(key)
    if lib is None:
        d = tempfile.mkdtemp(prefix="keops_host_")
        cpp, so = os.path.join(d, "f.cpp"), os.path.join(d, "f.so")
        with open(cpp, "w") as f:
            f.write(src)
        subprocess.run(["g++", "-O1", "-shared", "-fPIC", "-ffp-contract=off", cpp, "-o", so], check=True)
        lib = _cache[key] = ctypes.CDLL(so)
    arrs = [np.ascontiguousarray(a, dtype=dtype) for a in args]
    ptrs = (ctypes.c_void_p * max(1, len(arrs)))(*[a.ctypes.data for a in arrs])
    out = np.empty((M, N, op.dim), dtype=dtype)
    lib.dense(ctypes.c_int64(M), ctypes.c_int64(N), ptrs, out.ctypes.data_as(ctypes.c_void_p))
    return out
