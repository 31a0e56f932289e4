// Shared device-side definitions for the map-reduce kernel templates (gfx950, wave64).
//
// A kernel module is the concatenation of a generated "plug-in" (typedefs T / TACC, the KEOPS_*
// geometry macros, the variable tables and struct KeopsFormula) followed by one of the
// hand-written templates in this directory.  This header is included by every template.
#pragma once

typedef long long i64;

#ifndef INFINITY
#define INFINITY __builtin_huge_valf()
#endif
#ifndef NAN
#define NAN __builtin_nanf("")
#endif

// ---- scalar math used by generated formula bodies (slow-path spellings; the fast paths are
// ---- emitted as __builtin_amdgcn_* calls by the code generator) ---------------------------
__device__ __forceinline__ float keops_exp(float x) { return __ocml_exp_f32(x); }
__device__ __forceinline__ double keops_exp(double x) { return __ocml_exp_f64(x); }
__device__ __forceinline__ float keops_log(float x) { return __ocml_log_f32(x); }
__device__ __forceinline__ double keops_log(double x) { return __ocml_log_f64(x); }
__device__ __forceinline__ float keops_sqrt(float x) { return __ocml_sqrt_f32(x); }
__device__ __forceinline__ double keops_sqrt(double x) { return __ocml_sqrt_f64(x); }
__device__ __forceinline__ float keops_abs(float x) { return __builtin_fabsf(x); }
__device__ __forceinline__ double keops_abs(double x) { return __builtin_fabs(x); }
__device__ __forceinline__ float keops_sin(float x) { return __ocml_sin_f32(x); }
__device__ __forceinline__ double keops_sin(double x) { return __ocml_sin_f64(x); }
__device__ __forceinline__ float keops_cos(float x) { return __ocml_cos_f32(x); }
__device__ __forceinline__ double keops_cos(double x) { return __ocml_cos_f64(x); }
__device__ __forceinline__ float keops_asin(float x) { return __ocml_asin_f32(x); }
__device__ __forceinline__ double keops_asin(double x) { return __ocml_asin_f64(x); }
__device__ __forceinline__ float keops_acos(float x) { return __ocml_acos_f32(x); }
__device__ __forceinline__ double keops_acos(double x) { return __ocml_acos_f64(x); }
__device__ __forceinline__ float keops_atan(float x) { return __ocml_atan_f32(x); }
__device__ __forceinline__ double keops_atan(double x) { return __ocml_atan_f64(x); }
__device__ __forceinline__ float keops_atan2(float y, float x) { return __ocml_atan2_f32(y, x); }
__device__ __forceinline__ double keops_atan2(double y, double x) { return __ocml_atan2_f64(y, x); }
__device__ __forceinline__ float keops_pow(float x, float y) { return __ocml_pow_f32(x, y); }
__device__ __forceinline__ double keops_pow(double x, double y) { return __ocml_pow_f64(x, y); }
// a sum, a difference, a product rounded on its own: never contracted into a fused multiply-add with a neighbour
// (the arguments of exponentials: an exponential magnifies a relative error of its argument by the argument's size)
template <typename U> __device__ __forceinline__ U keops_add_rounded(U a, U b) {
#pragma clang fp contract(off)
  return a + b;
}
template <typename U> __device__ __forceinline__ U keops_sub_rounded(U a, U b) {
#pragma clang fp contract(off)
  return a - b;
}
template <typename U> __device__ __forceinline__ U keops_mul_rounded(U a, U b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float keops_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double keops_fma(double a, double b, double c) { return __builtin_fma(a, b, c); }
__device__ __forceinline__ float keops_floor(float x) { return __builtin_floorf(x); }
__device__ __forceinline__ double keops_floor(double x) { return __builtin_floor(x); }
__device__ __forceinline__ float keops_round(float x) { return __builtin_roundf(x); }
__device__ __forceinline__ double keops_round(double x) { return __builtin_round(x); }

// exp used inside reductions (online log-sum-exp): hardware exp2 for float, libm for double
__device__ __forceinline__ float keops_red_exp(float x) {
#if KEOPS_FAST_MATH
  return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
#else
  return __ocml_exp_f32(x);
#endif
}
__device__ __forceinline__ double keops_red_exp(double x) { return __ocml_exp_f64(x); }

__device__ __forceinline__ float keops_fmax(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double keops_fmax(double a, double b) { return __builtin_fmax(a, b); }

template <typename A> __device__ __forceinline__ A keops_inf() { return (A)__builtin_huge_valf(); }

__device__ __forceinline__ i64 keops_min(i64 a, i64 b) { return a < b ? a : b; }
__device__ __forceinline__ i64 keops_max(i64 a, i64 b) { return a > b ? a : b; }

// ---- block-sparse / batched geometry of the matrix-core schemes ------------------------------------
//
// Same tables as the generic block-sparse kernel (keopscore/keopscore/mapreduce/gpu/GpuReduc1D_ranges.py:74-173,
// keopscore/keopscore/binders/nvrtc/keops_nvrtc.cpp:152-248): one lookup entry (range id, first row,
// end row) per workgroup, the reduced-index ranges of every row range, and, with batch dimensions, the
// first-row offset of every argument for every workgroup (here indexed by argument number).
// A module built with KEOPS_MC_RANGES = 0 ignores the tables: every helper folds to the dense case.
#ifndef KEOPS_MC_RANGES
#define KEOPS_MC_RANGES 0
#endif

// A value that is the same in every lane of a wavefront (loaded from a table at a wave-uniform address): kept in
// scalar registers
__device__ __forceinline__ i64 keops_uniform(i64 v) {
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)(v & 0xffffffffll));
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)((unsigned long long)v >> 32));
  return (i64)(((unsigned long long)hi << 32) | lo);
}

// true when the predicate holds in some lane: one compare into a scalar register pair and a scalar test (the
// library's __any goes through an integer per lane: two more vector instructions)
__device__ __forceinline__ bool keops_any(bool p) { return __builtin_amdgcn_ballot_w64(p) != 0ull; }

struct KeopsRangeTables {
  const i64* lookup;    // [nblocks][3] = (range id, first row, end row)
  const i64* slices_x;  // end slice of every row range
  const i64* ranges_y;  // [*][2] reduced-index ranges
  const i64* offsets;   // batch mode: [nblocks][nargs] first-row offsets by argument
  int nbatchdims;
  int nargs;
};

// rows owned by a workgroup and the index arithmetic of its arguments
struct KeopsTileGeom {
  i64 row_first, row_end;  // global output rows [row_first, row_end) of this workgroup
  i64 slice_first, slice_end;
  const i64* offs;         // batch mode: this workgroup's per-argument offsets, else null

  __device__ __forceinline__ void init(const KeopsRangeTables& R, i64 nx, int rows_per_block) {
#if KEOPS_MC_RANGES
    const i64 bid = blockIdx.x;
    const i64 range_id = keops_uniform(R.lookup[3 * bid]);
    row_first = keops_uniform(R.lookup[3 * bid + 1]);
    row_end = keops_uniform(R.lookup[3 * bid + 2]);
    slice_first = range_id < 1 ? 0 : keops_uniform(R.slices_x[range_id - 1]);
    slice_end = keops_uniform(R.slices_x[range_id]);
    offs = R.nbatchdims > 0 ? R.offsets + (i64)R.nargs * bid : nullptr;
#else
    row_first = (i64)blockIdx.x * rows_per_block;
    row_end = keops_min(nx, row_first + rows_per_block);
    slice_first = slice_end = 0;
    offs = nullptr;
#endif
  }
  // row of argument `arg` that holds global output row q / reduced row j / the parameter
  __device__ __forceinline__ i64 row(int arg, i64 q) const {
#if KEOPS_MC_RANGES
    return offs ? keops_uniform(offs[arg]) + (q - row_first) : q;
#else
    return q;
#endif
  }
  __device__ __forceinline__ i64 col(int arg, i64 j) const {
#if KEOPS_MC_RANGES
    return offs ? keops_uniform(offs[arg]) + j : j;
#else
    return j;
#endif
  }
  __device__ __forceinline__ i64 par(int arg) const {
#if KEOPS_MC_RANGES
    return offs ? keops_uniform(offs[arg]) : 0;
#else
    return 0;
#endif
  }
  // Cursor over the maximal runs of contiguous reduced-index ranges of this workgroup: next() yields [jbeg, jend)
  // until the ranges are exhausted.  With batch dimensions the single range of the batch is swept as [0, length)
  // (batch-relative indices, the offsets move the arguments).  A dense module yields its one interval once.
  // (A loop around the sweep instead of a callback: the sweep must be inlined, or the register tiles it updates
  // would live in scratch memory.)
  i64 cur_index, cur_start;
  __device__ __forceinline__ void rewind(const KeopsRangeTables& R) {
    cur_index = slice_first;
#if KEOPS_MC_RANGES
    cur_start = slice_first < slice_end ? keops_uniform(R.ranges_y[2 * slice_first]) : 0;
#else
    cur_start = 0;
#endif
  }
  __device__ __forceinline__ bool next(const KeopsRangeTables& R, i64& jbeg, i64& jend) {
#if KEOPS_MC_RANGES
    for (; cur_index < slice_end; cur_index++) {
      if (cur_index + 1 >= slice_end || R.ranges_y[2 * cur_index + 2] != R.ranges_y[2 * cur_index + 1]) {
        const i64 end_y = keops_uniform(R.ranges_y[2 * cur_index + 1]);
        jbeg = offs ? (i64)0 : cur_start;
        jend = offs ? end_y - cur_start : end_y;
        if (cur_index + 1 < slice_end) cur_start = keops_uniform(R.ranges_y[2 * cur_index + 2]);
        cur_index++;
        return true;
      }
    }
#endif
    return false;
  }
};
