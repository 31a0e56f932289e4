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
