// Reduction policies for the map-reduce kernel templates.
//
// Each policy restates, for register-resident accumulators, the semantics of one reference
// reduction class (keopscore/keopscore/formulas/reductions/):
//   KEOPS_RED_KIND 0  Sum_Reduction.py:21-40                  acc += f            (+ Kahan)
//   KEOPS_RED_KIND 1  Max_SumShiftExpWeight_Reduction.py:35-61 (m, s) online log-sum-exp
//   KEOPS_RED_KIND 2  Min_ArgMin_Reduction_Base.py:21-49      (min, argmin), strict <
//   KEOPS_RED_KIND 3  Max_ArgMax_Reduction_Base.py            (max, argmax), strict >
//   KEOPS_RED_KIND 4  KMin_ArgKMin_Reduction.py:34-100        K smallest (value, index), ties keep
//                                                             the lower index first
// The accumulator of one output row is the POD struct KeopsAcc<A>; A is T for the per-tile
// temporary of the block_sum scheme (sum_schemes.py:44-71) and TACC for the running value.
// Index parts are kept as integers in registers and written out as floating point, which is the
// storage convention of the reference (the Python layer casts them back to int64).
#pragma once
#include "keops_common.h"

#define KEOPS_FD KEOPS_DIMFOUT

#if KEOPS_RED_KIND == 0 || KEOPS_RED_KIND == 5
// ------------------------------------------------------------------------------------ Sum
template <typename A> struct KeopsAcc {
  A v[KEOPS_FD];
#if KEOPS_SUM_SCHEME == 2
  A c[KEOPS_FD];  // Kahan compensation
#endif
  __device__ __forceinline__ void init() {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) {
      v[k] = (A)0;
#if KEOPS_SUM_SCHEME == 2
      c[k] = (A)0;
#endif
    }
  }
  __device__ __forceinline__ void push(const T (&f)[KEOPS_FD], i64) {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) {
#if KEOPS_SUM_SCHEME == 2
      A a = (A)f[k] - c[k];
      A b = v[k] + a;
      c[k] = (b - v[k]) - a;
      v[k] = b;
#else
      v[k] += (A)f[k];
#endif
    }
  }
  template <typename B> __device__ __forceinline__ void merge(const KeopsAcc<B>& o) {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) v[k] += (A)o.v[k];
  }
  __device__ __forceinline__ void store_partial(TACC* dst) const {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) dst[k] = (TACC)v[k];
  }
  __device__ __forceinline__ void load_partial(const TACC* src) {
    init();
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) v[k] = (A)src[k];
  }
  __device__ __forceinline__ void finalize(T* out) const {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) out[k] = (T)v[k];
  }
};

#elif KEOPS_RED_KIND == 1
// --------------------------------------------------------------- Max_SumShiftExp(Weight)
// f = [f0, g_1..g_{FD-1}];  acc = [m, s_1..s_{FD-1}]  represents  exp(m) * s.
template <typename A> struct KeopsAcc {
  A m;
  A s[KEOPS_FD - 1];
#if KEOPS_SUM_SCHEME == 2
  A c[KEOPS_FD - 1];
#endif
  __device__ __forceinline__ void init() {
    m = -keops_inf<A>();
#pragma unroll
    for (int k = 0; k < KEOPS_FD - 1; k++) {
      s[k] = (A)0;
#if KEOPS_SUM_SCHEME == 2
      c[k] = (A)0;
#endif
    }
  }
  // (m, s) <- (m, s) (+) (fm, g):  if m > fm: s += g*exp(fm-m)  else: s = g + exp(m-fm)*s, m = fm.
  // Branch-free form of the same update: one exponential of -|fm - m| and selects.
  template <typename B> __device__ __forceinline__ void absorb(B fm, const B* g) {
    const bool keep = m > (A)fm;  // false when equal or when m is still -inf
    // both sides still empty (-inf - -inf): the maximum with a finite bound drops the NaN, the factor is 0
    const A d = keops_fmax(keep ? (A)fm - m : m - (A)fm, (A)(-3.0e38f));
    A e = (A)keops_red_exp((T)d);
    // (the maximum above must not drop a value that is not a number: it makes the sums NaN for good, as the reference's
    // update does, Max_SumShiftExpWeight_Reduction.py:35-61)
    if (!((A)fm == (A)fm)) e = (A)fm;
#pragma unroll
    for (int k = 0; k < KEOPS_FD - 1; k++) {
#if KEOPS_SUM_SCHEME == 2
      // Max_SumShiftExpWeight_Reduction.py:63-87
      if (keep) {
        A a = (A)g[k] * e - c[k];
        A b = s[k] + a;
        c[k] = (b - s[k]) - a;
        s[k] = b;
      } else {
        A u = e * s[k];
        A a = (A)g[k] - e * c[k];
        A b = u + a;
        c[k] = (b - u) - a;
        s[k] = b;
      }
#else
      const A hi = keep ? s[k] : (A)g[k];
      const A lo = keep ? (A)g[k] : s[k];
      s[k] = hi + lo * e;
#endif
    }
    m = keep ? m : (A)fm;
  }
  __device__ __forceinline__ void push(const T (&f)[KEOPS_FD], i64) { absorb<T>(f[0], &f[1]); }
  template <typename B> __device__ __forceinline__ void merge(const KeopsAcc<B>& o) { absorb<B>(o.m, o.s); }
#if KEOPS_SUM_SCHEME != 2
  // G pairs at once: one running-maximum update and one rescaling of s per group, then per pair a
  // single exponential of (f - max) and one accumulation (the difference is formed first, as in the
  // reference: folding the shift into a multiply-add would lose accuracy when |max| is large).  Same function as G calls of push (the
  // running maximum only moves up, sums are shifted consistently); entries with f = -inf add nothing.
  template <int G> __device__ __forceinline__ void push_group(const T (&f)[G][KEOPS_FD]) {
    T mx = f[0][0];
#pragma unroll
    for (int g = 1; g < G; g++) mx = keops_fmax(mx, f[g][0]);
    // the lower bound keeps (f - mnew) and (m - mnew) well defined when everything seen so far is -inf
    const A mnew = keops_fmax(keops_fmax(m, (A)mx), (A)(-3.0e38f));
    const A scale = (A)keops_red_exp((T)(m - mnew));
#pragma unroll
    for (int k = 0; k < KEOPS_FD - 1; k++) s[k] *= scale;
#pragma unroll
    for (int g = 0; g < G; g++) {
      const A e = (A)keops_red_exp((T)((A)f[g][0] - mnew));
#pragma unroll
      for (int k = 0; k < KEOPS_FD - 1; k++) s[k] += (A)f[g][1 + k] * e;
    }
    m = mnew;
  }
#endif
  __device__ __forceinline__ void store_partial(TACC* dst) const {
    dst[0] = (TACC)m;
#pragma unroll
    for (int k = 0; k < KEOPS_FD - 1; k++) dst[1 + k] = (TACC)s[k];
  }
  __device__ __forceinline__ void load_partial(const TACC* src) {
    init();
    m = (A)src[0];
#pragma unroll
    for (int k = 0; k < KEOPS_FD - 1; k++) s[k] = (A)src[1 + k];
  }
  __device__ __forceinline__ void finalize(T* out) const {
    out[0] = (T)m;
#pragma unroll
    for (int k = 0; k < KEOPS_FD - 1; k++) out[1 + k] = (T)s[k];
  }
};

#elif KEOPS_RED_KIND == 2 || KEOPS_RED_KIND == 3
// ----------------------------------------------------------- Min_ArgMin / Max_ArgMax family
#if KEOPS_RED_KIND == 2
#define KEOPS_BETTER(a, b) ((a) < (b))
#define KEOPS_WORST(A) keops_inf<A>()
#else
#define KEOPS_BETTER(a, b) ((a) > (b))
#define KEOPS_WORST(A) (-keops_inf<A>())
#endif
template <typename A> struct KeopsAcc {
  A v[KEOPS_FD];
  int idx[KEOPS_FD];
  __device__ __forceinline__ void init() {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) {
      v[k] = KEOPS_WORST(A);
      idx[k] = 0;
    }
  }
  __device__ __forceinline__ void push(const T (&f)[KEOPS_FD], i64 j) {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) {
      const bool b = KEOPS_BETTER((A)f[k], v[k]);
      v[k] = b ? (A)f[k] : v[k];
      idx[k] = b ? (int)j : idx[k];
    }
  }
  // partials are merged in increasing order of their column slab, so strict comparison keeps
  // the lowest index on ties exactly like the sequential loop
  template <typename B> __device__ __forceinline__ void merge(const KeopsAcc<B>& o) {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) {
      const bool b = KEOPS_BETTER((A)o.v[k], v[k]);
      v[k] = b ? (A)o.v[k] : v[k];
      idx[k] = b ? o.idx[k] : idx[k];
    }
  }
  __device__ __forceinline__ void store_partial(TACC* dst) const {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) {
      dst[k] = (TACC)v[k];
      dst[KEOPS_FD + k] = (TACC)idx[k];
    }
  }
  __device__ __forceinline__ void load_partial(const TACC* src) {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) {
      v[k] = (A)src[k];
      idx[k] = (int)src[KEOPS_FD + k];
    }
  }
  __device__ __forceinline__ void finalize(T* out) const {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) {
#if KEOPS_RED_KEEP == 0
      out[k] = (T)v[k];
      out[KEOPS_FD + k] = (T)idx[k];
#elif KEOPS_RED_KEEP == 1
      out[k] = (T)v[k];
#else
      out[k] = (T)idx[k];
#endif
    }
  }
};

#elif KEOPS_RED_KIND == 4
// ------------------------------------------------------------- KMin / ArgKMin / KMin_ArgKMin
// Register-resident sorted list of the K best (value, index) per component.  A candidate enters
// at the tail and bubbles up through a fully unrolled compare-exchange chain; strict "<" leaves
// an equal, earlier candidate in front, which is the order of the reference's sequential
// insertion (KMin_ArgKMin_Reduction.py:72-100).
template <typename A> struct KeopsAcc {
  A v[KEOPS_FD][KEOPS_RED_K];
  int idx[KEOPS_FD][KEOPS_RED_K];
  __device__ __forceinline__ void init() {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++)
#pragma unroll
      for (int l = 0; l < KEOPS_RED_K; l++) {
        v[k][l] = keops_inf<A>();
        idx[k][l] = 0;
      }
  }
  // entry l becomes old[l-1] when the candidate goes before old[l-1], the candidate when it goes before old[l]
  // only, and stays otherwise: one compare per entry, shared by two neighbours, and for float32 values the new
  // entry is the median of (candidate, old[l-1], old[l]) in one instruction
  static __device__ __forceinline__ float mid(float x, float a, float b, bool, bool) { return __builtin_amdgcn_fmed3f(x, a, b); }
  static __device__ __forceinline__ double mid(double x, double a, double b, bool before_a, bool before_b) {
    return before_a ? a : (before_b ? x : b);
  }
  __device__ __forceinline__ void insert(int k, A x, int j) {
    if (x < v[k][KEOPS_RED_K - 1]) {
      bool before_cur = true;
#pragma unroll
      for (int l = KEOPS_RED_K - 1; l > 0; l--) {
        const bool before_prev = x < v[k][l - 1];
        idx[k][l] = before_prev ? idx[k][l - 1] : (before_cur ? j : idx[k][l]);
        v[k][l] = mid(x, v[k][l - 1], v[k][l], before_prev, before_cur);
        before_cur = before_prev;
      }
      idx[k][0] = before_cur ? j : idx[k][0];
      v[k][0] = before_cur ? x : v[k][0];
    }
  }
  __device__ __forceinline__ void push(const T (&f)[KEOPS_FD], i64 j) {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++) insert(k, (A)f[k], (int)j);
  }
  // o comes from a later column slab: inserting its entries in rank order reproduces the merge of
  // two sorted lists with priority to the earlier one on ties (KMin_ArgKMin_Reduction.py:47-69)
  template <typename B> __device__ __forceinline__ void merge(const KeopsAcc<B>& o) {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++)
#pragma unroll
      for (int l = 0; l < KEOPS_RED_K; l++) insert(k, (A)o.v[k][l], o.idx[k][l]);
  }
  // storage layout of the reference: acc[k + 2*FD*l] = value, acc[k + 2*FD*l + FD] = index
  __device__ __forceinline__ void store_partial(TACC* dst) const {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++)
#pragma unroll
      for (int l = 0; l < KEOPS_RED_K; l++) {
        dst[k + 2 * KEOPS_FD * l] = (TACC)v[k][l];
        dst[k + 2 * KEOPS_FD * l + KEOPS_FD] = (TACC)idx[k][l];
      }
  }
  __device__ __forceinline__ void load_partial(const TACC* src) {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++)
#pragma unroll
      for (int l = 0; l < KEOPS_RED_K; l++) {
        v[k][l] = (A)src[k + 2 * KEOPS_FD * l];
        idx[k][l] = (int)src[k + 2 * KEOPS_FD * l + KEOPS_FD];
      }
  }
  __device__ __forceinline__ void finalize(T* out) const {
#pragma unroll
    for (int k = 0; k < KEOPS_FD; k++)
#pragma unroll
      for (int l = 0; l < KEOPS_RED_K; l++) {
#if KEOPS_RED_KEEP == 0
        out[k + 2 * KEOPS_FD * l] = (T)v[k][l];
        out[k + 2 * KEOPS_FD * l + KEOPS_FD] = (T)idx[k][l];
#elif KEOPS_RED_KEEP == 1
        out[k + KEOPS_FD * l] = (T)v[k][l];
#else
        out[k + KEOPS_FD * l] = (T)idx[k][l];
#endif
      }
  }
};
#else
#error "unknown KEOPS_RED_KIND"
#endif

// block_sum keeps a per-tile temporary in the data type; direct_sum and kahan_scheme fold
// every pair straight into the running accumulator (sum_schemes.py:33-86).
#if KEOPS_SUM_SCHEME == 1
#define KEOPS_USE_TILE_TMP 1
#else
#define KEOPS_USE_TILE_TMP 0
#endif
