/*
 * TEST INFRASTRUCTURE ONLY - CPU restatement of the KeOps CpuReduc map-reduce path.
 *
 * This file is the parity oracle for the HIP kernels in keops_amd/csrc.  It is never part of
 * the shipped product path: only the test-suite, the smoke test and the cpu_baseline leg of
 * the benchmark load it.  It restates, in plain C, the loop nests that the reference emits as
 * C++ text:
 *
 *   keopscore/keopscore/mapreduce/cpu/CpuReduc.py:43-64         (dense i/j loop, OpenMP over i)
 *   keopscore/keopscore/mapreduce/cpu/CpuReduc_ranges.py:102-230 (block-sparse ranges loop)
 *   keopscore/keopscore/formulas/reductions/sum_schemes.py:33-86 (direct / block / kahan)
 *   keopscore/keopscore/formulas/reductions/Sum_Reduction.py:21-40
 *   keopscore/keopscore/formulas/reductions/Max_SumShiftExpWeight_Reduction.py:35-61
 *   keopscore/keopscore/formulas/reductions/Min_ArgMin_Reduction_Base.py:21-49 (+ Max_ArgMax twin)
 *   keopscore/keopscore/formulas/reductions/KMin_ArgKMin_Reduction.py:34-100
 *   keopscore/keopscore/formulas/reductions/ArgKMin_Reduction.py:21-30, KMin_Reduction.py:24-31
 *
 * The pair formula F(x_i, y_j, p) is either one of a few hand-written bodies that follow the
 * reference's per-op evaluation order (Subtract.py:21-24, Square.py:17-18, Sum.py:20-24,
 * Mult.py:25, Minus.py:20-23, Exp.py + math_functions.py:86, Sqrt.py:17, Abs.py, Scalprod.py:32-36
 * with its fused multiply-add chain), or a dense table
 * F[i][j][:] computed by the caller (numpy / torch closed form), so that every reduction can be
 * exercised on any formula.
 *
 * Pinning status (checked by tests/test_oracle.py against float64 closed forms, scipy
 * logsumexp, numpy stable argsort, brute force, invariants): every formula body and every
 * reduction below is pinned; nothing here is "parity unpinned".
 *
 * The file is compiled twice: -DTYPE=float -DSUFFIX=f32 and -DTYPE=double -DSUFFIX=f64.
 * Build flags follow the reference (g++ -O3 -fopenmp, no fast-math; base_config.py:210-212,
 * 281,291) plus -ffp-contract=off so that no FMA is formed where the reference's baseline
 * x86-64 build has none.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef TYPE
#define TYPE float
#define SUFFIX f32
#endif

#define CAT_(a, b) a##_##b
#define CAT(a, b) CAT_(a, b)
#define NAME(base) CAT(base, SUFFIX)

typedef TYPE real;

static inline real r_exp(real x) { return sizeof(real) == 4 ? (real)expf((float)x) : (real)exp((double)x); }
static inline real r_sqrt(real x) { return sizeof(real) == 4 ? (real)sqrtf((float)x) : (real)sqrt((double)x); }
#define R_INF ((real)INFINITY)

/* ------------------------------------------------------------------ formulas */

enum {
  F_DENSE = 0,      /* args[0] = F table [nx][ny][dimfout]                                   */
  F_GAUSS = 1,      /* Exp(-g*SqDist(x,y))*b          args: x[D] y[D] b[Dv] g[1]   -> Dv     */
  F_GAUSS_GRADX = 2,/* Grad of F_GAUSS wrt x, gradin G args: x y b g G[Dv]         -> D      */
  F_SQDIST = 3,     /* SqDist(x,y)                    args: x[D] y[D]              -> 1      */
  F_LSE_GAUSS = 4,  /* Concat(l - SqDist(x,y)*e, 1)   args: x[D] y[D] l[1] e[1]    -> 2      */
  F_LAPLACE = 5,    /* Exp(-Norm2(x-y))*b             args: x[D] y[D] b[Dv]        -> Dv     */
  F_L1DIST = 6,     /* Sum(Abs(x-y))                  args: x[D] y[D]              -> 1      */
  F_EXP_L1 = 7,     /* Exp(-Sum(Abs(x-y)))*b          args: x[D] y[D] b[Dv]        -> Dv     */
  F_SCALPROD = 8,   /* (x|y)*b                        args: x[D] y[D] b[Dv]        -> Dv     */
  F_GAUSS_GRADX_ABS = 9 /* |F_GAUSS_GRADX| term by term: the condition scale sum_j |F_ij| of the tests */
};

typedef struct {
  int formula;
  int nargs;
  const real *const *args; /* row-major [rows][dim] arrays; parameters are [dim]              */
  const int *dims;         /* dim of every arg                                                */
  long ny_table;           /* F_DENSE only: row stride (= ny of the table)                    */
  int dimfout;
} fctx;

/* SqDist(x,y) = Sum(Square(Subtract(x,y))): out = 0; out += d_k*d_k in order (Sum.py:20-24) */
static inline real sqdist_seq(const real *x, const real *y, int D) {
  real s = (real)0;
  for (int k = 0; k < D; k++) {
    real d = x[k] - y[k];
    real q = d * d;
    s += q;
  }
  return s;
}

/* Sum(Abs(Subtract(x,y))): out = 0; out += |x_k - y_k| in order (Subtract.py:21-24, Abs.py +
   math_functions.py keops_abs, Sum.py:20-24) */
static inline real l1dist_seq(const real *x, const real *y, int D) {
  real s = (real)0;
  for (int k = 0; k < D; k++) {
    real d = x[k] - y[k];
    real q = sizeof(real) == 4 ? (real)fabsf((float)d) : (real)fabs((double)d);
    s += q;
  }
  return s;
}

/* Scalprod(x,y): out = 0; out = fma(x_k, y_k, out) in order (Scalprod.py:32-36, keops_fma) */
static inline real scalprod_fma(const real *x, const real *y, int D) {
  real s = (real)0;
  for (int k = 0; k < D; k++) s = sizeof(real) == 4 ? (real)fmaf((float)x[k], (float)y[k], (float)s) : (real)fma((double)x[k], (double)y[k], (double)s);
  return s;
}

static void eval_pair(const fctx *c, long i, long j, real *fout) {
  const real *const *a = c->args;
  const int *dm = c->dims;
  switch (c->formula) {
  case F_DENSE: {
    const real *src = a[0] + ((size_t)i * (size_t)c->ny_table + (size_t)j) * (size_t)c->dimfout;
    for (int k = 0; k < c->dimfout; k++) fout[k] = src[k];
  } break;
  case F_GAUSS: {
    int D = dm[0], Dv = dm[2];
    real s = sqdist_seq(a[0] + i * D, a[1] + j * D, D);
    real t = a[3][0] * s; /* g * SqDist  (Mult.py:25)  */
    real u = -t;          /* Minus       (Minus.py:20) */
    real e = r_exp(u);    /* Exp                        */
    const real *b = a[2] + j * Dv;
    for (int k = 0; k < Dv; k++) fout[k] = e * b[k];
  } break;
  case F_GAUSS_GRADX: {
    /* d/dx_i < G_i , sum_j K_ij b_j >  =  sum_j  -2 g K_ij (G_i . b_j) (x_i - y_j) */
    int D = dm[0], Dv = dm[2];
    const real *x = a[0] + i * D, *y = a[1] + j * D, *b = a[2] + j * Dv, *G = a[4] + i * Dv;
    real s = sqdist_seq(x, y, D);
    real e = r_exp(-(a[3][0] * s));
    real gb = (real)0;
    for (int k = 0; k < Dv; k++) gb += G[k] * b[k];
    real coef = -((real)2 * (a[3][0] * (e * gb)));
    for (int k = 0; k < D; k++) fout[k] = coef * (x[k] - y[k]);
  } break;
  case F_GAUSS_GRADX_ABS: {
    int D = dm[0], Dv = dm[2];
    const real *x = a[0] + i * D, *y = a[1] + j * D, *b = a[2] + j * Dv, *G = a[4] + i * Dv;
    real e = r_exp(-(a[3][0] * sqdist_seq(x, y, D)));
    real gb = (real)0;
    for (int k = 0; k < Dv; k++) gb += (real)fabs((double)(G[k] * b[k]));
    real coef = (real)2 * (real)fabs((double)a[3][0]) * (e * gb);
    for (int k = 0; k < D; k++) fout[k] = coef * (real)fabs((double)(x[k] - y[k]));
  } break;
  case F_SQDIST: {
    int D = dm[0];
    fout[0] = sqdist_seq(a[0] + i * D, a[1] + j * D, D);
  } break;
  case F_LSE_GAUSS: {
    int D = dm[0];
    real s = sqdist_seq(a[0] + i * D, a[1] + j * D, D);
    fout[0] = a[2][j] - s * a[3][0];
    fout[1] = (real)1; /* formula2 = IntCst(1), Max_SumShiftExpWeight_Reduction.py:24-29 */
  } break;
  case F_LAPLACE: {
    int D = dm[0], Dv = dm[2];
    real s = sqdist_seq(a[0] + i * D, a[1] + j * D, D);
    real e = r_exp(-r_sqrt(s));
    const real *b = a[2] + j * Dv;
    for (int k = 0; k < Dv; k++) fout[k] = e * b[k];
  } break;
  case F_L1DIST: {
    int D = dm[0];
    fout[0] = l1dist_seq(a[0] + i * D, a[1] + j * D, D);
  } break;
  case F_EXP_L1: {
    int D = dm[0], Dv = dm[2];
    real s = l1dist_seq(a[0] + i * D, a[1] + j * D, D);
    real e = r_exp(-s);
    const real *b = a[2] + j * Dv;
    for (int k = 0; k < Dv; k++) fout[k] = e * b[k];
  } break;
  case F_SCALPROD: {
    int D = dm[0], Dv = dm[2];
    real s = scalprod_fma(a[0] + i * D, a[1] + j * D, D);
    const real *b = a[2] + j * Dv;
    for (int k = 0; k < Dv; k++) fout[k] = s * b[k];
  } break;
  }
}

/* ---------------------------------------------------------------- reductions */

enum {
  R_SUM = 0,
  R_MAX_SUMSHIFTEXPWEIGHT = 1, /* fout = [f, g_0..]; acc = [m, s_0..]                        */
  R_MIN_ARGMIN = 2,            /* acc = [vals(fd), idx(fd)]                                    */
  R_MAX_ARGMAX = 3,
  R_KMIN_ARGKMIN = 4,          /* acc[2*K*fd] interleaved (val, idx) per rank                  */
  R_MIN = 5, R_ARGMIN = 6, R_MAX = 7, R_ARGMAX = 8, R_KMIN = 9, R_ARGKMIN = 10
};
enum { S_DIRECT = 0, S_BLOCK = 1, S_KAHAN = 2 };

typedef struct {
  int red, K, fd; /* fd = dim of the pair formula */
} rctx;

static int red_base(int red) {
  switch (red) {
  case R_MIN: case R_ARGMIN: return R_MIN_ARGMIN;
  case R_MAX: case R_ARGMAX: return R_MAX_ARGMAX;
  case R_KMIN: case R_ARGKMIN: return R_KMIN_ARGKMIN;
  default: return red;
  }
}
static int red_dimred(const rctx *r) {
  switch (red_base(r->red)) {
  case R_SUM: case R_MAX_SUMSHIFTEXPWEIGHT: return r->fd;
  case R_MIN_ARGMIN: case R_MAX_ARGMAX: return 2 * r->fd;
  default: return 2 * r->K * r->fd;
  }
}
static int red_dimout(const rctx *r) {
  switch (r->red) {
  case R_SUM: case R_MAX_SUMSHIFTEXPWEIGHT: return r->fd;
  case R_MIN_ARGMIN: case R_MAX_ARGMAX: return 2 * r->fd;
  case R_MIN: case R_ARGMIN: case R_MAX: case R_ARGMAX: return r->fd;
  case R_KMIN_ARGKMIN: return 2 * r->K * r->fd;
  default: return r->K * r->fd;
  }
}

/* The accumulator type may be wider than the data type (dtype_acc="float64"); the macro below
   instantiates every reduction primitive for an accumulator type A and a pair-value type real. */
#define DEFINE_RED(A, TAG)                                                                       \
  static void init_##TAG(const rctx *r, A *acc) {                                                \
    int fd = r->fd;                                                                              \
    switch (red_base(r->red)) {                                                                  \
    case R_SUM: for (int k = 0; k < fd; k++) acc[k] = 0; break;                                  \
    case R_MAX_SUMSHIFTEXPWEIGHT:                                                                \
      acc[0] = -(A)INFINITY; for (int k = 1; k < fd; k++) acc[k] = 0; break;                     \
    case R_MIN_ARGMIN:                                                                           \
      for (int k = 0; k < fd; k++) { acc[k] = (A)INFINITY; acc[fd + k] = 0; } break;             \
    case R_MAX_ARGMAX:                                                                           \
      for (int k = 0; k < fd; k++) { acc[k] = -(A)INFINITY; acc[fd + k] = 0; } break;            \
    default:                                                                                     \
      for (int k = 0; k < fd; k++)                                                               \
        for (int l = k; l < k + 2 * r->K * fd; l += 2 * fd) { acc[l] = (A)INFINITY; acc[l + fd] = 0; } \
    }                                                                                            \
  }                                                                                              \
  /* ReducePairShort(acc, fout, j): fold one pair value in */                                    \
  static void push_##TAG(const rctx *r, A *acc, const real *xi, long ind) {                      \
    int fd = r->fd;                                                                              \
    switch (red_base(r->red)) {                                                                  \
    case R_SUM: for (int k = 0; k < fd; k++) acc[k] += xi[k]; break;                             \
    case R_MAX_SUMSHIFTEXPWEIGHT:                                                                \
      if (acc[0] > xi[0]) {                                                                      \
        A e = (A)r_exp((real)(xi[0] - acc[0]));                                                  \
        for (int k = 1; k < fd; k++) acc[k] += xi[k] * e;                                        \
      } else {                                                                                   \
        A e = (A)r_exp((real)(acc[0] - xi[0]));                                                  \
        for (int k = 1; k < fd; k++) acc[k] = xi[k] + e * acc[k];                                \
        acc[0] = xi[0];                                                                          \
      } break;                                                                                   \
    case R_MIN_ARGMIN:                                                                           \
      for (int k = 0; k < fd; k++) if (xi[k] < acc[k]) { acc[k] = xi[k]; acc[fd + k] = (A)ind; } \
      break;                                                                                     \
    case R_MAX_ARGMAX:                                                                           \
      for (int k = 0; k < fd; k++) if (xi[k] > acc[k]) { acc[k] = xi[k]; acc[fd + k] = (A)ind; } \
      break;                                                                                     \
    default: /* sequential insertion from the tail, strict < (KMin_ArgKMin_Reduction.py:72-100) */ \
      for (int k = 0; k < fd; k++) {                                                             \
        A xik = xi[k];                                                                           \
        for (int l = k + (r->K - 1) * 2 * fd; l >= k && xik < acc[l]; l -= 2 * fd) {             \
          A tmpl = acc[l]; A indtmpl = acc[l + fd];                                              \
          acc[l] = xik; acc[l + fd] = (A)ind;                                                    \
          if (l < k + 2 * fd * (r->K - 1)) { acc[l + 2 * fd] = tmpl; acc[l + 2 * fd + fd] = indtmpl; } \
        }                                                                                        \
      }                                                                                          \
    }                                                                                            \
  }

DEFINE_RED(real, r)
DEFINE_RED(double, d)

/* ReducePair(acc, tmp): merge a partial accumulator (always of type real: block_sum keeps tmp
   in dtype, sum_schemes.py:44-47) into acc of type A.  Only Sum and Max_SumShiftExpWeight
   accept block_sum (parse_type.py:161-186). */
#define DEFINE_MERGE(A, TAG)                                                                     \
  static void merge_##TAG(const rctx *r, A *acc, const real *xi) {                               \
    int fd = r->fd;                                                                              \
    if (r->red == R_SUM) { for (int k = 0; k < fd; k++) acc[k] += xi[k]; return; }               \
    if (acc[0] > xi[0]) {                                                                        \
      A e = (A)r_exp((real)(xi[0] - acc[0]));                                                    \
      for (int k = 1; k < fd; k++) acc[k] += xi[k] * e;                                          \
    } else {                                                                                     \
      A e = (A)r_exp((real)(acc[0] - xi[0]));                                                    \
      for (int k = 1; k < fd; k++) acc[k] = xi[k] + e * acc[k];                                  \
      acc[0] = xi[0];                                                                            \
    }                                                                                            \
  }
DEFINE_MERGE(real, r)
DEFINE_MERGE(double, d)

/* KahanScheme for Sum (Sum_Reduction.py:31-40) and Max_SumShiftExpWeight (:63-87) */
#define DEFINE_KAHAN(A, TAG)                                                                     \
  static void kahan_##TAG(const rctx *r, A *acc, const real *xi, A *tmp) {                       \
    int fd = r->fd;                                                                              \
    if (r->red == R_SUM) {                                                                       \
      for (int k = 0; k < fd; k++) {                                                             \
        A a = xi[k] - tmp[k]; A b = acc[k] + a; tmp[k] = (b - acc[k]) - a; acc[k] = b;           \
      }                                                                                          \
      return;                                                                                    \
    }                                                                                            \
    if (acc[0] > xi[0]) {                                                                        \
      A e = (A)r_exp((real)(xi[0] - acc[0]));                                                    \
      for (int k = 1; k < fd; k++) {                                                             \
        A a = xi[k] * e - tmp[k - 1]; A b = acc[k] + a; tmp[k - 1] = (b - acc[k]) - a; acc[k] = b; \
      }                                                                                          \
    } else {                                                                                     \
      A e = (A)r_exp((real)(acc[0] - xi[0]));                                                    \
      for (int k = 1; k < fd; k++) {                                                             \
        A u = e * acc[k]; A a = xi[k] - e * tmp[k - 1]; A b = u + a;                             \
        tmp[k - 1] = (b - u) - a; acc[k] = b;                                                    \
      }                                                                                          \
      acc[0] = xi[0];                                                                            \
    }                                                                                            \
  }
DEFINE_KAHAN(real, r)
DEFINE_KAHAN(double, d)

#define DEFINE_FINAL(A, TAG)                                                                     \
  static void final_##TAG(const rctx *r, const A *acc, real *out) {                              \
    int fd = r->fd, K = r->K;                                                                    \
    switch (r->red) {                                                                            \
    case R_SUM: case R_MAX_SUMSHIFTEXPWEIGHT: for (int k = 0; k < fd; k++) out[k] = (real)acc[k]; break; \
    case R_MIN_ARGMIN: case R_MAX_ARGMAX: case R_KMIN_ARGKMIN:                                   \
      for (int k = 0; k < red_dimred(r); k++) out[k] = (real)acc[k]; break;                      \
    case R_MIN: case R_MAX: for (int k = 0; k < fd; k++) out[k] = (real)acc[k]; break;           \
    case R_ARGMIN: case R_ARGMAX: for (int k = 0; k < fd; k++) out[k] = (real)acc[fd + k]; break; \
    case R_KMIN:                                                                                 \
      for (int k = 0; k < fd; k++) { int p = k;                                                  \
        for (int l = k; l < k + 2 * fd * K; l += 2 * fd) { out[p] = (real)acc[l]; p += fd; } }   \
      break;                                                                                     \
    case R_ARGKMIN:                                                                              \
      for (int k = 0; k < fd; k++) { int p = k;                                                  \
        for (int l = k; l < k + 2 * fd * K; l += 2 * fd) { out[p] = (real)acc[l + fd]; p += fd; } } \
      break;                                                                                     \
    }                                                                                            \
  }
DEFINE_FINAL(real, r)
DEFINE_FINAL(double, d)

#define MAXRED 512

/* One output row of the dense scheme, CpuReduc.py:46-61. */
#define DEFINE_ROW(A, TAG)                                                                       \
  static void row_dense_##TAG(const fctx *f, const rctx *r, int scheme, long i, long ny, real *out) { \
    real fout[MAXRED]; A acc[MAXRED]; real tmp[MAXRED]; A ktmp[MAXRED];                          \
    init_##TAG(r, acc);                                                                          \
    long period = ny < 10 ? 100 : (long)sqrt((double)ny);                                        \
    if (scheme == S_BLOCK) init_r(r, tmp);                                                       \
    if (scheme == S_KAHAN) for (int k = 0; k < MAXRED; k++) ktmp[k] = 0;                         \
    for (long j = 0; j < ny; j++) {                                                              \
      eval_pair(f, i, j, fout);                                                                  \
      if (scheme == S_DIRECT) push_##TAG(r, acc, fout, j);                                       \
      else if (scheme == S_KAHAN) kahan_##TAG(r, acc, fout, ktmp);                               \
      else {                                                                                     \
        push_r(r, tmp, fout, j);                                                                 \
        if (!((j + 1) % period)) { merge_##TAG(r, acc, tmp); init_r(r, tmp); }                   \
      }                                                                                          \
    }                                                                                            \
    if (scheme == S_BLOCK) merge_##TAG(r, acc, tmp);                                             \
    final_##TAG(r, acc, out);                                                                    \
  }                                                                                              \
  /* One output row of the block-sparse scheme, CpuReduc_ranges.py:178-225 (nbatchdims == 0):   \
     no periodic fold there, the temporary is folded once at the end. */                         \
  static void row_ranges_##TAG(const fctx *f, const rctx *r, int scheme, long i,                 \
                               long start_slice, long end_slice, const int64_t *ranges_y, real *out) { \
    real fout[MAXRED]; A acc[MAXRED]; real tmp[MAXRED]; A ktmp[MAXRED];                          \
    init_##TAG(r, acc);                                                                          \
    if (scheme == S_BLOCK) init_r(r, tmp);                                                       \
    if (scheme == S_KAHAN) for (int k = 0; k < MAXRED; k++) ktmp[k] = 0;                         \
    for (long s = start_slice; s < end_slice; s++) {                                             \
      for (long j = ranges_y[2 * s]; j < ranges_y[2 * s + 1]; j++) {                             \
        eval_pair(f, i, j, fout);                                                                \
        if (scheme == S_DIRECT) push_##TAG(r, acc, fout, j);                                     \
        else if (scheme == S_KAHAN) kahan_##TAG(r, acc, fout, ktmp);                             \
        else push_r(r, tmp, fout, j);                                                            \
      }                                                                                          \
    }                                                                                            \
    if (scheme == S_BLOCK) merge_##TAG(r, acc, tmp);                                             \
    final_##TAG(r, acc, out);                                                                    \
  }                                                                                              \
  static void row_empty_##TAG(const rctx *r, real *out) {                                        \
    A acc[MAXRED]; init_##TAG(r, acc); final_##TAG(r, acc, out);                                 \
  }
DEFINE_ROW(real, r)
DEFINE_ROW(double, d)

/* ------------------------------------------------------------------ entry points */

/*
 * Dense reduction over j for the rows listed in `rows` (or all nx rows when rows == NULL):
 *   out[r][0..dimout) = Finalize( Reduce_j F(x_rows[r], y_j, p) ).
 * Returns 0, or -1 on bad arguments.
 */
int NAME(oracle_cpu_reduc)(int formula, int red, int K, int scheme, int acc_double, long nx, long ny,
                           int dimfout, int nargs, const real *const *args, const int *dims,
                           const int64_t *rows, long nrows, real *out) {
  fctx f = {formula, nargs, args, dims, ny, dimfout};
  rctx r = {red, K, dimfout};
  if (red_dimred(&r) > MAXRED || dimfout > MAXRED) return -1;
  long n = rows ? nrows : nx;
  int dimout = red_dimout(&r);
#pragma omp parallel for schedule(dynamic, 16)
  for (long q = 0; q < n; q++) {
    long i = rows ? rows[q] : q;
    if (acc_double) row_dense_d(&f, &r, scheme, i, ny, out + q * dimout);
    else row_dense_r(&f, &r, scheme, i, ny, out + q * dimout);
  }
  return 0;
}

/*
 * Block-sparse reduction (no batch dimensions).  ranges_x [nranges][2], slices_x [nranges],
 * ranges_y [*][2] are the three arrays CpuReduc_ranges.py:159-167 selects.  Rows that no
 * x-range covers receive Finalize(Initialize()) (CpuReduc_ranges.py:150-153).
 */
int NAME(oracle_cpu_reduc_ranges)(int formula, int red, int K, int scheme, int acc_double, long nx,
                                  long ny, int dimfout, int nargs, const real *const *args,
                                  const int *dims, long nranges, const int64_t *ranges_x,
                                  const int64_t *slices_x, const int64_t *ranges_y,
                                  const int64_t *rows, long nrows, real *out) {
  fctx f = {formula, nargs, args, dims, ny, dimfout};
  rctx r = {red, K, dimfout};
  if (red_dimred(&r) > MAXRED || dimfout > MAXRED) return -1;
  long n = rows ? nrows : nx;
  int dimout = red_dimout(&r);
  /* row -> last range that contains it (the reference's ranges are disjoint) */
  int64_t *owner = (int64_t *)malloc(sizeof(int64_t) * (size_t)(nx > 0 ? nx : 1));
  for (long i = 0; i < nx; i++) owner[i] = -1;
  for (long k = 0; k < nranges; k++)
    for (long i = ranges_x[2 * k]; i < ranges_x[2 * k + 1]; i++) owner[i] = k;
#pragma omp parallel for schedule(dynamic, 16)
  for (long q = 0; q < n; q++) {
    long i = rows ? rows[q] : q;
    long k = owner[i];
    real *o = out + q * dimout;
    if (k < 0) { if (acc_double) row_empty_d(&r, o); else row_empty_r(&r, o); continue; }
    long s0 = k < 1 ? 0 : slices_x[k - 1], s1 = slices_x[k];
    if (acc_double) row_ranges_d(&f, &r, scheme, i, s0, s1, ranges_y, o);
    else row_ranges_r(&f, &r, scheme, i, s0, s1, ranges_y, o);
  }
  free(owner);
  return 0;
}

int NAME(oracle_dimout)(int red, int K, int dimfout) {
  rctx r = {red, K, dimfout};
  return red_dimout(&r);
}
