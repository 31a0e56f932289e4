// Tiled map-reduce kernels:  out_i = Finalize( Reduce_j F(x_i, y_j, p) ).
//
// These templates replace the kernel text that the reference generates per formula
//   keopscore/keopscore/mapreduce/gpu/GpuReduc1D.py:43-96          (keops_conv_dense, one slab)
//   keopscore/keopscore/mapreduce/gpu/GpuReduc2D.py:81-200         (keops_conv_dense with column
//                                                                   slabs + keops_reduce_partials)
//   keopscore/keopscore/mapreduce/gpu/GpuReduc1D_ranges.py:74-173  (keops_conv_ranges)
// with a design for CDNA wave64 hardware:
//   * every lane owns KEOPS_ROWS output rows whose variables x_i stay in VGPRs for the whole
//     kernel, so one y_j fetched from LDS feeds KEOPS_ROWS formula evaluations;
//   * the reduced-index variables y_j of a tile are staged once per workgroup in LDS, packed row
//     by row (stride KEOPS_DIMY_PAD, a multiple of 4 floats) and read back with 128-bit
//     wave-uniform (broadcast, conflict-free) loads;
//   * the formula is straight-line scalar code, so all temporaries live in registers;
//   * the reduced axis can be cut into column slabs (blockIdx.y) whose partial accumulators are
//     merged in slab order by keops_reduce_partials: this fills the chip when there are few rows.
//
// The plug-in that precedes this header defines:  T, TACC, KEOPS_NARGS, KEOPS_DIMX, KEOPS_DIMY,
// KEOPS_DIMY_PAD, KEOPS_DIMP, KEOPS_DIMFOUT, KEOPS_DIMRED, KEOPS_DIMOUT, KEOPS_RED_KIND,
// KEOPS_RED_KEEP, KEOPS_RED_K, KEOPS_SUM_SCHEME, KEOPS_FAST_MATH, KEOPS_BLOCK, KEOPS_ROWS,
// KEOPS_TILE_J, KEOPS_UNROLL_J, KEOPS_LSE_GROUP, the tables keops_{row,col,par}_{arg,dim,off}[] with their counts
// KEOPS_NROWVARS / KEOPS_NCOLVARS / KEOPS_NPARVARS, and struct KeopsFormula.
//
// KEOPS_VCHUNK (formulas with one long elementwise sum, the vector-ALU counterpart of GpuReduc1D_chunks.py:19-118):
// the plug-in also defines VCH_D (components), VCH_DPAD, VCH_NROW / VCH_NCOL (long output-indexed / reduced-index
// variables), the flags keops_{row,col}_long[] and positions keops_vch_{row,col}[] of those variables in the
// tables, VCH_USES_YJ, VCH_FMA (the sum is a scalar product folded with explicit fused multiply-adds, as the reference's
// Scalprod: eval then returns the two factors), and struct KeopsChunkFormula (one component of the sum).  Long variables are not copied to
// x_i / y_j: the reduced-index ones are staged whole in LDS for a short tile of columns, the output-indexed ones are
// read from memory 16 bytes at a time (one cache line serves four such reads), each read feeding KEOPS_TILE_J
// running sums held in registers; KeopsFormula::eval takes the finished sum as an extra argument.
#pragma once
#include "keops_reductions.h"
#ifndef KEOPS_VCHUNK
#define KEOPS_VCHUNK 0
#endif

// Kernel argument block; the host library fills the same layout (keops_hip.cpp: LaunchParams).
struct KeopsParams {
  i64 nx;             // number of output rows (after the i/j swap when the reduction runs over i)
  i64 ny;             // number of reduced rows
  T* out;             // [nx][KEOPS_DIMOUT]
  TACC* partial;      // [nslabs][nx][KEOPS_DIMRED], only when nslabs > 1
  i64 slab_len;       // reduced rows per column slab
  int nslabs;
  int nbatchdims;
  const i64* lookup;    // ranges: [nblocks][3] = (range id, first row, end row)
  const i64* slices_x;  // ranges: end slice of every row range
  const i64* ranges_y;  // ranges: [*][2] column ranges
  const i64* offsets;   // batch mode: [nblocks][nvars] first-row offsets per variable
  const unsigned* guard;  // not null: the dense kernels return at once when *guard == 1 (another kernel of the
                          // module has produced the result: kernels/keops_radial_mfma.h)
  const T* arg[KEOPS_NARGS > 0 ? KEOPS_NARGS : 1];
};

#define KEOPS_ROWS_PER_BLOCK (KEOPS_BLOCK * KEOPS_ROWS)

// ---- loading -------------------------------------------------------------------------------

// x_i of one output row: concatenation of the row variables (code_gen_utils.py:663-731 layout)
__device__ __forceinline__ void keops_load_row(const KeopsParams& P, const i64* rowoff, i64 i, T (&xi)[KEOPS_DIMX > 0 ? KEOPS_DIMX : 1]) {
#pragma unroll
  for (int v = 0; v < KEOPS_NROWVARS; v++) {
#if KEOPS_VCHUNK
    if (keops_row_long[v]) continue;
#endif
    const T* src = P.arg[keops_row_arg[v]] + (rowoff[v] + i) * keops_row_dim[v];
#pragma unroll
    for (int d = 0; d < keops_row_dim[v]; d++) xi[keops_row_off[v] + d] = src[d];
  }
}

__device__ __forceinline__ void keops_load_params(const KeopsParams& P, const i64* paroff, T (&p)[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1]) {
#pragma unroll
  for (int v = 0; v < KEOPS_NPARVARS; v++) {
    const T* src = P.arg[keops_par_arg[v]] + paroff[v] * keops_par_dim[v];
#pragma unroll
    for (int d = 0; d < keops_par_dim[v]; d++) p[keops_par_off[v] + d] = src[d];
  }
}

// Stage rows [j0, j0+n) of every reduced-index variable into LDS.  Each variable is a dense
// row-major array, so the n*dim values of a tile are contiguous in HBM and the workgroup reads
// them with fully coalesced loads; they are scattered to the packed per-row LDS layout.
__device__ __forceinline__ void keops_stage_tile(const KeopsParams& P, const i64* coloff, i64 j0, int n, T* ys) {
#pragma unroll
  for (int v = 0; v < KEOPS_NCOLVARS; v++) {
#if KEOPS_VCHUNK
    if (keops_col_long[v]) continue;
#endif
    const int dim = keops_col_dim[v];
    const T* src = P.arg[keops_col_arg[v]] + (coloff[v] + j0) * dim;
    const int total = n * dim;
    for (int e = threadIdx.x; e < total; e += KEOPS_BLOCK) {
      const int row = e / dim, c = e - row * dim;
      ys[row * KEOPS_DIMY_PAD + keops_col_off[v] + c] = src[e];
    }
  }
}

__device__ __forceinline__ void keops_read_col(const T* ys, int jj, T (&yj)[KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1]) {
  const T* row = ys + jj * KEOPS_DIMY_PAD;
  constexpr int VEC = 16 / sizeof(T);
  typedef T vecT __attribute__((ext_vector_type(VEC)));
#pragma unroll
  for (int q = 0; q < KEOPS_DIMY_PAD / VEC; q++) {
    const vecT w = *reinterpret_cast<const vecT*>(row + q * VEC);
#pragma unroll
    for (int c = 0; c < VEC; c++) yj[q * VEC + c] = w[c];
  }
}

#if KEOPS_VCHUNK
// ---- the pair loop of formulas with one long elementwise sum -----------------------------------

static_assert(KEOPS_ROWS == 1, "one output row per lane");
constexpr int VCH_VEC = 16 / sizeof(T);
typedef T vch_vec __attribute__((ext_vector_type(VCH_VEC)));

// Folds columns [jbeg, jend) into acc[0].  xlong[v]: this lane's row of the v-th long output-indexed variable.
__device__ __forceinline__ void keops_sweep(const KeopsParams& P, const i64* coloff, i64 jbeg, i64 jend, i64 jshift,
                                            const T (&xi)[KEOPS_ROWS][KEOPS_DIMX > 0 ? KEOPS_DIMX : 1],
                                            const T (&p)[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1],
                                            KeopsAcc<TACC> (&acc)[KEOPS_ROWS], T* ys, T* yl,
                                            const T* const (&xlong)[VCH_NROW > 0 ? VCH_NROW : 1]) {
#if KEOPS_RED_KIND >= 2
#pragma clang fp contract(off)  // index-carrying reductions: the running sum keeps the reference's roundings
#endif
  constexpr int NR = VCH_NROW > 0 ? VCH_NROW : 1, NC = VCH_NCOL > 0 ? VCH_NCOL : 1;
  for (i64 j0 = jbeg; j0 < jend; j0 += KEOPS_TILE_J) {
    const int n = (int)keops_min((i64)KEOPS_TILE_J, jend - j0);
    __syncthreads();  // the previous tile has been consumed by every wave
    keops_stage_tile(P, coloff, j0, n, ys);
    // long reduced-index variables: row jj of variable v at yl + (jj * VCH_NCOL + v) * VCH_DPAD
#pragma unroll
    for (int v = 0; v < VCH_NCOL; v++) {
      const T* src = P.arg[keops_col_arg[keops_vch_col[v]]] + (coloff[keops_vch_col[v]] + j0) * VCH_D;
      for (int e = threadIdx.x; e < n * VCH_D; e += KEOPS_BLOCK) {
        const int row = e / VCH_D, c = e - row * VCH_D;
        yl[(row * VCH_NCOL + v) * VCH_DPAD + c] = src[e];
      }
    }
    __syncthreads();
    T s[KEOPS_TILE_J];
#pragma unroll
    for (int jj = 0; jj < KEOPS_TILE_J; jj++) s[jj] = (T)0;
    T yj0[KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1] = {};
    // whole groups of VCH_VEC components, in order (a sequential sum, as the reference's)
    for (int k0 = 0; k0 + VCH_VEC <= VCH_D; k0 += VCH_VEC) {
      T xk[NR][VCH_VEC];
#pragma unroll
      for (int v = 0; v < VCH_NROW; v++)
#pragma unroll
        for (int c = 0; c < VCH_VEC; c++) xk[v][c] = xlong[v][k0 + c];
#pragma unroll
      for (int jj = 0; jj < KEOPS_TILE_J; jj++) {
        T yk[NC][VCH_VEC];
#pragma unroll
        for (int v = 0; v < VCH_NCOL; v++) {
          const vch_vec w = *reinterpret_cast<const vch_vec*>(yl + (jj * VCH_NCOL + v) * VCH_DPAD + k0);
#pragma unroll
          for (int c = 0; c < VCH_VEC; c++) yk[v][c] = w[c];
        }
#if VCH_USES_YJ
        T yj[KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1];
        keops_read_col(ys, jj, yj);
#else
        const T (&yj)[KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1] = yj0;
#endif
#pragma unroll
        for (int c = 0; c < VCH_VEC; c++) {
          T xc[NR], yc[NC];
#pragma unroll
          for (int v = 0; v < NR; v++) xc[v] = xk[v][c];
#pragma unroll
          for (int v = 0; v < NC; v++) yc[v] = yk[v][c];
#if VCH_FMA
          T fb;
          const T fa = KeopsChunkFormula::eval(xc, yc, xi[0], yj, p, fb);
          s[jj] = keops_fma(fa, fb, s[jj]);  // the reference's scalar-product chain (Scalprod.py:32-36)
#else
          s[jj] = s[jj] + KeopsChunkFormula::eval(xc, yc, xi[0], yj, p);
#endif
        }
      }
    }
    // the last VCH_D % VCH_VEC components
    if (VCH_D % VCH_VEC != 0) {
      constexpr int k0 = VCH_D / VCH_VEC * VCH_VEC;
#pragma unroll
      for (int jj = 0; jj < KEOPS_TILE_J; jj++) {
#if VCH_USES_YJ
        T yj[KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1];
        keops_read_col(ys, jj, yj);
#else
        const T (&yj)[KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1] = yj0;
#endif
#pragma unroll
        for (int c = 0; c < VCH_D % VCH_VEC; c++) {
          T xc[NR] = {}, yc[NC] = {};
#pragma unroll
          for (int v = 0; v < VCH_NROW; v++) xc[v] = xlong[v][k0 + c];
#pragma unroll
          for (int v = 0; v < VCH_NCOL; v++) yc[v] = yl[(jj * VCH_NCOL + v) * VCH_DPAD + k0 + c];
#if VCH_FMA
          T fb;
          const T fa = KeopsChunkFormula::eval(xc, yc, xi[0], yj, p, fb);
          s[jj] = keops_fma(fa, fb, s[jj]);  // the reference's scalar-product chain (Scalprod.py:32-36)
#else
          s[jj] = s[jj] + KeopsChunkFormula::eval(xc, yc, xi[0], yj, p);
#endif
        }
      }
    }
#if KEOPS_USE_TILE_TMP
    KeopsAcc<T> tmp;
    tmp.init();
#endif
#pragma unroll
    for (int jj = 0; jj < KEOPS_TILE_J; jj++) {
      if (jj < n) {
        T yj[KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1];
        keops_read_col(ys, jj, yj);
        T fout[KEOPS_DIMFOUT];
        KeopsFormula::eval(xi[0], yj, p, s[jj], fout);
#if KEOPS_USE_TILE_TMP
        tmp.push(fout, j0 + jj - jshift);
#else
        acc[0].push(fout, j0 + jj - jshift);
#endif
      }
    }
#if KEOPS_USE_TILE_TMP
    acc[0].merge(tmp);
#endif
  }
}
#define KEOPS_SWEEP_EXTRA , yl, xlong
#else
#define KEOPS_SWEEP_EXTRA
// ---- the pair loop over one contiguous column range ----------------------------------------

// Folds columns [jbeg, jend) into acc[].  jshift is subtracted from the column index handed to
// index-carrying reductions (batch mode reports batch-relative indices).
__device__ __forceinline__ void keops_sweep(const KeopsParams& P, const i64* coloff, i64 jbeg, i64 jend, i64 jshift,
                                            const T (&xi)[KEOPS_ROWS][KEOPS_DIMX > 0 ? KEOPS_DIMX : 1],
                                            const T (&p)[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1],
                                            KeopsAcc<TACC> (&acc)[KEOPS_ROWS], T* ys) {
  for (i64 j0 = jbeg; j0 < jend; j0 += KEOPS_TILE_J) {
    const int n = (int)keops_min((i64)KEOPS_TILE_J, jend - j0);
    __syncthreads();  // the previous tile has been consumed by every wave
    keops_stage_tile(P, coloff, j0, n, ys);
    __syncthreads();
#if KEOPS_USE_TILE_TMP
    KeopsAcc<T> tmp[KEOPS_ROWS];
#pragma unroll
    for (int r = 0; r < KEOPS_ROWS; r++) tmp[r].init();
#endif
#if KEOPS_RED_KIND == 1 && KEOPS_SUM_SCHEME != 2
    // log-sum-exp: columns are folded KEOPS_LSE_GROUP at a time (one maximum update per group);
    // the last n % KEOPS_LSE_GROUP columns of a tile go one by one
    constexpr int G = KEOPS_LSE_GROUP;
    int jj0 = 0;
    for (; jj0 + G <= n; jj0 += G) {
      T yj[G][KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1];
#pragma unroll
      for (int g = 0; g < G; g++) keops_read_col(ys, jj0 + g, yj[g]);
#pragma unroll
      for (int r = 0; r < KEOPS_ROWS; r++) {
        T f[G][KEOPS_DIMFOUT];
#pragma unroll
        for (int g = 0; g < G; g++) KeopsFormula::eval(xi[r], yj[g], p, f[g]);
#if KEOPS_USE_TILE_TMP
        tmp[r].template push_group<G>(f);
#else
        acc[r].template push_group<G>(f);
#endif
      }
    }
    for (int jj = jj0; jj < n; jj++) {
      T yj[KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1];
      keops_read_col(ys, jj, yj);
#pragma unroll
      for (int r = 0; r < KEOPS_ROWS; r++) {
        T fout[KEOPS_DIMFOUT];
        KeopsFormula::eval(xi[r], yj, p, fout);
#if KEOPS_USE_TILE_TMP
        tmp[r].push(fout, 0);
#else
        acc[r].push(fout, 0);
#endif
      }
    }
#else
#pragma unroll KEOPS_UNROLL_J
    for (int jj = 0; jj < n; jj++) {
      T yj[KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1];
      keops_read_col(ys, jj, yj);
      const i64 jind = j0 + jj - jshift;
#pragma unroll
      for (int r = 0; r < KEOPS_ROWS; r++) {
        T fout[KEOPS_DIMFOUT];
        KeopsFormula::eval(xi[r], yj, p, fout);
#if KEOPS_USE_TILE_TMP
        tmp[r].push(fout, jind);
#else
        acc[r].push(fout, jind);
#endif
      }
    }
#endif
#if KEOPS_USE_TILE_TMP
#pragma unroll
    for (int r = 0; r < KEOPS_ROWS; r++) acc[r].merge(tmp[r]);
#endif
  }
}

#endif  // KEOPS_VCHUNK

// ---- dense scheme ---------------------------------------------------------------------------

extern "C" __global__ void __launch_bounds__(KEOPS_BLOCK) keops_conv_dense(const KeopsParams P) {
  if (P.guard != nullptr && *P.guard == 1u) return;
  __shared__ __attribute__((aligned(16))) T ys[KEOPS_TILE_J * (KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1)];
  const i64 zero_off[8 + KEOPS_NARGS] = {};
  const i64 row0 = (i64)blockIdx.x * KEOPS_ROWS_PER_BLOCK + threadIdx.x;

  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  keops_load_params(P, zero_off, p);
  T xi[KEOPS_ROWS][KEOPS_DIMX > 0 ? KEOPS_DIMX : 1];
  KeopsAcc<TACC> acc[KEOPS_ROWS];
#pragma unroll
  for (int r = 0; r < KEOPS_ROWS; r++) {
    const i64 i = row0 + (i64)r * KEOPS_BLOCK;
    keops_load_row(P, zero_off, i < P.nx ? i : P.nx - 1, xi[r]);  // clamped rows compute, never store
    acc[r].init();
  }

  const i64 jbeg = (i64)blockIdx.y * P.slab_len;
  const i64 jend = keops_min(P.ny, jbeg + P.slab_len);
#if KEOPS_VCHUNK
  __shared__ __attribute__((aligned(16))) T yl[KEOPS_TILE_J * (VCH_NCOL > 0 ? VCH_NCOL : 1) * VCH_DPAD];
  const T* xlong[VCH_NROW > 0 ? VCH_NROW : 1] = {};
#pragma unroll
  for (int v = 0; v < VCH_NROW; v++)
    xlong[v] = P.arg[keops_row_arg[keops_vch_row[v]]] + (row0 < P.nx ? row0 : P.nx - 1) * VCH_D;
#endif
  keops_sweep(P, zero_off, jbeg, jend, 0, xi, p, acc, ys KEOPS_SWEEP_EXTRA);

#pragma unroll
  for (int r = 0; r < KEOPS_ROWS; r++) {
    const i64 i = row0 + (i64)r * KEOPS_BLOCK;
    if (i < P.nx) {
      if (P.nslabs > 1)
        acc[r].store_partial(P.partial + ((i64)blockIdx.y * P.nx + i) * KEOPS_DIMRED);
      else
        acc[r].finalize(P.out + i * KEOPS_DIMOUT);
    }
  }
}

// Second pass of the slab scheme: merge the per-slab partial accumulators of every row in slab
// order (ReducePair) and finalize (GpuReduc2D.py:85-125).
extern "C" __global__ void __launch_bounds__(KEOPS_BLOCK) keops_reduce_partials(const KeopsParams P) {
  if (P.guard != nullptr && *P.guard == 1u) return;
  const i64 i = (i64)blockIdx.x * KEOPS_BLOCK + threadIdx.x;
  if (i >= P.nx) return;
  KeopsAcc<TACC> acc;
  acc.load_partial(P.partial + i * KEOPS_DIMRED);
  for (int s = 1; s < P.nslabs; s++) {
    KeopsAcc<TACC> o;
    o.load_partial(P.partial + ((i64)s * P.nx + i) * KEOPS_DIMRED);
    acc.merge(o);
  }
  acc.finalize(P.out + i * KEOPS_DIMOUT);
}

// Writes Finalize(Initialize()) to every output row: block-sparse launches call it first because
// the row ranges need not cover the output (the CPU reference does the same,
// keopscore/keopscore/mapreduce/cpu/CpuReduc_ranges.py:139-153).
extern "C" __global__ void __launch_bounds__(KEOPS_BLOCK) keops_fill_neutral(const KeopsParams P) {
  const i64 i = (i64)blockIdx.x * KEOPS_BLOCK + threadIdx.x;
  if (i >= P.nx) return;
  KeopsAcc<TACC> acc;
  acc.init();
  acc.finalize(P.out + i * KEOPS_DIMOUT);
}

// ---- block-sparse / batched scheme ----------------------------------------------------------

// One workgroup = up to KEOPS_ROWS_PER_BLOCK consecutive rows of one row range; it sweeps the
// column ranges [slices_x[r-1], slices_x[r]) of ranges_y, merging ranges that touch
// (GpuReduc1D_ranges.py:127-165).  With batch dimensions, rows and columns are addressed relative
// to per-variable offsets (broadcasting over batch dimensions, keops_nvrtc.cpp:75-149).
extern "C" __global__ void __launch_bounds__(KEOPS_BLOCK) keops_conv_ranges(const KeopsParams P) {
  if (P.guard != nullptr && *P.guard == 1u) return;
  __shared__ __attribute__((aligned(16))) T ys[KEOPS_TILE_J * (KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1)];
  constexpr int NV = KEOPS_NROWVARS + KEOPS_NCOLVARS + KEOPS_NPARVARS;
  i64 offs[NV > 0 ? NV : 1];
#pragma unroll
  for (int k = 0; k < NV; k++) offs[k] = P.nbatchdims > 0 ? P.offsets[(i64)NV * blockIdx.x + k] : 0;
  const i64* rowoff = offs;
  const i64* coloff = offs + KEOPS_NROWVARS;
  const i64* paroff = offs + KEOPS_NROWVARS + KEOPS_NCOLVARS;

  const i64 range_id = P.lookup[3 * (i64)blockIdx.x];
  const i64 start_x = P.lookup[3 * (i64)blockIdx.x + 1];
  const i64 end_x = P.lookup[3 * (i64)blockIdx.x + 2];
  if (end_x <= start_x) return;  // empty entry: tables built on the device round the grid up
  const i64 start_slice = range_id < 1 ? 0 : P.slices_x[range_id - 1];
  const i64 end_slice = P.slices_x[range_id];
  const bool batched = P.nbatchdims > 0;

  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  keops_load_params(P, paroff, p);
  T xi[KEOPS_ROWS][KEOPS_DIMX > 0 ? KEOPS_DIMX : 1];
  KeopsAcc<TACC> acc[KEOPS_ROWS];
#pragma unroll
  for (int r = 0; r < KEOPS_ROWS; r++) {
    i64 rel = (i64)threadIdx.x + (i64)r * KEOPS_BLOCK;  // row inside this block
    if (start_x + rel >= end_x) rel = end_x - start_x - 1;
    keops_load_row(P, rowoff, batched ? rel : start_x + rel, xi[r]);
    acc[r].init();
  }

#if KEOPS_VCHUNK
  __shared__ __attribute__((aligned(16))) T yl[KEOPS_TILE_J * (VCH_NCOL > 0 ? VCH_NCOL : 1) * VCH_DPAD];
  const T* xlong[VCH_NROW > 0 ? VCH_NROW : 1] = {};
  {
    i64 rel = (i64)threadIdx.x;
    if (start_x + rel >= end_x) rel = end_x - start_x - 1;
#pragma unroll
    for (int v = 0; v < VCH_NROW; v++)
      xlong[v] = P.arg[keops_row_arg[keops_vch_row[v]]] + (rowoff[keops_vch_row[v]] + (batched ? rel : start_x + rel)) * VCH_D;
  }
#endif
  if (start_slice < end_slice) {
    i64 start_y = P.ranges_y[2 * start_slice];
    for (i64 index = start_slice; index < end_slice; index++) {
      if (index + 1 >= end_slice || P.ranges_y[2 * index + 2] != P.ranges_y[2 * index + 1]) {
        const i64 end_y = P.ranges_y[2 * index + 1];
        // batch mode: variables are read at (offset + j - start_y) and indices are batch-relative
        if (batched)
          keops_sweep(P, coloff, 0, end_y - start_y, 0, xi, p, acc, ys KEOPS_SWEEP_EXTRA);
        else
          keops_sweep(P, coloff, start_y, end_y, 0, xi, p, acc, ys KEOPS_SWEEP_EXTRA);
        if (index + 1 < end_slice) start_y = P.ranges_y[2 * index + 2];
      }
    }
  }

#pragma unroll
  for (int r = 0; r < KEOPS_ROWS; r++) {
    const i64 i = start_x + threadIdx.x + (i64)r * KEOPS_BLOCK;
    if (i < end_x) acc[r].finalize(P.out + i * KEOPS_DIMOUT);
  }
}
