// High-dimensional map-reduce in double precision: the inner contraction runs on the float64 matrix instruction
// v_mfma_f64_16x16x4_f64, the rest of the formula and the reduction on the vector ALU.
//
// Counterpart, for KeOps_module<double> (keopscore/keopscore/binders/nvrtc/keops_nvrtc.cpp:646-648), of the chunked
// scheme keopscore/keopscore/mapreduce/gpu/GpuReduc1D_chunks.py:19-118: the chunked sub-formula
//     s_ij = SqDist(x_i, y_j) = |x_i|^2 + |y_j|^2 - 2 <x_i, y_j>      (CHK_MODE 0)
//     s_ij = <x_i, y_j>                                                (CHK_MODE 1)
// is produced for a 16 x 16 tile of pairs by CHK_DPAD / 4 matrix instructions, and the post-chunk formula
// F'(s_ij, other variables) is the generated straight-line code of KeopsFormula::eval.  The arithmetic is plain
// float64 (no operand splitting); for SqDist the rows are first centred on the column mean of y, which keeps the
// expansion well conditioned (error about 2^-52 (|x^|^2 + |y^|^2)), and values that are small compared with the norms
// (identical or neighbouring points) are recomputed from the differences.  On the vector ALU a squared distance costs
// a subtraction and a fused multiply-add per component; the matrix instruction does one multiply-add per component
// and keeps both operands in registers / LDS: about twice the vector rate at the same published peak.
//
// Register layout of the instruction (wavefront of 64 lanes, lane l): A[i = l % 16][k = l / 16], B[k = l / 16][j = l % 16],
// D[i = 4 v + l / 16][j = l % 16] for the lane's four accumulators v.  Here A rows are the staged reduced rows and B
// columns the output rows: lane l works for output row l % 16 of its block and, after the instructions of a
// sub-tile, holds s for the reduced rows 4 v + l / 16.  The four lanes of an output row merge their accumulators at
// the end in a fixed order (deterministic sums).
//
// Copies of the operands: rows are stored (centred, the row variable times -2 in CHK_MODE 0) with the components
// of every group of 8 permuted as [0, 4, 1, 5, 2, 6, 3, 7], so that the 16 bytes at position 2 g of the group hold the
// operands of lane group g = l / 16 for two consecutive instructions (components 8 p + g and 8 p + 4 + g).
//
// The plug-in defines: T = TACC = double, KEOPS_NARGS, CHK_D, CHK_DPAD (multiple of 8), CHK_MODE, CHK_XARG, CHK_YARG,
// CHK_WAVES, CHK_RB (blocks of 16 output rows per wavefront), the KEOPS_DIM* / KEOPS_RED_* / KEOPS_SUM_SCHEME macros,
// the row/col/par variable tables of the *other* variables, and KeopsFormula::eval(xi, yj, p, s, fout).
#pragma once
#include "keops_reductions.h"

typedef double c64_d4 __attribute__((ext_vector_type(4)));
typedef double c64_d2 __attribute__((ext_vector_type(2)));

#define C64_KP (CHK_DPAD / 8)                 // pairs of 4-wide k blocks: one 16-byte operand read each
#define C64_BLOCK (64 * CHK_WAVES)
#define C64_QB (16 * CHK_RB * CHK_WAVES)      // output rows per workgroup
#define C64_TJ 32                             // reduced rows per staged tile
#define C64_ROWBYTES (CHK_DPAD * 8)
#define C64_STRIDE (C64_ROWBYTES + 16)        // padded LDS row: the 16 rows a half-wavefront reads fall in distinct banks
#define C64_DY (KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1)
#ifndef C64_NEAR
#define C64_NEAR 0.0009765625                 // 2^-10: below this fraction of the norms a squared distance is recomputed
#endif

struct C64Params {
  i64 nx, ny;           // output rows, reduced rows
  double* xs;           // [nxs][CHK_DPAD] copies of the chunked row variable (see the head of this file)
  double* ys;           // [nys][CHK_DPAD]
  double* xn;           // [nxs] |x - mu|^2      (CHK_MODE 0)
  double* yn;           // [nys]
  double* colsum;       // [CHK_DPAD] column sums of y
  double* colpart;      // [nparts][CHK_DPAD]
  T* out;               // [nx][KEOPS_DIMOUT]
  i64 nxs, nys;         // rows of the chunked arguments (fewer than nx, ny when a batch dimension is broadcast)
  KeopsRangeTables rt;  // block-sparse / batch geometry (KEOPS_MC_RANGES)
  const T* arg[KEOPS_NARGS > 0 ? KEOPS_NARGS : 1];
};

// position of component k inside a stored row
__device__ __forceinline__ int c64_pos(int k) { return (k & ~7) + 2 * (k & 3) + ((k >> 2) & 1); }

// ---- pre-pass -----------------------------------------------------------------------------------

// column sums of y in two deterministic stages (no atomics: the same inputs always give the same centring)
extern "C" __global__ void __launch_bounds__(256) keops_c64_colsum(const C64Params P) {
  const i64 rows_per_block = (P.nys + gridDim.x - 1) / gridDim.x;
  const i64 r0 = (i64)blockIdx.x * rows_per_block, r1 = keops_min(P.nys, r0 + rows_per_block);
  const T* y = P.arg[CHK_YARG];
  for (int c = threadIdx.x; c < CHK_DPAD; c += 256) {
    double s = 0.0;
    if (c < CHK_D)
      for (i64 r = r0; r < r1; r++) s += y[r * CHK_D + c];
    P.colpart[(i64)blockIdx.x * CHK_DPAD + c] = s;
  }
}

extern "C" __global__ void __launch_bounds__(256) keops_c64_colsum_final(const C64Params P, int nparts) {
  for (int c = threadIdx.x; c < CHK_DPAD; c += 256) {
    double s = 0.0;
    for (int b = 0; b < nparts; b++) s += P.colpart[(i64)b * CHK_DPAD + c];
    P.colsum[c] = s;
  }
}

// One row per group of 8 lanes, 8 components per lane and pass; which = 0: row variable (stored times -2 in
// CHK_MODE 0), 1: column variable.  The squared norm is reduced inside the lane group (deterministic).
extern "C" __global__ void __launch_bounds__(256) keops_c64_prep(const C64Params P, int which) {
  const i64 n = which ? P.nys : P.nxs;
  const T* src = P.arg[which ? CHK_YARG : CHK_XARG];
  double* dst = which ? P.ys : P.xs;
  const int q = threadIdx.x % 8;
  const i64 row = ((i64)blockIdx.x * 256 + threadIdx.x) / 8;
  const bool live = row < n;
  const double inv = 1.0 / (double)P.nys;
  const double scale = (CHK_MODE == 0 && !which) ? -2.0 : 1.0;
  double nrm = 0.0;
  for (int c0 = q * 8; c0 < CHK_DPAD && live; c0 += 64) {
    double v[8];
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int c = c0 + e;
      double t = 0.0;
      if (c < CHK_D) {
        t = src[row * CHK_D + c];
        if (CHK_MODE == 0) t -= P.colsum[c] * inv;
      }
      nrm += t * t;
      v[e] = t * scale;
    }
#pragma unroll
    for (int e = 0; e < 8; e++) dst[row * CHK_DPAD + c0 + 2 * (e & 3) + (e >> 2)] = v[e];
  }
#pragma unroll
  for (int o = 4; o > 0; o >>= 1) nrm += __shfl_xor(nrm, o, 8);
  if (CHK_MODE == 0 && live && q == 0) (which ? P.yn : P.xn)[row] = nrm;
}

// ---- main kernel --------------------------------------------------------------------------------

extern "C" __global__ void __launch_bounds__(C64_BLOCK) keops_c64_main(const C64Params P) {
  // staged tile; after the sweep the same memory holds the accumulators that the four lanes of a row merge
  constexpr int TILE_BYTES = C64_TJ * C64_STRIDE;
  constexpr int MERGE_BYTES = (int)sizeof(TACC) * C64_QB * 3 * KEOPS_DIMRED;
  __shared__ __attribute__((aligned(16))) unsigned char as[TILE_BYTES > MERGE_BYTES ? TILE_BYTES : MERGE_BYTES];
  __shared__ __attribute__((aligned(16))) double yn_s[C64_TJ];
  __shared__ __attribute__((aligned(16))) T yo_s[C64_TJ * C64_DY];  // other column variables
  TACC (*merge_s)[3][KEOPS_DIMRED] = reinterpret_cast<TACC (*)[3][KEOPS_DIMRED]>(as);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, col = lane & 15;
  KeopsTileGeom G;
  G.init(P.rt, P.nx, C64_QB);
  if (G.row_first >= G.row_end) return;  // empty entry: tables built on the device round the grid up
  const i64 row0 = G.row_first + (i64)wave * (16 * CHK_RB);  // first output row of this wavefront
  const bool wave_live = row0 < G.row_end;                   // a wavefront without rows only helps staging the tiles

  // B operands: rows of the chunked row variable, CHK_RB blocks of 16
  c64_d2 bx[CHK_RB][C64_KP];
  i64 qrow[CHK_RB], qx[CHK_RB];
  bool valid[CHK_RB];
  double xnq[CHK_RB];
  T xi[CHK_RB][KEOPS_DIMX > 0 ? KEOPS_DIMX : 1];
  KeopsAcc<TACC> acc[CHK_RB];
#pragma unroll
  for (int rb = 0; rb < CHK_RB; rb++) {
    i64 q = row0 + rb * 16 + col;
    valid[rb] = q < G.row_end;
    if (!valid[rb]) q = G.row_end - 1;  // clamped rows compute, never store
    qrow[rb] = q;
    qx[rb] = G.row(CHK_XARG, q);
#pragma unroll
    for (int p = 0; p < C64_KP; p++) bx[rb][p] = *reinterpret_cast<const c64_d2*>(P.xs + qx[rb] * CHK_DPAD + p * 8 + 2 * g);
    xnq[rb] = CHK_MODE == 0 ? P.xn[qx[rb]] : 0.0;
#pragma unroll
    for (int v = 0; v < KEOPS_NROWVARS; v++) {
      const T* src = P.arg[keops_row_arg[v]] + G.row(keops_row_arg[v], q) * keops_row_dim[v];
#pragma unroll
      for (int d = 0; d < keops_row_dim[v]; d++) xi[rb][keops_row_off[v] + d] = src[d];
    }
    acc[rb].init();
  }
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
#pragma unroll
  for (int v = 0; v < KEOPS_NPARVARS; v++) {
    const T* src = P.arg[keops_par_arg[v]] + G.par(keops_par_arg[v]) * keops_par_dim[v];
#pragma unroll
    for (int d = 0; d < keops_par_dim[v]; d++) p[keops_par_off[v] + d] = src[d];
  }

  // software pipeline: tile t+1 travels to registers while tile t is consumed
  constexpr int CH = C64_ROWBYTES / 16;
  constexpr int NPF = (C64_TJ * CH + C64_BLOCK - 1) / C64_BLOCK;
  uint4 pf[NPF];
  double pfn = 0.0;
  auto prefetch = [&](i64 j0, i64 jend) {
    const int n = (int)keops_min((i64)C64_TJ, jend - j0);
    const i64 jy = G.col(CHK_YARG, j0);
    const uint4* src = reinterpret_cast<const uint4*>(P.ys + jy * CHK_DPAD);
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * C64_BLOCK;
      pf[u] = (e < n * CH) ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
    if (CHK_MODE == 0) pfn = (tid < n) ? P.yn[jy + tid] : 0.0;
  };
  const T* xorig = P.arg[CHK_XARG];
  const T* yorig = P.arg[CHK_YARG];
  // folds the reduced rows [jbeg, jend) into the accumulators
  i64 jbeg, jend;
#if KEOPS_MC_RANGES
  G.rewind(P.rt);
  while (G.next(P.rt, jbeg, jend)) {
#else
  jbeg = 0;
  jend = P.ny;
  {
#endif
  if (jbeg < jend) prefetch(jbeg, jend);
  for (i64 j0 = jbeg; j0 < jend; j0 += C64_TJ) {
    const int n = (int)keops_min((i64)C64_TJ, jend - j0);
    __syncthreads();
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * C64_BLOCK;
      if (e < C64_TJ * CH) {
        const int row = e / CH, c = e - row * CH;
        *reinterpret_cast<uint4*>(as + row * C64_STRIDE + c * 16) = pf[u];
      }
    }
    if (CHK_MODE == 0 && tid < C64_TJ) yn_s[tid] = pfn;
    // the other reduced-index variables of this tile (small: loaded directly)
#pragma unroll
    for (int v = 0; v < KEOPS_NCOLVARS; v++) {
      const int dim = keops_col_dim[v];
      const T* src = P.arg[keops_col_arg[v]] + G.col(keops_col_arg[v], j0) * dim;
      for (int e = tid; e < n * dim; e += C64_BLOCK) {
        const int row = e / dim, c = e - row * dim;
        yo_s[row * C64_DY + keops_col_off[v] + c] = src[e];
      }
    }
    __syncthreads();
    if (j0 + C64_TJ < jend) prefetch(j0 + C64_TJ, jend);
    const i64 jy0 = G.col(CHK_YARG, j0);
    if (!wave_live) continue;

    const int nsub = (n + 15) / 16;
    for (int sub = 0; sub < nsub; sub++) {
      // accumulator v of this lane is reduced row 4 v + g of the sub-tile: start from the norms of those rows
      c64_d4 s[CHK_RB];
#pragma unroll
      for (int rb = 0; rb < CHK_RB; rb++)
#pragma unroll
        for (int v = 0; v < 4; v++) s[rb][v] = CHK_MODE == 0 ? yn_s[sub * 16 + 4 * v + g] : 0.0;
      const unsigned char* arow = as + (sub * 16 + col) * C64_STRIDE + 16 * g;
#pragma unroll
      for (int pp = 0; pp < C64_KP; pp++) {
        const c64_d2 a = *reinterpret_cast<const c64_d2*>(arow + pp * 64);
#pragma unroll
        for (int rb = 0; rb < CHK_RB; rb++) {
          s[rb] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[0], bx[rb][pp][0], s[rb], 0, 0, 0);
          s[rb] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[1], bx[rb][pp][1], s[rb], 0, 0, 0);
        }
      }
#pragma unroll
      for (int rb = 0; rb < CHK_RB; rb++) {
#if KEOPS_USE_TILE_TMP
        KeopsAcc<T> tmp;
        tmp.init();
#endif
#pragma unroll
        for (int v = 0; v < 4; v++) {
          const int r = sub * 16 + 4 * v + g;
          if (r < n) {
            double sv = s[rb][v];
            if (CHK_MODE == 0) {
              sv = __builtin_fmax(sv + xnq[rb], 0.0);
              if (sv < C64_NEAR * (xnq[rb] + yn_s[r])) {
                // close compared with the norms: the expansion has lost its leading digits, take the differences
                const T* x = xorig + qx[rb] * CHK_D;
                const T* y = yorig + (jy0 + r) * CHK_D;
                double d = 0.0;
#pragma nounroll
                for (int k = 0; k < CHK_D; k++) {
                  const double t = x[k] - y[k];
                  d = __builtin_fma(t, t, d);
                }
                sv = d;
              }
            }
            T yj[C64_DY];
#pragma unroll
            for (int c = 0; c < KEOPS_DIMY_PAD; c++) yj[c] = yo_s[r * C64_DY + c];
            T fout[KEOPS_DIMFOUT];
            KeopsFormula::eval(xi[rb], yj, p, (T)sv, fout);
#if KEOPS_USE_TILE_TMP
            tmp.push(fout, j0 + r);
#else
            acc[rb].push(fout, j0 + r);
#endif
          }
        }
#if KEOPS_USE_TILE_TMP
        acc[rb].merge(tmp);
#endif
      }
    }
  }
  }

  // the four lanes of an output row merge their accumulators in a fixed order
  __syncthreads();
#pragma unroll
  for (int rb = 0; rb < CHK_RB; rb++) {
    const int slot = (wave * CHK_RB + rb) * 16 + col;
    if (g > 0) acc[rb].store_partial(merge_s[slot][g - 1]);
  }
  __syncthreads();
  if (g == 0) {
#pragma unroll
    for (int rb = 0; rb < CHK_RB; rb++) {
      const int slot = (wave * CHK_RB + rb) * 16 + col;
#pragma unroll
      for (int k = 0; k < 3; k++) {
        KeopsAcc<TACC> other;
        other.load_partial(merge_s[slot][k]);
        acc[rb].merge(other);
      }
      if (valid[rb] && wave_live) acc[rb].finalize(P.out + qrow[rb] * KEOPS_DIMOUT);
    }
  }
}

#if KEOPS_MC_RANGES
// rows that no range covers receive the neutral element of the reduction
extern "C" __global__ void __launch_bounds__(256) keops_c64_fill_neutral(const C64Params P) {
  const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
  if (i >= P.nx) return;
  KeopsAcc<TACC> acc;
  acc.init();
  acc.finalize(P.out + i * KEOPS_DIMOUT);
}
#endif
