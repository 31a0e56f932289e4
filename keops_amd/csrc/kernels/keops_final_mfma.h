// Sum reductions whose formula is a scalar kernel times a high-dimensional reduced-index variable,
//     out_i[0..DV) = sum_j f(x_i, y_j, p) * v_j[0..DV),
// i.e. a dense (M x N) by (N x DV) product whose left factor is generated on the fly.
//
// Counterpart of the reference's "final chunk" schemes
//   keopscore/keopscore/mapreduce/gpu/GpuReduc1D_finalchunks.py:19-69,72-225
// which evaluate f once per pair into shared memory and then stream 64-wide chunks of v_j through
// per-thread accumulators.  Here the product runs on the matrix cores in full float32:
//   * a wavefront owns 32 output rows; at every step lane l evaluates the scalar
//     f(x_{l%32}, y_{j0 + l/32}) -- this *is* the A operand layout of v_mfma_f32_32x32x2_f32 (row
//     l%32, k = l/32), so the 64 pair values of a step never leave their registers;
//   * the B operand of the same instruction is v[j0 + l/32][32 b + l%32], one conflict-free 4-byte
//     LDS read per lane and 32-column block b of the staged v tile;
//   * the 32 x 32 float32 accumulator tiles (one per column block, FIN_NB of them) stay in VGPRs
//     for the whole sweep; column blocks beyond FIN_NB are handled by further workgroups
//     (blockIdx.z), which re-evaluate f: it is cheap next to 2*DV flop per pair;
//   * block summation: every FIN_PERIOD reduced rows the register tiles are folded into the
//     output rows (owned by this workgroup, plain read-modify-write) and cleared, so rounding
//     errors do not grow with the number of reduced rows;
//   * few output rows: the reduced axis is cut in slabs (blockIdx.y) with one partial output per
//     slab, summed in slab order by keops_fin_reduce (deterministic);
//   * FIN_ACC64 (dtype_acc = float64, or the Kahan scheme, whose compensated float32 sum this replaces): the folds
//     and the slab sum run in double on a buffer of their own, with a short FIN_PERIOD, and keops_fin_reduce rounds
//     once to float32 (sum_schemes.py:44-71 with a double accumulator).
//
// The plug-in defines: T (float), TACC (float, double with FIN_ACC64), KEOPS_NARGS, FIN_DV, FIN_VARG, FIN_NB, FIN_WAVES, FIN_TJ,
// FIN_PERIOD, FIN_BLOCKSUM, the KEOPS_DIM* macros and row/col/par variable tables of the scalar
// kernel f, and KeopsFormula::eval(xi, yj, p, fout[1]).
#pragma once
#include "keops_common.h"
#ifndef FIN_ACC64
#define FIN_ACC64 0
#endif

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float fin_f32x16;

#define FIN_BLOCK (64 * FIN_WAVES)
#define FIN_QB (32 * FIN_WAVES)                    // output rows per workgroup
#define FIN_NBTOT ((FIN_DV + 31) / 32)             // 32-column blocks of v
#define FIN_VS (FIN_NB * 32)                       // floats per staged v row
#define FIN_DY (KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1)

struct FinParams {
  i64 nx, ny;
  T* out;          // [nx][FIN_DV]
  TACC* partial;   // [nslabs][nx][FIN_DV] when nslabs > 1, and always when the sums are kept in double (FIN_ACC64)
  i64 slab_len;    // reduced rows per slab (multiple of FIN_TJ)
  int nslabs;
  int pad_;
  __bf16* vsplit;       // keops_fin_split: v as three bfloat16 terms, [tile][term][column][row in tile]
  i64 vrows;            // rows of the array v (all batches)
  KeopsRangeTables rt;  // block-sparse / batch geometry (KEOPS_MC_RANGES)
  const T* arg[KEOPS_NARGS > 0 ? KEOPS_NARGS : 1];
};

extern "C" __global__ void __launch_bounds__(FIN_BLOCK) keops_fin_main(const FinParams P) {
  __shared__ __attribute__((aligned(16))) T vt[FIN_TJ * FIN_VS];   // v tile, this workgroup's column blocks
  __shared__ __attribute__((aligned(16))) T ys[FIN_TJ * FIN_DY];   // reduced-index variables of f

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  KeopsTileGeom G;
  G.init(P.rt, P.nx, FIN_QB);
  if (G.row_first >= G.row_end) return;  // empty entry: tables built on the device round the grid up
  const i64 row0 = G.row_first + wave * 32;  // first output row of this wavefront
  const bool wave_live = row0 < G.row_end;   // a wavefront without rows only helps staging the tiles
  i64 q = row0 + col;
  if (q >= G.row_end) q = G.row_end - 1;  // clamped rows compute, never store
  const int cb0 = blockIdx.z * FIN_NB;                      // first column block of this workgroup
  const int c0 = cb0 * 32;                                  // first column
  const int ncols = (int)keops_min((i64)FIN_VS, (i64)FIN_DV - c0);

  T xi[KEOPS_DIMX > 0 ? KEOPS_DIMX : 1];
#pragma unroll
  for (int v = 0; v < KEOPS_NROWVARS; v++) {
    const T* src = P.arg[keops_row_arg[v]] + G.row(keops_row_arg[v], q) * keops_row_dim[v];
#pragma unroll
    for (int d = 0; d < keops_row_dim[v]; d++) xi[keops_row_off[v] + d] = src[d];
  }
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
#pragma unroll
  for (int v = 0; v < KEOPS_NPARVARS; v++) {
    const T* src = P.arg[keops_par_arg[v]] + G.par(keops_par_arg[v]) * keops_par_dim[v];
#pragma unroll
    for (int d = 0; d < keops_par_dim[v]; d++) p[keops_par_off[v] + d] = src[d];
  }

  fin_f32x16 acc[FIN_NB];
#pragma unroll
  for (int b = 0; b < FIN_NB; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[b][r] = 0.f;

  TACC* dst = (P.nslabs > 1 || FIN_ACC64) ? P.partial + (i64)blockIdx.y * P.nx * FIN_DV : reinterpret_cast<TACC*>(P.out);
  bool first = true;
  // folds the register tiles into the output rows of this wavefront and clears them
  auto fold = [&]() {
    const i64 ibase = row0 + 4 * half;
    TACC* o = dst + ibase * FIN_DV + c0 + col;
    // folds are rare: keep their address arithmetic here instead of in registers across the sweep
    asm volatile("" : "+v"(o));
#pragma unroll
    for (int b = 0; b < FIN_NB; b++) {
      const int d = c0 + 32 * b + col;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ir = 8 * (r >> 2) + (r & 3);
        if (ibase + ir < G.row_end && d < FIN_DV) {
          TACC* oo = o + (i64)ir * FIN_DV + 32 * b;
          *oo = first ? (TACC)acc[b][r] : *oo + (TACC)acc[b][r];
        }
        acc[b][r] = 0.f;
      }
    }
    first = false;
  };

  const T* vsrc = P.arg[FIN_VARG];

  // software pipeline: the v rows of tile t+1 travel to registers while tile t is consumed
  constexpr int NPF = (FIN_TJ * FIN_VS + FIN_BLOCK - 1) / FIN_BLOCK;
  T pf[NPF];
  auto prefetch = [&](i64 j0, i64 jend) {
    const int n = (int)keops_min((i64)FIN_TJ, jend - j0);
    const i64 jv = G.col(FIN_VARG, j0);
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * FIN_BLOCK;
      const int row = e / FIN_VS, c = e - row * FIN_VS;
      pf[u] = (row < n && c < ncols) ? vsrc[(jv + row) * FIN_DV + c0 + c] : (T)0;  // zero rows/columns past the end
    }
  };
  int since_fold = 0;
  // folds the reduced rows [jbeg, jend) into the register tiles
  i64 jbeg, jend;
#if KEOPS_MC_RANGES
  G.rewind(P.rt);
  while (G.next(P.rt, jbeg, jend)) {
#else
  jbeg = (i64)blockIdx.y * P.slab_len;
  jend = keops_min(P.ny, ((i64)blockIdx.y + 1) * P.slab_len);
  {
#endif
  if (jbeg < jend) prefetch(jbeg, jend);
  for (i64 j0 = jbeg; j0 < jend; j0 += FIN_TJ) {
    const int n = (int)keops_min((i64)FIN_TJ, jend - j0);
    __syncthreads();  // the previous tile has been consumed by every wavefront
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * FIN_BLOCK;
      if (e < FIN_TJ * FIN_VS) vt[e] = pf[u];
    }
#pragma unroll
    for (int v = 0; v < KEOPS_NCOLVARS; v++) {
      const int dim = keops_col_dim[v];
      const T* src = P.arg[keops_col_arg[v]] + G.col(keops_col_arg[v], j0) * dim;
      for (int e = tid; e < n * dim; e += FIN_BLOCK) {
        const int row = e / dim, c = e - row * dim;
        ys[row * FIN_DY + keops_col_off[v] + c] = src[e];
      }
    }
    __syncthreads();
    if (j0 + FIN_TJ < jend) prefetch(j0 + FIN_TJ, jend);
    if (!wave_live) continue;

    // operands of step s+1 (pair value and v entries) are fetched while the MFMAs of step s execute
    auto operands = [&](int s, float& fv, float (&bv)[FIN_NB]) {
      const int jr = 2 * s + half;  // reduced row of this lane's pair
      const T* vrow = vt + jr * FIN_VS + col;
#pragma unroll
      for (int b = 0; b < FIN_NB; b++) bv[b] = vrow[32 * b];
      T yj[FIN_DY];
      constexpr int VEC = 4;
      typedef T vecT __attribute__((ext_vector_type(VEC)));
#pragma unroll
      for (int c4 = 0; c4 < KEOPS_DIMY_PAD / VEC; c4++) {
        const vecT w = *reinterpret_cast<const vecT*>(ys + jr * FIN_DY + c4 * VEC);
#pragma unroll
        for (int c = 0; c < VEC; c++) yj[c4 * VEC + c] = w[c];
      }
      T fout[1];
      KeopsFormula::eval(xi, yj, p, fout);
      fv = jr < n ? fout[0] : 0.f;  // select, never multiply: rows past the end hold garbage
    };
    float fcur, bcur[FIN_NB];
    operands(0, fcur, bcur);
#pragma unroll 2
    for (int s = 0; s < FIN_TJ / 2; s++) {
      float fnext = 0.f, bnext[FIN_NB];
      if (s + 1 < FIN_TJ / 2) operands(s + 1, fnext, bnext);
#pragma unroll
      for (int b = 0; b < FIN_NB; b++) acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(fcur, bcur[b], acc[b], 0, 0, 0);
      fcur = fnext;
#pragma unroll
      for (int b = 0; b < FIN_NB; b++) bcur[b] = bnext[b];
    }
#if FIN_BLOCKSUM
    since_fold += FIN_TJ;
    if (since_fold >= FIN_PERIOD) {
      fold();
      since_fold = 0;
    }
#endif
  }
  }
  fold();
}

// sums the per-slab partial outputs in slab order
extern "C" __global__ void __launch_bounds__(256) keops_fin_reduce(const FinParams P) {
  const i64 e = (i64)blockIdx.x * 256 + threadIdx.x;
  const i64 total = P.nx * FIN_DV;
  if (e >= total) return;
  TACC s = P.partial[e];
  for (int k = 1; k < P.nslabs; k++) s += P.partial[(i64)k * total + e];
  P.out[e] = (T)s;
}

#if KEOPS_MC_RANGES
// block-sparse mode: output rows that belong to no row range are zero
extern "C" __global__ void __launch_bounds__(256) keops_fin_fill_neutral(const FinParams P) {
  const i64 e = (i64)blockIdx.x * 256 + threadIdx.x;
  if (e < P.nx * FIN_DV) P.out[e] = (T)0;
}
#endif

// ---- the same product with every operand written as three bfloat16 terms ------------------------------
//
// x = h + m + l with h = bf16(x), m = bf16(x - h), l = bf16(x - h - m) carries the 24 significant bits of a
// float32, and f * v ~ hh + (hm + mh) + (hl + lh + mm) drops terms below 2^-24 |f v| only: float32 accuracy
// from six v_mfma_f32_32x32x16_bf16 (6 x 32 cycles per 32 x 32 x 16 block) where the float32 instruction
// v_mfma_f32_32x32x2_f32 needs 8 x 64 cycles.
//   * keops_fin_split writes v once as [tile][term][column][row in tile] bfloat16, zero past the last row and
//     column, so that a workgroup stages a tile with straight 16-byte copies; a tile is FIN_TJ consecutive rows of
//     the array v from a multiple of FIN_TJ on.  Block-sparse and batched launches (ranges start anywhere, a batch
//     moves its arguments) sweep the tiles that cover a range and give the rows outside it the pair value 0.  A lane
//     reads the 8 consecutive reduced rows of its B operand (column l % 32, rows 8 (l / 32) ..) with one
//     ds_read_b128 (columns padded to FIN_TS elements: conflict-free);
//   * lane l evaluates f for output row l % 32 and the 8 reduced rows 8 (l / 32) .. of a 16-row block -- the A
//     operand layout -- and splits the 8 values in registers.
// keops_fin_main above (float32 instruction) remains for modules built without FIN_SPLIT3.
#if defined(FIN_SPLIT3) && FIN_SPLIT3
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 fin_bf16x8;
#define FIN_TS (FIN_TJ + 8)            // bfloat16 elements per staged column (padded)
#define FIN_DVP (FIN_NBTOT * 32)       // columns of the split copy

extern "C" __global__ void __launch_bounds__(256) keops_fin_split(const FinParams P) {
  const i64 e = (i64)blockIdx.x * 256 + threadIdx.x;   // one (tile, column, row in tile)
  const i64 ntiles = (P.vrows + FIN_TJ - 1) / FIN_TJ;
  if (e >= ntiles * FIN_DVP * FIN_TJ) return;
  const int r = (int)(e % FIN_TJ);
  const int c = (int)((e / FIN_TJ) % FIN_DVP);
  const i64 tile = e / ((i64)FIN_TJ * FIN_DVP);
  const i64 j = tile * FIN_TJ + r;
  const float x = (j < P.vrows && c < FIN_DV) ? P.arg[FIN_VARG][j * FIN_DV + c] : 0.f;
  const __bf16 h = (__bf16)x;
  const float r1 = x - (float)h;
  const __bf16 m = (__bf16)r1;
  const __bf16 l = (__bf16)(r1 - (float)m);
  __bf16* dst = P.vsplit + (tile * 3 * FIN_DVP + c) * FIN_TJ + r;
  dst[0] = h;
  dst[(i64)FIN_DVP * FIN_TJ] = m;
  dst[(i64)2 * FIN_DVP * FIN_TJ] = l;
}

extern "C" __global__ void __launch_bounds__(FIN_BLOCK, 2) keops_fin_main3(const FinParams P) {
  // two copies of a tile, [term][column][row] of this workgroup's column blocks and the reduced-index variables of f:
  // a wavefront writes its share of the next tile while the others still read the current one
  __shared__ __attribute__((aligned(16))) __bf16 vt2[2][3 * FIN_VS * FIN_TS];
  __shared__ __attribute__((aligned(16))) T ys2[2][FIN_TJ * FIN_DY];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  KeopsTileGeom G;
  G.init(P.rt, P.nx, FIN_QB);
  if (G.row_first >= G.row_end) return;  // empty entry: tables built on the device round the grid up
  const i64 row0 = G.row_first + wave * 32;  // first output row of this wavefront
  const bool wave_live = row0 < G.row_end;   // a wavefront without rows only helps staging the tiles
  i64 q = row0 + col;
  if (q >= G.row_end) q = G.row_end - 1;     // clamped rows compute, never store
  const int cb0 = blockIdx.z * FIN_NB;
  const int c0 = cb0 * 32;

  T xi[KEOPS_DIMX > 0 ? KEOPS_DIMX : 1];
#pragma unroll
  for (int v = 0; v < KEOPS_NROWVARS; v++) {
    const T* src = P.arg[keops_row_arg[v]] + G.row(keops_row_arg[v], q) * keops_row_dim[v];
#pragma unroll
    for (int d = 0; d < keops_row_dim[v]; d++) xi[keops_row_off[v] + d] = src[d];
  }
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
#pragma unroll
  for (int v = 0; v < KEOPS_NPARVARS; v++) {
    const T* src = P.arg[keops_par_arg[v]] + G.par(keops_par_arg[v]) * keops_par_dim[v];
#pragma unroll
    for (int d = 0; d < keops_par_dim[v]; d++) p[keops_par_off[v] + d] = src[d];
  }

  fin_f32x16 acc[FIN_NB];
#pragma unroll
  for (int b = 0; b < FIN_NB; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[b][r] = 0.f;

  TACC* dst = (P.nslabs > 1 || FIN_ACC64) ? P.partial + (i64)blockIdx.y * P.nx * FIN_DV : reinterpret_cast<TACC*>(P.out);
  bool first = true;
  // folds the register tiles into the output rows of this wavefront and clears them
  auto fold = [&]() {
    const i64 ibase = row0 + 4 * half;
    TACC* o = dst + ibase * FIN_DV + c0 + col;
    asm volatile("" : "+v"(o));
#pragma unroll
    for (int b = 0; b < FIN_NB; b++) {
      const int d = c0 + 32 * b + col;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ir = 8 * (r >> 2) + (r & 3);
        if (ibase + ir < G.row_end && d < FIN_DV) {
          TACC* oo = o + (i64)ir * FIN_DV + 32 * b;
          *oo = first ? (TACC)acc[b][r] : *oo + (TACC)acc[b][r];
        }
        acc[b][r] = 0.f;
      }
    }
    first = false;
  };

  // a staged tile: per term FIN_VS columns of FIN_TJ rows, 16-byte chunks of the split copy
  constexpr int CPC = FIN_TJ / 8;                         // chunks per column
  constexpr int NCH = 3 * FIN_VS * CPC;                   // chunks per tile
  constexpr int NPF = (NCH + FIN_BLOCK - 1) / FIN_BLOCK;
  uint4 pf[NPF];
  auto prefetch = [&](i64 tile) {
    const uint4* base = reinterpret_cast<const uint4*>(P.vsplit + tile * 3 * FIN_DVP * FIN_TJ);
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * FIN_BLOCK;
      const int term = e / (FIN_VS * CPC), rest = e - term * (FIN_VS * CPC);
      const int c = rest / CPC, part = rest - c * CPC;
      // columns past the padded width of the split copy belong to no block of v
      pf[u] = (e < NCH && c0 + c < FIN_DVP) ? base[((i64)term * FIN_DVP + c0 + c) * CPC + part] : make_uint4(0u, 0u, 0u, 0u);
    }
  };
  auto store_tile = [&](__bf16* vt) {
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * FIN_BLOCK;
      if (e < NCH) {
        const int term = e / (FIN_VS * CPC), rest = e - term * (FIN_VS * CPC);
        const int c = rest / CPC, part = rest - c * CPC;
        *reinterpret_cast<uint4*>(vt + ((term * FIN_VS + c) * FIN_TS + part * 8)) = pf[u];
      }
    }
  };

  int since_fold = 0, cur = 0;
  // folds the reduced rows [jbeg, jend) into the register tiles
  i64 jbeg, jend;
#if KEOPS_MC_RANGES
  G.rewind(P.rt);
  while (G.next(P.rt, jbeg, jend)) {
#else
  jbeg = (i64)blockIdx.y * P.slab_len;
  jend = keops_min(P.ny, ((i64)blockIdx.y + 1) * P.slab_len);
  {
#endif
  // row of v that holds reduced row j: j + shift (a batch moves its arguments); tiles are counted along v
  const i64 shift = G.col(FIN_VARG, 0);
  i64 tile = (jbeg + shift) / FIN_TJ;
  const i64 tile_end = (jend + shift + FIN_TJ - 1) / FIN_TJ;
  if (tile < tile_end) prefetch(tile);
  for (; tile < tile_end; tile++) {
    const i64 j0 = tile * FIN_TJ - shift;  // reduced row of the tile's first row: before jbeg when the range starts inside
#if KEOPS_MC_RANGES
    const int lo = (int)keops_max((i64)0, jbeg - j0);
#else
    constexpr int lo = 0;                  // slabs start at multiples of FIN_TJ
#endif
    const int n = (int)keops_min((i64)FIN_TJ, jend - j0);
    // (the copy written here was last read two tiles ago, and every wavefront has passed the barrier of the
    // previous tile since)
    __bf16* vt = vt2[cur];
    T* ys = ys2[cur];
    cur ^= 1;
    store_tile(vt);
#pragma unroll
    for (int v = 0; v < KEOPS_NCOLVARS; v++) {
      const int dim = keops_col_dim[v];
      const T* src = P.arg[keops_col_arg[v]] + G.col(keops_col_arg[v], j0) * dim;  // rows [lo, n) of it exist
      for (int e = tid; e < n * dim; e += FIN_BLOCK) {
        const int row = e / dim, c = e - row * dim;
        if (row >= lo) ys[row * FIN_DY + keops_col_off[v] + c] = src[e];
      }
    }
    __syncthreads();
    if (tile + 1 < tile_end) prefetch(tile + 1);
    if (!wave_live) continue;

#pragma unroll
    for (int kb = 0; kb < FIN_TJ / 16; kb++) {
      // A operand: the pair values of output row `col` and the 8 reduced rows 16 kb + 8 half + e, in three terms
      fin_bf16x8 ah, am, al;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const int jr = 16 * kb + 8 * half + e;
        T yj[FIN_DY];
        constexpr int VEC = 4;
        typedef T vecT __attribute__((ext_vector_type(VEC)));
#pragma unroll
        for (int c4 = 0; c4 < KEOPS_DIMY_PAD / VEC; c4++) {
          const vecT w = *reinterpret_cast<const vecT*>(ys + jr * FIN_DY + c4 * VEC);
#pragma unroll
          for (int c = 0; c < VEC; c++) yj[c4 * VEC + c] = w[c];
        }
        T fout[1];
        KeopsFormula::eval(xi, yj, p, fout);
        // select, never multiply: rows outside the range hold garbage
        const float f = (jr >= lo && jr < n) ? fout[0] : 0.f;
        const __bf16 h = (__bf16)f;
        const float r1 = f - (float)h;
        const __bf16 m = (__bf16)r1;
        ah[e] = h;
        am[e] = m;
        al[e] = (__bf16)(r1 - (float)m);
      }
      const __bf16* brow = vt + col * FIN_TS + 16 * kb + 8 * half;
#pragma unroll
      for (int b = 0; b < FIN_NB; b++) {
        const fin_bf16x8 bh = *reinterpret_cast<const fin_bf16x8*>(brow + (0 * FIN_VS + 32 * b) * FIN_TS);
        const fin_bf16x8 bm = *reinterpret_cast<const fin_bf16x8*>(brow + (1 * FIN_VS + 32 * b) * FIN_TS);
        const fin_bf16x8 bl = *reinterpret_cast<const fin_bf16x8*>(brow + (2 * FIN_VS + 32 * b) * FIN_TS);
        // smallest terms first
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(am, bm, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bh, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bl, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(am, bh, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bm, acc[b], 0, 0, 0);
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh, acc[b], 0, 0, 0);
      }
    }
#if FIN_BLOCKSUM
    since_fold += FIN_TJ;
    if (since_fold >= FIN_PERIOD) {
      fold();
      since_fold = 0;
    }
#endif
  }
  }
  fold();
}
#endif
