// High-dimensional map-reduce: the inner contraction over a large vector dimension runs on the
// matrix cores, the rest of the formula and the reduction on the vector ALU.
//
// Counterpart of the reference's "chunked" schemes
//   keopscore/keopscore/mapreduce/gpu/GpuReduc1D_chunks.py:19-118,255-330
//   keopscore/keopscore/mapreduce/Chunk_Mode_Constants.py:6-140
// which cut a Sum / Scalprod over a dimension >= 146 into 64-wide chunks accumulated per thread in
// a local array, and then evaluate the "post-chunk" formula in which the chunked sub-formula has
// become a scalar variable.  Here the chunked sub-formula
//     s_ij = SqDist(x_i, y_j) = |x_i|^2 + |y_j|^2 - 2 <x_i, y_j>      (CHK_MODE 0)
//     s_ij = <x_i, y_j>                                                (CHK_MODE 1)
// is produced for a 32 x 32 tile of pairs by v_mfma_f32_32x32x16_f16, and the post-chunk formula
// F'(s_ij, other variables) is the generated straight-line code of KeopsFormula::eval.
//
// Precision: every float32 operand is split once as x = hi + lo with hi = half(a x), lo = half(a x - hi)
// (two 11-bit significands, 22 bits in total; a is a power of two chosen per launch from the largest
// component so that the terms sit high in the half-precision range: keops_chk_absmax, chk_pow2_scale) and
// <x, y> is accumulated in float32 from the three products hi*hi + hi*lo + lo*hi; the dropped lo*lo term and
// the split residuals are below 3 * 2^-22 |x||y| = 7.2e-7 |x||y|.  For SqDist the rows are first centred on the
// column mean of y, which keeps |x|^2 + |y|^2 - 2<x,y> well conditioned: the squared distance is off by at
// most 7.2e-7 (|x^|^2 + |y^|^2), the order of what the float32 sum of D squared differences of the reference
// itself carries (sqrt(D) 2^-24 s).  With use_fast_math=False the engine does not select this scheme.
//
// Work decomposition: a wavefront owns 32 output rows ("queries") whose split operands stay in
// VGPRs as the MFMA B matrix; the workgroup stages 32 reduced rows at a time in LDS (A matrix plus
// the other reduced-index variables of the formula).  After the MFMAs lane l holds, for output row
// l % 32, the 16 values s of reduced rows 8*(v/4) + 4*(l/32) + v%4; it evaluates the formula and
// folds them in its private accumulator; the two lanes of a row merge their accumulators at the end
// (ReducePair), so sums are deterministic.
//
// When the post-chunk formula of a Sum reduction is itself "scalar times reduced-index variable",
//     F'(s, ...) = g(s, ...) * v_j,
// (CHK_FINAL, kernel keops_chk_final) the weighted accumulation also runs on the matrix cores, in
// float32: register v of the s tile, once mapped through g, is the A operand of
// v_mfma_f32_32x32x2_f32 (output row l % 32, k = l / 32 <-> reduced rows r_v and r_v + 4) and
// v_j[r][32 b + l % 32] its B operand, one 4-byte LDS read per lane instead of dim(v) wave-wide
// broadcast reads.  The 32 x 32 float32 output tiles stay in registers, are folded into the output
// rows every CHK_PERIOD reduced rows (block summation) and the reduced axis can be cut in slabs
// summed in order by keops_chk_reduce.
//
// The plug-in defines: T (float), TACC, KEOPS_NARGS, CHK_D, CHK_DPAD, CHK_MODE, CHK_XARG, CHK_YARG,
// CHK_WAVES, the KEOPS_DIM* / KEOPS_RED_* / KEOPS_SUM_SCHEME macros, the row/col/par variable
// tables of the *other* variables, and KeopsFormula::eval(xi, yj, p, s, fout); with CHK_FINAL also
// CHK_FV_ARG, CHK_FV_DIM (argument index and dimension of v), CHK_FNB (32-column blocks),
// CHK_PERIOD, CHK_BLOCKSUM, and eval returns the scalar g in fout[0].
#pragma once
#include "keops_reductions.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 chk_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 chk_bf16x4;
typedef _Float16 chk_half;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 chk_h8;
typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 chk_h4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float chk_f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float chk_f32x4;

#ifndef CHK_NC
#define CHK_NC 1                             // wavefronts that share 32 output rows and split the contraction
#endif
#define CHK_BLOCK (64 * CHK_WAVES)
#define CHK_QB (32 * CHK_WAVES / CHK_NC)     // output rows per workgroup
#define CHK_KB (CHK_DPAD / 16)
#define CHK_KBC (CHK_KB / CHK_NC)            // 16-wide k blocks per wavefront
#define CHK_VS (16 / CHK_NC)                 // values of a 32 x 32 tile each lane evaluates
// CHK_SINGLE: the data are half-precision numbers (use_half launches: float32 copies of float16 arrays).  Their
// products are exact in float32, so one term per operand is enough: no lo parts, one matrix instruction per k block
// instead of three, and no centring (which would leave values that one half-precision number cannot hold).
#ifndef CHK_SINGLE
#define CHK_SINGLE 0
#endif
#define CHK_RW (CHK_DPAD * (CHK_SINGLE ? 1 : 2))  // half-precision elements per stored row: [hi] or [hi | lo]
#define CHK_ROWBYTES (CHK_RW * 2)
#define CHK_STRIDE (CHK_ROWBYTES + 16)       // padded LDS row
#define CHK_TJ 32                            // reduced rows per staged tile
#define CHK_DY (KEOPS_DIMY_PAD > 0 ? KEOPS_DIMY_PAD : 1)

struct ChkParams {
  i64 nx, ny;           // output rows, reduced rows
  chk_half* xs;         // [nx][2*CHK_DPAD] split (and centred, scaled) rows of the chunked row variable
  chk_half* ys;         // [ny][2*CHK_DPAD]
  float* xn;            // [nx] |x - mu|^2      (CHK_MODE 0)
  float* yn;            // [ny]
  float* colsum;        // [CHK_DPAD]
  float* colpart;       // [nparts][CHK_DPAD] partial column sums
  T* out;               // [nx][KEOPS_DIMOUT]
  T* partial;           // keops_chk_final: [nslabs][nx][KEOPS_DIMOUT] when nslabs > 1
  i64 slab_len;         // keops_chk_final: reduced rows per slab (multiple of CHK_TJ)
  int nslabs;
  int pad_;
  i64 nxs, nys;         // rows of the chunked row / column arguments (fewer than nx, ny when a batch dimension is broadcast)
  __bf16* vsplit;       // CHK_SPLIT3: v as three bfloat16 terms, [tile][term][column][CHK_TS positions]
  float* scal;          // [2] bound of the |components| of the chunked row / column arguments that sets their scale (keops_chk_absmax,
                        // keops_chk_robust), then at byte 16 int[2][256]: rows per exponent of their largest component
  KeopsRangeTables rt;  // block-sparse / batch geometry (KEOPS_MC_RANGES)
  const T* arg[KEOPS_NARGS > 0 ? KEOPS_NARGS : 1];
};

// ---- pre-pass -----------------------------------------------------------------------------------

// Column sums of the chunked column variable in two deterministic stages: per-workgroup partial
// sums, then one workgroup adds the partials in a fixed order (no atomics: the same inputs always
// give the same centring, hence bit-identical results from call to call).
#define CHK_CW (CHK_D > 128 ? 256 : (CHK_D > 64 ? 128 : (CHK_D > 32 ? 64 : 32)))
extern "C" __global__ void __launch_bounds__(256) keops_chk_colsum(const ChkParams P) {
  // lanes run along the columns (coalesced rows), 256 / CHK_CW row groups per block
  __shared__ float part[256];
  constexpr int RG = 256 / CHK_CW;
  const int cw = threadIdx.x % CHK_CW, rg = threadIdx.x / CHK_CW;
  const i64 rows_per_block = (P.nys + gridDim.x - 1) / gridDim.x;
  const i64 r0 = (i64)blockIdx.x * rows_per_block, r1 = keops_min(P.nys, r0 + rows_per_block);
  const T* y = P.arg[CHK_YARG];
  for (int c0 = 0; c0 < CHK_DPAD; c0 += CHK_CW) {  // every workgroup: all columns of its own rows
    const int c = c0 + cw;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (c < CHK_D) {
      i64 r = r0 + rg;
      for (; r + 3 * RG < r1; r += 4 * RG) {
        s0 += (float)y[r * CHK_D + c];
        s1 += (float)y[(r + RG) * CHK_D + c];
        s2 += (float)y[(r + 2 * RG) * CHK_D + c];
        s3 += (float)y[(r + 3 * RG) * CHK_D + c];
      }
      for (; r < r1; r += RG) s0 += (float)y[r * CHK_D + c];
    }
    part[threadIdx.x] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (rg == 0 && c < CHK_DPAD) {
      float s = 0.f;
#pragma unroll
      for (int g = 0; g < RG; g++) s += part[g * CHK_CW + cw];
      P.colpart[(i64)blockIdx.x * CHK_DPAD + c] = s;
    }
    __syncthreads();
  }
}

extern "C" __global__ void __launch_bounds__(256) keops_chk_colsum_final(const ChkParams P, int nparts) {
  __shared__ float part[256];
  constexpr int RG = 256 / CHK_CW;
  const int cw = threadIdx.x % CHK_CW, rg = threadIdx.x / CHK_CW;
  for (int c0 = blockIdx.x * CHK_CW; c0 < CHK_DPAD; c0 += gridDim.x * CHK_CW) {  // one group of columns per workgroup
    const int c = c0 + cw;
    // eight interleaved partial sums, added in a fixed order: the loads of one thread do not wait for each other
    float s8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (c < CHK_DPAD) {
      int b = rg;
      for (; b + 7 * RG < nparts; b += 8 * RG) {
#pragma unroll
        for (int u = 0; u < 8; u++) s8[u] += P.colpart[(i64)(b + u * RG) * CHK_DPAD + c];
      }
      for (; b < nparts; b += RG) s8[0] += P.colpart[(i64)b * CHK_DPAD + c];
    }
    const float s = ((s8[0] + s8[1]) + (s8[2] + s8[3])) + ((s8[4] + s8[5]) + (s8[6] + s8[7]));
    part[threadIdx.x] = s;
    __syncthreads();
    if (rg == 0 && c < CHK_DPAD) {
      float t = 0.f;
#pragma unroll
      for (int g = 0; g < RG; g++) t += part[g * CHK_CW + cw];
      P.colsum[c] = t;
    }
    __syncthreads();
  }
}

// The rows are centred to keep the norms, hence the error of the expansion, small: any point inside the cloud will do,
// and the mean is not one when a few rows are far away (one component of 1e30 moves it by 1e30 / n: every centred row
// would then leave the half-precision range and be computed pair by pair).  keops_chk_centre takes, per component, the
// median and the quartiles of 1024 evenly spaced rows of the column variable (bitonic sort in LDS, values that are not
// finite last) and raises a flag (fourth word of P.scal) when the mean is further than four interquartile ranges from
// the median, or not a number; keops_chk_centre_apply then replaces every mean by the median.  Ordinary data keep their
// mean, bit for bit.  Row nparts of colpart holds the medians.
extern "C" __global__ void __launch_bounds__(256) keops_chk_centre(const ChkParams P, int nparts) {
  __shared__ float v[1024];
  __shared__ int nfin;
  const int c = blockIdx.x, tid = threadIdx.x;
  if (c >= CHK_D) return;
  if (tid == 0) nfin = 0;
  __syncthreads();
  const T* y = P.arg[CHK_YARG];
  const i64 ns = P.nys < 1024 ? P.nys : 1024, step = ns > 0 ? P.nys / ns : 1;
  int mine = 0;
#pragma unroll
  for (int t = 0; t < 4; t++) {
    const int k = tid + 256 * t;
    float a = __builtin_inff();
    if (k < ns) {
      const float w = (float)y[(i64)k * step * CHK_D + c];
      if (__builtin_fabsf(w) < __builtin_inff()) { a = w; mine++; }
    }
    v[k] = a;
  }
  atomicAdd(&nfin, mine);
  __syncthreads();
  for (int k = 2; k <= 1024; k <<= 1)
    for (int j = k >> 1; j > 0; j >>= 1) {
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const int i = tid + 256 * t, l = i ^ j;
        if (l > i) {
          const float a = v[i], b = v[l];
          const bool up = (i & k) == 0;
          if ((a > b) == up) { v[i] = b; v[l] = a; }
        }
      }
      __syncthreads();
    }
  if (tid == 0) {
    const int n = nfin;
    const float med = n > 0 ? v[(n - 1) / 2] : 0.f, iqr = n > 0 ? v[(3 * n) / 4 < n ? (3 * n) / 4 : n - 1] - v[n / 4] : 0.f;
    const float mean = P.colsum[c] / (float)P.nys;
    P.colpart[(i64)nparts * CHK_DPAD + c] = med;
    if (!(__builtin_fabsf(mean - med) <= 4.f * iqr + 1e-3f * __builtin_fabsf(med) + 1e-30f))
      atomicOr(reinterpret_cast<unsigned*>(P.scal) + 3, 1u);
  }
}

extern "C" __global__ void __launch_bounds__(256) keops_chk_centre_apply(const ChkParams P, int nparts) {
  if (reinterpret_cast<const unsigned*>(P.scal)[3] == 0u) return;
  for (int c = threadIdx.x; c < CHK_D; c += 256) P.colsum[c] = P.colpart[(i64)nparts * CHK_DPAD + c] * (float)P.nys;
}

// Largest |component| of the two chunked arguments: atomic maximum on the bit patterns of non-negative floats
// (order-independent, hence deterministic).  The host zeroes P.scal before the launch.
extern "C" __global__ void __launch_bounds__(256) keops_chk_absmax(const ChkParams P) {
  const T* x = P.arg[CHK_XARG];
  const T* y = P.arg[CHK_YARG];
  const i64 nxe = P.nxs * CHK_D, nye = P.nys * CHK_D, step = (i64)gridDim.x * 256;
  float mx = 0.f, my = 0.f;
  for (i64 e = (i64)blockIdx.x * 256 + threadIdx.x; e < nxe; e += step) mx = __builtin_fmaxf(mx, __builtin_fabsf((float)x[e]));
  for (i64 e = (i64)blockIdx.x * 256 + threadIdx.x; e < nye; e += step) my = __builtin_fmaxf(my, __builtin_fabsf((float)y[e]));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mx = __builtin_fmaxf(mx, __shfl_xor(mx, o));
    my = __builtin_fmaxf(my, __shfl_xor(my, o));
  }
  if ((threadIdx.x & 63) == 0) {
    atomicMax(reinterpret_cast<unsigned*>(P.scal), __float_as_uint(mx));
    atomicMax(reinterpret_cast<unsigned*>(P.scal) + 1, __float_as_uint(my));
  }
}

// Outliers.  One scale per operand means that a single row with a component 2^k times the others' costs every other
// row k bits, and one component of 1e30 (or an infinite one) leaves nothing of them.  For squared distances (CHK_MODE 0,
// where single pairs can be recomputed from the float32 rows, chk_fix_near) the scale is therefore taken from the bulk
// of the rows when the largest component is far beyond it: keops_chk_rowhist counts the rows by the exponent of their
// largest component (integer atomics: the counts do not depend on the order), keops_chk_robust finds the exponent E
// below which all but max(4, n / 1024) rows lie and, when the largest component exceeds 64 * 2^(E+1), replaces the bound
// by 8 * 2^(E+1).  Rows that then leave the half-precision range get a NaN norm from keops_chk_prep, which sends every
// pair they take part in through chk_fix_near: they cost D operations per pair, the other rows keep their accuracy.
// Data without such rows (largest component within 64 times the bulk's) are scaled exactly as before.
#ifndef CHK_ROBUST
#define CHK_ROBUST 1
#endif
#define CHK_HIST(scal) (reinterpret_cast<int*>(scal) + 4)
extern "C" __global__ void __launch_bounds__(256) keops_chk_rowhist(const ChkParams P, int which) {
  __shared__ int h[256];
  h[threadIdx.x] = 0;
  __syncthreads();
  const i64 n = which ? P.nys : P.nxs;
  const T* src = P.arg[which ? CHK_YARG : CHK_XARG];
  // one row per group of 8 lanes
  const int q = threadIdx.x & 7;
  for (i64 row = ((i64)blockIdx.x * 256 + threadIdx.x) >> 3; row < n; row += (i64)gridDim.x * 32) {
    float m = 0.f;
    bool odd = false;  // NaN or infinite
    for (int c = q; c < CHK_D; c += 8) {
      const float a = __builtin_fabsf((float)src[row * CHK_D + c]);
      odd |= !(a < __builtin_inff());
      m = __builtin_fmaxf(m, a);
    }
    unsigned key = odd ? 255u : ((__float_as_uint(m) >> 23) & 0xffu);
#pragma unroll
    for (int o = 4; o > 0; o >>= 1) {
      const unsigned other = (unsigned)__shfl_xor((int)key, o, 8);
      key = other > key ? other : key;
    }
    if (q == 0) atomicAdd(&h[key], 1);
  }
  __syncthreads();
  if (h[threadIdx.x] != 0) atomicAdd(CHK_HIST(P.scal) + which * 256 + threadIdx.x, h[threadIdx.x]);
}

extern "C" __global__ void __launch_bounds__(64) keops_chk_robust(const ChkParams P) {
  if (threadIdx.x >= 2) return;
  const int which = threadIdx.x;
  const i64 n = which ? P.nys : P.nxs;
  const int* h = CHK_HIST(P.scal) + which * 256;
  i64 budget = n / 1024 > 4 ? n / 1024 : 4;
  if (budget > n / 2) budget = n / 2;
  i64 cum = 0;
  int E = 255;
  for (int e = 0; e < 256; e++) {
    cum += h[e];
    if (cum >= n - budget) { E = e; break; }
  }
  if (E >= 254 - 7) return;  // the bulk itself is huge or not finite: nothing to protect
  const float bulk = __uint_as_float((unsigned)(E + 1) << 23);  // every row but the budget has components below this
  const float top = P.scal[which];
  // Squared distances: rows that leave the half-precision range are computed pair by pair, so the scale can follow
  // the bulk closely.  Scalar products have no such path: there the scale only lets go of the largest component when
  // it is 2^20 times the bulk's (the other rows would keep fewer than 17 bits), and rows up to that ratio stay
  // representable; beyond it a row overflows to infinity in its own results and leaves the others theirs.
  if (CHK_MODE == 0) {
    if (!(top <= 64.f * bulk)) P.scal[which] = 8.f * bulk;
  } else {
    if (!(top <= 1048576.f * bulk)) P.scal[which] = 131072.f * bulk;
  }
}

// Power of two that brings components bounded by B into [2^12, 2^13) (1 for B = 0, clamped to 2^+-60): the split
// terms then sit high in the half-precision range (lo terms stay normal down to components 2^-15 of the largest,
// below that they lose absolute accuracy 2^-25 against a largest component of 2^12) and nothing can overflow
// (|-2 a x| < 2^14, products < 2^27 per component, accumulated in float32).
__device__ __forceinline__ float chk_pow2_scale(float B) {
  const int e = (int)((__float_as_uint(B) >> 23) & 0xffu);
  if (e == 0 || e == 255) return 1.f;
  int t = 266 - e;  // 127 + 12 - (e - 127)
  t = t < 67 ? 67 : (t > 187 ? 187 : t);
  return __uint_as_float((unsigned)t << 23);
}
// scales of the row (which = 0) and column (1) operands.  Centred rows (CHK_MODE 0) are bounded by
// |x| + |mean y| <= max|x| + max|y| and |y| + |mean y| <= 2 max|y|.
__device__ __forceinline__ float chk_operand_scale(const float* scal, int which) {
  const float ax = scal[0], ay = scal[1];
  if (CHK_MODE == 0) return chk_pow2_scale(which ? 2.f * ay : ax + ay);
  return chk_pow2_scale(which ? ay : ax);
}

// One row per group of CHK_LPR lanes, 4 columns per lane and pass; which = 0: row variable (stored times -2
// in CHK_MODE 0), 1: column variable.  The squared norm is reduced inside the lane group
// (deterministic).
#define CHK_LPR (CHK_DPAD / 4 <= 4 ? 4 : (CHK_DPAD / 4 <= 8 ? 8 : (CHK_DPAD / 4 <= 16 ? 16 : (CHK_DPAD / 4 <= 32 ? 32 : 64))))
extern "C" __global__ void __launch_bounds__(256) keops_chk_prep(const ChkParams P, int which) {
  const i64 n = which ? P.nys : P.nxs;
  const T* src = P.arg[which ? CHK_YARG : CHK_XARG];
  chk_half* dst = which ? P.ys : P.xs;
  const int q = threadIdx.x % CHK_LPR;
  const i64 row = ((i64)blockIdx.x * 256 + threadIdx.x) / CHK_LPR;
  const bool live = row < n;
  const float inv = 1.0f / (float)P.nys;
  const float scale = ((CHK_MODE == 0 && !which) ? -2.0f : 1.0f) * chk_operand_scale(P.scal, which);
  float nrm = 0.f;
  bool over = false;
  for (int c0 = q * 4; c0 < CHK_DPAD && live; c0 += CHK_LPR * 4) {
    chk_h4 hi, lo;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int c = c0 + e;
      float v = 0.f;
      if (c < CHK_D) {
        v = src[row * CHK_D + c];
        if (CHK_MODE == 0 && !CHK_SINGLE) v -= P.colsum[c] * inv;
      }
      nrm += v * v;
      v *= scale;
      over |= !(__builtin_fabsf(v) < 65504.f);  // leaves the half-precision range (or is not a number)
      hi[e] = (_Float16)v;
      // (an infinite hi part has no remainder: infinity minus infinity would turn every product of the row into NaN)
      lo[e] = __builtin_fabsf((float)hi[e]) < __builtin_inff() ? (_Float16)(v - (float)hi[e]) : (_Float16)0.0f;
    }
    *reinterpret_cast<chk_h4*>(dst + row * CHK_RW + c0) = hi;
    if (!CHK_SINGLE) *reinterpret_cast<chk_h4*>(dst + row * CHK_RW + CHK_DPAD + c0) = lo;
  }
#pragma unroll
  for (int o = CHK_LPR / 2; o > 0; o >>= 1) nrm += __shfl_xor(nrm, o, CHK_LPR);
  // a row that does not fit the half-precision operand: its norm says so, and chk_fix_near computes its pairs from the
  // float32 rows
  int ov = over ? 1 : 0;
#pragma unroll
  for (int o = CHK_LPR / 2; o > 0; o >>= 1) ov |= __shfl_xor(ov, o, CHK_LPR);
  if (ov && CHK_ROBUST) nrm = __builtin_nanf("");
  if (CHK_MODE == 0 && live && q == 0) (which ? P.yn : P.xn)[row] = nrm;
}

// Squared distances come out of the expansion |x^|^2 + |y^|^2 - 2 <x^, y^> with 22-bit operands and float32
// accumulation: an absolute error of about 1.4e-7 (|x^|^2 + |y^|^2) (bound: 7.2e-7), harmless unless the pair is
// close compared with the norms (identical or neighbouring points, kernels narrower than the cloud), where it would
// be a large relative error.  A value below CHK_NEAR (1/4; 1/8 below 32 components) of the sum of the squared
// norms is therefore recomputed from the float32 rows: every squared distance is then good to a relative 6e-7, the
// order of the rounding of the reference's own float32 sum of D squared differences.  In high dimension random
// pairs never come that close, so the branch costs one compare; clustered data pay for their accuracy.
#ifndef CHK_NEAR
#define CHK_NEAR 0.125f
#endif
// near_bound: CHK_NEAR (xn + largest yn of the staged tile), the only test on the common path.
__device__ __forceinline__ float chk_near_bound(const float* yn_s, float xn, int col) {
  float m = yn_s[col];
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) m = __builtin_fmaxf(m, __shfl_xor(m, o));
  return CHK_NEAR * (xn + m);
}
// sv[u]: squared distance of this lane's output row to reduced row 8*(v/4) + 4*half + v%4 of the tile, v = v0 + u,
// from the expansion; entries that are small compared with the norms are replaced by the float32 value.
template <int NV>
__device__ __forceinline__ void chk_fix_near(const ChkParams& P, float (&sv)[NV], int v0, int half, int n, float xn,
                                             const float* yn_s, float near_bound, i64 ix, i64 jy0) {
  float m = sv[0];
#pragma unroll
  for (int u = 1; u < NV; u++) m = __builtin_fminf(m, sv[u]);
  // (comparisons written so that a NaN - a row that left the half-precision range, keops_chk_prep - takes the slow path)
#if CHK_ROBUST
  if (__builtin_expect(!keops_any(!(m >= near_bound)), 1)) return;
#else
  if (__builtin_expect(!keops_any(m < near_bound), 1)) return;
#endif
  unsigned mask = 0u;
#pragma unroll
  for (int u = 0; u < NV; u++) {
    const int v = v0 + u, r = 8 * (v >> 2) + 4 * half + (v & 3);
#if CHK_ROBUST
    if (r < n && !(sv[u] >= CHK_NEAR * (xn + yn_s[r]))) mask |= 1u << u;
#else
    if (r < n && sv[u] < CHK_NEAR * (xn + yn_s[r])) mask |= 1u << u;
#endif
  }
  const T* x = P.arg[CHK_XARG] + ix * CHK_D;
  while (mask != 0u) {
    const int u0 = __ffs(mask) - 1;
    mask &= mask - 1u;
    const int v = v0 + u0, r = 8 * (v >> 2) + 4 * half + (v & 3);
    const T* y = P.arg[CHK_YARG] + (jy0 + r) * CHK_D;
    float d = 0.f;
#pragma nounroll
    for (int k = 0; k < CHK_D; k++) {
      const float t = x[k] - y[k];
      d = __builtin_fmaf(t, t, d);
    }
#pragma unroll
    for (int u = 0; u < NV; u++) sv[u] = (u == u0) ? d : sv[u];
  }
}

// ---- main kernel --------------------------------------------------------------------------------

#if !(defined(CHK_FINAL) && CHK_FINAL) && !(defined(CHK_SOFTMAX) && CHK_SOFTMAX)
extern "C" __global__ void __launch_bounds__(CHK_BLOCK) keops_chk_main(const ChkParams P) {
  // A tile (hi|lo); after the sweep the same memory holds the accumulators that the lanes of a row merge
  constexpr int TILE_BYTES = CHK_TJ * CHK_STRIDE;
  constexpr int MERGE_BYTES = (int)sizeof(TACC) * CHK_QB * (2 * CHK_NC - 1) * KEOPS_DIMRED;
  __shared__ __attribute__((aligned(16))) unsigned char as[TILE_BYTES > MERGE_BYTES ? TILE_BYTES : MERGE_BYTES];
  __shared__ __attribute__((aligned(16))) float yn_s[CHK_TJ];
  __shared__ __attribute__((aligned(16))) float yns_s[CHK_TJ];  // the same norms times chk_sc: initial value of the s tile
  __shared__ __attribute__((aligned(16))) T yo_s[CHK_TJ * CHK_DY];                // other column variables
  TACC (*merge_s)[2 * CHK_NC - 1][KEOPS_DIMRED] = reinterpret_cast<TACC (*)[2 * CHK_NC - 1][KEOPS_DIMRED]>(as);
#if CHK_NC > 1
  __shared__ float xch[CHK_WAVES * 16 * 64];  // partial 32 x 32 tiles of the wavefronts that split the contraction
#endif

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  KeopsTileGeom G;
  G.init(P.rt, P.nx, CHK_QB);
  if (G.row_first >= G.row_end) return;  // empty entry: tables built on the device round the grid up
  // CHK_NC wavefronts share 32 output rows: wavefront `chunk` of group `grp` contracts k blocks
  // [chunk * CHK_KBC, (chunk + 1) * CHK_KBC) and evaluates values [chunk * CHK_VS, (chunk + 1) * CHK_VS) of each tile
  const int grp = wave / CHK_NC, chunk = wave % CHK_NC;
  const i64 row0 = G.row_first + grp * 32;   // first output row of this wavefront
  const bool wave_live = row0 < G.row_end;   // a wavefront without rows only helps staging the tiles
  i64 q = row0 + col;
  const bool valid = q < G.row_end;
  if (!valid) q = G.row_end - 1;
  const i64 qx = G.row(CHK_XARG, q);

  // B operands: split rows of the chunked row variable
  chk_h8 bh[CHK_KBC], bl[CHK_SINGLE ? 1 : CHK_KBC];
#pragma unroll
  for (int kb = 0; kb < CHK_KBC; kb++) {
    const int k0 = (chunk * CHK_KBC + kb) * 16 + 8 * half;
    bh[kb] = *reinterpret_cast<const chk_h8*>(P.xs + qx * CHK_RW + k0);
#if !CHK_SINGLE
    bl[kb] = *reinterpret_cast<const chk_h8*>(P.xs + qx * CHK_RW + CHK_DPAD + k0);
#endif
  }
  const float xnq = CHK_MODE == 0 ? P.xn[qx] : 0.f;
  // the tile comes out of the matrix cores times chk_sc (a power of two: the scales of the two operands)
  const float chk_sc = chk_operand_scale(P.scal, 0) * chk_operand_scale(P.scal, 1), chk_inv = 1.0f / chk_sc;
  // other row variables and parameters of the post-chunk formula
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
  KeopsAcc<TACC> acc;
  acc.init();
#if defined(CHK_KNN_K)
  // K-nearest-neighbour sweep: the 2 * CHK_NC lanes of an output row keep separate candidate lists.  The row's
  // KEOPS_RED_K-th smallest value overall cannot exceed the last entry of any of them, so the smallest of those last
  // entries (exchanged through tau_s once per tile; an older value is only looser) screens the candidates of all:
  // far fewer wave-wide list insertions than with each lane's own last entry.
  __shared__ float tau_s[CHK_WAVES][32];
  if (half == 0) tau_s[wave][col] = __builtin_huge_valf();
  float tau_row = __builtin_huge_valf();
#endif

  // software pipeline: tile t+1 travels to registers while tile t is consumed
  constexpr int CH = CHK_ROWBYTES / 16;
  constexpr int NPF = (CHK_TJ * CH + CHK_BLOCK - 1) / CHK_BLOCK;
  uint4 pf[NPF];
  float pfn = 0.f;
  auto prefetch = [&](i64 j0, i64 jend) {
    const int n = (int)keops_min((i64)CHK_TJ, jend - j0);
    const i64 jy = G.col(CHK_YARG, j0);
    const uint4* src = reinterpret_cast<const uint4*>(P.ys + jy * CHK_RW);
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * CHK_BLOCK;
      pf[u] = (e < n * CH) ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
    if (CHK_MODE == 0) pfn = (tid < n) ? P.yn[jy + tid] : 0.f;
  };
  // folds the reduced rows [jbeg, jend) into the accumulators
  i64 jbeg, jend;
#if KEOPS_MC_RANGES
  G.rewind(P.rt);
  while (G.next(P.rt, jbeg, jend)) {
#else
  // (the K-nearest-neighbour variant cuts the reduced axis in slabs, one list of candidates per slab)
  jbeg = (i64)blockIdx.y * P.slab_len;
  jend = keops_min(P.ny, jbeg + P.slab_len);
  {
#endif
  if (jbeg < jend) prefetch(jbeg, jend);
  for (i64 j0 = jbeg; j0 < jend; j0 += CHK_TJ) {
    const int n = (int)keops_min((i64)CHK_TJ, jend - j0);
    __syncthreads();
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * CHK_BLOCK;
      if (e < CHK_TJ * CH) {
        const int row = e / CH, c = e - row * CH;
        *reinterpret_cast<uint4*>(as + row * CHK_STRIDE + c * 16) = pf[u];
      }
    }
    if (CHK_MODE == 0 && tid < CHK_TJ) { yn_s[tid] = pfn; yns_s[tid] = pfn * chk_sc; }
    // the other reduced-index variables of this tile (small: loaded directly)
#pragma unroll
    for (int v = 0; v < KEOPS_NCOLVARS; v++) {
      const int dim = keops_col_dim[v];
      const T* src = P.arg[keops_col_arg[v]] + G.col(keops_col_arg[v], j0) * dim;
      for (int e = tid; e < n * dim; e += CHK_BLOCK) {
        const int row = e / dim, c = e - row * dim;
        yo_s[row * CHK_DY + keops_col_off[v] + c] = src[e];
      }
    }
    __syncthreads();
    if (j0 + CHK_TJ < jend) prefetch(j0 + CHK_TJ, jend);
    const float near_bound = CHK_MODE == 0 ? chk_near_bound(yn_s, xnq, col) : 0.f;
    const i64 jy0 = G.col(CHK_YARG, j0);
#if defined(CHK_KNN_K)
#pragma unroll
    for (int c = 0; c < CHK_NC; c++) tau_row = __builtin_fminf(tau_row, tau_s[grp * CHK_NC + c][col]);
#endif
#if CHK_NC == 1
    if (!wave_live) continue;

    // s tile: accumulator register v of this lane is reduced row 8*(v/4) + 4*half + v%4
    chk_f32x16 s;
    if (CHK_MODE == 0) {
      chk_f32x4 kk[4];
#pragma unroll
      for (int b = 0; b < 4; b++) kk[b] = *reinterpret_cast<const chk_f32x4*>(yns_s + 8 * b + 4 * half);
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] = kk[v >> 2][v & 3];
    } else {
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] = 0.f;
    }
    const unsigned char* arow = as + col * CHK_STRIDE + 16 * half;
#pragma unroll
    for (int kb = 0; kb < CHK_KB; kb++) {
      const chk_h8 ah = *reinterpret_cast<const chk_h8*>(arow + kb * 32);
#if !CHK_SINGLE
      const chk_h8 al = *reinterpret_cast<const chk_h8*>(arow + CHK_DPAD * 2 + kb * 32);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bh[kb], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bl[kb], s, 0, 0, 0);
#endif
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh[kb], s, 0, 0, 0);
    }
#else
    // partial tile of this wavefront's k blocks, handed to the group through LDS
    if (wave_live) {
      chk_f32x16 s;
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] = 0.f;
      const unsigned char* arow = as + col * CHK_STRIDE + 16 * half + chunk * CHK_KBC * 32;
#pragma unroll
      for (int kb = 0; kb < CHK_KBC; kb++) {
        const chk_h8 ah = *reinterpret_cast<const chk_h8*>(arow + kb * 32);
#if !CHK_SINGLE
        const chk_h8 al = *reinterpret_cast<const chk_h8*>(arow + CHK_DPAD * 2 + kb * 32);
        s = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bh[kb], s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bl[kb], s, 0, 0, 0);
#endif
        s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh[kb], s, 0, 0, 0);
      }
#pragma unroll
      for (int v = 0; v < 16; v++) xch[(wave * 16 + v) * 64 + lane] = s[v];
    }
    __syncthreads();
    if (!wave_live) continue;
    // this wavefront's share of the tile: partial sums added in chunk order (deterministic)
    float s[CHK_VS];
#pragma unroll
    for (int vv = 0; vv < CHK_VS; vv++) {
      const int v = chunk * CHK_VS + vv;
      float t = CHK_MODE == 0 ? yns_s[8 * (v >> 2) + 4 * half + (v & 3)] : 0.f;
#pragma unroll
      for (int c = 0; c < CHK_NC; c++) t += xch[((grp * CHK_NC + c) * 16 + v) * 64 + lane];
      s[vv] = t;
    }
#endif
#if KEOPS_USE_TILE_TMP
    KeopsAcc<T> tmp;
    tmp.init();
#endif
    float sq[CHK_VS];
#pragma unroll
    for (int vv = 0; vv < CHK_VS; vv++) sq[vv] = CHK_MODE == 0 ? __builtin_fmaxf(__builtin_fmaf(s[vv], chk_inv, xnq), 0.f) : s[vv] * chk_inv;
    if (CHK_MODE == 0) chk_fix_near<CHK_VS>(P, sq, chunk * CHK_VS, half, n, xnq, yn_s, near_bound, qx, jy0);
#pragma unroll
    for (int vv = 0; vv < CHK_VS; vv++) {
      const int v = chunk * CHK_VS + vv;
      const int r = 8 * (v >> 2) + 4 * half + (v & 3);
      if (r < n) {
        T sv = sq[vv];
        T yj[CHK_DY];
        constexpr int VEC = 16 / sizeof(T);
        typedef T vecT __attribute__((ext_vector_type(VEC)));
#pragma unroll
        for (int c4 = 0; c4 < KEOPS_DIMY_PAD / VEC; c4++) {
          const vecT w = *reinterpret_cast<const vecT*>(yo_s + r * CHK_DY + c4 * VEC);
#pragma unroll
          for (int c = 0; c < VEC; c++) yj[c4 * VEC + c] = w[c];
        }
        T fout[KEOPS_DIMFOUT];
        KeopsFormula::eval(xi, yj, p, sv, fout);
#if defined(CHK_KNN_K)
        if (fout[0] < tau_row) acc.push(fout, j0 + r);
#elif KEOPS_USE_TILE_TMP
        tmp.push(fout, j0 + r);
#else
        acc.push(fout, j0 + r);
#endif
      }
    }
#if KEOPS_USE_TILE_TMP && !defined(CHK_KNN_K)
    acc.merge(tmp);
#endif
#if defined(CHK_KNN_K)
    {
      // last entry of this lane's list and of the partner lane (the other 16 reduced rows of the tile)
      float mine = (float)acc.v[0][KEOPS_RED_K - 1];
      mine = __builtin_fminf(mine, __shfl_xor(mine, 32));
      tau_row = __builtin_fminf(tau_row, mine);
      if (half == 0) tau_s[wave][col] = mine;
    }
#endif
  }
  }

  // the 2 * CHK_NC lanes of an output row merge their accumulators in a fixed order
  __syncthreads();
  const int part = chunk * 2 + half;
  if (part > 0) acc.store_partial(merge_s[grp * 32 + col][part - 1]);
  __syncthreads();
  if (part == 0) {
#pragma unroll
    for (int k = 0; k < 2 * CHK_NC - 1; k++) {
      KeopsAcc<TACC> other;
      other.load_partial(merge_s[grp * 32 + col][k]);
      acc.merge(other);
    }
    if (valid) acc.finalize(P.out + ((i64)blockIdx.y * P.nx + q) * KEOPS_DIMOUT);
  }
}
#endif

// ---- K nearest neighbours in high dimension: exact re-rank of the lists of the sweep -----------------
//
// CHK_KNN_K: the module serves a KMin-family reduction of SqDist(x, y) with K = CHK_KNN_K.  keops_chk_main keeps the
// KEOPS_RED_K > K smallest *approximate* squared distances per row and column slab (split bfloat16 operands: |approx - d| <=
// CHK_KNN_C (|x^|^2 + |y^|^2) for the centred rows x^, y^) in the reference's (value, index) list layout.  Here
// one lane per row computes the float32 distances of its candidates in the reference's operation order (sequential
// sum of squared differences, no fused multiply-add), sorts them under (distance, index) and writes the K best.
// The result is certified when every reference left out of the list is provably farther than the K-th neighbour:
// (a_last - eps) (1 - 1e-4) > d_K with a_last the largest approximate distance kept and eps the bound above at the
// largest |y^|^2; rows that fail the test are counted and the caller recomputes the call on the exact kernel.
#if defined(CHK_KNN_K)
#define CHK_KNN_C 2.0e-4f
struct ChkKnnExtra {
  const float* lists;  // [nslabs][nx][2 * KEOPS_RED_K] approximate (value, index) pairs of the sweep
  T* out;              // [nx][CHK_KNN_DIMOUT]
  int* flag;           // flag[0]: rows that are not certified; flag[1] (as float): max_j |y^_j|^2
};

extern "C" __global__ void __launch_bounds__(256) keops_chk_knn_ymax(const ChkParams P, const ChkKnnExtra E) {
  __shared__ float red[256];
  float m = 0.f;
  for (i64 j = threadIdx.x; j < P.ny; j += 256) m = __builtin_fmaxf(m, P.yn[j]);
  red[threadIdx.x] = m;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) red[threadIdx.x] = __builtin_fmaxf(red[threadIdx.x], red[threadIdx.x + o]);
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    E.flag[0] = 0;
    reinterpret_cast<float*>(E.flag)[1] = red[0];
  }
}

// One wavefront per row; lane c re-examines candidate c % KEOPS_RED_K of slab c / KEOPS_RED_K (the launcher keeps
// nslabs * KEOPS_RED_K <= 64), ranks are counted across the lanes under (distance, index, lane).
extern "C" __global__ void __launch_bounds__(256) keops_chk_knn_rerank(const ChkParams P, const ChkKnnExtra E) {
  const int lane = threadIdx.x & 63;
  const i64 q = (i64)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (q >= P.nx) return;
  const float inf = __builtin_huge_valf();
  const int ncand = P.nslabs * KEOPS_RED_K;
  const int slab = lane / KEOPS_RED_K, entry = lane - slab * KEOPS_RED_K;
  const T* xq = P.arg[CHK_XARG] + q * CHK_D;
  float a = inf, d = inf;
  int j = 0x7fffffff;
  if (lane < ncand) {
    const float* L = E.lists + ((i64)slab * P.nx + q) * 2 * KEOPS_RED_K;
    a = L[2 * entry];
    if (a < inf) {
      j = (int)L[2 * entry + 1];
      const T* yr = P.arg[CHK_YARG] + (i64)j * CHK_D;
      float t = 0.f;
      {
#pragma clang fp contract(off)
        for (int k = 0; k < CHK_D; k++) {
          const float u = xq[k] - yr[k];
          t = t + u * u;
        }
      }
      d = t;
    }
  }
  // what was left out of slab s has an approximate distance >= the last entry of its list (inf: nothing left out)
  float a_last = (lane < ncand && entry == KEOPS_RED_K - 1) ? a : inf;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) a_last = __builtin_fminf(a_last, __shfl_xor(a_last, o));
  int rank = 0;
  for (int c = 0; c < ncand; c++) {
    const float dc = __shfl(d, c);
    const int jc = __shfl(j, c);
    rank += (dc < d || (dc == d && (jc < j || (jc == j && c < lane)))) ? 1 : 0;
  }
  T* o = E.out + q * CHK_KNN_DIMOUT;
  if (lane < ncand && rank < CHK_KNN_K) {
    const T jv = d < inf ? (T)j : (T)0;
    if (CHK_KNN_KEEP == 0) {
      o[2 * rank] = d;
      o[2 * rank + 1] = jv;
    } else {
      o[rank] = CHK_KNN_KEEP == 1 ? (T)d : jv;
    }
  }
  // K-th exact distance: held by the lane of rank K - 1
  float dk = (lane < ncand && rank == CHK_KNN_K - 1) ? d : -inf;
#pragma unroll
  for (int o2 = 32; o2 > 0; o2 >>= 1) dk = __builtin_fmaxf(dk, __shfl_xor(dk, o2));
  if (lane == 0 && a_last < inf) {
    const float eps = CHK_KNN_C * (P.xn[q] + reinterpret_cast<const float*>(E.flag)[1]);
    if (!((a_last - eps) * (1.0f - 1.0e-4f) > dk)) atomicAdd(E.flag, 1);
  }
}
#endif

// ---- weighted sums with every operand in three bfloat16 terms ----------------------------------------
//
// Dense launches of the two variants below (CHK_SPLIT3).  x = h + m + l with h = bf16(x), m = bf16(x - h),
// l = bf16(x - h - m) carries the 24 significant bits of a float32 and w * v ~ hh + (hm + mh) + (hl + lh + mm)
// drops terms below 2^-24 |w v| only: float32 accuracy from six v_mfma_f32_32x32x16_bf16 (6 x 32 cycles per
// 32 x 32 x 16 block) where v_mfma_f32_32x32x2_f32 needs 8 x 64.  The pair weights sit in the accumulator layout
// of the s tile (register v of lane l: reduced row 8 (v/4) + 4 (l/32) + v%4 of output row l % 32); registers
// 8 kb .. 8 kb + 7 are the A operand of k block kb when the contraction index runs over the reduced rows in the
// order 16 kb + {0,1,2,3,8,9,10,11} for lanes 0-31 and 16 kb + {4,..,7,12,..,15} for lanes 32-63, so
// keops_chk_split stores v with its rows in that order: row r of a 32-row tile at position
// 16 (r/16) + 8 ((r>>2)&1) + 4 ((r>>3)&1) + r%4 of [tile][term][column][CHK_TS], and a lane reads the 8 rows of
// its B operand with one ds_read_b128 (CHK_TS = 40 elements per column: conflict-free).
#if defined(CHK_SPLIT3) && CHK_SPLIT3
#define CHK_V3 1
#ifndef CHK_PRESPLIT
#define CHK_PRESPLIT 1
#endif
#define CHK_V3_PRESPLIT (CHK_PRESPLIT && !KEOPS_MC_RANGES)  // block-sparse / batched launches split the tile while staging it
#define CHK_TS 40
#define CHK_VCOLS (CHK_FNB * 32)

#if CHK_V3_PRESPLIT
extern "C" __global__ void __launch_bounds__(256) keops_chk_split(const ChkParams P) {
  const i64 e = (i64)blockIdx.x * 256 + threadIdx.x;   // one (tile, column, row in tile)
  const i64 ntiles = (P.ny + CHK_TJ - 1) / CHK_TJ;
  if (e >= ntiles * CHK_VCOLS * CHK_TJ) return;
  const int r = (int)(e % CHK_TJ);
  const int c = (int)((e / CHK_TJ) % CHK_VCOLS);
  const i64 tile = e / ((i64)CHK_TJ * CHK_VCOLS);
  const i64 j = tile * CHK_TJ + r;
  const float x = (j < P.ny && c < CHK_FV_DIM) ? P.arg[CHK_FV_ARG][j * CHK_FV_DIM + c] : 0.f;
  const __bf16 h = (__bf16)x;
  const float r1 = x - (float)h;
  const __bf16 m = (__bf16)r1;
  const __bf16 l = (__bf16)(r1 - (float)m);
  const int pos = 16 * (r >> 4) + 8 * ((r >> 2) & 1) + 4 * ((r >> 3) & 1) + (r & 3);
  __bf16* dst = P.vsplit + (tile * 3 * CHK_VCOLS + c) * CHK_TS + pos;
  dst[0] = h;
  dst[(i64)CHK_VCOLS * CHK_TS] = m;
  dst[(i64)2 * CHK_VCOLS * CHK_TS] = l;
}

// 16-byte chunks of one staged tile and their prefetch registers
#define CHK_V3_CHUNKS (3 * CHK_VCOLS * CHK_TS / 8)
#define CHK_V3_NPF ((CHK_V3_CHUNKS + CHK_BLOCK - 1) / CHK_BLOCK)

__device__ __forceinline__ void chk_v3_prefetch(const ChkParams& P, i64 j0, int tid, uint4 (&pf)[CHK_V3_NPF]) {
  const uint4* base = reinterpret_cast<const uint4*>(P.vsplit + (j0 / CHK_TJ) * 3 * CHK_VCOLS * CHK_TS);
#pragma unroll
  for (int u = 0; u < CHK_V3_NPF; u++) {
    const int e = tid + u * CHK_BLOCK;
    pf[u] = e < CHK_V3_CHUNKS ? base[e] : make_uint4(0u, 0u, 0u, 0u);
  }
}

__device__ __forceinline__ void chk_v3_store(__bf16* bt3, int tid, const uint4 (&pf)[CHK_V3_NPF]) {
#pragma unroll
  for (int u = 0; u < CHK_V3_NPF; u++) {
    const int e = tid + u * CHK_BLOCK;
    if (e < CHK_V3_CHUNKS) reinterpret_cast<uint4*>(bt3)[e] = pf[u];
  }
}
#endif

// Block-sparse and batched launches (reduced-index ranges start anywhere, no pre-split copy): the tile is split
// while it is staged.  A task is one column and the 8 reduced rows of one (k block, lane half) group, i.e. 8
// consecutive positions of the LDS layout: 8 coalesced float32 loads (prefetched one tile ahead), one
// ds_write_b128 per term.
#define CHK_V3_TASKS (CHK_VCOLS * 4)
#define CHK_V3_NT ((CHK_V3_TASKS + CHK_BLOCK - 1) / CHK_BLOCK)

__device__ __forceinline__ void chk_v3_gather(const T* vsrc, i64 jv, int n, int tid, float (&pfv)[CHK_V3_NT * 8]) {
#pragma unroll
  for (int u = 0; u < CHK_V3_NT; u++) {
    const int t = tid + u * CHK_BLOCK;
    const int c = t % CHK_VCOLS, g = t / CHK_VCOLS;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const int r = 16 * (g >> 1) + 4 * (g & 1) + (e < 4 ? e : e + 4);
      pfv[u * 8 + e] = (t < CHK_V3_TASKS && r < n && c < CHK_FV_DIM) ? vsrc[(jv + r) * CHK_FV_DIM + c] : 0.f;
    }
  }
}

__device__ __forceinline__ void chk_v3_scatter(__bf16* bt3, int tid, const float (&pfv)[CHK_V3_NT * 8]) {
#pragma unroll
  for (int u = 0; u < CHK_V3_NT; u++) {
    const int t = tid + u * CHK_BLOCK;
    if (t < CHK_V3_TASKS) {
      const int c = t % CHK_VCOLS, g = t / CHK_VCOLS;
      chk_bf16x8 h8, m8, l8;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float x = pfv[u * 8 + e];
        const __bf16 h = (__bf16)x;
        const float r1 = x - (float)h;
        const __bf16 m = (__bf16)r1;
        h8[e] = h;
        m8[e] = m;
        l8[e] = (__bf16)(r1 - (float)m);
      }
      __bf16* dst = bt3 + c * CHK_TS + 8 * g;
      *reinterpret_cast<chk_bf16x8*>(dst) = h8;
      *reinterpret_cast<chk_bf16x8*>(dst + CHK_VCOLS * CHK_TS) = m8;
      *reinterpret_cast<chk_bf16x8*>(dst + 2 * CHK_VCOLS * CHK_TS) = l8;
    }
  }
}

// acc[b] += W (32 output rows x 32 reduced rows, the 16 weights w of this lane) * v (staged terms bt3).
// CHK_WTERMS bfloat16 terms per weight: 3 (24 bits, six term products) or 2 (w = h + m with both terms rounded to
// nearest: |w - h - m| <= 2^-17 |w|, either sign; five term products, less vector work; not the float32 class).
#ifndef CHK_WTERMS
#define CHK_WTERMS 3
#endif
__device__ __forceinline__ void chk_v3_product(const float (&w)[16], const __bf16* bt3, int col, int half,
                                               chk_f32x16 (&acc)[CHK_FNB]) {
#pragma unroll
  for (int kb = 0; kb < 2; kb++) {
    chk_bf16x8 ah, am, al;
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float x = w[8 * kb + e];
      const __bf16 h = (__bf16)x;
      const float r1 = x - (float)h;
      const __bf16 m = (__bf16)r1;
      ah[e] = h;
      am[e] = m;
      if (CHK_WTERMS == 3) al[e] = (__bf16)(r1 - (float)m);
    }
    const __bf16* brow = bt3 + col * CHK_TS + 16 * kb + 8 * half;
#pragma unroll
    for (int b = 0; b < CHK_FNB; b++) {
      const chk_bf16x8 bh = *reinterpret_cast<const chk_bf16x8*>(brow + (0 * CHK_VCOLS + 32 * b) * CHK_TS);
      const chk_bf16x8 bm = *reinterpret_cast<const chk_bf16x8*>(brow + (1 * CHK_VCOLS + 32 * b) * CHK_TS);
      const chk_bf16x8 bl = *reinterpret_cast<const chk_bf16x8*>(brow + (2 * CHK_VCOLS + 32 * b) * CHK_TS);
      // smallest terms first
      acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(am, bm, acc[b], 0, 0, 0);
      if (CHK_WTERMS == 3) acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bh, acc[b], 0, 0, 0);
      acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bl, acc[b], 0, 0, 0);
      acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(am, bh, acc[b], 0, 0, 0);
      acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bm, acc[b], 0, 0, 0);
      acc[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah, bh, acc[b], 0, 0, 0);
    }
  }
}
#else
#define CHK_V3 0
#endif

// ---- variant with the final product on the matrix cores -------------------------------------------

#if defined(CHK_FINAL) && CHK_FINAL
#define CHK_FVS (CHK_FNB * 32)  // floats per staged v row (columns past CHK_FV_DIM are zero)

extern "C" __global__ void __launch_bounds__(CHK_BLOCK) keops_chk_final(const ChkParams P) {
  __shared__ __attribute__((aligned(16))) unsigned char as[CHK_TJ * CHK_STRIDE];  // A tile (hi|lo)
  __shared__ __attribute__((aligned(16))) float yn_s[CHK_TJ];
  __shared__ __attribute__((aligned(16))) float yns_s[CHK_TJ];  // the same norms times chk_sc: initial value of the s tile
  __shared__ __attribute__((aligned(16))) T yo_s[CHK_TJ * CHK_DY];                // other column variables of g
#if CHK_V3
  __shared__ __attribute__((aligned(16))) __bf16 bt3[3 * CHK_VCOLS * CHK_TS];       // v tile in three terms
#else
  __shared__ __attribute__((aligned(16))) T bt[CHK_TJ * CHK_FVS];                 // v tile
#endif

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  KeopsTileGeom G;
  G.init(P.rt, P.nx, CHK_QB);
  if (G.row_first >= G.row_end) return;  // empty entry: tables built on the device round the grid up
  const i64 row0 = G.row_first + wave * 32;  // first output row of this wavefront
  const bool wave_live = row0 < G.row_end;   // a wavefront without rows only helps staging the tiles
  i64 q = row0 + col;
  if (q >= G.row_end) q = G.row_end - 1;
  const i64 qx = G.row(CHK_XARG, q);  // clamped rows compute, never store

  chk_h8 bh[CHK_KB], bl[CHK_SINGLE ? 1 : CHK_KB];
#pragma unroll
  for (int kb = 0; kb < CHK_KB; kb++) {
    bh[kb] = *reinterpret_cast<const chk_h8*>(P.xs + qx * CHK_RW + kb * 16 + 8 * half);
#if !CHK_SINGLE
    bl[kb] = *reinterpret_cast<const chk_h8*>(P.xs + qx * CHK_RW + CHK_DPAD + kb * 16 + 8 * half);
#endif
  }
  const float xnq = CHK_MODE == 0 ? P.xn[qx] : 0.f;
  // the tile comes out of the matrix cores times chk_sc (a power of two: the scales of the two operands)
  const float chk_sc = chk_operand_scale(P.scal, 0) * chk_operand_scale(P.scal, 1), chk_inv = 1.0f / chk_sc;
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

  chk_f32x16 acc[CHK_FNB];
#pragma unroll
  for (int b = 0; b < CHK_FNB; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[b][r] = 0.f;

  T* dst = P.nslabs > 1 ? P.partial + (i64)blockIdx.y * P.nx * CHK_FV_DIM : P.out;
  bool first = true;
  // folds the register tiles into the output rows of this wavefront and clears them
  auto fold = [&]() {
    const i64 ibase = row0 + 4 * half;
    T* o = dst + ibase * CHK_FV_DIM + col;
    asm volatile("" : "+v"(o));  // folds are rare: keep their address arithmetic out of the sweep's registers
#pragma unroll
    for (int b = 0; b < CHK_FNB; b++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ir = 8 * (r >> 2) + (r & 3);
        if (ibase + ir < G.row_end && 32 * b + col < CHK_FV_DIM) {
          T* oo = o + (i64)ir * CHK_FV_DIM + 32 * b;
          *oo = first ? acc[b][r] : *oo + acc[b][r];
        }
        acc[b][r] = 0.f;
      }
    }
    first = false;
  };

  const T* vsrc = P.arg[CHK_FV_ARG];

  constexpr int CH = CHK_ROWBYTES / 16;
  constexpr int NPF = (CHK_TJ * CH + CHK_BLOCK - 1) / CHK_BLOCK;
  uint4 pf[NPF];
#if CHK_V3 && CHK_V3_PRESPLIT
  uint4 pf3[CHK_V3_NPF];
#elif CHK_V3
  float pfv[CHK_V3_NT * 8];
#else
  constexpr int NPV = (CHK_TJ * CHK_FVS + CHK_BLOCK - 1) / CHK_BLOCK;
  T pfv[NPV];
#endif
  float pfn = 0.f;
  auto prefetch = [&](i64 j0, i64 jend) {
    const int n = (int)keops_min((i64)CHK_TJ, jend - j0);
    const i64 jy = G.col(CHK_YARG, j0), jv = G.col(CHK_FV_ARG, j0);
    const uint4* src = reinterpret_cast<const uint4*>(P.ys + jy * CHK_RW);
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * CHK_BLOCK;
      pf[u] = (e < n * CH) ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
    if (CHK_MODE == 0) pfn = (tid < n) ? P.yn[jy + tid] : 0.f;
    // v tile, zero past the last row / column (the matrix product must not see stale values)
#if CHK_V3 && CHK_V3_PRESPLIT
    chk_v3_prefetch(P, j0, tid, pf3);
#elif CHK_V3
    chk_v3_gather(vsrc, jv, n, tid, pfv);
#else
#pragma unroll
    for (int u = 0; u < NPV; u++) {
      const int e = tid + u * CHK_BLOCK;
      const int row = e / CHK_FVS, c = e - row * CHK_FVS;
      pfv[u] = (row < n && c < CHK_FV_DIM) ? vsrc[(jv + row) * CHK_FV_DIM + c] : (T)0;
    }
#endif
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
  for (i64 j0 = jbeg; j0 < jend; j0 += CHK_TJ) {
    const int n = (int)keops_min((i64)CHK_TJ, jend - j0);
    __syncthreads();
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * CHK_BLOCK;
      if (e < CHK_TJ * CH) {
        const int row = e / CH, c = e - row * CH;
        *reinterpret_cast<uint4*>(as + row * CHK_STRIDE + c * 16) = pf[u];
      }
    }
    if (CHK_MODE == 0 && tid < CHK_TJ) { yn_s[tid] = pfn; yns_s[tid] = pfn * chk_sc; }
#pragma unroll
    for (int v = 0; v < KEOPS_NCOLVARS; v++) {
      const int dim = keops_col_dim[v];
      const T* src = P.arg[keops_col_arg[v]] + G.col(keops_col_arg[v], j0) * dim;
      for (int e = tid; e < n * dim; e += CHK_BLOCK) {
        const int row = e / dim, c = e - row * dim;
        yo_s[row * CHK_DY + keops_col_off[v] + c] = src[e];
      }
    }
#if CHK_V3 && CHK_V3_PRESPLIT
    chk_v3_store(bt3, tid, pf3);
#elif CHK_V3
    chk_v3_scatter(bt3, tid, pfv);
#else
#pragma unroll
    for (int u = 0; u < NPV; u++) {
      const int e = tid + u * CHK_BLOCK;
      if (e < CHK_TJ * CHK_FVS) bt[e] = pfv[u];
    }
#endif
    __syncthreads();
    if (j0 + CHK_TJ < jend) prefetch(j0 + CHK_TJ, jend);
    const float near_bound = CHK_MODE == 0 ? chk_near_bound(yn_s, xnq, col) : 0.f;
    const i64 jy0 = G.col(CHK_YARG, j0);
    if (!wave_live) continue;

    chk_f32x16 s;
    if (CHK_MODE == 0) {
      chk_f32x4 kk[4];
#pragma unroll
      for (int b = 0; b < 4; b++) kk[b] = *reinterpret_cast<const chk_f32x4*>(yns_s + 8 * b + 4 * half);
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] = kk[v >> 2][v & 3];
    } else {
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] = 0.f;
    }
    const unsigned char* arow = as + col * CHK_STRIDE + 16 * half;
#pragma unroll
    for (int kb = 0; kb < CHK_KB; kb++) {
      const chk_h8 ah = *reinterpret_cast<const chk_h8*>(arow + kb * 32);
#if !CHK_SINGLE
      const chk_h8 al = *reinterpret_cast<const chk_h8*>(arow + CHK_DPAD * 2 + kb * 32);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bh[kb], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bl[kb], s, 0, 0, 0);
#endif
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh[kb], s, 0, 0, 0);
    }
    float sq[16];
#pragma unroll
    for (int v = 0; v < 16; v++) sq[v] = CHK_MODE == 0 ? __builtin_fmaxf(__builtin_fmaf(s[v], chk_inv, xnq), 0.f) : s[v] * chk_inv;
    if (CHK_MODE == 0) chk_fix_near<16>(P, sq, 0, half, n, xnq, yn_s, near_bound, qx, jy0);
#if CHK_V3
    float gw[16];
#endif
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int r = 8 * (v >> 2) + 4 * half + (v & 3);
      T sv = sq[v];
      T yj[CHK_DY];
      constexpr int VEC = 16 / sizeof(T);
      typedef T vecT __attribute__((ext_vector_type(VEC)));
#pragma unroll
      for (int c4 = 0; c4 < KEOPS_DIMY_PAD / VEC; c4++) {
        const vecT w = *reinterpret_cast<const vecT*>(yo_s + r * CHK_DY + c4 * VEC);
#pragma unroll
        for (int c = 0; c < VEC; c++) yj[c4 * VEC + c] = w[c];
      }
      T fout[1];
      KeopsFormula::eval(xi, yj, p, sv, fout);
      const float g = r < n ? fout[0] : 0.f;  // select, never multiply: rows past the end hold garbage
#if CHK_V3
      gw[v] = g;
#else
#pragma unroll
      for (int b = 0; b < CHK_FNB; b++)
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(g, bt[r * CHK_FVS + 32 * b + col], acc[b], 0, 0, 0);
#endif
    }
#if CHK_V3
    chk_v3_product(gw, bt3, col, half, acc);
#endif
#if CHK_BLOCKSUM
    since_fold += CHK_TJ;
    if (since_fold >= CHK_PERIOD) {
      fold();
      since_fold = 0;
    }
#endif
  }
  }
  fold();
}

// sums the per-slab partial outputs in slab order
extern "C" __global__ void __launch_bounds__(256) keops_chk_reduce(const ChkParams P) {
  const i64 e = (i64)blockIdx.x * 256 + threadIdx.x;
  const i64 total = P.nx * CHK_FV_DIM;
  if (e >= total) return;
  T s = P.partial[e];
  for (int k = 1; k < P.nslabs; k++) s += P.partial[(i64)k * total + e];
  P.out[e] = s;
}
#endif

// ---- variant for softmax-weighted sums (online log-sum-exp with the weighted sum on the matrix cores) ----
//
// Max_SumShiftExpWeight reduction whose post-chunk formulas are F'(s, ...) (scalar) and a weight that is
// a plain reduced-index variable v_j, optionally preceded by a constant 1 (the SumSoftMaxWeight layout
// [1, v_j] of the Python layer):   m_i = max_j F'_ij,   l_i = sum_j exp(F'_ij - m_i),
// O_i = sum_j exp(F'_ij - m_i) v_j.  Per 32-row tile and wavefront: the running maximum of every output
// row moves up (tile maximum over the lane's 16 values and its partner lane), the 32 x 32 float32 output
// tiles and l are rescaled by exp(m_old - m_new) when any maximum of the wavefront moved (the factors
// travel through LDS to the accumulator layout), then p = exp(F' - m_new) is the A operand of
// v_mfma_f32_32x32x2_f32 against the staged v tile, exactly as in keops_chk_final.
#if defined(CHK_SOFTMAX) && CHK_SOFTMAX
#define CHK_SVS (CHK_FNB * 32)

extern "C" __global__ void __launch_bounds__(CHK_BLOCK) keops_chk_softmax(const ChkParams P) {
  __shared__ __attribute__((aligned(16))) unsigned char as[CHK_TJ * CHK_STRIDE];
  __shared__ __attribute__((aligned(16))) float yn_s[CHK_TJ];
  __shared__ __attribute__((aligned(16))) float yns_s[CHK_TJ];  // the same norms times chk_sc: initial value of the s tile
  __shared__ __attribute__((aligned(16))) T yo_s[CHK_TJ * CHK_DY];
#if CHK_V3
  __shared__ __attribute__((aligned(16))) __bf16 bt3[3 * CHK_VCOLS * CHK_TS];       // v tile in three terms
#else
  __shared__ __attribute__((aligned(16))) T bt[CHK_TJ * CHK_SVS];
#endif
  __shared__ __attribute__((aligned(16))) float al_s[CHK_WAVES][32];  // rescaling factors of a wavefront's rows

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  KeopsTileGeom G;
  G.init(P.rt, P.nx, CHK_QB);
  if (G.row_first >= G.row_end) return;  // empty entry: tables built on the device round the grid up
  const i64 row0 = G.row_first + wave * 32;  // first output row of this wavefront
  const bool wave_live = row0 < G.row_end;   // a wavefront without rows only helps staging the tiles
  i64 q = row0 + col;
  if (q >= G.row_end) q = G.row_end - 1;
  const i64 qx = G.row(CHK_XARG, q);

  chk_h8 bh[CHK_KB], bl[CHK_SINGLE ? 1 : CHK_KB];
#pragma unroll
  for (int kb = 0; kb < CHK_KB; kb++) {
    bh[kb] = *reinterpret_cast<const chk_h8*>(P.xs + qx * CHK_RW + kb * 16 + 8 * half);
#if !CHK_SINGLE
    bl[kb] = *reinterpret_cast<const chk_h8*>(P.xs + qx * CHK_RW + CHK_DPAD + kb * 16 + 8 * half);
#endif
  }
  const float xnq = CHK_MODE == 0 ? P.xn[qx] : 0.f;
  // the tile comes out of the matrix cores times chk_sc (a power of two: the scales of the two operands)
  const float chk_sc = chk_operand_scale(P.scal, 0) * chk_operand_scale(P.scal, 1), chk_inv = 1.0f / chk_sc;
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

  chk_f32x16 acc[CHK_FNB];
#pragma unroll
  for (int b = 0; b < CHK_FNB; b++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[b][r] = 0.f;
  const float ninf = -__builtin_huge_valf();
  float m_run = ninf;   // running maximum of output row `col` (identical in both halves)
  float l_run = 0.f;    // this lane's share of sum_j exp(F' - m_run)

  const T* vsrc = P.arg[CHK_FV_ARG];

  constexpr int CH = CHK_ROWBYTES / 16;
  constexpr int NPF = (CHK_TJ * CH + CHK_BLOCK - 1) / CHK_BLOCK;
  uint4 pf[NPF];
#if CHK_V3 && CHK_V3_PRESPLIT
  uint4 pf3[CHK_V3_NPF];
#elif CHK_V3
  float pfv[CHK_V3_NT * 8];
#else
  constexpr int NPV = (CHK_TJ * CHK_SVS + CHK_BLOCK - 1) / CHK_BLOCK;
  T pfv[NPV];
#endif
  float pfn = 0.f;
  auto prefetch = [&](i64 j0, i64 jend) {
    const int n = (int)keops_min((i64)CHK_TJ, jend - j0);
    const i64 jy = G.col(CHK_YARG, j0), jv = G.col(CHK_FV_ARG, j0);
    const uint4* src = reinterpret_cast<const uint4*>(P.ys + jy * CHK_RW);
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * CHK_BLOCK;
      pf[u] = (e < n * CH) ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
    if (CHK_MODE == 0) pfn = (tid < n) ? P.yn[jy + tid] : 0.f;
#if CHK_V3 && CHK_V3_PRESPLIT
    chk_v3_prefetch(P, j0, tid, pf3);
#elif CHK_V3
    chk_v3_gather(vsrc, jv, n, tid, pfv);
#else
#pragma unroll
    for (int u = 0; u < NPV; u++) {
      const int e = tid + u * CHK_BLOCK;
      const int row = e / CHK_SVS, c = e - row * CHK_SVS;
      pfv[u] = (row < n && c < CHK_FV_DIM) ? vsrc[(jv + row) * CHK_FV_DIM + c] : (T)0;
    }
#endif
  };
  // folds the reduced rows [jbeg, jend) into the running maxima, sums and register tiles
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
  for (i64 j0 = jbeg; j0 < jend; j0 += CHK_TJ) {
    const int n = (int)keops_min((i64)CHK_TJ, jend - j0);
    __syncthreads();
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * CHK_BLOCK;
      if (e < CHK_TJ * CH) {
        const int row = e / CH, c = e - row * CH;
        *reinterpret_cast<uint4*>(as + row * CHK_STRIDE + c * 16) = pf[u];
      }
    }
    if (CHK_MODE == 0 && tid < CHK_TJ) { yn_s[tid] = pfn; yns_s[tid] = pfn * chk_sc; }
#pragma unroll
    for (int v = 0; v < KEOPS_NCOLVARS; v++) {
      const int dim = keops_col_dim[v];
      const T* src = P.arg[keops_col_arg[v]] + G.col(keops_col_arg[v], j0) * dim;
      for (int e = tid; e < n * dim; e += CHK_BLOCK) {
        const int row = e / dim, c = e - row * dim;
        yo_s[row * CHK_DY + keops_col_off[v] + c] = src[e];
      }
    }
#if CHK_V3 && CHK_V3_PRESPLIT
    chk_v3_store(bt3, tid, pf3);
#elif CHK_V3
    chk_v3_scatter(bt3, tid, pfv);
#else
#pragma unroll
    for (int u = 0; u < NPV; u++) {
      const int e = tid + u * CHK_BLOCK;
      if (e < CHK_TJ * CHK_SVS) bt[e] = pfv[u];
    }
#endif
    __syncthreads();
    if (j0 + CHK_TJ < jend) prefetch(j0 + CHK_TJ, jend);
    const float near_bound = CHK_MODE == 0 ? chk_near_bound(yn_s, xnq, col) : 0.f;
    const i64 jy0 = G.col(CHK_YARG, j0);
    if (!wave_live) continue;

    chk_f32x16 s;
    if (CHK_MODE == 0) {
      chk_f32x4 kk[4];
#pragma unroll
      for (int b = 0; b < 4; b++) kk[b] = *reinterpret_cast<const chk_f32x4*>(yns_s + 8 * b + 4 * half);
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] = kk[v >> 2][v & 3];
    } else {
#pragma unroll
      for (int v = 0; v < 16; v++) s[v] = 0.f;
    }
    const unsigned char* arow = as + col * CHK_STRIDE + 16 * half;
#pragma unroll
    for (int kb = 0; kb < CHK_KB; kb++) {
      const chk_h8 ah = *reinterpret_cast<const chk_h8*>(arow + kb * 32);
#if !CHK_SINGLE
      const chk_h8 al = *reinterpret_cast<const chk_h8*>(arow + CHK_DPAD * 2 + kb * 32);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bh[kb], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bl[kb], s, 0, 0, 0);
#endif
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh[kb], s, 0, 0, 0);
    }
    float sq[16];
#pragma unroll
    for (int v = 0; v < 16; v++) sq[v] = CHK_MODE == 0 ? __builtin_fmaxf(__builtin_fmaf(s[v], chk_inv, xnq), 0.f) : s[v] * chk_inv;
    if (CHK_MODE == 0) chk_fix_near<16>(P, sq, 0, half, n, xnq, yn_s, near_bound, qx, jy0);
    // F' for the lane's 16 pairs (rows past the end: -inf, they weigh nothing) and the tile maximum
    float mx = ninf;
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int r = 8 * (v >> 2) + 4 * half + (v & 3);
      T sv = sq[v];
      T yj[CHK_DY];
      constexpr int VEC = 16 / sizeof(T);
      typedef T vecT __attribute__((ext_vector_type(VEC)));
#pragma unroll
      for (int c4 = 0; c4 < KEOPS_DIMY_PAD / VEC; c4++) {
        const vecT w = *reinterpret_cast<const vecT*>(yo_s + r * CHK_DY + c4 * VEC);
#pragma unroll
        for (int c = 0; c < VEC; c++) yj[c4 * VEC + c] = w[c];
      }
      T fout[1];
      KeopsFormula::eval(xi, yj, p, sv, fout);
      s[v] = r < n ? fout[0] : ninf;
      mx = __builtin_fmaxf(mx, s[v]);
    }
    mx = __builtin_fmaxf(mx, __shfl_xor(mx, 32));  // the partner lane holds the other 16 reduced rows of this output row
    const float m_new = __builtin_fmaxf(__builtin_fmaxf(m_run, mx), -3.0e38f);
    if (keops_any(m_new != m_run)) {
      // rescale: alpha_i = exp(m_old - m_new) for the rows of this wavefront, moved to the accumulator layout
      const float alpha = keops_red_exp(m_run - m_new);
      l_run *= alpha;
      volatile float* aw = al_s[wave];
      if (half == 0) aw[col] = alpha;
      __threadfence_block();
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float a = aw[8 * (r >> 2) + 4 * half + (r & 3)];
#pragma unroll
        for (int b = 0; b < CHK_FNB; b++) acc[b][r] *= a;
      }
      __threadfence_block();
      m_run = m_new;
    }
#if CHK_V3
    float pw[16];
#endif
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const int r = 8 * (v >> 2) + 4 * half + (v & 3);
      const float pv = keops_red_exp(s[v] - m_run);
      l_run += pv;
#if CHK_V3
      pw[v] = pv;
#else
#pragma unroll
      for (int b = 0; b < CHK_FNB; b++)
        acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(pv, bt[r * CHK_SVS + 32 * b + col], acc[b], 0, 0, 0);
#endif
    }
#if CHK_V3
    chk_v3_product(pw, bt3, col, half, acc);
#endif
  }
  }

  // results of this slab: [m, (l,) O_0 .. O_{dv-1}] per output row
  l_run += __shfl_xor(l_run, 32);
  T* dst = P.nslabs > 1 ? P.partial + (i64)blockIdx.y * P.nx * KEOPS_DIMRED : P.out;
  if (half == 0 && row0 + col < G.row_end) {
    T* o = dst + (row0 + col) * KEOPS_DIMRED;
    o[0] = m_run;
    if (CHK_SM_ONE) o[1] = l_run;
  }
  {
    const i64 ibase = row0 + 4 * half;
    T* o = dst + ibase * KEOPS_DIMRED + 1 + CHK_SM_ONE + col;
#pragma unroll
    for (int b = 0; b < CHK_FNB; b++) {
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int ir = 8 * (r >> 2) + (r & 3);
        if (ibase + ir < G.row_end && 32 * b + col < CHK_FV_DIM) o[(i64)ir * KEOPS_DIMRED + 32 * b] = acc[b][r];
      }
    }
  }
}

// merges the per-slab (m, s) results in slab order: m = max_k m_k, s = sum_k exp(m_k - m) s_k
extern "C" __global__ void __launch_bounds__(256) keops_chk_softmax_reduce(const ChkParams P) {
  const i64 e = (i64)blockIdx.x * 256 + threadIdx.x;
  const i64 total = P.nx * KEOPS_DIMRED;
  if (e >= total) return;
  const i64 i = e / KEOPS_DIMRED;
  const int c = (int)(e - i * KEOPS_DIMRED);
  float m = -__builtin_huge_valf();
  for (int k = 0; k < P.nslabs; k++) m = __builtin_fmaxf(m, P.partial[(i64)k * total + i * KEOPS_DIMRED]);
  if (c == 0) {
    P.out[e] = m;
    return;
  }
  const float mm = __builtin_fmaxf(m, -3.0e38f);
  float s = 0.f;
  for (int k = 0; k < P.nslabs; k++) {
    const float mk = P.partial[(i64)k * total + i * KEOPS_DIMRED];
    s += keops_red_exp(mk - mm) * P.partial[(i64)k * total + e];
  }
  P.out[e] = s;
}
#endif

#if KEOPS_MC_RANGES
// block-sparse mode: output rows that belong to no row range keep the neutral element of the reduction
extern "C" __global__ void __launch_bounds__(256) keops_chk_fill_neutral(const ChkParams P) {
  const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
  if (i >= P.nx) return;
#if defined(CHK_FINAL) && CHK_FINAL
  for (int d = 0; d < CHK_FV_DIM; d++) P.out[i * CHK_FV_DIM + d] = (T)0;
#elif defined(CHK_SOFTMAX) && CHK_SOFTMAX
  P.out[i * KEOPS_DIMRED] = -__builtin_huge_valf();
  for (int d = 1; d < KEOPS_DIMRED; d++) P.out[i * KEOPS_DIMRED + d] = (T)0;
#else
  KeopsAcc<TACC> acc;
  acc.init();
  acc.finalize(P.out + i * KEOPS_DIMOUT);
#endif
}
#endif
