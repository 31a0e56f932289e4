// Block-sparse radial sums on the matrix cores: the scheme of keops_radial_mfma.h for launches with ranges
// (counterpart of keopscore/keopscore/mapreduce/gpu/GpuReduc1D_ranges.py:74-173 for the Gaussian family).
//
// A block-sparse pattern exists because the kernel is much narrower than the cloud, which is exactly when one
// centre for the whole cloud leaves exponents too large for the matrix cores.  Here every row range has its own
// centre c_r (the mean of a sample of its rows): its rows are formatted as x^ = x - c_r, and the columns that the
// range sweeps are copied, formatted as y~ = y - c_r, to a "virtual" column operand of their own, padded to whole
// tiles: the range's reduced-index ranges one after the other.  A workgroup (one entry of the lookup table: up to
// RAD_ROWS_PER_BLOCK rows of one range) then runs the dense sweep over the virtual tiles of its range.  The copy
// costs one formatted column per (row range, column) pair, against rows-of-the-range pairs of work: the host only
// takes this path when the row ranges are long enough for that to be small.
//
// Accuracy: as in the dense scheme the error of an exponent is at most 8 * 2^-24 |k| (|x^|^2 + |y~|^2).  With
// R_x, R_y the largest |x^|, |y~| of a range and k < 0, a pair with |y~| > R_x + sqrt(RADR_CUT / |k|) has an
// exponent below -RADR_CUT (a kernel value below 2^-48 = 3.6e-15), so keops_radr_decide asks, for every range,
//     |k| (R_x^2 + min(R_y, R_x + sqrt(RADR_CUT / |k|))^2) <= RAD_LIMIT:
// kernel values above 2^-48 are as accurate as in the dense scheme; the smaller ones may carry up to
// (R_x + R_y)^2 |k| / RAD_LIMIT times its error bound (a block-sparse mask that keeps clusters ten kernel widths
// apart, as the reference's benchmark does, is the case; an exponent t is only known to a few 2^-24 |t| in any
// float32 implementation, the general-purpose kernel and the reference's fast exponential included).  When a
// range fails the check, or when the virtual operand does not fit its workspace (the ranges' contents changed since
// the host measured them), the flag stays 0 and keops_conv_ranges of the same module, launched right behind, does
// the work from exact differences.
#pragma once

#define RADR_CUT 48.0f
#define RADR_NCH 8   // workgroups that share the columns of one row range in keops_radr_prep_cols

struct RadRParams {
  i64 nx, ny;            // rows of the output axis, of the reduced axis
  i64 nranges, nblocks;  // row ranges; entries of the lookup table (empty ones included)
  const i64* rx;         // [nranges][2] row ranges as the caller passed them (clamped where they are read)
  KeopsRangeTables rt;   // lookup (one entry per workgroup), slices and reduced-index ranges, validated or clamped
  __bf16* xa;            // [nblocks * RAD_ROWS_PER_BLOCK][RAD_SLOTS] row-side slot vectors, by lookup entry
  __bf16* yb;            // [virtual tile][RAD_NKB][2][RAD_TJ][8]
  float* bw;             // [virtual tile * RAD_TJ][RAD_WS] (RAD_MM: the operand layout of rad_store_weights_mm)
  float* ctr;            // [nranges][RAD_D] centre of every row range
  i64* vt;               // [nranges][2] = (first virtual tile, number of virtual tiles)
  unsigned* rmax;        // [nranges][2] bit patterns of max |x^|^2 and max |y~|^2
  unsigned* scal;        // [2]: 1 when the matrix-core path is taken; [3]: 1 when the virtual operand does not fit
  i64 vt_capacity;       // virtual tiles that yb / bw hold
  T* out;
  float* partial;        // [nblocks * RAD_ROWS_PER_BLOCK][RAD_DV]
  const T* arg[KEOPS_NARGS > 0 ? KEOPS_NARGS : 1];
};

__device__ __forceinline__ void radr_load_params(const RadRParams& P, T (&p)[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1]) {
#pragma unroll
  for (int v = 0; v < KEOPS_NPARVARS; v++) {
    const T* src = P.arg[keops_par_arg[v]];
#pragma unroll
    for (int d = 0; d < keops_par_dim[v]; d++) p[keops_par_off[v] + d] = src[d];
  }
}

__device__ __forceinline__ i64 radr_clamp(i64 v, i64 lo, i64 hi) { return v < lo ? lo : (v > hi ? hi : v); }

__device__ __forceinline__ void radr_slices(const RadRParams& P, i64 r, i64& k0, i64& k1) {
  k0 = r < 1 ? 0 : P.rt.slices_x[r - 1];
  k1 = P.rt.slices_x[r];
}

// Slot vector of one point relative to a centre; returns the squared norm of the centred point.
// (RAD_BIL: bil holds the RAD_DW components of u_i resp. v_j, whose terms fill the slots of kind 4)
__device__ __forceinline__ float radr_slots(const T* src, const float* ctr, double kappa, bool column, __bf16 (&slot)[RAD_SLOTS],
                                            float (&cf)[RAD_D], const T* bil = nullptr) {
  __bf16 ct[RAD_D][3], nt[4];
#if RAD_BIL
  __bf16 bt[RAD_DW][3];
#pragma unroll
  for (int d = 0; d < RAD_DW; d++) rad_split3((float)bil[d], bt[d]);
#endif
  double nrm = 0.0;
#pragma unroll
  for (int k = 0; k < RAD_D; k++) {
    const double c = (double)src[k] - (double)ctr[k];
    cf[k] = (float)c;
    nrm += c * c;
    rad_split3((float)(column ? c : -2.0 * kappa * c), ct[k]);
  }
  rad_split4(kappa * nrm, nt);
#pragma unroll
  for (int s = 0; s < RAD_SLOTS; s++) {
    const int kind = column ? rad_col_kind[s] : rad_row_kind[s];
    const int comp = column ? rad_col_comp[s] : rad_row_comp[s];
    const int term = column ? rad_col_term[s] : rad_row_term[s];
#if RAD_BIL
    slot[s] = kind == 0 ? (__bf16)0.0f : (kind == 1 ? (__bf16)1.0f : (kind == 2 ? ct[comp][term] : (kind == 3 ? nt[term] : bt[comp][term])));
#else
    slot[s] = kind == 0 ? (__bf16)0.0f : (kind == 1 ? (__bf16)1.0f : (kind == 2 ? ct[comp][term] : nt[term]));
#endif
  }
  return (float)nrm * 1.000001f;
}

// largest value of the wavefront (non-negative floats order like their bit patterns), one atomic per wavefront
__device__ __forceinline__ void radr_atomic_max(unsigned* dst, float v) {
  unsigned b = __float_as_uint(v);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const unsigned other = (unsigned)__shfl_xor((int)b, o);
    b = other > b ? other : b;
  }
  if ((threadIdx.x & 63) == 0) atomicMax(dst, b);
}

// ---- pre-pass ---------------------------------------------------------------------------------------------------

// One workgroup per row range: its centre (mean of at most 4096 evenly spaced rows, summed in a fixed order) and
// the number of virtual tiles its columns need.
extern "C" __global__ void __launch_bounds__(256) keops_radr_centres(const RadRParams P) {
  __shared__ double part[256];
  __shared__ i64 cnt[256];
  const i64 r = blockIdx.x;
  const int tid = threadIdx.x;
  const i64 a = radr_clamp(P.rx[2 * r], 0, P.nx), b = radr_clamp(P.rx[2 * r + 1], a, P.nx);
  const i64 len = b - a, step = len > 4096 ? len / 4096 : 1, nsamp = len > 0 ? (len + step - 1) / step : 0;
  const T* x = P.arg[RAD_XARG];
#pragma unroll
  for (int c = 0; c < RAD_D; c++) {
    double s = 0.0;
    for (i64 q = tid; q < nsamp; q += 256) s += (double)x[(a + q * step) * RAD_D + c];
    part[tid] = s;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
      if (tid < o) part[tid] += part[tid + o];
      __syncthreads();
    }
    if (tid == 0) P.ctr[r * RAD_D + c] = nsamp > 0 ? (float)(part[0] / (double)nsamp) : 0.f;
    __syncthreads();
  }
  i64 k0, k1;
  radr_slices(P, r, k0, k1);
  i64 n = 0;
  for (i64 k = k0 + tid; k < k1; k += 256) {
    const i64 l = P.rt.ranges_y[2 * k + 1] - P.rt.ranges_y[2 * k];
    n += l > 0 ? l : 0;
  }
  cnt[tid] = n;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (tid < o) cnt[tid] += cnt[tid + o];
    __syncthreads();
  }
  if (tid == 0) {
    P.vt[2 * r + 1] = len > 0 ? (cnt[0] + RAD_TJ - 1) / RAD_TJ : 0;  // a range without rows needs no columns
    P.rmax[2 * r] = 0u;
    P.rmax[2 * r + 1] = 0u;
  }
}

// first virtual tile of every range (exclusive scan, one workgroup, chunks of 1024 ranges); scal[3] = 1 when the
// operand does not fit
extern "C" __global__ void __launch_bounds__(1024) keops_radr_scan(const RadRParams P) {
  __shared__ i64 part[1024];
  __shared__ i64 carry;
  const int tid = threadIdx.x;
  if (tid == 0) carry = 0;
  __syncthreads();
  for (i64 base = 0; base < P.nranges; base += 1024) {
    const i64 r = base + tid;
    const i64 v = r < P.nranges ? P.vt[2 * r + 1] : 0;
    part[tid] = v;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {
      const i64 t = tid >= o ? part[tid - o] : 0;
      __syncthreads();
      part[tid] += t;
      __syncthreads();
    }
    if (r < P.nranges) P.vt[2 * r] = carry + part[tid] - v;
    __syncthreads();
    if (tid == 1023) carry += part[1023];
    __syncthreads();
  }
  if (tid == 0) {
    P.scal[2] = 0u;
    P.scal[3] = carry > P.vt_capacity ? 1u : 0u;
  }
}

// one workgroup per lookup entry: slot vectors of its rows, zero past the last row of the entry
extern "C" __global__ void __launch_bounds__(RAD_ROWS_PER_BLOCK) keops_radr_prep_rows(const RadRParams P) {
  const i64 e = blockIdx.x;
  const i64 r = keops_uniform(P.rt.lookup[3 * e]), r0 = keops_uniform(P.rt.lookup[3 * e + 1]), r1 = keops_uniform(P.rt.lookup[3 * e + 2]);
  if (r1 <= r0) return;  // empty entry: the main kernel skips it too
  const i64 i = r0 + threadIdx.x;
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  radr_load_params(P, p);
  const double kappa = (double)KeopsRadFormula::kappa(p);
  __bf16 slot[RAD_SLOTS];
  float cf[RAD_D];
  float nrm = 0.f;
  if (i < r1) {
#if RAD_BIL
    T xi[RAD_DIMX > 0 ? RAD_DIMX : 1], uv[RAD_DW];
#pragma unroll
    for (int v = 0; v < RAD_NROWVARS; v++) {
      const T* a = P.arg[rad_row_arg[v]] + i * rad_row_dim[v];
#pragma unroll
      for (int d = 0; d < rad_row_dim[v]; d++) xi[rad_row_off[v] + d] = a[d];
    }
    KeopsRadFormula::rowvec(xi, p, uv);
    nrm = radr_slots(P.arg[RAD_XARG] + i * RAD_D, P.ctr + r * RAD_D, kappa, false, slot, cf, uv);
#else
    nrm = radr_slots(P.arg[RAD_XARG] + i * RAD_D, P.ctr + r * RAD_D, kappa, false, slot, cf);
#endif
  } else {
#pragma unroll
    for (int s = 0; s < RAD_SLOTS; s++) slot[s] = (__bf16)0.0f;
  }
  radr_atomic_max(P.rmax + 2 * r, nrm);
  __bf16* dst = P.xa + (e * RAD_ROWS_PER_BLOCK + threadIdx.x) * RAD_SLOTS;
#pragma unroll
  for (int c8 = 0; c8 < RAD_SLOTS / 8; c8++) {
    rad_bf16x8 v8;
#pragma unroll
    for (int q = 0; q < 8; q++) v8[q] = slot[c8 * 8 + q];
    *reinterpret_cast<rad_bf16x8*>(dst + c8 * 8) = v8;
  }
}

// Grid (row range, RADR_NCH): the columns of the range's reduced-index ranges, one after the other, go to the
// virtual tiles of the range; workgroup y takes the tiles t with t % RADR_NCH == y.  Places past the last column hold
// zero slot vectors and zero weights.
extern "C" __global__ void __launch_bounds__(256) keops_radr_prep_cols(const RadRParams P) {
  if (P.scal[3] != 0u) return;
  const i64 r = blockIdx.x;
  const i64 tile0 = keops_uniform(P.vt[2 * r]), ntiles = keops_uniform(P.vt[2 * r + 1]);
  if (ntiles == 0) return;
  const int tid = threadIdx.x, chunk = blockIdx.y;
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  radr_load_params(P, p);
  const double kappa = (double)KeopsRadFormula::kappa(p);
  const float* ctr = P.ctr + r * RAD_D;
  float nmax = 0.f;

  auto store = [&](i64 t, int c, const __bf16 (&slot)[RAD_SLOTS], const float (&w)[RAD_WS]) {
    const i64 tile = tile0 + t;
#pragma unroll
    for (int kb = 0; kb < RAD_NKB; kb++)
#pragma unroll
      for (int hf = 0; hf < 2; hf++) {
        rad_bf16x8 v8;
#pragma unroll
        for (int q = 0; q < 8; q++) v8[q] = slot[kb * 16 + hf * 8 + q];
        *reinterpret_cast<rad_bf16x8*>(P.yb + (((tile * RAD_NKB + kb) * 2 + hf) * RAD_TJ + c) * 8) = v8;
      }
#if RAD_MM
    rad_store_weights_mm(reinterpret_cast<__bf16*>(P.bw), tile * RAD_TJ + c, w);  // B operand of the second product
#else
#pragma unroll
    for (int d = 0; d < RAD_WS; d++) P.bw[(tile * RAD_TJ + c) * RAD_WS + d] = w[d];
#endif
  };

  i64 k0, k1;
  radr_slices(P, r, k0, k1);
  i64 base = 0;  // virtual column of the first column of the current reduced-index range
  for (i64 k = k0; k < k1; k++) {
    const i64 s = keops_uniform(P.rt.ranges_y[2 * k]), e = keops_uniform(P.rt.ranges_y[2 * k + 1]);
    const i64 len = e > s ? e - s : 0;
    if (len == 0) continue;
    i64 t = base / RAD_TJ;
    t += ((i64)chunk - t % RADR_NCH + RADR_NCH) % RADR_NCH;
    for (; t * RAD_TJ < base + len; t += RADR_NCH)
      for (int c = tid; c < RAD_TJ; c += 256) {
        const i64 v = t * RAD_TJ + c;
        if (v < base || v >= base + len) continue;
        const i64 j = s + (v - base);
        __bf16 slot[RAD_SLOTS];
        float cf[RAD_D], w[RAD_WS];
        T yj[RAD_DIMY > 0 ? RAD_DIMY : 1];
#pragma unroll
        for (int q = 0; q < RAD_NCOLVARS; q++) {
          const T* a = P.arg[rad_col_arg[q]] + j * rad_col_dim[q];
#pragma unroll
          for (int d = 0; d < rad_col_dim[q]; d++) yj[rad_col_off[q] + d] = a[d];
        }
        T wv[RAD_DW];
        KeopsRadFormula::weights(yj, p, wv);
        const float nrm = radr_slots(P.arg[RAD_YARG] + j * RAD_D, ctr, kappa, true, slot, cf, wv);
        nmax = nrm > nmax ? nrm : nmax;
#if RAD_BIL
        // the weights sit in the slot vectors: what is left per column is [y~_j, 1], or 1
#if RAD_DIFF != 0
#pragma unroll
        for (int q = 0; q < RAD_D; q++) w[q] = cf[q];
        w[RAD_D] = 1.f;
#else
        w[0] = 1.f;
#endif
#elif RAD_UPAIR
        // the weights as they are, then [y~_j, 1]: the sweep forms <u_i, v_j> itself
#pragma unroll
        for (int d = 0; d < RAD_DW; d++) w[d] = (float)wv[d];
#pragma unroll
        for (int q = 0; q < RAD_D; q++) w[RAD_DW + q] = cf[q];
        w[RAD_DW + RAD_D] = 1.f;
#elif RAD_DIFF != 0
        // component d of the weights against [y~_j, 1]
#pragma unroll
        for (int d = 0; d < RAD_DW; d++) {
#pragma unroll
          for (int q = 0; q < RAD_D; q++) w[d * (RAD_D + 1) + q] = (float)wv[d] * cf[q];
          w[d * (RAD_D + 1) + RAD_D] = (float)wv[d];
        }
#else
#pragma unroll
        for (int d = 0; d < RAD_DV; d++) w[d] = (float)wv[d];
#endif
        store(t, c, slot, w);
      }
    base += len;
  }
  // the rest of the last tile
  const i64 last = ntiles - 1;
  if (last % RADR_NCH == chunk) {
    __bf16 slot[RAD_SLOTS];
    float w[RAD_WS];
#pragma unroll
    for (int s = 0; s < RAD_SLOTS; s++) slot[s] = (__bf16)0.0f;
#pragma unroll
    for (int d = 0; d < RAD_WS; d++) w[d] = 0.f;
    for (int c = tid; c < RAD_TJ; c += 256)
      if (last * RAD_TJ + c >= base) store(last, c, slot, w);
  }
  radr_atomic_max(P.rmax + 2 * r + 1, nmax);
}

// one workgroup: every range must pass the check at the head of this file
extern "C" __global__ void __launch_bounds__(256) keops_radr_decide(const RadRParams P) {
  __shared__ int bad[256];
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  radr_load_params(P, p);
  const float kappa = (float)KeopsRadFormula::kappa(p), ak = __builtin_fabsf(kappa);
  int mine = 0;
  for (i64 r = threadIdx.x; r < P.nranges; r += 256) {
    const float rx2 = __uint_as_float(P.rmax[2 * r]), ry2 = __uint_as_float(P.rmax[2 * r + 1]);
    float ry = __builtin_sqrtf(ry2);
    if (kappa < 0.f) {
      const float reach = __builtin_sqrtf(rx2) + __builtin_sqrtf(RADR_CUT / ak);
      ry = ry < reach ? ry : reach;
    }
    if (!(ak * (rx2 + ry * ry) <= (float)RAD_LIMIT)) mine = 1;  // also for NaN
    // a column so far out that the terms of its exponent overflow (they would cancel to NaN instead of a large negative
    // number): the general-purpose kernel gives such pairs their zero
    if (!(ak * ry2 <= 1e30f)) mine = 1;
  }
  bad[threadIdx.x] = mine;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) bad[threadIdx.x] |= bad[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) P.scal[2] = (bad[0] == 0 && P.scal[3] == 0u) ? 1u : 0u;
}

// ---- main kernel: one workgroup per lookup entry --------------------------------------------------------------------

extern "C" __global__ void __launch_bounds__(RAD_BLOCK, RAD_MIN_WAVES) keops_radr_main(const RadRParams P) {
  if (P.scal[2] != 1u) return;
  __shared__ __attribute__((aligned(16))) __bf16 ys[RAD_NKB * 2 * RAD_TJ * 8];  // [kb][half][col][8]
#if RAD_MM
  __shared__ __attribute__((aligned(16))) __bf16 ws[RAD_TJ * 32 * RAD_MM_NB];  // [sub-tile][k block][half][operand column][8]
#else
  __shared__ __attribute__((aligned(16))) float bs[RAD_TJ * RAD_WS];
#endif
  const i64 e = blockIdx.x;
  const i64 r = keops_uniform(P.rt.lookup[3 * e]), r0 = keops_uniform(P.rt.lookup[3 * e + 1]), r1 = keops_uniform(P.rt.lookup[3 * e + 2]);
  if (r1 <= r0) return;
  const int wave = threadIdx.x >> 6;
  const i64 local0 = e * RAD_ROWS_PER_BLOCK + (i64)wave * (32 * RAD_RB);
  RadSweep S;
  S.xa = P.xa + local0 * RAD_SLOTS;   // padded with zero vectors up to the end of the entry
  S.rows_avail = 32 * RAD_RB;
  S.yb = P.yb;
  S.bw = P.bw;
  S.jbeg = keops_uniform(P.vt[2 * r]) * RAD_TJ;
  S.jend = S.jbeg + keops_uniform(P.vt[2 * r + 1]) * RAD_TJ;
  S.part = P.partial + local0 * RAD_DV;
  S.rows_store = 32 * RAD_RB;
  S.arg = P.arg;
  S.row_first = r0 + (i64)wave * (32 * RAD_RB);
  S.row_last = r1 - 1;
  S.rperm = nullptr;  // (the per-tile choice belongs to the dense launches: here every range has been checked)
  S.ctmax = nullptr;
  S.xq = 0.f;
#if RAD_MM
  rad_sweep_mm(S, ys, ws);
#else
  rad_sweep(S, ys, bs);
#endif
}

// the factors of the output index and, for the gradients with respect to the points, the difference
// x^_i S - sum_j K_ij w_j y~_j, once per output row
extern "C" __global__ void __launch_bounds__(RAD_ROWS_PER_BLOCK) keops_radr_finish(const RadRParams P) {
  if (P.scal[2] != 1u) return;
  const i64 e = blockIdx.x;
  const i64 r = keops_uniform(P.rt.lookup[3 * e]), r0 = keops_uniform(P.rt.lookup[3 * e + 1]), r1 = keops_uniform(P.rt.lookup[3 * e + 2]);
  const i64 i = r0 + threadIdx.x;
  if (i >= r1) return;
  const float* s = P.partial + (e * RAD_ROWS_PER_BLOCK + threadIdx.x) * RAD_DV;
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  radr_load_params(P, p);
  T xi[RAD_DIMX > 0 ? RAD_DIMX : 1];
#pragma unroll
  for (int v = 0; v < RAD_NROWVARS; v++) {
    const T* a = P.arg[rad_row_arg[v]] + i * rad_row_dim[v];
#pragma unroll
    for (int d = 0; d < rad_row_dim[v]; d++) xi[rad_row_off[v] + d] = a[d];
  }
  const float ai = (float)KeopsRadFormula::rowscale(xi, p) * RAD_SIGN;
  // a factor <u_i, v_j> of both indices: the sums were accumulated per component of v, u_i contracts them here
#if RAD_DU > 0 && !RAD_UPAIR && !RAD_BIL
  T uv[RAD_DU];
  KeopsRadFormula::rowvec(xi, p, uv);
#endif
#if RAD_DIFF != 0
  const T* x = P.arg[RAD_XARG] + i * RAD_D;
#pragma unroll
  for (int k = 0; k < RAD_D; k++) {
    const float xc = (float)((double)x[k] - (double)P.ctr[r * RAD_D + k]);
#if RAD_DU > 0 && !RAD_UPAIR && !RAD_BIL
    float acc = 0.f;
#pragma unroll
    for (int d = 0; d < RAD_DW; d++) acc = __builtin_fmaf((float)uv[d], __builtin_fmaf(xc, s[d * (RAD_D + 1) + RAD_D], -s[d * (RAD_D + 1) + k]), acc);
    P.out[i * RAD_DOUT + k] = (T)(ai * (float)RAD_DIFF * acc);
#else
    P.out[i * RAD_DOUT + k] = (T)(ai * (float)RAD_DIFF * __builtin_fmaf(xc, s[RAD_D], -s[k]));
#endif
  }
#elif RAD_DU > 0 && !RAD_BIL
  float acc = 0.f;
#pragma unroll
  for (int d = 0; d < RAD_DW; d++) acc = __builtin_fmaf((float)uv[d], s[d], acc);
  P.out[i] = (T)(ai * acc);
#else
#pragma unroll
  for (int d = 0; d < RAD_DOUT; d++) P.out[i * RAD_DOUT + d] = (T)(ai * s[d]);
#endif
}
