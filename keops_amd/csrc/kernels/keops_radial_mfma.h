// Low-dimensional radial sums on the matrix cores:
//     out_i = A(i-variables) sum_j exp(c * |x_i - y_j|^2) * W(j-variables),          x, y of RAD_D <= 8 components,
// and, with the difference factor of the gradients with respect to the points (RAD_DIFF = +-1),
//     out_i = +- A_i sum_j exp(c * |x_i - y_j|^2) w_j (x_i - y_j)  =  +- A_i (x^_i S_i - sum_j K_ij w_j y^_j),
// where the kernel accumulates the RAD_D + 1 sums of K_ij w_j [y^_j, 1] and x^, y^ are the points minus the mean of y
// (the two terms that are subtracted are then as small as the cloud allows; what remains is a cancellation of
// order 2^-24 |x^_i| / |x_i - y_j|, small wherever the device-side check below lets this path run).
//
// Counterpart of keopscore/keopscore/mapreduce/gpu/GpuReduc1D.py:43-96 for this family (the Gaussian kernel sum of
// the reference's benchmarks): the general-purpose kernel of keops_conv.h spends 3*D + 3 of its 9 vector
// instructions per pair on the exponent.  Here the exponent of a whole 32 x 32 tile of pairs,
//     t_ij = k |x_i - y_j|^2 = k |x_i|^2 + k |y_j|^2 - 2 k <x_i, y_j>,        k = c * log2(e),
// comes out of v_mfma_f32_32x32x16_bf16 as ONE scalar product of two "slot vectors", and the vector ALU is left
// with v_exp_f32 and one fused multiply-add per pair and output component.
//
// Exact operands.  bfloat16 products are exact in float32 (8 x 8 significant bits), so a float32 number split as
// h + m + l (three bfloat16 terms, 24 bits) multiplies exactly term by term.  Row side: u = -2 k x^ (x^ = x minus
// the mean of y, formed in double precision, rounded once to float32) in three terms, p = k |x^|^2 from double
// precision in four terms; column side: y^ in three terms, q = k |y^|^2 in four.  The slots of the scalar product
// are the term products (h,h) (h,m) (m,h) (m,m) (h,l) (l,h) (m,l) of every component plus (p_n, 1) and (1, q_n):
// 7 D + 8 slots, ordered by magnitude so that the big terms, which cancel, share one 8-slot group of the first
// instruction (the hardware adds the products of a group exactly up to 24 bits below the largest and truncates
// each instruction's result to float32; measured on a million pairs: |dt| <= 8 * 2^-24 |k| (|x^|^2 + |y^|^2), no
// bias).  Dropped: (l,m), (l,l), below 2^-24 |u||y|.  The error of a kernel value is therefore at most
// ln(2) |dt| <= 3.3e-7 |k| (|x^|^2 + |y^|^2), typically a third of it: the float32 class of the reference's own
// exponent as long as the kernel is not much narrower than the cloud.  keops_rad_decide checks exactly that on the
// device, |k| (max |x^|^2 + max |y^|^2) <= RAD_LIMIT, and sets a flag: when it does not hold, the kernels of this
// file return at once and the general-purpose kernel of the same module, which is launched behind them and returns
// at once in the other case, computes the sum from exact float32 differences.  No host synchronisation.
//
// Work decomposition: lane l of a wavefront owns column j = l % 32 of the staged sub-tile (its slot vector is the B
// operand, its weights B_j sit in registers) and, after the instruction, the 16 exponents of rows
// 8 (v / 4) + 4 (l / 32) + v % 4; it accumulates exp2(t) * B_j per row and component in registers for the whole
// sweep.  A wavefront holds RAD_RB blocks of 32 rows (A operands in VGPRs), RAD_WAVES wavefronts share the staged
// column tile (slot vectors pre-formatted by keops_rad_prep: straight 16-byte copies, conflict-free 16-byte reads).
// The lanes of a row are summed with shuffles once at the end; slabs over the reduced axis (blockIdx.y) are added
// in order by keops_rad_reduce: deterministic.
//
// RAD_FOLD (a scalar weight w_j and no difference factor: the plain Gaussian kernel sum): exp2(t) w_j =
// +- exp2(t + log2 |w_j|), so log2 |w_j| joins the column's squared-norm term (formed in double precision) and the
// columns are partitioned by the sign of their weight (stable, deterministic: keops_rad_sign_count / _scan, then
// keops_rad_prep scatters every column to its place; unused places hold "dead" columns whose exponent is -16384).
// Tiles of non-negative weights are accumulated with one v_add_f32 per pair, the others with one v_sub_f32: half
// the cost of the fused multiply-add (v_exp_f32 takes 8 issue cycles per wavefront, v_fmac_f32 4, v_add_f32 2).
// The sweep alternates between the two groups tile by tile (rad_tile_of), so that the running sums stay as small
// as with the weights in their original order: summing one sign after the other would carry rounding errors
// relative to sum_j K_ij |w_j| into a result that may be much smaller.
//
// The plug-in defines RAD_D, RAD_DV, RAD_NKB (16-slot blocks), RAD_RB, RAD_WAVES, RAD_XARG, RAD_YARG, RAD_LIMIT,
// the slot tables rad_slot_kind / rad_slot_comp / rad_slot_term for both sides, the tables of the variables of B
// (rad_col_arg / rad_col_dim / rad_col_off, RAD_NCOLVARS, RAD_DIMY) and of the parameters (keops_par_*), and
// the tables of the variables of A (rad_row_*, RAD_NROWVARS, RAD_DIMX), RAD_DW (components of W), RAD_DU (components of
// a row vector u_i that multiplies W as <u_i, W_j>: KeopsRadFormula::rowvec), RAD_DOUT, RAD_DIFF,
// RAD_SIGN and struct KeopsRadFormula { kappa(p); weights(yj, p, w); rowscale(xi, p) }.
#pragma once

typedef __bf16 rad_bf16x8 __attribute__((ext_vector_type(8)));
typedef float rad_f32x16 __attribute__((ext_vector_type(16)));
typedef float rad_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 rad_bf16x2 __attribute__((ext_vector_type(2)));

#ifndef RAD_TJ
#define RAD_TJ 128                 // columns per staged tile
#endif
#ifndef RAD_DU
#define RAD_DU 0                   // components of a row factor u_i that enters as <u_i, v_j> (0: none)
#endif
#ifndef RAD_UPAIR
#define RAD_UPAIR 0                // 1 (with RAD_DIFF and RAD_DU): <u_i, v_j> is formed per pair and D + 1 sums are kept
#endif
#define RAD_WS (RAD_UPAIR ? RAD_DW + RAD_D + 1 : RAD_DV)  // floats staged per column: the weights as the sweep needs them
// RAD_BIL: a factor <u_i, v_j> comes out of the matrix cores like the exponent: the k blocks RAD_NKE .. RAD_NKB - 1 of
// the slot vectors hold the term products of u_i (rows) and v_j (columns), slot kind 4, and a second accumulator
// receives their sum for the 32 x 32 tile; the vector ALU multiplies it with the kernel value.
#ifndef RAD_BIL
#define RAD_BIL 0
#endif
#ifndef RAD_NKE
#define RAD_NKE RAD_NKB            // k blocks of the exponent
#endif
#ifndef RAD_MM
#define RAD_MM 0                   // 1: the weighted sum runs on the matrix cores too (see rad_sweep_mm)
#endif
#define RAD_MM_FOLD 4096           // columns between two folds of the running sums (block summation)
#define RAD_MM_NB ((3 * RAD_DV + 31) / 32)  // 32-column blocks of the B operand of the second product
#ifndef RAD_MM_TERMS
#define RAD_MM_TERMS 3             // bfloat16 terms of a kernel value in the second product (3: truncated, exact; 2: rounded)
#endif
#define RAD_NSUB (RAD_TJ / 32)
#define RAD_SLOTS (16 * RAD_NKB)
#define RAD_BLOCK (64 * RAD_WAVES)
#define RAD_ROWS_PER_BLOCK (32 * RAD_RB * RAD_WAVES)

struct RadParams {
  i64 nx, ny;
  __bf16* xa;         // [nx][RAD_SLOTS] row-side slot vectors
  __bf16* yb;         // [tile][RAD_NKB][2][RAD_TJ][8] column-side slot vectors, tile by tile
  float* bw;          // [ntiles * RAD_TJ][RAD_DV] weights B_j (zero past the last column)
  float* colsum;      // [RAD_D] column sums of y
  float* colpart;     // [nparts][RAD_D]
  unsigned* scal;     // [0], [1]: bit patterns of max |x^|^2, max |y^|^2; [2]: 1 when the matrix-core path is taken;
                      // [3] (RAD_FOLD): number of tiles of columns with non-negative weights
  int* blk;           // RAD_FOLD: [nblk] non-negative weights per block of 256 columns, then their exclusive scan
  T* out;             // [nx][RAD_DV]
  float* partial;     // [nslabs][nx][RAD_DV]
  i64 slab_len;       // reduced rows per slab (multiple of RAD_TJ)
  int nslabs;
  int nparts;
  const T* arg[KEOPS_NARGS > 0 ? KEOPS_NARGS : 1];
};

__device__ __forceinline__ void rad_load_params(const RadParams& P, T (&p)[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1]) {
#pragma unroll
  for (int v = 0; v < KEOPS_NPARVARS; v++) {
    const T* src = P.arg[keops_par_arg[v]];
#pragma unroll
    for (int d = 0; d < keops_par_dim[v]; d++) p[keops_par_off[v] + d] = src[d];
  }
}

// ---- pre-pass ---------------------------------------------------------------------------------------------------

#ifndef RAD_RANGES
#define RAD_RANGES 0
#endif

#if !RAD_RANGES
// column sums of y in two deterministic stages (fixed order, no atomics)
extern "C" __global__ void __launch_bounds__(256) keops_rad_colsum(const RadParams P) {
  __shared__ float part[256];
  const T* y = P.arg[RAD_YARG];
  const i64 rows_per_block = (P.ny + gridDim.x - 1) / gridDim.x;
  const i64 r0 = (i64)blockIdx.x * rows_per_block, r1 = keops_min(P.ny, r0 + rows_per_block);
#pragma unroll
  for (int c = 0; c < RAD_D; c++) {
    float s = 0.f;
    for (i64 r = r0 + threadIdx.x; r < r1; r += 256) s += (float)y[r * RAD_D + c];
    part[threadIdx.x] = s;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
      if ((int)threadIdx.x < o) part[threadIdx.x] += part[threadIdx.x + o];
      __syncthreads();
    }
    if (threadIdx.x == 0) P.colpart[(i64)blockIdx.x * RAD_D + c] = part[0];
    __syncthreads();
  }
}

extern "C" __global__ void __launch_bounds__(64) keops_rad_colsum_final(const RadParams P) {
  const int c = threadIdx.x;
  if (c < RAD_D) {
    double s = 0.0;
    for (int b = 0; b < P.nparts; b++) s += (double)P.colpart[(i64)b * RAD_D + c];
    P.colsum[c] = (float)(s / (double)P.ny);  // the mean
  }
  if (c < 4) P.scal[c] = 0u;
}

#endif  // !RAD_RANGES

#ifndef RAD_FOLD
#define RAD_FOLD 0
#endif

__device__ __forceinline__ float rad_column_weight(const RadParams& P, i64 j, const T (&p)[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1]) {
  T yj[RAD_DIMY > 0 ? RAD_DIMY : 1];
#pragma unroll
  for (int v = 0; v < RAD_NCOLVARS; v++) {
    const T* a = P.arg[rad_col_arg[v]] + j * rad_col_dim[v];
#pragma unroll
    for (int d = 0; d < rad_col_dim[v]; d++) yj[rad_col_off[v] + d] = a[d];
  }
  T wv[RAD_DW];
  KeopsRadFormula::weights(yj, p, wv);
  return (float)wv[0];
}

#if RAD_FOLD
// columns with a non-negative weight, per block of 256 columns (a NaN weight counts as non-negative)
extern "C" __global__ void __launch_bounds__(256) keops_rad_sign_count(const RadParams P) {
  __shared__ int cnt[4];
  const i64 j = (i64)blockIdx.x * 256 + threadIdx.x;
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  rad_load_params(P, p);
  const bool pos = j < P.ny && !(rad_column_weight(P, j, p) < 0.f);
  const unsigned long long bal = __ballot(pos);
  if ((threadIdx.x & 63) == 0) cnt[threadIdx.x >> 6] = __popcll(bal);
  __syncthreads();
  if (threadIdx.x == 0) P.blk[blockIdx.x] = cnt[0] + cnt[1] + cnt[2] + cnt[3];
}

// exclusive scan of the block counts (one workgroup, sequential over chunks of 1024 blocks); scal[3] = tiles of
// non-negative columns
extern "C" __global__ void __launch_bounds__(1024) keops_rad_sign_scan(const RadParams P, int nblk) {
  __shared__ int part[1024];
  __shared__ int carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < nblk; base += 1024) {
    const int b = base + threadIdx.x;
    const int v = b < nblk ? P.blk[b] : 0;
    part[threadIdx.x] = v;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {  // inclusive scan in shared memory
      const int t = (int)threadIdx.x >= o ? part[threadIdx.x - o] : 0;
      __syncthreads();
      part[threadIdx.x] += t;
      __syncthreads();
    }
    if (b < nblk) P.blk[b] = carry + part[threadIdx.x] - v;
    __syncthreads();
    if (threadIdx.x == 1023) carry += part[1023];
    __syncthreads();
  }
  if (threadIdx.x == 0) P.scal[3] = (unsigned)((carry + RAD_TJ - 1) / RAD_TJ);
}

// every place of the column operand starts as a dead column: exponent -16384 for every row
extern "C" __global__ void __launch_bounds__(256) keops_rad_fill_dead(const RadParams P, i64 ncols) {
  const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
  if (i >= ncols) return;
  const i64 tile = i / RAD_TJ;
  const int c = (int)(i % RAD_TJ);
#pragma unroll
  for (int kb = 0; kb < RAD_NKB; kb++)
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
      rad_bf16x8 v8;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const int s = kb * 16 + hf * 8 + e;
        v8[e] = (rad_col_kind[s] == 3 && rad_col_term[s] == 0) ? (__bf16)(-16384.0f) : (__bf16)0.0f;
      }
      *reinterpret_cast<rad_bf16x8*>(P.yb + (((tile * RAD_NKB + kb) * 2 + hf) * RAD_TJ + c) * 8) = v8;
    }
}
#endif

__device__ __forceinline__ void rad_split3(float v, __bf16 (&t)[3]) {
  t[0] = (__bf16)v;
  const float r1 = v - (float)t[0];
  t[1] = (__bf16)r1;
  t[2] = (__bf16)(r1 - (float)t[1]);
}
__device__ __forceinline__ void rad_split4(double v, __bf16 (&t)[4]) {
  double r = v;
#pragma unroll
  for (int k = 0; k < 4; k++) {
    t[k] = (__bf16)(float)r;
    r -= (double)(float)t[k];
  }
}


#if RAD_MM
// Weights of column j in the layout of the B operand of the weighted sum (rad_sweep_mm): 32 operand columns
// [w_h | w_m | w_l | 0] (the three bfloat16 terms of the RAD_DV weights side by side), contraction index = the 32
// columns of a sub-tile in the order in which the exponent tile leaves them in the registers of a lane: registers
// 0-7 (k block 0) of lanes 0-31 hold columns {0,1,2,3,8,9,10,11}, of lanes 32-63 {4,...,7,12,...,15}; registers 8-15
// (k block 1) the same plus 16.  Layout [32-column sub-tile][k block][half][operand column][8]; beyond ten weights the
// 3 * RAD_DV operand columns take RAD_MM_NB blocks of 32.
__device__ __forceinline__ void rad_store_weights_mm(__bf16* bwm, i64 j, const float (&w)[RAD_DV]) {
  const int jj = (int)(j & 31), kb = jj >> 4, q = jj & 15, hf = (q >> 2) & 1, e = (q & 3) + 4 * (q >> 3);
  __bf16* dst = bwm + ((((j >> 5) * 2 + kb) * 2 + hf) * (32 * RAD_MM_NB)) * 8 + e;
#pragma unroll
  for (int n = 0; n < 32 * RAD_MM_NB; n++) {
    __bf16 v = (__bf16)0.0f;
    if (n < 3 * RAD_DV) {
      __bf16 t3[3];
      rad_split3(w[n % RAD_DV], t3);
      v = t3[n / RAD_DV];
    }
    dst[n * 8] = v;
  }
}
#endif

#if !RAD_RANGES
// Slot vector of one point.  which = 0: rows (x), 1: columns (y; one thread per column of the padded tile grid).
extern "C" __global__ void __launch_bounds__(256) keops_rad_prep(const RadParams P, int which) {
  const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
  const i64 n = which ? P.ny : P.nx;
#if RAD_FOLD
  const i64 ntot = which ? (P.ny + 255) / 256 * 256 : P.nx;  // whole blocks: every lane takes part in the ranking
#else
  const i64 ntot = which ? (P.ny + RAD_TJ - 1) / RAD_TJ * RAD_TJ : P.nx;
#endif
  if (i >= ntot) return;
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  rad_load_params(P, p);
  const double kappa = (double)KeopsRadFormula::kappa(p);
  __bf16 slot[RAD_SLOTS];
  float w[RAD_WS];
#pragma unroll
  for (int d = 0; d < RAD_WS; d++) w[d] = 0.f;
  if (i < n) {
    const T* src = P.arg[which ? RAD_YARG : RAD_XARG] + i * RAD_D;
    __bf16 ct[RAD_D][3], nt[4];
    float cf[RAD_D];
    double nrm = 0.0;
#pragma unroll
    for (int k = 0; k < RAD_D; k++) {
      const double c = (double)src[k] - (double)P.colsum[k];
      cf[k] = (float)c;
      nrm += c * c;
      rad_split3((float)(which ? c : -2.0 * kappa * c), ct[k]);
    }
#if RAD_FOLD
    // the weight joins the exponent: exp2(t) w = +- exp2(t + log2 |w|)
    float wfold = 1.f;
    if (which) {
      wfold = rad_column_weight(P, i, p);
      w[0] = wfold;
    }
    rad_split4(which ? kappa * nrm + (double)__ocml_log2_f64((double)__builtin_fabsf(wfold)) : kappa * nrm, nt);
#else
    rad_split4(kappa * nrm, nt);
#endif
#if RAD_BIL
    // three bfloat16 terms of every component of u_i (rows) or v_j (columns)
    __bf16 bt[RAD_DW][3];
    {
      T vals[RAD_DW];
      if (which) {
        T yj[RAD_DIMY > 0 ? RAD_DIMY : 1];
#pragma unroll
        for (int v = 0; v < RAD_NCOLVARS; v++) {
          const T* a = P.arg[rad_col_arg[v]] + i * rad_col_dim[v];
#pragma unroll
          for (int d = 0; d < rad_col_dim[v]; d++) yj[rad_col_off[v] + d] = a[d];
        }
        KeopsRadFormula::weights(yj, p, vals);
      } else {
        T xi[RAD_DIMX > 0 ? RAD_DIMX : 1];
#pragma unroll
        for (int v = 0; v < RAD_NROWVARS; v++) {
          const T* a = P.arg[rad_row_arg[v]] + i * rad_row_dim[v];
#pragma unroll
          for (int d = 0; d < rad_row_dim[v]; d++) xi[rad_row_off[v] + d] = a[d];
        }
        KeopsRadFormula::rowvec(xi, p, vals);
      }
#pragma unroll
      for (int d = 0; d < RAD_DW; d++) rad_split3((float)vals[d], bt[d]);
    }
#endif
    // largest centred squared norm (bit pattern of a non-negative float, rounded up): order-independent maximum
    atomicMax(P.scal + which, __float_as_uint((float)nrm * 1.000001f));
#pragma unroll
    for (int s = 0; s < RAD_SLOTS; s++) {
      const int kind = which ? rad_col_kind[s] : rad_row_kind[s];
      const int comp = which ? rad_col_comp[s] : rad_row_comp[s];
      const int term = which ? rad_col_term[s] : rad_row_term[s];
#if RAD_BIL
      slot[s] = kind == 0 ? (__bf16)0.0f : (kind == 1 ? (__bf16)1.0f : (kind == 2 ? ct[comp][term] : (kind == 3 ? nt[term] : bt[comp][term])));
#else
      slot[s] = kind == 0 ? (__bf16)0.0f : (kind == 1 ? (__bf16)1.0f : (kind == 2 ? ct[comp][term] : nt[term]));
#endif
    }
    if (which && !RAD_FOLD) {
      T yj[RAD_DIMY > 0 ? RAD_DIMY : 1];
#pragma unroll
      for (int v = 0; v < RAD_NCOLVARS; v++) {
        const T* a = P.arg[rad_col_arg[v]] + i * rad_col_dim[v];
#pragma unroll
        for (int d = 0; d < rad_col_dim[v]; d++) yj[rad_col_off[v] + d] = a[d];
      }
      T wv[RAD_DW];
      KeopsRadFormula::weights(yj, p, wv);
#if RAD_BIL
      // the weights sit in the slot vectors: what is left per column is [y^_j, 1], or 1
      (void)wv;
#if RAD_DIFF != 0
#pragma unroll
      for (int k = 0; k < RAD_D; k++) w[k] = cf[k];
      w[RAD_D] = 1.f;
#else
      w[0] = 1.f;
#endif
#elif RAD_UPAIR
      // the weights as they are, then [y^_j, 1]: the sweep forms <u_i, v_j> itself
#pragma unroll
      for (int d = 0; d < RAD_DW; d++) w[d] = (float)wv[d];
#pragma unroll
      for (int k = 0; k < RAD_D; k++) w[RAD_DW + k] = cf[k];
      w[RAD_DW + RAD_D] = 1.f;
#elif RAD_DIFF != 0
      // component d of the weights against [y^_j, 1]
#pragma unroll
      for (int d = 0; d < RAD_DW; d++) {
#pragma unroll
        for (int k = 0; k < RAD_D; k++) w[d * (RAD_D + 1) + k] = (float)wv[d] * cf[k];
        w[d * (RAD_D + 1) + RAD_D] = (float)wv[d];
      }
#else
#pragma unroll
      for (int d = 0; d < RAD_DV; d++) w[d] = (float)wv[d];
#endif
    }
  } else {
#pragma unroll
    for (int s = 0; s < RAD_SLOTS; s++) slot[s] = (__bf16)0.0f;
  }
  if (!which) {
#pragma unroll
    for (int c8 = 0; c8 < RAD_SLOTS / 8; c8++) {
      rad_bf16x8 v8;
#pragma unroll
      for (int e = 0; e < 8; e++) v8[e] = slot[c8 * 8 + e];
      *reinterpret_cast<rad_bf16x8*>(P.xa + i * RAD_SLOTS + c8 * 8) = v8;
    }
  } else {
#if RAD_FOLD
    // stable partition by the sign of the weight: rank of this column among the non-negative (or negative) ones
    __shared__ int wcnt[4];
    const bool real = i < n, posw = real && !(w[0] < 0.f);
    const unsigned long long bal = __ballot(posw);
    const int lane = threadIdx.x & 63, wv_ = threadIdx.x >> 6;
    if (lane == 0) wcnt[wv_] = __popcll(bal);
    __syncthreads();
    int before = __popcll(bal & ((1ull << lane) - 1ull));
    for (int k = 0; k < wv_; k++) before += wcnt[k];
    const i64 npos_before = (i64)P.blk[blockIdx.x] + before;
    if (!real || w[0] == 0.f) return;  // zero weights: the place stays dead
    const i64 dst = posw ? npos_before : (i64)P.scal[3] * RAD_TJ + (i - npos_before);
    const i64 tile = dst / RAD_TJ;
    const int c = (int)(dst % RAD_TJ);
#else
    const i64 tile = i / RAD_TJ;
    const int c = (int)(i % RAD_TJ);
#endif
#pragma unroll
    for (int kb = 0; kb < RAD_NKB; kb++)
#pragma unroll
      for (int hf = 0; hf < 2; hf++) {
        rad_bf16x8 v8;
#pragma unroll
        for (int e = 0; e < 8; e++) v8[e] = slot[kb * 16 + hf * 8 + e];
        *reinterpret_cast<rad_bf16x8*>(P.yb + (((tile * RAD_NKB + kb) * 2 + hf) * RAD_TJ + c) * 8) = v8;
      }
#if RAD_MM
    rad_store_weights_mm(reinterpret_cast<__bf16*>(P.bw), i, w);
#elif !RAD_FOLD
#pragma unroll
    for (int d = 0; d < RAD_WS; d++) P.bw[i * RAD_WS + d] = w[d];
#endif
  }
}

// the matrix-core path is taken when the kernel is not too narrow for the cloud (see the head of this file)
extern "C" __global__ void __launch_bounds__(64) keops_rad_decide(const RadParams P) {
  if (threadIdx.x != 0) return;
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  rad_load_params(P, p);
  const float kappa = (float)KeopsRadFormula::kappa(p);
  const float R = __uint_as_float(P.scal[0]) + __uint_as_float(P.scal[1]);
  P.scal[2] = (__builtin_fabsf(kappa) * R <= (float)RAD_LIMIT) ? 1u : 0u;  // false for NaN
}
#endif  // !RAD_RANGES

#if RAD_FOLD
// k-th tile of the sweep: tiles of the two sign groups alternate while both last, then the rest of the larger group
__device__ __forceinline__ i64 rad_tile_of(i64 k, i64 pos_tiles, i64 all_tiles, bool& negative) {
  const i64 neg_tiles = all_tiles - pos_tiles, m = pos_tiles < neg_tiles ? pos_tiles : neg_tiles;
  if (k < 2 * m) {
    negative = (k & 1) != 0;
    return negative ? pos_tiles + (k >> 1) : (k >> 1);
  }
  negative = pos_tiles <= neg_tiles;
  return (negative ? pos_tiles : 0) + m + (k - 2 * m);
}
#endif

// ---- main kernel ------------------------------------------------------------------------------------------------

// with at most 32 accumulators per lane the kernel fits 128 registers: four wavefronts per SIMD, two workgroups per CU
#if RAD_MM
#define RAD_MIN_WAVES (RAD_MM_NB > 1 ? 1 : (RAD_RB == 1 ? 4 : 2))  // (several operand blocks: 32 accumulators each)
#else
#define RAD_MIN_WAVES ((RAD_RB * 16 * RAD_DV <= 32) ? (RAD_BIL ? 2 : 4) : 1)  // (RAD_BIL: a second tile of 16 values per block)
#endif

// What one wavefront sweeps: its 32 * RAD_RB rows against the columns [jbeg, jend) of the pre-formatted operand.
struct RadSweep {
  const __bf16* xa;    // slot vectors of the wavefront's rows: [rows_avail][RAD_SLOTS]
  i64 rows_avail;      // rows past the last one are clamped to it (they compute, never store)
  const __bf16* yb;    // column tiles
  const float* bw;     // weights, padded to whole tiles
  i64 jbeg, jend;      // jbeg a multiple of RAD_TJ
  float* part;         // [rows_store][RAD_DV] sums of the wavefront's rows
  i64 rows_store;
  i64 pos_tiles, all_tiles;  // RAD_FOLD
  const T* const* arg;       // RAD_UPAIR: the arguments, for the row factor u_i of the wavefront's rows ...
  i64 row_first, row_last;   // ... which are rows row_first + k of the arguments, clamped to row_last
};

// parameters of the formula from the argument table
__device__ __forceinline__ void rad_params_of(const T* const* arg, T (&p)[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1]) {
#pragma unroll
  for (int v = 0; v < KEOPS_NPARVARS; v++) {
    const T* src = arg[keops_par_arg[v]];
#pragma unroll
    for (int d = 0; d < keops_par_dim[v]; d++) p[keops_par_off[v] + d] = src[d];
  }
}

// All wavefronts of the workgroup call this together with the same columns (they share the staged tile).
__device__ __forceinline__ void rad_sweep(const RadSweep& S, __bf16* ys, float* bs) {
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, col = lane & 31;
  rad_bf16x8 a[RAD_RB][RAD_NKB];
#pragma unroll
  for (int r = 0; r < RAD_RB; r++) {
    i64 i = r * 32 + col;
    if (i >= S.rows_avail) i = S.rows_avail - 1;
#pragma unroll
    for (int kb = 0; kb < RAD_NKB; kb++) a[r][kb] = *reinterpret_cast<const rad_bf16x8*>(S.xa + i * RAD_SLOTS + kb * 16 + 8 * half);
  }
  float acc[RAD_RB][16][RAD_DV];
#pragma unroll
  for (int r = 0; r < RAD_RB; r++)
#pragma unroll
    for (int v = 0; v < 16; v++)
#pragma unroll
      for (int d = 0; d < RAD_DV; d++) acc[r][v][d] = 0.f;
#if RAD_UPAIR
  // the row factor u_i of the 16 rows this lane accumulates, from the arguments themselves
  float ur[RAD_RB][16][RAD_DW];
  {
    T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
    rad_params_of(S.arg, p);
#pragma unroll
    for (int r = 0; r < RAD_RB; r++)
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const i64 gi = keops_min(S.row_first + r * 32 + 8 * (v >> 2) + 4 * half + (v & 3), S.row_last);
        T xi[RAD_DIMX > 0 ? RAD_DIMX : 1];
#pragma unroll
        for (int q = 0; q < RAD_NROWVARS; q++) {
          const T* a_ = S.arg[rad_row_arg[q]] + gi * rad_row_dim[q];
#pragma unroll
          for (int d = 0; d < rad_row_dim[q]; d++) xi[rad_row_off[q] + d] = a_[d];
        }
        T uv[RAD_DU > 0 ? RAD_DU : 1];
        KeopsRadFormula::rowvec(xi, p, uv);
#pragma unroll
        for (int d = 0; d < RAD_DW; d++) ur[r][v][d] = (float)uv[d];
      }
  }
#endif

  const i64 jbeg = S.jbeg, jend = S.jend;
  // software pipeline: tile t+1 travels to registers while tile t is consumed
  constexpr int CH = RAD_NKB * 2 * RAD_TJ;  // 16-byte chunks of the slot vectors of a tile
  constexpr int NPF = (CH + RAD_BLOCK - 1) / RAD_BLOCK;
  constexpr int NPW = (RAD_TJ * RAD_WS + RAD_BLOCK - 1) / RAD_BLOCK;
  uint4 pf[NPF];
#if !RAD_FOLD
  float pfw[NPW];
#endif
  auto prefetch = [&](i64 j0) {
#if RAD_FOLD
    bool neg_;
    const i64 tile = rad_tile_of(j0 / RAD_TJ, S.pos_tiles, S.all_tiles, neg_);
#else
    const i64 tile = j0 / RAD_TJ;
#endif
    const uint4* src = reinterpret_cast<const uint4*>(S.yb + tile * (RAD_NKB * 2 * RAD_TJ * 8));
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * RAD_BLOCK;
      pf[u] = e < CH ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
#if !RAD_FOLD
    const float* wsrc = S.bw + j0 * RAD_WS;  // padded to whole tiles
#pragma unroll
    for (int u = 0; u < NPW; u++) {
      const int e = tid + u * RAD_BLOCK;
      pfw[u] = e < RAD_TJ * RAD_WS ? wsrc[e] : 0.f;
    }
#endif
  };
  if (jbeg < jend) prefetch(jbeg);
  for (i64 j0 = jbeg; j0 < jend; j0 += RAD_TJ) {
    __syncthreads();  // the previous tile has been consumed by every wavefront
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * RAD_BLOCK;
      if (e < CH) reinterpret_cast<uint4*>(ys)[e] = pf[u];
    }
#if !RAD_FOLD
#pragma unroll
    for (int u = 0; u < NPW; u++) {
      const int e = tid + u * RAD_BLOCK;
      if (e < RAD_TJ * RAD_WS) bs[e] = pfw[u];
    }
#endif
    __syncthreads();
    if (j0 + RAD_TJ < jend) prefetch(j0 + RAD_TJ);
#if RAD_FOLD
    bool negative;  // uniform: one sign per tile
    (void)rad_tile_of(j0 / RAD_TJ, S.pos_tiles, S.all_tiles, negative);
#endif
#pragma unroll
    for (int sub = 0; sub < RAD_NSUB; sub++) {
      const int c = sub * 32 + col;
      rad_bf16x8 b[RAD_NKB];
#pragma unroll
      for (int kb = 0; kb < RAD_NKB; kb++) b[kb] = *reinterpret_cast<const rad_bf16x8*>(ys + ((kb * 2 + half) * RAD_TJ + c) * 8);
#if !RAD_FOLD
      float w[RAD_WS];
#pragma unroll
      for (int d = 0; d < RAD_WS; d++) w[d] = bs[c * RAD_WS + d];
#endif
      rad_f32x16 t[RAD_RB];
#if RAD_BIL
      rad_f32x16 t2[RAD_RB];  // <u_i, v_j> of the same pairs
#endif
#pragma unroll
      for (int r = 0; r < RAD_RB; r++) {
        rad_f32x16 z;
#pragma unroll
        for (int v = 0; v < 16; v++) z[v] = 0.f;
#pragma unroll
        for (int kb = 0; kb < RAD_NKE; kb++) z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r][kb], b[kb], z, 0, 0, 0);
        t[r] = z;
#if RAD_BIL
#pragma unroll
        for (int v = 0; v < 16; v++) z[v] = 0.f;
#pragma unroll
        for (int kb = RAD_NKE; kb < RAD_NKB; kb++) z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r][kb], b[kb], z, 0, 0, 0);
        t2[r] = z;
#endif
      }
#if RAD_FOLD
      if (!negative) {
#pragma unroll
        for (int r = 0; r < RAD_RB; r++)
#pragma unroll
          for (int v = 0; v < 16; v++) acc[r][v][0] += __builtin_amdgcn_exp2f(t[r][v]);
      } else {
#pragma unroll
        for (int r = 0; r < RAD_RB; r++)
#pragma unroll
          for (int v = 0; v < 16; v++) acc[r][v][0] -= __builtin_amdgcn_exp2f(t[r][v]);
      }
#else
#pragma unroll
      for (int r = 0; r < RAD_RB; r++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const float e = __builtin_amdgcn_exp2f(t[r][v]);
#if RAD_BIL
          const float es = e * t2[r][v];
#pragma unroll
          for (int d = 0; d < RAD_DV; d++) acc[r][v][d] = __builtin_fmaf(es, w[d], acc[r][v][d]);
#elif RAD_UPAIR
          // K_ij <u_i, v_j> [y^_j, 1]
          float sp = ur[r][v][0] * w[0];
#pragma unroll
          for (int d = 1; d < RAD_DW; d++) sp = __builtin_fmaf(ur[r][v][d], w[d], sp);
          const float es = e * sp;
#pragma unroll
          for (int d = 0; d < RAD_DV; d++) acc[r][v][d] = __builtin_fmaf(es, w[RAD_DW + d], acc[r][v][d]);
#else
#pragma unroll
          for (int d = 0; d < RAD_DV; d++) acc[r][v][d] = __builtin_fmaf(e, w[d], acc[r][v][d]);
#endif
        }
#endif
    }
  }
  // the 32 lanes of a half hold the same rows for different columns: shuffle sums, then one lane stores
#pragma unroll
  for (int r = 0; r < RAD_RB; r++)
#pragma unroll
    for (int v = 0; v < 16; v++) {
      const i64 i = r * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
#pragma unroll
      for (int d = 0; d < RAD_DV; d++) {
        float s = acc[r][v][d];
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o);
        if (col == 0 && i < S.rows_store) S.part[i * RAD_DV + d] = s;
      }
    }
}


#if RAD_MM
// The same sweep with the weighted sum on the matrix cores (3 * RAD_DV <= 32 accumulated components):
//     out[i][d] = sum_j K_ij w_j[d]   is the matrix product   K (32 rows x 32 columns of a sub-tile) x W (32 x RAD_DV).
// The exponent tile is computed transposed (columns as the A operand, the wavefront's rows as B), so that lane l
// receives the 16 values of ITS row l % 32: registers 0-7 and 8-15 are then A operands of two k blocks of the second
// product as they stand.  Float32 accuracy from bfloat16 products: K = h + m + l by truncation (two v_and, two exact
// v_sub, byte permutes to pack: the same vector work per pair whatever RAD_DV is, against v_exp_f32 + RAD_DV fma),
// and the three terms of the weights sit side by side in the 32 operand columns, so three instructions per k block
// form all nine term products; the column groups are added once at the end.  Running sums are folded into a second
// accumulator every RAD_MM_FOLD columns.
__device__ __forceinline__ void rad_sweep_mm(const RadSweep& S, __bf16* ys, __bf16* ws) {
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, col = lane & 31;
  rad_bf16x8 a[RAD_RB][RAD_NKB];
#pragma unroll
  for (int r = 0; r < RAD_RB; r++) {
    i64 i = r * 32 + col;
    if (i >= S.rows_avail) i = S.rows_avail - 1;
#pragma unroll
    for (int kb = 0; kb < RAD_NKB; kb++) a[r][kb] = *reinterpret_cast<const rad_bf16x8*>(S.xa + i * RAD_SLOTS + kb * 16 + 8 * half);
  }
  rad_f32x16 acc[RAD_RB][RAD_MM_NB], tot[RAD_RB][RAD_MM_NB];
#pragma unroll
  for (int r = 0; r < RAD_RB; r++)
#pragma unroll
    for (int nb = 0; nb < RAD_MM_NB; nb++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[r][nb][v] = tot[r][nb][v] = 0.f;

  const i64 jbeg = S.jbeg, jend = S.jend;
  constexpr int CH = RAD_NKB * 2 * RAD_TJ;  // 16-byte chunks of the slot vectors of a tile
  constexpr int NPF = (CH + RAD_BLOCK - 1) / RAD_BLOCK;
  constexpr int CW = RAD_TJ * 4 * RAD_MM_NB;  // 16-byte chunks of the weights of a tile (64 bytes per column and block)
  constexpr int NPW = (CW + RAD_BLOCK - 1) / RAD_BLOCK;
  uint4 pf[NPF], pfw[NPW];
  const __bf16* bwm = reinterpret_cast<const __bf16*>(S.bw);
  auto prefetch = [&](i64 j0) {
    const uint4* src = reinterpret_cast<const uint4*>(S.yb + (j0 / RAD_TJ) * (RAD_NKB * 2 * RAD_TJ * 8));
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * RAD_BLOCK;
      pf[u] = e < CH ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
    const uint4* wsrc = reinterpret_cast<const uint4*>(bwm + j0 * (32 * RAD_MM_NB));  // padded to whole tiles
#pragma unroll
    for (int u = 0; u < NPW; u++) {
      const int e = tid + u * RAD_BLOCK;
      pfw[u] = e < CW ? wsrc[e] : make_uint4(0u, 0u, 0u, 0u);
    }
  };
  if (jbeg < jend) prefetch(jbeg);
  i64 since_fold = 0;
  for (i64 j0 = jbeg; j0 < jend; j0 += RAD_TJ) {
    __syncthreads();  // the previous tile has been consumed by every wavefront
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * RAD_BLOCK;
      if (e < CH) reinterpret_cast<uint4*>(ys)[e] = pf[u];
    }
#pragma unroll
    for (int u = 0; u < NPW; u++) {
      const int e = tid + u * RAD_BLOCK;
      if (e < CW) reinterpret_cast<uint4*>(ws)[e] = pfw[u];
    }
    __syncthreads();
    if (j0 + RAD_TJ < jend) prefetch(j0 + RAD_TJ);
#pragma unroll
    for (int sub = 0; sub < RAD_NSUB; sub++) {
      const int c = sub * 32 + col;
      rad_bf16x8 b[RAD_NKB], wk[2][RAD_MM_NB];
#pragma unroll
      for (int kb = 0; kb < RAD_NKB; kb++) b[kb] = *reinterpret_cast<const rad_bf16x8*>(ys + ((kb * 2 + half) * RAD_TJ + c) * 8);
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int nb = 0; nb < RAD_MM_NB; nb++)
          wk[kb][nb] = *reinterpret_cast<const rad_bf16x8*>(ws + (((sub * 2 + kb) * 2 + half) * (32 * RAD_MM_NB) + 32 * nb + col) * 8);
#pragma unroll
      for (int r = 0; r < RAD_RB; r++) {
        rad_f32x16 z;
#pragma unroll
        for (int v = 0; v < 16; v++) z[v] = 0.f;
        // transposed: z[v] = exponent of (row l % 32, column 8 (v / 4) + 4 (l / 32) + v % 4 of the sub-tile)
#pragma unroll
        for (int kb = 0; kb < RAD_NKE; kb++) z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[kb], a[r][kb], z, 0, 0, 0);
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#if RAD_MM_TERMS == 2
          // K = h + m: h the bfloat16 nearest to K, m the bfloat16 nearest to the (exact) rest, |K - h - m| <= 2^-17 K
          // with either sign (an option: forty times the float32 rounding).  v_cvt_pk_bf16_f32 rounds and packs two values at once; a shift / a mask give h back as
          // a float.
          uint4 ph, pm;
          unsigned* php = reinterpret_cast<unsigned*>(&ph);
          unsigned* pmp = reinterpret_cast<unsigned*>(&pm);
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float x0 = __builtin_amdgcn_exp2f(z[8 * kb + 2 * e]), x1 = __builtin_amdgcn_exp2f(z[8 * kb + 2 * e + 1]);
            const rad_f32x2 xx = {x0, x1};
            const unsigned hp = __builtin_bit_cast(unsigned, __builtin_convertvector(xx, rad_bf16x2));
            php[e] = hp;
            const rad_f32x2 rr = {x0 - __uint_as_float(hp << 16), x1 - __uint_as_float(hp & 0xffff0000u)};
            pmp[e] = __builtin_bit_cast(unsigned, __builtin_convertvector(rr, rad_bf16x2));
          }
          const rad_bf16x8 kh = __builtin_bit_cast(rad_bf16x8, ph), km = __builtin_bit_cast(rad_bf16x8, pm);
#pragma unroll
          for (int nb = 0; nb < RAD_MM_NB; nb++) {
            acc[r][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(km, wk[kb][nb], acc[r][nb], 0, 0, 0);
            acc[r][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kh, wk[kb][nb], acc[r][nb], 0, 0, 0);
          }
#else
          // K = h + m + l, each the truncation of what is left to 8 significant bits (the subtractions are exact); a
          // byte permute packs the high halves of two floats: the bfloat16 terms.  (v_dot2_f32_bf16 against the pairs
          // (-1, 0) / (0, -1) subtracts a packed term in one instruction instead of v_and + v_sub: measured, same time.)
          uint4 ph, pm, pl;
          unsigned* php = reinterpret_cast<unsigned*>(&ph);
          unsigned* pmp = reinterpret_cast<unsigned*>(&pm);
          unsigned* plp = reinterpret_cast<unsigned*>(&pl);
#pragma unroll
          for (int e = 0; e < 4; e++) {
            const float x0 = __builtin_amdgcn_exp2f(z[8 * kb + 2 * e]), x1 = __builtin_amdgcn_exp2f(z[8 * kb + 2 * e + 1]);
            php[e] = __builtin_amdgcn_perm(__float_as_uint(x1), __float_as_uint(x0), 0x07060302u);
            const float r0 = x0 - __uint_as_float(__float_as_uint(x0) & 0xffff0000u);
            const float r1 = x1 - __uint_as_float(__float_as_uint(x1) & 0xffff0000u);
            pmp[e] = __builtin_amdgcn_perm(__float_as_uint(r1), __float_as_uint(r0), 0x07060302u);
            const float s0 = r0 - __uint_as_float(__float_as_uint(r0) & 0xffff0000u);
            const float s1 = r1 - __uint_as_float(__float_as_uint(r1) & 0xffff0000u);
            plp[e] = __builtin_amdgcn_perm(__float_as_uint(s1), __float_as_uint(s0), 0x07060302u);
          }
          const rad_bf16x8 kh = __builtin_bit_cast(rad_bf16x8, ph), km = __builtin_bit_cast(rad_bf16x8, pm),
                           kl = __builtin_bit_cast(rad_bf16x8, pl);
          // smallest terms first
#pragma unroll
          for (int nb = 0; nb < RAD_MM_NB; nb++) {
            acc[r][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kl, wk[kb][nb], acc[r][nb], 0, 0, 0);
            acc[r][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(km, wk[kb][nb], acc[r][nb], 0, 0, 0);
            acc[r][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kh, wk[kb][nb], acc[r][nb], 0, 0, 0);
          }
#endif
        }
      }
    }
    since_fold += RAD_TJ;
    if (since_fold >= RAD_MM_FOLD) {
      since_fold = 0;
#pragma unroll
      for (int r = 0; r < RAD_RB; r++)
#pragma unroll
        for (int nb = 0; nb < RAD_MM_NB; nb++)
#pragma unroll
          for (int v = 0; v < 16; v++) {
            tot[r][nb][v] += acc[r][nb][v];
            acc[r][nb][v] = 0.f;
          }
    }
  }
  // lane l holds operand column l % 32 of rows 8 (v / 4) + 4 (l / 32) + v % 4: the three column groups
  // (terms of the weights) are added with shuffles, lanes d < RAD_DV store
#pragma unroll
  for (int r = 0; r < RAD_RB; r++)
#pragma unroll
    for (int v = 0; v < 16; v++) {
      // term t of component d = lane % 32 sits in operand column t * RAD_DV + d: block (column / 32), lane (column % 32)
      // of the same half
      float term[3];
#pragma unroll
      for (int t = 0; t < 3; t++) {
        const int c = t * RAD_DV + col;
        float got = 0.f;
#pragma unroll
        for (int nb = 0; nb < RAD_MM_NB; nb++) {
          const float cand = __shfl(tot[r][nb][v] + acc[r][nb][v], 32 * half + (c & 31));
          got = (c >> 5) == nb ? cand : got;
        }
        term[t] = got;
      }
      // (smallest group first)
      const float s = (term[2] + term[1]) + term[0];
      const i64 i = r * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
      if (col < RAD_DV && i < S.rows_store) S.part[i * RAD_DV + col] = s;
    }
}
#endif

#if !RAD_RANGES
extern "C" __global__ void __launch_bounds__(RAD_BLOCK, RAD_MIN_WAVES) keops_rad_main(const RadParams P) {
  if (P.scal[2] != 1u) return;
  __shared__ __attribute__((aligned(16))) __bf16 ys[RAD_NKB * 2 * RAD_TJ * 8];  // [kb][half][col][8]
#if RAD_MM
  __shared__ __attribute__((aligned(16))) __bf16 ws[RAD_TJ * 32 * RAD_MM_NB];  // [sub-tile][k block][half][operand column][8]
#elif !RAD_FOLD
  __shared__ __attribute__((aligned(16))) float bs[RAD_TJ * RAD_WS];
#else
  float* bs = nullptr;
#endif
  const int wave = threadIdx.x >> 6;
  const i64 row0 = ((i64)blockIdx.x * RAD_WAVES + wave) * (32 * RAD_RB);
  // (RAD_FOLD: the partition by sign pads both groups to whole tiles: one more tile than the columns need)
  const i64 ncols = RAD_FOLD ? ((P.ny + RAD_TJ - 1) / RAD_TJ + 1) * RAD_TJ : P.ny;
  RadSweep S;
  // a wavefront past the last row sweeps the last row again (the workgroup's barriers need it) and stores nothing
  const i64 first = row0 < P.nx ? row0 : P.nx - 1;
  S.xa = P.xa + first * RAD_SLOTS;
  S.rows_avail = P.nx - first;
  S.yb = P.yb;
  S.bw = P.bw;
  S.jbeg = (i64)blockIdx.y * P.slab_len;
  S.jend = keops_min(ncols, S.jbeg + P.slab_len);
  S.part = P.partial + ((i64)blockIdx.y * P.nx + first) * RAD_DV;
  S.rows_store = row0 < P.nx ? P.nx - row0 : 0;
  S.pos_tiles = RAD_FOLD ? keops_uniform((i64)P.scal[3]) : 0;  // tiles of columns with non-negative weights come first
  S.all_tiles = ncols / RAD_TJ;
  S.arg = P.arg;
  S.row_first = first;
  S.row_last = P.nx - 1;
#if RAD_MM
  rad_sweep_mm(S, ys, ws);
#else
  rad_sweep(S, ys, bs);
#endif
}
#endif

#if !RAD_RANGES
// slabs are added in order; the factors of the output index and, for the gradients with respect to the points, the
// difference x^_i S - sum_j K_ij w_j y^_j are applied here, once per output row
extern "C" __global__ void __launch_bounds__(256) keops_rad_reduce(const RadParams P) {
  if (P.scal[2] != 1u) return;
  const i64 i = (i64)blockIdx.x * 256 + threadIdx.x;
  if (i >= P.nx) return;
  float s[RAD_DV];
#pragma unroll
  for (int d = 0; d < RAD_DV; d++) s[d] = P.partial[i * RAD_DV + d];
  for (int k = 1; k < P.nslabs; k++)
#pragma unroll
    for (int d = 0; d < RAD_DV; d++) s[d] += P.partial[((i64)k * P.nx + i) * RAD_DV + d];
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  rad_load_params(P, p);
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
    const float xc = (float)((double)x[k] - (double)P.colsum[k]);
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
#else
#include "keops_radial_ranges.h"
#endif
