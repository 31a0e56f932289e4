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
// exponent wherever |k| (|x^|^2 + |y^|^2) is moderate, which the kernels check PER TILE: both clouds are sorted by
// that quantity (a stable counting sort on RAD_NBK buckets, so that the points of a tile have similar norms and the
// summation order is reproducible), and a wavefront takes the exponents of a 32-column sub-tile from the matrix cores
// only when  max over its rows + max over the sub-tile's columns <= RAD_LIMIT  (a-priori error of a kernel value
// 3.3e-7 * RAD_LIMIT).  The other sub-tiles -- the shell of the cloud against itself, an outlier against everything --
// are left out by the sweep and computed by keops_rad_exact, launched behind it, from exact float32 differences in the
// reference's own operation order (difference, square, sum without contraction, one rounded product with the
// coefficient, then an exponential good to 2 ulp); it adds its sums to the sweep's.
// keops_rad_decide estimates the share of such pairs from the bucket counts and sets a flag: when more than
// RAD_EXACT_FRAC of the pairs would take the slow path (a kernel much narrower than the cloud), the kernels of this
// file return at once and the general-purpose kernel of the same module, which is launched behind them and returns
// at once in the other case, computes the whole sum from exact differences.  No host synchronisation.
//
// Work decomposition: lane l of a wavefront owns column j = l % 32 of the staged sub-tile (its slot vector is the B
// operand, its weights B_j sit in registers) and, after the instruction, the 16 exponents of rows
// 8 (v / 4) + 4 (l / 32) + v % 4; it accumulates exp2(t) * B_j per row and component in registers for the whole
// sweep.  A wavefront holds RAD_RB blocks of 32 rows (A operands in VGPRs), RAD_WAVES wavefronts share the staged
// column tile (slot vectors pre-formatted by keops_rad_prep: straight 16-byte copies, conflict-free 16-byte reads).
// The lanes of a row are summed with shuffles once at the end; slabs over the reduced axis (blockIdx.y) are added
// in order by keops_rad_reduce: deterministic.
//
// The plug-in defines RAD_D, RAD_DV, RAD_NKB (16-slot blocks), RAD_RB, RAD_WAVES, RAD_XARG, RAD_YARG, RAD_LIMIT,
// the slot tables rad_slot_kind / rad_slot_comp / rad_slot_term for both sides, the tables of the variables of B
// (rad_col_arg / rad_col_dim / rad_col_off, RAD_NCOLVARS, RAD_DIMY) and of the parameters (keops_par_*), and
// the tables of the variables of A (rad_row_*, RAD_NROWVARS, RAD_DIMX), RAD_DW (components of W), RAD_DU (components of
// a row vector u_i that multiplies W as <u_i, W_j>: KeopsRadFormula::rowvec), RAD_DOUT, RAD_DIFF,
// RAD_SIGN and struct KeopsRadFormula { coef(p); kappa(p); weights(yj, p, w); rowscale(xi, p) }.
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

#ifndef RAD_RANGES
#define RAD_RANGES 0
#endif
// Per-tile choice between matrix-core exponents and exact differences (dense launches; the block-sparse variant has
// one centre per row range and decides per range).
#define RAD_TILEWISE (!RAD_RANGES)
#define RAD_NBK 128                // buckets of the counting sort by |k| |x^|^2: [0, RAD_LIMIT) in equal parts, the last one open
#define RAD_SORT_CHUNK 1024        // points per workgroup of the sort (4 rounds of 256)
// keops_rad_exact: floats per column of its operand: original coordinates | centred coordinates (gradients with respect
// to the points) | the weights as the formula gives them, each part padded to 16 bytes
#define RADX_XD ((RAD_D + 3) / 4 * 4)
#define RADX_XC (RAD_DIFF != 0 ? RADX_XD : 0)
#define RADX_XWT ((RAD_DW + 3) / 4 * 4)
#define RADX_XW (RADX_XD + RADX_XC + RADX_XWT)
#ifndef RAD_EXACT_FRAC
#define RAD_EXACT_FRAC 0.25f       // largest estimated share of pairs from exact differences for which this family still runs
#endif

struct RadParams {
  i64 nx, ny;
  __bf16* xa;         // [nx][RAD_SLOTS] row-side slot vectors, rows in sorted order
  __bf16* yb;         // [tile][RAD_NKB][2][RAD_TJ][8] column-side slot vectors, tile by tile, columns in sorted order
  float* bw;          // [ntiles * RAD_TJ][RAD_DV] weights B_j (zero past the last column)
  float* colsum;      // [RAD_D] column sums of y
  float* colpart;     // [nparts][RAD_D]
  unsigned* scal;     // [0], [1]: bit patterns of max |x^|^2, max |y^|^2; [2]: 1 when the matrix-core path is taken
  int* hist[2];       // rows, columns: [RAD_NBK][nblk] points per bucket and sort chunk, then their exclusive scan per bucket
  int* btot[2];       // [RAD_NBK] points per bucket, then (keops_rad_decide) their exclusive scan: first sorted position of a bucket
  unsigned char* bkt[2];  // [n] bucket of every point
  int* perm[2];       // [n (columns: padded to whole tiles)] sorted position -> point (-1: padding)
  float* qn[2];       // ... and |k| |x^|^2 of that point, rounded up
  float* gmax[2];     // largest qn of every group of sorted points: rows by 32 * RAD_RB (a wavefront's rows), columns by RAD_TJ (a tile)
  T* out;             // [nx][RAD_DOUT]
  float* partial;     // [nslabs][nx][RAD_DV], rows in sorted order
  float* yo;          // [ntiles * RAD_TJ][RADX_XW] what keops_rad_exact needs of a column, columns in sorted order
  float* xpart;       // [nseg][nx][RAD_DV] sums of keops_rad_exact (only the rows that meet a tile beyond the bound are written)
  float* segmax;      // [nseg] largest qn of the columns of every segment
  i64 slab_len;       // reduced rows per slab (multiple of RAD_TJ)
  i64 seg_len;        // reduced rows per segment of keops_rad_exact (multiple of RAD_TJ)
  int nslabs;
  int nseg;
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

// The centre only has to lie inside the cloud (the bound of a tile grows with the centred norms); the mean does not
// when a few columns are very far away (one at 1e9 cloud radii among 1e6 moves it by 1e3 radii, and every tile is then
// beyond the bound).  One workgroup per component: median and quartiles of 1024 evenly spaced columns (bitonic sort
// in LDS, values that are not finite last); a mean further than four interquartile ranges from the median, or not a
// number, is replaced by the median.  Ordinary data keep their mean.
extern "C" __global__ void __launch_bounds__(256) keops_rad_centre(const RadParams P) {
  __shared__ float v[1024];
  __shared__ int nfin;
  const int c = blockIdx.x, tid = threadIdx.x;
  if (c >= RAD_D) return;
  if (tid == 0) nfin = 0;
  __syncthreads();
  const T* y = P.arg[RAD_YARG];
  const i64 ns = P.ny < 1024 ? P.ny : 1024, step = ns > 0 ? P.ny / ns : 1;
  int mine = 0;
#pragma unroll
  for (int t = 0; t < 4; t++) {
    const int k = tid + 256 * t;
    float a = __builtin_inff();
    if (k < ns) {
      const float w = (float)y[(i64)k * step * RAD_D + c];
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
    const float mean = P.colsum[c];
    if (!(__builtin_fabsf(mean - med) <= 4.f * iqr + 1e-3f * __builtin_fabsf(med) + 1e-30f)) P.colsum[c] = med;
  }
}

// |k| |x^|^2 of a point (x^: the point minus the mean of y, in double precision) and its bucket
__device__ __forceinline__ double rad_centred_norm(const RadParams& P, const T* src) {
  double nrm = 0.0;
#pragma unroll
  for (int k = 0; k < RAD_D; k++) {
    const double c = (double)src[k] - (double)P.colsum[k];
    nrm += c * c;
  }
  return nrm;
}
__device__ __forceinline__ int rad_bucket_of(double q) {
  // NaN and everything from RAD_LIMIT on: the last bucket
  return q < (double)RAD_LIMIT ? (int)(q * ((double)(RAD_NBK - 1) / (double)RAD_LIMIT)) : RAD_NBK - 1;
}

// Counting sort by |k| |x^|^2, pass 1: bucket of every point and points per (bucket, chunk of RAD_SORT_CHUNK points).
// which = 0: rows (x), 1: columns (y).
extern "C" __global__ void __launch_bounds__(256) keops_rad_bucket(const RadParams P, int which) {
  __shared__ int h[RAD_NBK];
  const i64 n = which ? P.ny : P.nx;
  for (int b = threadIdx.x; b < RAD_NBK; b += 256) h[b] = 0;
  __syncthreads();
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  rad_load_params(P, p);
  const double ak = __builtin_fabs((double)KeopsRadFormula::kappa(p));
  const T* base = P.arg[which ? RAD_YARG : RAD_XARG];
  float nmax = 0.f;
#pragma unroll
  for (int r = 0; r < RAD_SORT_CHUNK / 256; r++) {
    const i64 i = (i64)blockIdx.x * RAD_SORT_CHUNK + r * 256 + threadIdx.x;
    if (i < n) {
      const double nrm = rad_centred_norm(P, base + i * RAD_D);
      const int b = rad_bucket_of(ak * nrm);
      P.bkt[which][i] = (unsigned char)b;
      atomicAdd(&h[b], 1);
      const float nf = (float)nrm * 1.000001f;
      nmax = nf > nmax ? nf : nmax;
    }
  }
  // largest centred squared norm (bit pattern of a non-negative float, rounded up): order-independent maximum, one
  // atomic per wavefront
  {
    unsigned bits = __float_as_uint(nmax);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const unsigned other = (unsigned)__shfl_xor((int)bits, o);
      bits = other > bits ? other : bits;
    }
    if ((threadIdx.x & 63) == 0) atomicMax(P.scal + which, bits);
  }
  __syncthreads();
  for (int b = threadIdx.x; b < RAD_NBK; b += 256) P.hist[which][(i64)b * gridDim.x + blockIdx.x] = h[b];
}

// pass 2: exclusive scan of the counts of every bucket over the chunks (one workgroup per bucket and cloud, the
// counts of a bucket are contiguous) and the points per bucket.  The first sorted position of (bucket, chunk) is the
// scan of the bucket totals, done by keops_rad_decide, plus this.
extern "C" __global__ void __launch_bounds__(256) keops_rad_scan(const RadParams P, int nblk_r, int nblk_c) {
  __shared__ int part[256];
  const int which = blockIdx.y, b = blockIdx.x, t = threadIdx.x;
  const int nblk = which ? nblk_c : nblk_r;
  int* h = P.hist[which] + (i64)b * nblk;
  const int per = (nblk + 255) / 256, lo = keops_min(nblk, t * per), hi = keops_min(nblk, lo + per);
  int s = 0;
  for (int k = lo; k < hi; k++) s += h[k];
  part[t] = s;
  __syncthreads();
  for (int o = 1; o < 256; o <<= 1) {
    const int v = t >= o ? part[t - o] : 0;
    __syncthreads();
    part[t] += v;
    __syncthreads();
  }
  int run = part[t] - s;
  for (int k = lo; k < hi; k++) {
    const int c = h[k];
    h[k] = run;
    run += c;
  }
  if (t == 255) P.btot[which][b] = part[255];
}
#endif  // !RAD_RANGES

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
// pass 3: slot vector of every point, written at its sorted position.  which = 0: rows (x), 1: columns (y; the
// places past the last column of the padded tile grid receive zero vectors and zero weights).  Stable: the points of
// a bucket keep their order (chunks in order, rounds in order, wavefronts in order, lanes in order).
extern "C" __global__ void __launch_bounds__(256) keops_rad_prep(const RadParams P, int which) {
  __shared__ int cnt[RAD_NBK];
  const i64 n = which ? P.ny : P.nx;
  const i64 ntot = which ? (P.ny + RAD_TJ - 1) / RAD_TJ * RAD_TJ : P.nx;
  const int nblk = (int)((n + RAD_SORT_CHUNK - 1) / RAD_SORT_CHUNK);  // chunks that hold points (the grid may be longer)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int b = threadIdx.x; b < RAD_NBK; b += 256) cnt[b] = 0;
  __syncthreads();
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  rad_load_params(P, p);
  const double kappa = (double)KeopsRadFormula::kappa(p);
  for (int r = 0; r < RAD_SORT_CHUNK / 256; r++) {
    const i64 i = (i64)blockIdx.x * RAD_SORT_CHUNK + r * 256 + threadIdx.x;
    const bool real = i < n;
    // rank of the point among the points of its bucket in this chunk
    const int b = real ? (int)P.bkt[which][i] : 0;
    unsigned long long same = __ballot(real);
#pragma unroll
    for (int bit = 0; bit < 7; bit++) {
      const bool set = (b >> bit) & 1;
      const unsigned long long bal = __ballot(set);
      same &= set ? bal : ~bal;
    }
    int rank = 0;
    for (int w = 0; w < 4; w++) {
      if (wave == w && real) {
        const int before = cnt[b];
        rank = before + __popcll(same & ((1ull << lane) - 1ull));
        if ((same >> lane) == 1ull) cnt[b] = before + __popcll(same);  // the highest lane of the group
      }
      __syncthreads();
    }
    if (i >= ntot) continue;
    const i64 pos = real ? (i64)P.btot[which][b] + P.hist[which][(i64)b * nblk + blockIdx.x] + rank : i;

    __bf16 slot[RAD_SLOTS];
    float w[RAD_WS];
#pragma unroll
    for (int d = 0; d < RAD_WS; d++) w[d] = 0.f;
    float q = 0.f;
    if (real) {
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
      rad_split4(kappa * nrm, nt);
      q = (float)(__builtin_fabs(kappa) * nrm) * 1.000001f;
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
      if (which) {
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
    P.perm[which][pos] = real ? (int)i : -1;
    P.qn[which][pos] = q;
#if RAD_TILEWISE
    if (which) {
      // the column as keops_rad_exact reads it (zeros past the last column)
      float* yo = P.yo + pos * RADX_XW;
#pragma unroll
      for (int d = 0; d < RADX_XW; d++) yo[d] = 0.f;
      if (real) {
        const T* src = P.arg[RAD_YARG] + i * RAD_D;
#pragma unroll
        for (int d = 0; d < RAD_D; d++) yo[d] = (float)src[d];
#if RAD_DIFF != 0
#pragma unroll
        for (int d = 0; d < RAD_D; d++) yo[RADX_XD + d] = (float)((double)src[d] - (double)P.colsum[d]);
#endif
        T yj[RAD_DIMY > 0 ? RAD_DIMY : 1], wv[RAD_DW];
#pragma unroll
        for (int v = 0; v < RAD_NCOLVARS; v++) {
          const T* a = P.arg[rad_col_arg[v]] + i * rad_col_dim[v];
#pragma unroll
          for (int d = 0; d < rad_col_dim[v]; d++) yj[rad_col_off[v] + d] = a[d];
        }
        KeopsRadFormula::weights(yj, p, wv);
#pragma unroll
        for (int d = 0; d < RAD_DW; d++) yo[RADX_XD + RADX_XC + d] = (float)wv[d];
      }
    }
#endif
    if (!which) {
#pragma unroll
      for (int c8 = 0; c8 < RAD_SLOTS / 8; c8++) {
        rad_bf16x8 v8;
#pragma unroll
        for (int e = 0; e < 8; e++) v8[e] = slot[c8 * 8 + e];
        *reinterpret_cast<rad_bf16x8*>(P.xa + pos * RAD_SLOTS + c8 * 8) = v8;
      }
    } else {
      const i64 tile = pos / RAD_TJ;
      const int c = (int)(pos % RAD_TJ);
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
      rad_store_weights_mm(reinterpret_cast<__bf16*>(P.bw), pos, w);
#else
#pragma unroll
      for (int d = 0; d < RAD_WS; d++) P.bw[pos * RAD_WS + d] = w[d];
#endif
    }
  }
}

// pass 4: largest |k| |x^|^2 of the rows of every wavefront of the sweep (32 * RAD_RB sorted rows) and of the columns
// of every tile (RAD_TJ sorted columns); one wavefront per group
extern "C" __global__ void __launch_bounds__(256) keops_rad_groupmax(const RadParams P) {
  const i64 gr = (P.nx + 32 * RAD_RB - 1) / (32 * RAD_RB), gc = (P.ny + RAD_TJ - 1) / RAD_TJ;
  i64 g = (i64)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (g >= gr + gc) return;
  const int which = g >= gr, lane = threadIdx.x & 63;
  if (which) g -= gr;
  const i64 len = which ? RAD_TJ : 32 * RAD_RB, n = which ? gc * RAD_TJ : P.nx;
  const float* q = P.qn[which] + g * len;
  float m = 0.f;
  for (i64 k = lane; k < len && g * len + k < n; k += 64) m = q[k] > m ? q[k] : m;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float other = __shfl_xor(m, o);
    m = other > m ? other : m;
  }
  if (lane == 0) P.gmax[which][g] = m;
}

// largest |k| |y^|^2 of every column segment of keops_rad_exact (one wavefront per segment)
extern "C" __global__ void __launch_bounds__(64) keops_rad_segmax(const RadParams P) {
  const i64 ntile = (P.ny + RAD_TJ - 1) / RAD_TJ, per = P.seg_len / RAD_TJ;
  const i64 t0 = (i64)blockIdx.x * per, t1 = keops_min(ntile, t0 + per);
  float m = 0.f;
  for (i64 t = t0 + threadIdx.x; t < t1; t += 64) {
    const float q = P.gmax[1][t];
    m = q > m ? q : m;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float other = __shfl_xor(m, o);
    m = other > m ? other : m;
  }
  if (threadIdx.x == 0) P.segmax[blockIdx.x] = m;
}

// The matrix-core path is taken unless too many pairs would fall back to exact differences.  Estimate from the
// bucket counts: a pair of buckets (a, b) needs exact differences when a + b + 1 > RAD_NBK - 1 (mid-point rule on
// the bucket edges); the last bucket (everything from RAD_LIMIT on) is bad against every column.
extern "C" __global__ void __launch_bounds__(RAD_NBK) keops_rad_decide(const RadParams P) {
  __shared__ double hy[RAD_NBK], bad[RAD_NBK];
  __shared__ int cnt[2][RAD_NBK];
  const int b = threadIdx.x;
  cnt[0][b] = P.btot[0][b];
  cnt[1][b] = P.btot[1][b];
  hy[b] = (double)cnt[1][b];
  __syncthreads();
  double suffix = 0.0;  // columns in buckets >= RAD_NBK - 1 - b
  for (int k = RAD_NBK - 1 - b; k < RAD_NBK; k++) suffix += hy[k];
  bad[b] = (double)cnt[0][b] * suffix;
  // first sorted position of every bucket
  if (b < 2) {
    int run = 0;
    for (int k = 0; k < RAD_NBK; k++) {
      P.btot[b][k] = run;
      run += cnt[b][k];
    }
  }
  __syncthreads();
  if (b != 0) return;
  double total = 0.0;
  for (int k = 0; k < RAD_NBK; k++) total += bad[k];
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  rad_load_params(P, p);
  const float kappa = (float)KeopsRadFormula::kappa(p);
  const bool finite = __builtin_fabsf(kappa) <= 3.0e38f;  // false for NaN
  P.scal[2] = (finite && total <= (double)RAD_EXACT_FRAC * (double)P.nx * (double)P.ny) ? 1u : 0u;
}
#endif  // !RAD_RANGES

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
  const T* const* arg;       // the arguments (RAD_UPAIR: the row factor u_i of the wavefront's rows; exact sub-tiles: x, y) ...
  i64 row_first, row_last;   // ... whose rows row_first + k, clamped to row_last, are the wavefront's rows
  // RAD_TILEWISE: sorted position -> point for the rows (indexed by row_first + k), the largest |k| |y^|^2 of every
  // tile of sorted columns and the largest |k| |x^|^2 of the wavefront's rows
  const int* rperm;
  const float* ctmax;
  float xq;
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

// exp(coef * s) the way the reference evaluates it: one rounded product, then an exponential good to 2 ulp whatever the
// size of the argument (the product with log2(e) in two parts: the hardware exp2 of a single rounded product would be
// off by 2^-24 |argument|)
__device__ __forceinline__ float rad_exp_of(float coef, float s) {
#pragma clang fp contract(off)
  const float u = coef * s;
  const float th = u * 1.44269502162933349609375f;
  const float tl = __builtin_fmaf(u, 1.925963033500011e-08f, __builtin_fmaf(u, 1.44269502162933349609375f, -th));
  const float e = __builtin_amdgcn_exp2f(th);
  // (an infinite argument leaves tl undefined: exp2 has already given 0 or infinity)
  return (e > 0.f && e < __builtin_inff()) ? __builtin_fmaf(e, tl * 0.693147180559945f, e) : e;
}

// squared distance in the reference's operation order (difference, square, sequential sum; no contraction)
__device__ __forceinline__ float rad_sqdist_exact(const float* x, const float (&y)[RAD_D]) {
#pragma clang fp contract(off)
  const float d0 = x[0] - y[0];
  float s = d0 * d0;
#pragma unroll
  for (int k = 1; k < RAD_D; k++) {
    const float d = x[k] - y[k];
    const float sq = d * d;
    s = s + sq;
  }
  return s;
}

// original row of the wavefront's k-th row
__device__ __forceinline__ i64 rad_row_of(const RadSweep& S, i64 k) {
  const i64 i = keops_min(S.row_first + k, S.row_last);
#if RAD_TILEWISE
  return (i64)S.rperm[i];
#else
  return i;
#endif
}

// All wavefronts of the workgroup call this together with the same columns (they share the staged tile).
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
        const i64 gi = rad_row_of(S, r * 32 + 8 * (v >> 2) + 4 * half + (v & 3));
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
  float pfw[NPW];
#if RAD_TILEWISE
  float pfq = 0.f;  // largest |k| |y^|^2 of the tile in flight
#endif
  auto prefetch = [&](i64 j0) {
    const i64 tile = j0 / RAD_TJ;
    const uint4* src = reinterpret_cast<const uint4*>(S.yb + tile * (RAD_NKB * 2 * RAD_TJ * 8));
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * RAD_BLOCK;
      pf[u] = e < CH ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
    const float* wsrc = S.bw + j0 * RAD_WS;  // padded to whole tiles
#pragma unroll
    for (int u = 0; u < NPW; u++) {
      const int e = tid + u * RAD_BLOCK;
      pfw[u] = e < RAD_TJ * RAD_WS ? wsrc[e] : 0.f;
    }
#if RAD_TILEWISE
    pfq = S.ctmax[tile];
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
#pragma unroll
    for (int u = 0; u < NPW; u++) {
      const int e = tid + u * RAD_BLOCK;
      if (e < RAD_TJ * RAD_WS) bs[e] = pfw[u];
    }
#if RAD_TILEWISE
    // the tile's norms, with those of the wavefront's rows, beyond what the matrix-core exponents are good for: the
    // wavefront leaves the tile to keops_rad_exact (same test there; wavefront-uniform)
    const bool skip = !(pfq + S.xq <= (float)RAD_LIMIT);
#endif
    __syncthreads();
    if (j0 + RAD_TJ < jend) prefetch(j0 + RAD_TJ);
#if RAD_TILEWISE
    if (skip) continue;
#endif
#pragma unroll
    for (int sub = 0; sub < RAD_NSUB; sub++) {
      const int c = sub * 32 + col;
      rad_bf16x8 b[RAD_NKB];
#pragma unroll
      for (int kb = 0; kb < RAD_NKB; kb++) b[kb] = *reinterpret_cast<const rad_bf16x8*>(ys + ((kb * 2 + half) * RAD_TJ + c) * 8);
      float w[RAD_WS];
#pragma unroll
      for (int d = 0; d < RAD_WS; d++) w[d] = bs[c * RAD_WS + d];
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
    }
  }
  // the 32 lanes of a half hold the same rows for different columns: shuffle sums; lane v of the half keeps the sum
  // of row v, so that one store per row block covers its 32 rows
#pragma unroll
  for (int r = 0; r < RAD_RB; r++) {
    float keep[RAD_DV];
#pragma unroll
    for (int d = 0; d < RAD_DV; d++) keep[d] = 0.f;
#pragma unroll
    for (int v = 0; v < 16; v++) {
#pragma unroll
      for (int d = 0; d < RAD_DV; d++) {
        float s = acc[r][v][d];
#pragma unroll
        for (int o = 16; o > 0; o >>= 1) s += __shfl_xor(s, o);
        if (col == v) keep[d] = s;
      }
    }
    const i64 i = r * 32 + 8 * (col >> 2) + 4 * half + (col & 3);
    if (col < 16 && i < S.rows_store) {
#pragma unroll
      for (int d = 0; d < RAD_DV; d++) S.part[i * RAD_DV + d] = keep[d];
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
#if RAD_TILEWISE
  float pfq = 0.f;  // largest |k| |y^|^2 of the tile in flight
#endif
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
#if RAD_TILEWISE
    pfq = S.ctmax[j0 / RAD_TJ];
#endif
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
#if RAD_TILEWISE
    const bool skip = !(pfq + S.xq <= (float)RAD_LIMIT);  // left to keops_rad_exact (see rad_sweep)
#endif
    __syncthreads();
    if (j0 + RAD_TJ < jend) prefetch(j0 + RAD_TJ);
#if RAD_TILEWISE
    if (skip) continue;
#endif
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
#else
  __shared__ __attribute__((aligned(16))) float bs[RAD_TJ * RAD_WS];
#endif
  const int wave = threadIdx.x >> 6;
  // (both clouds are sorted by increasing norm: the workgroups of the last rows and the last slab leave the most
  // tiles to keops_rad_exact, so the launch ends on the workgroups that have the least to do)
  const i64 bx = (i64)blockIdx.x, by = (i64)blockIdx.y;
  const i64 row0 = (bx * RAD_WAVES + wave) * (32 * RAD_RB);
  RadSweep S;
  // a wavefront past the last row sweeps the last row again (the workgroup's barriers need it) and stores nothing
  const i64 first = row0 < P.nx ? row0 : P.nx - 1;
  S.xa = P.xa + first * RAD_SLOTS;
  S.rows_avail = P.nx - first;
  S.yb = P.yb;
  S.bw = P.bw;
  S.jbeg = by * P.slab_len;
  S.jend = keops_min(P.ny, S.jbeg + P.slab_len);
  S.part = P.partial + (by * P.nx + first) * RAD_DV;
  S.rows_store = row0 < P.nx ? P.nx - row0 : 0;
  S.arg = P.arg;
  S.row_first = first;
  S.row_last = P.nx - 1;
  S.rperm = P.perm[0];
  S.ctmax = P.gmax[1];
  // largest |k| |x^|^2 of the wavefront's rows (a wavefront past the last row recomputes the last row: that row's group)
  S.xq = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, P.gmax[0][first / (32 * RAD_RB)])));
#if RAD_MM
  rad_sweep_mm(S, ys, ws);
#else
  rad_sweep(S, ys, bs);
#endif
}

// The tiles that the sweep left out, from exact differences.  RADX_LPR lanes share an output row (its original
// coordinates in their registers) and take every RADX_LPR-th column of a staged chunk.  keops_rad_prep has written,
// in sorted order, everything a pair needs of a column -- original coordinates, centred coordinates (gradients with
// respect to the points) and the weights as the formula gives them: chunks of RADX_CHUNK columns travel through
// registers into one of two LDS buffers while the previous chunk is computed (one barrier per chunk), and are read back
// 16 bytes at a time.  The test of a (wavefront of the sweep, tile) pair is the sweep's own, on the same numbers, so
// every pair is computed exactly once.  The work sits where both norms are large (the last rows against the last
// columns): it is cut finer than the sweep, in workgroups of 256 / RADX_LPR rows and column segments of seg_len,
// heaviest first, and the sums of a segment go to their own array, which keops_rad_reduce adds for the rows that
// have any (same test again).
#define RADX_LPR 4
#define RADX_ROWS (256 / RADX_LPR)
#define RADX_CHUNK (RADX_XW <= 16 ? (RAD_TJ < 256 ? RAD_TJ : 256) : (RAD_TJ < 128 ? RAD_TJ : 128))  // columns per staged chunk (divides RAD_TJ)
#define RADX_MAXT 1024   // tiles of a segment whose numbers fit the workgroup's list (longer segments are walked in parts)
extern "C" __global__ void __launch_bounds__(256) keops_rad_exact(const RadParams P) {
  if (P.scal[2] != 1u) return;
  constexpr int XD = RADX_XD, XC = RADX_XC, XWT = RADX_XWT, XW = RADX_XW, CH = RADX_CHUNK, NF4 = XW / 4;
  constexpr int CPT = RAD_TJ / CH;  // chunks per tile
  __shared__ __attribute__((aligned(16))) float cs[2][CH * XW];
  __shared__ float wgmax[4];
  __shared__ int slow_tile[RADX_MAXT];
  __shared__ float slow_q[RADX_MAXT];
  __shared__ int nslow_s;
  const int tid = threadIdx.x, lane = tid & 63, sub = tid % RADX_LPR;
  // (the last rows and the last segment hold the work: they are issued first)
  const i64 bx = (i64)gridDim.x - 1 - blockIdx.x, seg = (i64)gridDim.y - 1 - blockIdx.y;
  const i64 k = bx * RADX_ROWS + tid / RADX_LPR;  // sorted position of the lane's row
  const bool valid = k < P.nx;
  const float xq = valid ? P.gmax[0][k / (32 * RAD_RB)] : 0.f;
  // nothing to do for the whole workgroup?  (the rows are sorted: most workgroups meet no tile beyond the bound)
  {
    float m = valid ? xq : 0.f;
    m = !(m == m) ? 3.0e38f : m;  // a NaN norm: every tile
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float other = __shfl_xor(m, o);
      m = other > m ? other : m;
    }
    if (lane == 0) wgmax[tid >> 6] = m;
  }
  __syncthreads();
  const float xq_wg = fmaxf(fmaxf(wgmax[0], wgmax[1]), fmaxf(wgmax[2], wgmax[3]));
  if (P.segmax[seg] + xq_wg <= (float)RAD_LIMIT) return;  // (uniform over the workgroup)
  const i64 jbeg = seg * P.seg_len, jend = keops_min(P.ny, jbeg + P.seg_len);
  const i64 tile0 = jbeg / RAD_TJ, ntile = jend > jbeg ? (jend - jbeg + RAD_TJ - 1) / RAD_TJ : 0;
  T p[KEOPS_DIMP > 0 ? KEOPS_DIMP : 1];
  rad_load_params(P, p);
  const float coef = (float)KeopsRadFormula::coef(p);
  const i64 i = valid ? (i64)P.perm[0][k] : 0;
  float xv[RAD_D];
#pragma unroll
  for (int d = 0; d < RAD_D; d++) xv[d] = (float)P.arg[RAD_XARG][i * RAD_D + d];
#if RAD_BIL || RAD_UPAIR
  float uv[RAD_DW];
  {
    T xi[RAD_DIMX > 0 ? RAD_DIMX : 1], u_[RAD_DU > 0 ? RAD_DU : 1];
#pragma unroll
    for (int v = 0; v < RAD_NROWVARS; v++) {
      const T* a = P.arg[rad_row_arg[v]] + i * rad_row_dim[v];
#pragma unroll
      for (int d = 0; d < rad_row_dim[v]; d++) xi[rad_row_off[v] + d] = a[d];
    }
    KeopsRadFormula::rowvec(xi, p, u_);
#pragma unroll
    for (int d = 0; d < RAD_DW; d++) uv[d] = (float)u_[d];
  }
#endif
  float acc[RAD_DV];
#pragma unroll
  for (int d = 0; d < RAD_DV; d++) acc[d] = 0.f;

  // one pair: column `col` of the staged chunk against the lane's row
  auto pair = [&](const float* col) {
    float yv[RAD_D];
    {
      float yy[XD];
#pragma unroll
      for (int q = 0; q < XD / 4; q++) *reinterpret_cast<float4*>(yy + 4 * q) = reinterpret_cast<const float4*>(col)[q];
#pragma unroll
      for (int d = 0; d < RAD_D; d++) yv[d] = yy[d];
    }
    float wv[XWT];
#pragma unroll
    for (int q = 0; q < XWT / 4; q++) *reinterpret_cast<float4*>(wv + 4 * q) = reinterpret_cast<const float4*>(col + XD + XC)[q];
#if RAD_DIFF != 0
    float cf[XD];
#pragma unroll
    for (int q = 0; q < XD / 4; q++) *reinterpret_cast<float4*>(cf + 4 * q) = reinterpret_cast<const float4*>(col + XD)[q];
#endif
    const float e = rad_exp_of(coef, rad_sqdist_exact(xv, yv));
#if RAD_BIL || RAD_UPAIR
    float sp = uv[0] * wv[0];
#pragma unroll
    for (int d = 1; d < RAD_DW; d++) sp = __builtin_fmaf(uv[d], wv[d], sp);
    const float es = e * sp;
#if RAD_DIFF != 0
#pragma unroll
    for (int d = 0; d < RAD_D; d++) acc[d] = __builtin_fmaf(es, cf[d], acc[d]);
    acc[RAD_D] += es;
#else
    acc[0] += es;
#endif
#elif RAD_DIFF != 0
    // component d of the weights against [y^_j, 1]
#pragma unroll
    for (int d = 0; d < RAD_DW; d++) {
      const float ew = e * wv[d];
#pragma unroll
      for (int q = 0; q < RAD_D; q++) acc[d * (RAD_D + 1) + q] = __builtin_fmaf(ew, cf[q], acc[d * (RAD_D + 1) + q]);
      acc[d * (RAD_D + 1) + RAD_D] += ew;
    }
#else
#pragma unroll
    for (int d = 0; d < RAD_DV; d++) acc[d] = __builtin_fmaf(e, wv[d], acc[d]);
#endif
  };

  for (i64 part0 = 0; part0 < ntile; part0 += RADX_MAXT) {
    const int npart = (int)keops_min((i64)RADX_MAXT, ntile - part0);
    // the tiles that some row of the workgroup needs, in order (first wavefront: 64 tiles at a time)
    __syncthreads();
    if (tid < 64) {
      int n = 0;
      for (int base = 0; base < npart; base += 64) {
        const int t = base + lane;
        const float tq = t < npart ? P.gmax[1][tile0 + part0 + t] : 0.f;
        const bool need = t < npart && !(tq + xq_wg <= (float)RAD_LIMIT);
        const unsigned long long bal = __ballot(need);
        if (need) {
          const int at = n + __popcll(bal & ((1ull << lane) - 1ull));
          slow_tile[at] = t;
          slow_q[at] = tq;
        }
        n += __popcll(bal);
      }
      if (lane == 0) nslow_s = n;
    }
    __syncthreads();
    const int nitems = nslow_s * CPT;
    // chunk `it` of the list: columns [col0, col0 + ncol) of the sorted operand
    auto chunk_of = [&](int it, i64& col0, int& ncol) __attribute__((always_inline)) {
      const i64 j0 = (tile0 + part0 + slow_tile[it / CPT]) * RAD_TJ + (i64)(it % CPT) * CH;
      col0 = j0;
      ncol = (int)keops_max((i64)0, keops_min((i64)CH, P.ny - j0));  // places past the last column are left out
    };
    float4 pf[NF4];
    auto fetch = [&](int it) __attribute__((always_inline)) {
      i64 col0;
      int ncol;
      chunk_of(it, col0, ncol);
      // (a thread past the last column of the chunk reads a column it will not stash: yo is padded to whole tiles)
      const float4* src = reinterpret_cast<const float4*>(P.yo + (col0 + (tid < CH ? tid : 0)) * XW);
#pragma unroll
      for (int q = 0; q < NF4; q++) pf[q] = src[q];
    };
    auto stash = [&](int it) __attribute__((always_inline)) {
      i64 col0;
      int ncol;
      chunk_of(it, col0, ncol);
      if (tid < ncol) {
        float4* dst = reinterpret_cast<float4*>(cs[it & 1] + tid * XW);
#pragma unroll
        for (int q = 0; q < NF4; q++) dst[q] = pf[q];
      }
    };
    if (nitems > 0) {
      fetch(0);
      stash(0);
    }
    __syncthreads();
    for (int it = 0; it < nitems; it++) {
      if (it + 1 < nitems) fetch(it + 1);  // in flight while this chunk is computed
      i64 col0;
      int ncol;
      chunk_of(it, col0, ncol);
      const bool mine = valid && !(slow_q[it / CPT] + xq <= (float)RAD_LIMIT);  // the sweep's test for this row's wavefront
      if (mine) {
        const float* buf = cs[it & 1];
        int c = sub;
        for (; c + 3 * RADX_LPR < ncol; c += 4 * RADX_LPR) {  // four independent pairs in flight
#pragma unroll
          for (int u = 0; u < 4; u++) pair(buf + (c + u * RADX_LPR) * XW);
        }
        for (; c < ncol; c += RADX_LPR) pair(buf + c * XW);
      }
      if (it + 1 < nitems) stash(it + 1);
      __syncthreads();
    }
  }
  // the RADX_LPR lanes of a row are neighbours
#pragma unroll
  for (int d = 0; d < RAD_DV; d++) {
#pragma unroll
    for (int o = 1; o < RADX_LPR; o <<= 1) acc[d] += __shfl_xor(acc[d], o);
  }
  if (valid && sub == 0 && !(P.segmax[seg] + xq <= (float)RAD_LIMIT)) {
    float* dst = P.xpart + (seg * P.nx + k) * RAD_DV;
#pragma unroll
    for (int d = 0; d < RAD_DV; d++) dst[d] = acc[d];
  }
}
#endif

#if !RAD_RANGES
// slabs are added in order; the factors of the output index and, for the gradients with respect to the points, the
// difference x^_i S - sum_j K_ij w_j y^_j are applied here, once per output row (the sweep's rows are in sorted order:
// row k of the sums belongs to point perm[k])
extern "C" __global__ void __launch_bounds__(256) keops_rad_reduce(const RadParams P) {
  if (P.scal[2] != 1u) return;
  const i64 k = (i64)blockIdx.x * 256 + threadIdx.x;
  if (k >= P.nx) return;
  const i64 i = (i64)P.perm[0][k];
  float s[RAD_DV];
#pragma unroll
  for (int d = 0; d < RAD_DV; d++) s[d] = P.partial[k * RAD_DV + d];
  for (int sl = 1; sl < P.nslabs; sl++)
#pragma unroll
    for (int d = 0; d < RAD_DV; d++) s[d] += P.partial[((i64)sl * P.nx + k) * RAD_DV + d];
  // the sums of keops_rad_exact, for the segments in which this row's wavefront left tiles out (its test)
  {
    const float xq = P.gmax[0][k / (32 * RAD_RB)];
    for (int sg = 0; sg < P.nseg; sg++)
      if (!(P.segmax[sg] + xq <= (float)RAD_LIMIT)) {
#pragma unroll
        for (int d = 0; d < RAD_DV; d++) s[d] += P.xpart[((i64)sg * P.nx + k) * RAD_DV + d];
      }
  }
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
  for (int c = 0; c < RAD_D; c++) {
    const float xc = (float)((double)x[c] - (double)P.colsum[c]);
#if RAD_DU > 0 && !RAD_UPAIR && !RAD_BIL
    float acc = 0.f;
#pragma unroll
    for (int d = 0; d < RAD_DW; d++) acc = __builtin_fmaf((float)uv[d], __builtin_fmaf(xc, s[d * (RAD_D + 1) + RAD_D], -s[d * (RAD_D + 1) + c]), acc);
    P.out[i * RAD_DOUT + c] = (T)(ai * (float)RAD_DIFF * acc);
#else
    P.out[i * RAD_DOUT + c] = (T)(ai * (float)RAD_DIFF * __builtin_fmaf(xc, s[RAD_D], -s[c]));
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
