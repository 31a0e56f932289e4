// K-nearest-neighbour search (KMin / ArgKMin / KMin_ArgKMin of SqDist(x_i, y_j)): matrix-core filter +
// exact re-rank.  One bf16 per component for D >= 32; for lower dimensions (dense point clouds, where
// neighbours are close compared with the norms) every component is split as hi + lo (KNN_SPLIT) and the
// inner product takes three MFMAs per k-block, which tightens the filter slack from 8e-3 to 5e-5.
//
// Replaces, for this formula, the generic kernel the reference would generate from
//   keopscore/keopscore/mapreduce/gpu/GpuReduc1D.py:43-96 with
//   keopscore/keopscore/formulas/reductions/KMin_ArgKMin_Reduction.py:34-100,
// whose per-thread K-list insertion evaluates all 3*D flops per pair on the vector ALU.
//
// Design (CDNA4 / gfx950):
//   1. keops_knn_prep rewrites queries and references once as centred bfloat16 rows
//      x^ = bf16(x - mu), y^ = bf16(y - mu) (mu = column mean of the references) together with the
//      scalar keys (1-c)|x^|^2, (1-c)|y^|^2.
//   2. keops_knn_main: a wavefront owns 32*KNN_QSETS queries held as MFMA "B" operands in VGPRs;
//      reference rows are staged in LDS (padded rows, conflict-free 128-bit reads) and fed as "A"
//      operands to v_mfma_f32_32x32x16_bf16, which yields the inner products S = <y^_j, x^_i>.
//      A pair survives the filter when  (1-c)|y^_j|^2 - 2 S  <=  tau_i (1+delta) - (1-c)|x^_i|^2,
//      tau_i being the current K-th best exact distance of query i.  The constant c bounds the bf16
//      rounding of both operands and the fp32 accumulation error, so that every pair whose exact
//      distance is <= tau_i survives (no false negative); the filter only decides what is
//      re-examined, never what is returned.
//   3. Survivors are queued per wavefront and re-examined 64 at a time, one per lane: the distance
//      is recomputed from the original float32 rows in the reference's own operation order
//      (sequential sum of squared differences, no fused multiply-add; Sum.py:20-24,
//      Square.py:17-18, Subtract.py:21-24) and inserted in the query's sorted K-list (LDS) under the
//      lexicographic key (distance, index).  That key reproduces the reference's sequential
//      strict-"<" insertion (KMin_ArgKMin_Reduction.py:72-100) whatever the arrival order, so
//      indices and distances are bit-identical to the CPU path.
//   4. The reference axis can be cut in slabs (blockIdx.y); keops_knn_merge merges the per-slab
//      lists under the same key and writes the output in the reference's layout.
//   5. Large problems run in two phases so that the matrix-core sweep never waits for a re-rank:
//      (a) keops_knn_sample sweeps every step-th reference (step <= KNN_SAMPLE) and keeps, per query, the K
//      smallest *upper bounds* U = L + 2c(|x^|^2 + |y^|^2) of the pair distances, straight from the
//      matrix-core values (no exact distance, no memory access per candidate); the K-th of them bounds the
//      final K-th distance from above and becomes a *fixed* threshold;
//      (b) keops_knn_filter sweeps all references against the fixed thresholds and only logs the
//      surviving (query, reference) pairs, each wavefront in a private region of global memory (no
//      atomics, no list updates); (c) keops_knn_rerank replays every log with the exact distance and
//      the same K-list insertion.  With enough slabs, (b)-(c) run twice: first on every 4th slab, whose
//      replayed lists tighten the thresholds (K-th distance among a quarter of the references instead of
//      among the sample), then on the other slabs, which then log about four times fewer survivors.
//      If a log overflows (pathological ties) the adaptive kernel, launched behind and idle otherwise, redoes all
//      references.
//
// The plug-in defines: T (float), KEOPS_NARGS, KNN_D, KNN_DPAD (D rounded up to 16), KNN_K,
// KEOPS_RED_KEEP, KEOPS_DIMOUT, KNN_QSETS, KNN_WAVES (wavefronts per workgroup), KNN_TJ, KNN_FTJ, KNN_SPLIT,
// KNN_FWAVES / KNN_FQSETS (filter geometry), KNN_SWAVES / KNN_SQSETS (sampling pass geometry).
#pragma once
#include "keops_common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 knn_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 knn_bf16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float knn_f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float knn_f32x4;

#ifndef KNN_RANGES
#define KNN_RANGES 0                   // 1: module for block-sparse launches (adaptive kernel with a range cursor)
#endif
#ifndef KNN_SPLIT
#define KNN_SPLIT 0
#endif
static_assert(KNN_FQSETS <= 4 && KNN_SQSETS <= 2, "a lane owns the lists of at most two queries in the replay kernel, of one in the sampling kernel");
#ifndef KNN_FTJ
#define KNN_FTJ KNN_TJ                 // reference rows per staged tile of the fixed-threshold filter
#endif
#ifndef KNN_I8
#define KNN_I8 0                       // 1: the fixed-threshold filter also exists on signed bytes (keops_knn_filter_i8)
#endif
#define KNN_DP8 ((KNN_D + 31) / 32 * 32)  // bytes per quantised row: whole k blocks of v_mfma_i32_32x32x32_i8
#define KNN_I8_ETA 0.08f               // the byte filter is used when its slack is below this fraction of the search radius
#define KNN_KB (KNN_DPAD / 16)         // 16-wide k blocks
#define KNN_RW (KNN_DPAD * (1 + KNN_SPLIT))  // bf16 elements per stored row: [hi] or [hi | lo]
#define KNN_STRIDE (KNN_RW * 2 + 16)   // bytes per staged reference row (16 B pad: conflict-free b128 reads)
// Filter slack c.  One bf16 per component (D >= 32): 4u(1+3u) + 2(D+1) 2^-24 with u = 2^-9, rounded up.
// Split operands x^ = hi + lo (KNN_SPLIT, low dimensions, where neighbours are close compared with the
// norms): representation error 2^-18 per vector, the dropped lo*lo product 2^-18 |x^||y^|, fp32
// accumulation of at most 100 exact bf16 products: 5 2^-18 + 200 2^-24 = 3.1e-5, rounded up.
#if KNN_SPLIT
#define KNN_C 5.0e-5f
#else
#define KNN_C 0.0082f
#endif
#define KNN_DELTA 2e-5f
// distance of the upper bound U to the lower bound L of a pair: U - L = 2c (|x^|^2 + |y^|^2) = KNN_E (xkey + ykey)
#define KNN_E (2.0f * KNN_C / (1.0f - KNN_C))
#define KNN_FLT_MAX 3.402823466e38f

struct KnnParams {
  i64 nq, nr;            // queries (output rows), references (reduced rows)
  const float* xq;       // [nq][KNN_D] original queries
  const float* yr;       // [nr][KNN_D] original references
  __bf16* xh;            // [nq][KNN_RW] centred bf16 queries (times -2)
  __bf16* yh;            // [nr][KNN_RW]
  float* xkey;           // [nq]  (1-c)|x^|^2
  float* ykey;           // [nr]
  float* colsum;         // [KNN_DPAD] column sums of the references
  float* colpart;        // [nparts][KNN_DPAD] partial column sums
  float* plist_d;        // [nslabs][nq][K] partial lists: distances
  int* plist_i;          //                                indices
  i64 slab_len;
  int nslabs;
  int ref_step;          // reference row j of this pass is row j*ref_step of yr (sub-sampled pass: > 1)
  T* out;                // [nq][KEOPS_DIMOUT]
  float* thr;            // [nq] fixed filter thresholds of the two-phase scheme
  int2* log;             // candidate logs of the filter pass: [nlogs][logcap] (local query, reference)
  int* logcount;         // [nlogs] entries written (clamped to logcap)
  int* overflow;         // set to 1 when a log was too small
  i64 logcap;
  int stage;             // filter / replay: which slabs this launch covers (knn_stage_slab)
  int fb;                // fallback of the two-phase schedule, decided on the device: keops_knn_main with fb = 1 runs only
                         // when a candidate log overflowed (*overflow != 0); keops_knn_merge with fb > 0 then merges the
                         // fb slabs of that pass instead of nslabs
  // filter on signed bytes (KNN_I8; null otherwise)
  signed char* xq8;      // [nq][KNN_DP8] minus the quantised centred queries
  signed char* yq8;      // [nr][KNN_DP8] quantised centred references
  int* ykey_i;           // [nr] floor(|y~|^2 / 2) in quantisation steps
  int* xnorm_i;          // [nq] |x~|^2
  float* xres;           // [nq] distance between a centred query and its quantised copy (rounded up)
  int* thr_i;            // [nq] integer thresholds
  unsigned* scal;        // [0]: bit pattern of the largest |centred component|; [1]: queries for which the byte filter
                         // would be too loose; [2]: bit pattern of the largest distance between a centred reference
                         // and its quantised copy; [3]: 1 when the byte filter served the call (written at the end)
  i64 batch_rows, batch_cols;  // > 0: the row ranges are batches of that many queries / references, and the indices
                         // returned are relative to the batch (GpuReduc1D_ranges.py:151-158)
#if KNN_RANGES
  KeopsRangeTables rt;   // block-sparse launches: workgroup table and reduced-index ranges (keops_knn_main only)
#endif
};

// Slab handled by workgroup row y of a filter (or replay) launch.  stage 0: all slabs in order;
// stage 1: every 4th slab (0, 4, 8, ...), whose exact replay tightens the thresholds; stage 2: the others.
__device__ __forceinline__ int knn_stage_slab(int stage, int y) { return stage == 0 ? y : (stage == 1 ? 4 * y : y + y / 3 + 1); }

// ---- pre-pass ---------------------------------------------------------------------------------

// Column sums of the references in two deterministic stages (per-workgroup partials, then a
// fixed-order final sum): no atomics.
#define KNN_CW (KNN_D > 128 ? 256 : (KNN_D > 64 ? 128 : (KNN_D > 32 ? 64 : 32)))
extern "C" __global__ void __launch_bounds__(256) keops_knn_colsum(const KnnParams P) {
  // lanes run along the columns (coalesced rows), 256 / KNN_CW row groups per block; fixed summation order
  __shared__ float part[256];
  constexpr int RG = 256 / KNN_CW;
  const int cw = threadIdx.x % KNN_CW, rg = threadIdx.x / KNN_CW;
  const i64 rows_per_block = (P.nr + gridDim.x - 1) / gridDim.x;
  const i64 r0 = (i64)blockIdx.x * rows_per_block, r1 = keops_min(P.nr, r0 + rows_per_block);
  for (int c0 = 0; c0 < KNN_DPAD; c0 += KNN_CW) {
    const int c = c0 + cw;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (c < KNN_D) {
      i64 r = r0 + rg;
      for (; r + 3 * RG < r1; r += 4 * RG) {
        s0 += P.yr[r * KNN_D + c];
        s1 += P.yr[(r + RG) * KNN_D + c];
        s2 += P.yr[(r + 2 * RG) * KNN_D + c];
        s3 += P.yr[(r + 3 * RG) * KNN_D + c];
      }
      for (; r < r1; r += RG) s0 += P.yr[r * KNN_D + c];
    }
    part[threadIdx.x] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (rg == 0 && c < KNN_DPAD) {
      float s = 0.f;
#pragma unroll
      for (int g = 0; g < RG; g++) s += part[g * KNN_CW + cw];
      P.colpart[(i64)blockIdx.x * KNN_DPAD + c] = s;
    }
    __syncthreads();
  }
}

extern "C" __global__ void __launch_bounds__(256) keops_knn_colsum_final(const KnnParams P, int nparts) {
  __shared__ float part[256];
  if (KNN_I8 && P.scal != nullptr && threadIdx.x < 4) P.scal[threadIdx.x] = 0u;
  if (threadIdx.x == 0) *reinterpret_cast<unsigned*>(P.colpart + (i64)(nparts + 1) * KNN_DPAD) = 0u;  // keops_knn_centre
  constexpr int RG = 256 / KNN_CW;
  const int cw = threadIdx.x % KNN_CW, rg = threadIdx.x / KNN_CW;
  for (int c0 = 0; c0 < KNN_DPAD; c0 += KNN_CW) {
    const int c = c0 + cw;
    float s = 0.f;
    if (c < KNN_DPAD)
      for (int b = rg; b < nparts; b += RG) s += P.colpart[(i64)b * KNN_DPAD + c];
    part[threadIdx.x] = s;
    __syncthreads();
    if (rg == 0 && c < KNN_DPAD) {
      float t = 0.f;
#pragma unroll
      for (int g = 0; g < RG; g++) t += part[g * KNN_CW + cw];
      P.colsum[c] = t;
    }
    __syncthreads();
  }
}

// The centre only has to lie inside the cloud: the filters' error bounds grow with the centred norms, the result does
// not depend on it.  The mean does not when a few references are far away (one point at 1e30 moves it by 1e30 / n,
// and every centred point is then that number: no neighbour would be found; one infinite component makes it NaN).
// keops_knn_centre takes, per component, the median and the quartiles of 1024 evenly spaced references (bitonic sort
// in LDS, values that are not finite last) and raises a flag when the mean is further than four interquartile ranges
// from the median (or not a number); keops_knn_centre_apply then replaces every mean by the median.  Ordinary data keep
// their mean, bit for bit.  Scratch: row nparts of colpart holds the medians, the first word of row nparts + 1 the flag.
extern "C" __global__ void __launch_bounds__(256) keops_knn_centre(const KnnParams P, int nparts) {
  __shared__ float v[1024];
  __shared__ int nfin;
  const int c = blockIdx.x, tid = threadIdx.x;
  if (c >= KNN_D) return;
  if (tid == 0) nfin = 0;
  __syncthreads();
  const i64 ns = P.nr < 1024 ? P.nr : 1024, step = P.nr / ns;
  int mine = 0;
#pragma unroll
  for (int t = 0; t < 4; t++) {
    const int k = tid + 256 * t;
    float a = __builtin_inff();
    if (k < ns) {
      const float y = P.yr[(i64)k * step * KNN_D + c];
      if (__builtin_fabsf(y) < __builtin_inff()) { a = y; mine++; }
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
    const float mean = P.colsum[c] / (float)P.nr;
    P.colpart[(i64)nparts * KNN_DPAD + c] = med;
    if (!(__builtin_fabsf(mean - med) <= 4.f * iqr + 1e-3f * __builtin_fabsf(med) + 1e-30f))
      atomicOr(reinterpret_cast<unsigned*>(P.colpart + (i64)(nparts + 1) * KNN_DPAD), 1u);
  }
}

extern "C" __global__ void __launch_bounds__(256) keops_knn_centre_apply(const KnnParams P, int nparts) {
  if (*reinterpret_cast<const unsigned*>(P.colpart + (i64)(nparts + 1) * KNN_DPAD) == 0u) return;
  for (int c = threadIdx.x; c < KNN_D; c += 256) P.colsum[c] = P.colpart[(i64)nparts * KNN_DPAD + c] * (float)P.nr;
}

// which = 0: queries, 1: references.  One row per group of KNN_LPR lanes, 4 columns per lane.
#define KNN_LPR (KNN_DPAD / 4 <= 4 ? 4 : (KNN_DPAD / 4 <= 8 ? 8 : (KNN_DPAD / 4 <= 16 ? 16 : (KNN_DPAD / 4 <= 32 ? 32 : 64))))
extern "C" __global__ void __launch_bounds__(256) keops_knn_prep(const KnnParams P, int which) {
  const i64 n = which ? P.nr : P.nq;
  const float* src = which ? P.yr : P.xq;
  __bf16* dst = which ? P.yh : P.xh;
  float* key = which ? P.ykey : P.xkey;
  const int sub = threadIdx.x % KNN_LPR;
  const i64 row = ((i64)blockIdx.x * 256 + threadIdx.x) / KNN_LPR;
  const float inv = 1.0f / (float)P.nr;
  float nrm = 0.f, vmax = 0.f;
  const bool live = row < n && sub * 4 < KNN_DPAD;
  if (live) {
    knn_bf16x4 h, l;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int c = sub * 4 + e;
      float v = 0.f;
      if (c < KNN_D) v = src[row * KNN_D + c] - P.colsum[c] * inv;
      vmax = __builtin_fmaxf(vmax, __builtin_fabsf(v));
      h[e] = (__bf16)v;
      float r = (float)h[e];
      if (KNN_SPLIT) {
        l[e] = (__bf16)(v - r);
        r += (float)l[e];  // exact: the two parts do not overlap
      }
      nrm += r * r;
      // queries are stored as -2 x^ (exact in bf16) so that the MFMA accumulator, initialised with
      // the reference keys, directly holds (1-c)|y^|^2 - 2 <y^, x^>
      if (!which) {
        h[e] = (__bf16)(-2.0f * (float)h[e]);
        if (KNN_SPLIT) l[e] = (__bf16)(-2.0f * (float)l[e]);
      }
    }
    *reinterpret_cast<knn_bf16x4*>(dst + row * KNN_RW + sub * 4) = h;
    if (KNN_SPLIT) *reinterpret_cast<knn_bf16x4*>(dst + row * KNN_RW + KNN_DPAD + sub * 4) = l;
  }
#pragma unroll
  for (int o = KNN_LPR / 2; o > 0; o >>= 1) nrm += __shfl_xor(nrm, o, KNN_LPR);
  if (live && sub == 0) key[row] = (1.0f - KNN_C) * nrm;
  if (KNN_I8 && P.scal != nullptr) {
    // largest centred component of both sets (a NaN never wins: the byte filter is then simply not exact about
    // that row, as the bf16 one, and the exact re-rank decides); one atomic per wavefront
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) vmax = __builtin_fmaxf(vmax, __shfl_xor(vmax, o));
    // (most wavefronts find the current maximum at least as large and skip the atomic)
    if ((threadIdx.x & 63) == 0 && __float_as_uint(vmax) > *const_cast<volatile unsigned*>(P.scal)) atomicMax(P.scal, __float_as_uint(vmax));
  }
}

// ---- exact re-rank ----------------------------------------------------------------------------

// SqDist in the reference's operation order, without contraction
__device__ __forceinline__ float knn_exact_sqdist(const float* __restrict__ x, const float* __restrict__ y) {
#pragma clang fp contract(off)
  float s = 0.f;
  if (KNN_D % 4 == 0) {
#pragma unroll 4
    for (int k = 0; k < KNN_D; k += 4) {
      const knn_f32x4 a = *reinterpret_cast<const knn_f32x4*>(x + k);
      const knn_f32x4 b = *reinterpret_cast<const knn_f32x4*>(y + k);
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const float d = a[e] - b[e];
        const float q = d * d;
        s = s + q;
      }
    }
  } else {
    for (int k = 0; k < KNN_D; k++) {
      const float d = x[k] - y[k];
      const float q = d * d;
      s = s + q;
    }
  }
  return s;
}

__device__ __forceinline__ bool knn_better(float d, int j, float d2, int j2) { return d < d2 || (d == d2 && j < j2); }

// sorted insertion of (d, j) in a K-list stored in LDS
__device__ __forceinline__ void knn_insert(float* lv, int* li, float d, int j) {
  if (!knn_better(d, j, lv[KNN_K - 1], li[KNN_K - 1])) return;
  int pos = KNN_K - 1;
  while (pos > 0 && knn_better(d, j, lv[pos - 1], li[pos - 1])) {
    lv[pos] = lv[pos - 1];
    li[pos] = li[pos - 1];
    pos--;
  }
  lv[pos] = d;
  li[pos] = j;
}

// ---- sweep of the references: staging, MFMA filter, candidate queue ----------------------------

// MODE 0 (adaptive): thresholds follow the K-lists, full queues are re-examined at once.
// MODE 1 (fixed thresholds): full queues are appended to the wavefront's log in global memory.
// MODE 2 (threshold estimate): adaptive, but nothing is re-examined: the K-lists hold the upper bounds
//   U = L + KNN_E (xkey + ykey) of the pair distances, computed from the matrix-core values alone (no memory
//   access per candidate); their K-th smallest bounds the K-th exact distance from above.  Lane l of a
//   wavefront owns the sorted list of query l in registers (one v_med3_f32 per entry and insertion).
//   Candidates wait in the wavefront's queue; when 64 are waiting they are dealt to small per-query bins in
//   LDS (`cand`, counters in `owner`; one LDS atomic per candidate, all 64 in flight together) and every
//   owner folds its bin into its list.
#define KNN_BIN 8  // candidates per query bin
template <int MODE, int WAVES, int QSETS, int TJ = KNN_TJ>
__device__ __forceinline__ void knn_sweep(const KnnParams& P, unsigned char* ys, float* ykey_s, float (*lv)[KNN_K],
                                          int (*li)[KNN_K], int* owner, int (*qq)[64], int (*qj)[64],
                                          float* cand = nullptr) {
  constexpr int BLOCK = 64 * WAVES, QW = 32 * QSETS, QB = WAVES * QW;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
#if KNN_RANGES
  // block-sparse launch (adaptive kernel only): the workgroup serves a patch of one row range and sweeps the
  // reduced-index ranges of that row range, as GpuReduc1D_ranges.py:127-165 does for any reduction
  static_assert(MODE == 0, "block-sparse launches run the adaptive kernel");
  KeopsTileGeom G;
  G.init(P.rt, P.nq, QB);
  if (G.row_first >= G.row_end) return;  // empty entry: tables built on the device round the grid up
  const i64 qbase = G.row_first, qlimit = G.row_end;
#else
  const i64 qbase = (i64)blockIdx.x * QB, qlimit = P.nq;
#endif
  const i64 qw0 = qbase + (i64)wave * QW;  // first query of this wavefront
  const float inf = __builtin_huge_valf();

  // queries of this wavefront as MFMA B operands
  knn_bf16x8 bq[QSETS][KNN_KB];
  knn_bf16x8 bql[QSETS][KNN_SPLIT ? KNN_KB : 1];  // low parts (split operands)
  float xk[QSETS], t[QSETS];
  bool valid[QSETS];
#pragma unroll
  for (int h = 0; h < QSETS; h++) {
    i64 q = qw0 + h * 32 + col;
    valid[h] = q < qlimit;
    if (!valid[h]) q = qlimit - 1;
#pragma unroll
    for (int kb = 0; kb < KNN_KB; kb++) {
      bq[h][kb] = *reinterpret_cast<const knn_bf16x8*>(P.xh + q * KNN_RW + kb * 16 + 8 * half);
      if (KNN_SPLIT) bql[h][kb] = *reinterpret_cast<const knn_bf16x8*>(P.xh + q * KNN_RW + KNN_DPAD + kb * 16 + 8 * half);
    }
    xk[h] = P.xkey[q];
    // finite start value: padded rows carry an infinite key and never pass
    if (MODE != 1) t[h] = valid[h] ? KNN_FLT_MAX : -inf;
    else t[h] = valid[h] ? P.thr[q] : -inf;
  }
  if (MODE == 0) {
    for (int e = tid; e < QB * KNN_K; e += BLOCK) {
      (&lv[0][0])[e] = inf;
      (&li[0][0])[e] = 0;
    }
  }
  // MODE 2: sorted list of upper bounds of query `lane` of this wavefront (lanes < QW), bins empty
  float lst[MODE == 2 ? KNN_K : 1];
  volatile int* bin_n = MODE == 2 ? owner + wave * QW : nullptr;
  volatile float* bin_v = MODE == 2 ? cand + wave * QW * KNN_BIN : nullptr;
  if (MODE == 2) {
#pragma unroll
    for (int k = 0; k < KNN_K; k++) lst[k] = inf;
    if (lane < QW) bin_n[lane] = 0;
    __threadfence_block();
  }
  // MODE 2: the nb queued upper bounds are dealt to the bins of their queries, every owner lane folds its bin
  // into its list (a bin that overflows is emptied and refilled), then all lanes get the new thresholds
  auto drain = [&](int nb) {
    __threadfence_block();
    bool pending = lane < nb;
    int ql = 0;
    float u = inf;
    if (pending) {
      ql = qq[wave][lane];
      u = __int_as_float(qj[wave][lane]);
    }
    while (keops_any(pending)) {
      if (pending) {
        const int pos = atomicAdd(const_cast<int*>(&bin_n[ql]), 1);
        if (pos < KNN_BIN) {
          bin_v[ql * KNN_BIN + pos] = u;
          pending = false;
        }
      }
      __threadfence_block();
      if (lane < QW) {
        const int n = min(bin_n[lane], KNN_BIN);
        bin_n[lane] = 0;
        for (int i = 0; i < n; i++) {
          const float c = bin_v[lane * KNN_BIN + i];
          // sorted insertion: new[k] = median(c, old[k-1], old[k]), new[0] = min(c, old[0])
#pragma unroll
          for (int k = (MODE == 2 ? KNN_K : 1) - 1; k > 0; k--) lst[k] = __builtin_amdgcn_fmed3f(c, lst[k - 1], lst[k]);
          lst[0] = __builtin_fminf(c, lst[0]);
        }
      }
      __threadfence_block();
    }
    const float tau = lst[(MODE == 2 ? KNN_K : 1) - 1];
#pragma unroll
    for (int h = 0; h < QSETS; h++) {
      const float tq = __shfl(tau, h * 32 + col);
      // a pair can only enter the list of upper bounds when its lower bound is below the K-th of them
      t[h] = valid[h] ? __builtin_fminf(tq - xk[h], KNN_FLT_MAX) : -inf;
    }
  };
  int qcount = 0;    // wave-uniform number of queued candidates
  i64 logged = 0;    // wave-uniform number of entries already in this wavefront's log
  const int slab = MODE == 1 ? knn_stage_slab(P.stage, blockIdx.y) : (int)blockIdx.y;
  const i64 logid = ((i64)slab * gridDim.x + blockIdx.x) * WAVES + wave;
  int2* mylog = MODE == 1 ? P.log + logid * P.logcap : nullptr;

  // MODE 0: re-examine the queued candidates (one per lane) and refresh the thresholds
  auto process = [&](int nb) {
    const bool act = lane < nb;
    int ql = 0, j = 0;
    float d = inf;
    if (act) {
      ql = qq[wave][lane];
      j = qj[wave][lane];
      d = knn_exact_sqdist(P.xq + (qw0 + ql) * KNN_D, P.yr + (i64)j * KNN_D);
    }
    // several lanes may hold candidates of the same query: elect one owner per query and round
    const int slot = wave * QW + ql;
    volatile int* ow = owner;
    bool done = !act;
    while (keops_any(!done)) {
      if (!done) ow[slot] = lane;
      __threadfence_block();
      if (!done && ow[slot] == lane) {
        knn_insert(lv[slot], li[slot], d, j);
        done = true;
      }
      __threadfence_block();
    }
#pragma unroll
    for (int h = 0; h < QSETS; h++) {
      const float tau = lv[wave * QW + h * 32 + col][KNN_K - 1];
      t[h] = valid[h] ? __builtin_fminf((tau + tau * KNN_DELTA) - xk[h], KNN_FLT_MAX) : -inf;
    }
  };
  // MODE 1: append the queued candidates to the log (coalesced 8-byte stores, fire and forget)
  auto flush = [&](int nb) {
    if (logged + nb <= P.logcap) {
      if (lane < nb) mylog[logged + lane] = make_int2(qq[wave][lane], qj[wave][lane]);
      logged += nb;
    } else {
      if (lane == 0) *P.overflow = 1;
    }
  };

#if KNN_RANGES
  i64 jbeg = 0, jend = 0;
#else
  const i64 jbeg = (i64)slab * P.slab_len;
  const i64 jend = keops_min(P.nr, jbeg + P.slab_len);
#endif
  // software pipeline: the rows of tile t+1 travel from HBM/L2 to registers while tile t is consumed
  constexpr int CH = KNN_RW / 8;                            // 16-byte chunks per staged row
  constexpr int NPF = (TJ * CH + BLOCK - 1) / BLOCK;    // chunks per thread and tile
  uint4 pf[NPF];
  float pfkey = inf;
  auto prefetch = [&](i64 j0) {
    const int n = (int)keops_min((i64)TJ, jend - j0);
    const uint4* src = reinterpret_cast<const uint4*>(P.yh + j0 * KNN_RW);
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * BLOCK;
      pf[u] = (e < n * CH) ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
    pfkey = (tid < n) ? P.ykey[j0 + tid] : inf;
  };
  static_assert(TJ <= BLOCK, "one key per thread");
  // this lane's operand row and keys inside a sub-tile of 32 staged rows
  const unsigned char* const abase = ys + col * KNN_STRIDE + 16 * half;
  const float* const kbase = ykey_s + 4 * half;
#if KNN_RANGES
  G.rewind(P.rt);
  while (G.next(P.rt, jbeg, jend)) {
#else
  {
#endif
  if (jbeg < jend) prefetch(jbeg);
  for (i64 j0 = jbeg; j0 < jend; j0 += TJ) {
    const int n = (int)keops_min((i64)TJ, jend - j0);
    __syncthreads();  // every wavefront is done with the previous tile
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * BLOCK;
      if (e < TJ * CH) {
        const int row = e / CH, c = e - row * CH;
        *reinterpret_cast<uint4*>(ys + row * KNN_STRIDE + c * 16) = pf[u];
      }
    }
    if (tid < TJ) ykey_s[tid] = pfkey;
    __syncthreads();
    if (j0 + TJ < jend) prefetch(j0 + TJ);
    const int nsub = (n + 31) / 32;
    for (int sub = 0; sub < nsub; sub++) {
      // accumulator register v of this lane is reference row 8*(v/4) + 4*half + v%4 of the sub-tile:
      // start from the keys of those rows
      knn_f32x4 kk[4];
#pragma unroll
      for (int b = 0; b < 4; b++) kk[b] = *reinterpret_cast<const knn_f32x4*>(kbase + sub * 32 + 8 * b);
      knn_f32x16 acc[QSETS];
#pragma unroll
      for (int h = 0; h < QSETS; h++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[h][v] = kk[v >> 2][v & 3];
      const unsigned char* arow = abase + sub * (32 * KNN_STRIDE);
#pragma unroll
      for (int kb = 0; kb < KNN_KB; kb++) {
        const knn_bf16x8 a = *reinterpret_cast<const knn_bf16x8*>(arow + kb * 32);
        if (KNN_SPLIT) {
          // <hi + lo, hi + lo> without the lo * lo term, smallest products first
          const knn_bf16x8 al = *reinterpret_cast<const knn_bf16x8*>(arow + KNN_DPAD * 2 + kb * 32);
#pragma unroll
          for (int h = 0; h < QSETS; h++) {
            acc[h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al, bq[h][kb], acc[h], 0, 0, 0);
            acc[h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bql[h][kb], acc[h], 0, 0, 0);
          }
        }
#pragma unroll
        for (int h = 0; h < QSETS; h++) acc[h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bq[h][kb], acc[h], 0, 0, 0);
      }
      // one v_cmp per pair; its wave-wide result lands in an SGPR pair and is tested on the scalar
      // unit, so the common case (no survivor) costs no further vector work
#pragma unroll
      for (int h = 0; h < QSETS; h++) {
        // cheap screen first: the smallest of the lane's 16 values against the threshold (min3 tree)
        // (three-operand minima only: a two-operand v_min_f32 of matrix-core results costs two more instructions
        // that quiet its inputs)
        float m = __builtin_fminf(__builtin_fminf(acc[h][0], acc[h][1]), acc[h][2]);
#pragma unroll
        for (int v = 3; v < 15; v += 2) m = __builtin_fminf(__builtin_fminf(m, acc[h][v]), acc[h][v + 1]);
        m = __builtin_fminf(__builtin_fminf(m, acc[h][15]), KNN_FLT_MAX);
        if (__builtin_expect(!keops_any(m <= t[h]), 1)) continue;
        if (MODE == 2) {
          // A threshold estimate may ignore candidates (the bound only gets looser): every lane offers the
          // smallest of its 16 pairs of this sub-tile, which is nearly every candidate once they are sparse.
          float yk = 0.f;  // key of the row that holds the minimum
#pragma unroll
          for (int v = 0; v < 16; v++) yk = acc[h][v] == m ? kk[v >> 2][v & 3] : yk;
          const float u = (m + xk[h]) + KNN_E * (xk[h] + yk);
          bool mine = m <= t[h];
          unsigned long long bal = __ballot(mine);
          while (bal != 0ull) {
            const int slot = qcount + __popcll(bal & ((1ull << lane) - 1ull));
            if (mine && slot < 64) {
              qq[wave][slot] = h * 32 + col;
              qj[wave][slot] = __float_as_int(u);
              mine = false;
            }
            qcount += __popcll(bal);
            if (qcount >= 64) {
              drain(64);
              qcount = 0;
              mine = mine && (m <= t[h]);  // lanes that found the queue full retry unless excluded now
              bal = __ballot(mine);
            } else {
              bal = 0ull;
            }
          }
          continue;
        }
        // all 16 compares first (independent, pipelined), then scalar tests of their wave-wide masks
        unsigned long long bals[16];
#pragma unroll
        for (int v = 0; v < 16; v++) bals[v] = __ballot(acc[h][v] <= t[h]);
#pragma unroll
        for (int v = 0; v < 16; v++) {
          unsigned long long bal = bals[v];
          bool mine = (bal >> lane) & 1ull;
          while (__builtin_expect(bal != 0ull, 0)) {
            const int slot = qcount + __popcll(bal & ((1ull << lane) - 1ull));
            if (mine && slot < 64) {
              qq[wave][slot] = h * 32 + col;
              qj[wave][slot] = (int)(j0 + sub * 32 + 8 * (v >> 2) + 4 * half + (v & 3)) * P.ref_step;
              mine = false;
            }
            qcount += __popcll(bal);
            if (qcount >= 64) {
              if (MODE == 0) process(64);
              else flush(64);
              qcount = 0;
              // lanes that found the queue full retry (MODE 0: unless the new threshold excludes them)
              if (MODE == 0) mine = mine && (acc[h][v] <= t[h]);
              bal = __ballot(mine);
            } else {
              bal = 0ull;
            }
          }
        }
      }
    }
  }
  }
  if (MODE == 2) {
    // lists of this slab straight from the owners' registers
    drain(qcount);
    const i64 q = qw0 + lane;
    if (lane < QW && q < P.nq) {
#pragma unroll
      for (int l = 0; l < (MODE == 2 ? KNN_K : 1); l++) {
        const i64 o = ((i64)blockIdx.y * P.nq + q) * KNN_K + l;
        P.plist_d[o] = lst[l];
        P.plist_i[o] = 0;
      }
    }
    return;
  }
  if (qcount > 0) {
    if (MODE == 0) process(qcount);
    else flush(qcount);
  }
  if (MODE == 1) {
    if (lane == 0) P.logcount[logid] = (int)logged;
    return;
  }
  __syncthreads();
  // partial lists of this slab
  for (int e = tid; e < QB * KNN_K; e += BLOCK) {
    const int ql = e / KNN_K, l = e - ql * KNN_K;
    const i64 q = qbase + ql;
    if (q < qlimit) {
      const i64 o = ((i64)blockIdx.y * P.nq + q) * KNN_K + l;
      P.plist_d[o] = lv[ql][l];
      P.plist_i[o] = li[ql][l];
    }
  }
}

// adaptive kernel: KNN_WAVES wavefronts of 32*KNN_QSETS queries
extern "C" __global__ void __launch_bounds__(64 * KNN_WAVES) keops_knn_main(const KnnParams P) {
  __shared__ __attribute__((aligned(16))) unsigned char ys[KNN_TJ * KNN_STRIDE];
  __shared__ __attribute__((aligned(16))) float ykey_s[KNN_TJ];
  __shared__ float lv[KNN_WAVES * 32 * KNN_QSETS][KNN_K];
  __shared__ int li[KNN_WAVES * 32 * KNN_QSETS][KNN_K];
  __shared__ int owner[KNN_WAVES * 32 * KNN_QSETS];
  __shared__ int qq[KNN_WAVES][64];  // queued candidates: local query
  __shared__ int qj[KNN_WAVES][64];  //                    reference index
#if !KNN_RANGES
  if (P.fb == 1 && *P.overflow == 0) return;  // the two-phase schedule went through: nothing to redo
#endif
  knn_sweep<0, KNN_WAVES, KNN_QSETS>(P, ys, ykey_s, lv, li, owner, qq, qj);
}

#if KNN_I8 && !KNN_RANGES
typedef int knn_i32x16 __attribute__((ext_vector_type(16)));
typedef int knn_i32x4 __attribute__((ext_vector_type(4)));
#ifndef KNN_I8_PAD
#define KNN_I8_PAD 16
#endif
#define KNN_I8_STRIDE (KNN_DP8 + KNN_I8_PAD)   // bytes per staged byte row (padded against bank conflicts)
#define KNN_I8_KB (KNN_DP8 / 32)       // 32-wide k blocks

// Quantisation step of the byte filter: the largest centred component of both sets maps to 127.
__device__ __forceinline__ float knn_i8_step(const KnnParams& P) {
  return __builtin_fmaxf(__uint_as_float(P.scal[0]), 1e-30f) * (1.0f / 127.0f);
}
// The distance between two quantised points differs from the true one by at most the distances of the two points to
// their quantised copies (triangle inequality): the query's own, the largest one among the references
__device__ __forceinline__ float knn_i8_slack(const KnnParams& P, i64 q) { return P.xres[q] + __uint_as_float(P.scal[2]); }
// true while the byte filter serves this call (few queries for which its slack is large against their search radius)
__device__ __forceinline__ bool knn_i8_taken(const KnnParams& P) { return (i64)P.scal[1] * 8 <= P.nq; }

// Rows as signed bytes: round((v - mean) / step), the queries negated, with the integer squared norms.  The metric is
// exact on the quantised points (integer products), so the filter only needs the triangle inequality:
// | |x - y| - step |x~ - y~| | <= slack.  which = 0: queries, 1: references; one row per group of KNN_LPR8 lanes.
#define KNN_LPR8 (KNN_DP8 / 4 <= 8 ? 8 : (KNN_DP8 / 4 <= 16 ? 16 : (KNN_DP8 / 4 <= 32 ? 32 : 64)))
extern "C" __global__ void __launch_bounds__(256) keops_knn_quant(const KnnParams P, int which) {
  const i64 n = which ? P.nr : P.nq;
  const float* src = which ? P.yr : P.xq;
  signed char* dst = which ? P.yq8 : P.xq8;
  const int sub = threadIdx.x % KNN_LPR8;
  const i64 row = ((i64)blockIdx.x * 256 + threadIdx.x) / KNN_LPR8;
  const float inv = 1.0f / (float)P.nr, step = knn_i8_step(P), rstep = 1.0f / step;
  int nrm = 0;
  float res2 = 0.f;
  const bool live = row < n && sub * 4 < KNN_DP8;
  if (live) {
    unsigned packed = 0u;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int c = sub * 4 + e;
      int q = 0;
      if (c < KNN_D) {
        const float v = src[row * KNN_D + c] - P.colsum[c] * inv;
        q = (int)__builtin_rintf(__builtin_fminf(__builtin_fmaxf(v * rstep, -127.0f), 127.0f));  // (NaN -> -127 -> a finite byte)
        const float r = v - (float)q * step;
        res2 = __builtin_fmaf(r, r, res2);
      }
      nrm += q * q;
      packed |= ((unsigned)((which ? q : -q) & 0xff)) << (8 * e);
    }
    *reinterpret_cast<unsigned*>(dst + row * KNN_DP8 + sub * 4) = packed;
  }
#pragma unroll
  for (int o = KNN_LPR8 / 2; o > 0; o >>= 1) {
    nrm += __shfl_xor(nrm, o, KNN_LPR8);
    res2 += __shfl_xor(res2, o, KNN_LPR8);
  }
  // distance to the quantised copy, rounded up (float32 evaluation of the sum; the centring itself is rounded to 2^-24
  // of the uncentred component, counted as 2^-20 of the largest centred one per component)
  const float res = __builtin_sqrtf(res2) * 1.00001f + 1.0e-6f * __builtin_sqrtf((float)KNN_D) * (127.0f * step);
  if (live && sub == 0) {
    if (which) P.ykey_i[row] = nrm >> 1;  // floor: never excludes a pair
    else {
      P.xnorm_i[row] = nrm;
      P.xres[row] = res;
    }
  }
  if (which) {
    // largest one among the references (a NaN row is left out: its exact distances are NaN and never inserted)
    float rmax = (live && res == res) ? res : 0.f;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) rmax = __builtin_fmaxf(rmax, __shfl_xor(rmax, o));
    if ((threadIdx.x & 63) == 0 && __float_as_uint(rmax) > *const_cast<volatile unsigned*>(P.scal + 2)) atomicMax(P.scal + 2, __float_as_uint(rmax));
  }
}

// Integer threshold of query q for the K-th distance bound tau (squared, already inflated for rounding): a pair
// with |x - y|^2 <= tau has step |x~ - y~| <= sqrt(tau) + slack, i.e. |y~|^2 / 2 - <x~, y~> <= (R^2 - |x~|^2) / 2 with
// R = (sqrt(tau) + slack) / step.
__device__ __forceinline__ int knn_i8_threshold(const KnnParams& P, i64 q, float tau) {
  const double R = ((double)__builtin_sqrtf(__builtin_fmaxf(tau, 0.f)) * 1.000001 + (double)knn_i8_slack(P, q)) / (double)knn_i8_step(P);
  const double t = (R * R * 1.000001 - (double)P.xnorm_i[q]) * 0.5 + 1.0;
  return t >= 1.0e9 ? 1000000000 : (t <= -1.0e9 ? -1000000000 : (int)t);  // (NaN: the last branch, 0 on this hardware)
}

// Fixed-threshold filter on signed bytes: the geometry, the logs and the replay of keops_knn_filter, with
// v_mfma_i32_32x32x32_i8 (half as many matrix instructions and staged bytes per pair).  The accumulators start from
// floor(|y~|^2 / 2), the B operands hold -x~: a lane's 16 results are |y~|^2 / 2 - <x~, y~> for 16 references.
extern "C" __global__ void __launch_bounds__(64 * KNN_FWAVES) keops_knn_filter_i8(const KnnParams P) {
  if (!knn_i8_taken(P)) return;
  constexpr int WAVES = KNN_FWAVES, QSETS = KNN_FQSETS, TJ = KNN_FTJ;
  constexpr int BLOCK = 64 * WAVES, QW = 32 * QSETS, QB = WAVES * QW;
  __shared__ __attribute__((aligned(16))) unsigned char ys[TJ * KNN_I8_STRIDE];
  __shared__ __attribute__((aligned(16))) int ykey_s[TJ];
  __shared__ int qq[WAVES][64];
  __shared__ int qj[WAVES][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, col = lane & 31;
  const i64 qw0 = (i64)blockIdx.x * QB + (i64)wave * QW;
  knn_i32x4 bq[QSETS][KNN_I8_KB];
  int t[QSETS];
#pragma unroll
  for (int h = 0; h < QSETS; h++) {
    i64 q = qw0 + h * 32 + col;
    const bool valid = q < P.nq;
    if (!valid) q = P.nq - 1;
#pragma unroll
    for (int kb = 0; kb < KNN_I8_KB; kb++) bq[h][kb] = *reinterpret_cast<const knn_i32x4*>(P.xq8 + q * KNN_DP8 + kb * 32 + 16 * half);
    t[h] = valid ? P.thr_i[q] : -2147483647 - 1;
  }
  int qcount = 0;    // wave-uniform number of queued candidates
  i64 logged = 0;    // wave-uniform number of entries already in this wavefront's log
  const int slab = knn_stage_slab(P.stage, blockIdx.y);
  const i64 logid = ((i64)slab * gridDim.x + blockIdx.x) * WAVES + wave;
  int2* mylog = P.log + logid * P.logcap;
  auto flush = [&](int nb) {
    if (logged + nb <= P.logcap) {
      if (lane < nb) mylog[logged + lane] = make_int2(qq[wave][lane], qj[wave][lane]);
      logged += nb;
    } else {
      if (lane == 0) *P.overflow = 1;
    }
  };
  const i64 jbeg = (i64)slab * P.slab_len, jend = keops_min(P.nr, jbeg + P.slab_len);
  constexpr int CH = KNN_DP8 / 16;                       // 16-byte chunks per staged row
  constexpr int NPF = (TJ * CH + BLOCK - 1) / BLOCK;
  uint4 pf[NPF];
  int pfkey = 1000000000;
  auto prefetch = [&](i64 j0) {
    const int n = (int)keops_min((i64)TJ, jend - j0);
    const uint4* src = reinterpret_cast<const uint4*>(P.yq8 + j0 * KNN_DP8);
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * BLOCK;
      pf[u] = (e < n * CH) ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
    pfkey = (tid < n) ? P.ykey_i[j0 + tid] : 1000000000;  // padded rows never pass
  };
  static_assert(TJ <= BLOCK, "one key per thread");
  const unsigned char* const abase = ys + col * KNN_I8_STRIDE + 16 * half;
  const int* const kbase = ykey_s + 4 * half;
  if (jbeg < jend) prefetch(jbeg);
  for (i64 j0 = jbeg; j0 < jend; j0 += TJ) {
    const int n = (int)keops_min((i64)TJ, jend - j0);
    __syncthreads();  // every wavefront is done with the previous tile
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * BLOCK;
      if (e < TJ * CH) {
        const int row = e / CH, c = e - row * CH;
        *reinterpret_cast<uint4*>(ys + row * KNN_I8_STRIDE + c * 16) = pf[u];
      }
    }
    if (tid < TJ) ykey_s[tid] = pfkey;
    __syncthreads();
    if (j0 + TJ < jend) prefetch(j0 + TJ);
    const int nsub = (n + 31) / 32;
    for (int sub = 0; sub < nsub; sub++) {
      // accumulator register v of this lane is reference row 8*(v/4) + 4*half + v%4 of the sub-tile:
      // start from the keys of those rows (they are the C operand of the first matrix instruction)
      knn_i32x4 kk[4];
#pragma unroll
      for (int b = 0; b < 4; b++) kk[b] = *reinterpret_cast<const knn_i32x4*>(kbase + sub * 32 + 8 * b);
      knn_i32x16 acc[QSETS];
#pragma unroll
      for (int h = 0; h < QSETS; h++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[h][v] = kk[v >> 2][v & 3];
      const unsigned char* arow = abase + sub * (32 * KNN_I8_STRIDE);
#pragma unroll
      for (int kb = 0; kb < KNN_I8_KB; kb++) {
        const knn_i32x4 a = *reinterpret_cast<const knn_i32x4*>(arow + kb * 32);
#pragma unroll
        for (int h = 0; h < QSETS; h++) acc[h] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, bq[h][kb], acc[h], 0, 0, 0);
      }
#pragma unroll
      for (int h = 0; h < QSETS; h++) {
        // cheap screen first: the smallest of the lane's 16 values against the threshold (three-operand minima)
        int m = min(min(acc[h][0], acc[h][1]), acc[h][2]);
#pragma unroll
        for (int v = 3; v < 15; v += 2) m = min(min(m, acc[h][v]), acc[h][v + 1]);
        m = min(m, acc[h][15]);
        if (__builtin_expect(!keops_any(m <= t[h]), 1)) continue;
        unsigned long long bals[16];
#pragma unroll
        for (int v = 0; v < 16; v++) bals[v] = __ballot(acc[h][v] <= t[h]);
#pragma unroll
        for (int v = 0; v < 16; v++) {
          unsigned long long bal = bals[v];
          bool mine = (bal >> lane) & 1ull;
          while (__builtin_expect(bal != 0ull, 0)) {
            const int slot = qcount + __popcll(bal & ((1ull << lane) - 1ull));
            if (mine && slot < 64) {
              qq[wave][slot] = h * 32 + col;
              qj[wave][slot] = (int)(j0 + sub * 32 + 8 * (v >> 2) + 4 * half + (v & 3));
              mine = false;
            }
            qcount += __popcll(bal);
            if (qcount >= 64) {
              flush(64);
              qcount = 0;
              bal = __ballot(mine);  // lanes that found the queue full retry
            } else {
              bal = 0ull;
            }
          }
        }
      }
    }
  }
  if (qcount > 0) flush(qcount);
  if (lane == 0) P.logcount[logid] = (int)logged;
}
#endif

#if !KNN_RANGES
// threshold estimate from a subset of the references: K-lists of upper bounds, no memory access per candidate
extern "C" __global__ void __launch_bounds__(64 * KNN_SWAVES) keops_knn_sample(const KnnParams P) {
  __shared__ __attribute__((aligned(16))) unsigned char ys[KNN_TJ * KNN_STRIDE];
  __shared__ __attribute__((aligned(16))) float ykey_s[KNN_TJ];
  __shared__ int qq[KNN_SWAVES][64];                              // queued candidates: local query
  __shared__ int qj[KNN_SWAVES][64];                              //                    upper bound (float bits)
  __shared__ int bin_n[KNN_SWAVES * 32 * KNN_SQSETS];             // candidates dealt to every query
  __shared__ float bin_v[KNN_SWAVES * 32 * KNN_SQSETS * KNN_BIN];  // their upper bounds
  knn_sweep<2, KNN_SWAVES, KNN_SQSETS>(P, ys, ykey_s, nullptr, nullptr, bin_n, qq, qj, bin_v);
}

// fixed-threshold filter: KNN_FWAVES wavefronts of 32*KNN_FQSETS queries share every staged tile
extern "C" __global__ void __launch_bounds__(64 * KNN_FWAVES) keops_knn_filter(const KnnParams P) {
#if KNN_I8
  if (P.scal != nullptr && knn_i8_taken(P)) return;  // keops_knn_filter_i8 serves this call
#endif
  __shared__ __attribute__((aligned(16))) unsigned char ys[KNN_FTJ * KNN_STRIDE];
  __shared__ __attribute__((aligned(16))) float ykey_s[KNN_FTJ];
  __shared__ int qq[KNN_FWAVES][64];
  __shared__ int qj[KNN_FWAVES][64];
  knn_sweep<1, KNN_FWAVES, KNN_FQSETS, KNN_FTJ>(P, ys, ykey_s, nullptr, nullptr, nullptr, qq, qj);
}

// every step-th reference row (bf16 row + key) gathered in a compact array for the sampling pass
extern "C" __global__ void __launch_bounds__(256) keops_knn_gather_sample(const KnnParams P, __bf16* yh_s, float* ykey_sm,
                                                                           i64 nsample, int step) {
  constexpr int CH = KNN_RW / 8;
  const i64 e = (i64)blockIdx.x * 256 + threadIdx.x;
  const i64 row = e / CH;
  const int c = (int)(e - row * CH);
  if (row >= nsample) return;
  reinterpret_cast<uint4*>(yh_s)[e] = reinterpret_cast<const uint4*>(P.yh)[row * step * CH + c];
  if (c == 0) ykey_sm[row] = P.ykey[row * step];
}

#endif  // !KNN_RANGES

// ---- merge of the per-slab lists ----------------------------------------------------------------

// merges the sorted lists of slabs first, first + stride, ... (count of them) of query q
__device__ __forceinline__ void knn_merge_lists(const KnnParams& P, i64 q, float (&bv)[KNN_K], int (&bi)[KNN_K],
                                                int first, int stride, int count) {
#pragma unroll
  for (int l = 0; l < KNN_K; l++) {
    bv[l] = P.plist_d[((i64)first * P.nq + q) * KNN_K + l];
    bi[l] = P.plist_i[((i64)first * P.nq + q) * KNN_K + l];
  }
  for (int t = 1; t < count; t++) {
    const int s = first + t * stride;
    for (int l = 0; l < KNN_K; l++) {
      const float d = P.plist_d[((i64)s * P.nq + q) * KNN_K + l];
      const int j = P.plist_i[((i64)s * P.nq + q) * KNN_K + l];
      if (!knn_better(d, j, bv[KNN_K - 1], bi[KNN_K - 1])) break;  // slab lists are sorted
      // unrolled bubble insertion (registers only)
      bv[KNN_K - 1] = d;
      bi[KNN_K - 1] = j;
#pragma unroll
      for (int p = KNN_K - 1; p > 0; p--) {
        const bool sw = knn_better(bv[p], bi[p], bv[p - 1], bi[p - 1]);
        const float a = bv[p], b = bv[p - 1];
        const int ia = bi[p], ib = bi[p - 1];
        bv[p - 1] = sw ? a : b;
        bv[p] = sw ? b : a;
        bi[p - 1] = sw ? ia : ib;
        bi[p] = sw ? ib : ia;
      }
    }
  }
}

#if KNN_RANGES
// block-sparse launches: queries that no row range covers (and lists that fewer than K references reach) keep the
// neutral entries (infinite distance, index 0)
extern "C" __global__ void __launch_bounds__(256) keops_knn_fill_lists(const KnnParams P) {
  const i64 e = (i64)blockIdx.x * 256 + threadIdx.x;
  if (e >= P.nq * KNN_K) return;
  P.plist_d[e] = __builtin_huge_valf();
  P.plist_i[e] = 0;
}
#endif

extern "C" __global__ void __launch_bounds__(256) keops_knn_merge(const KnnParams P) {
  const i64 q = (i64)blockIdx.x * 256 + threadIdx.x;
#if KNN_I8 && !KNN_RANGES
  if (q == 0 && P.scal != nullptr) P.scal[3] = knn_i8_taken(P) ? 1u : 0u;  // which filter served the call
#endif
  if (q >= P.nq) return;
  float bv[KNN_K];
  int bi[KNN_K];
#if KNN_RANGES
  knn_merge_lists(P, q, bv, bi, 0, 1, P.nslabs);
#else
  knn_merge_lists(P, q, bv, bi, 0, 1, (P.fb > 0 && *P.overflow != 0) ? P.fb : P.nslabs);
#endif
  T* out = P.out + q * KEOPS_DIMOUT;
#if KNN_RANGES
  if (P.batch_rows > 0) {
    // (neutral entries, infinite distance and index 0, stay as they are)
    const int first = (int)((q / P.batch_rows) * P.batch_cols);
#pragma unroll
    for (int l = 0; l < KNN_K; l++) bi[l] = bv[l] < __builtin_huge_valf() ? bi[l] - first : bi[l];
  }
#endif
#pragma unroll
  for (int l = 0; l < KNN_K; l++) {
#if KEOPS_RED_KEEP == 0
    out[2 * l] = (T)bv[l];
    out[2 * l + 1] = (T)bi[l];
#elif KEOPS_RED_KEEP == 1
    out[l] = (T)bv[l];
#else
    out[l] = (T)bi[l];
#endif
  }
}

#if !KNN_RANGES
// Thresholds of a filter pass from K-lists of a subset of the references (any such K-th distance is
// an upper bound of the final one).  refine = 0: lists of upper bounds U of the sampling pass (slabs
// 0 .. nslabs-1): K references have an exact float32 distance <= U_K (1 + delta), so every final neighbour has a
// lower bound L <= U_K (1 + delta)^2; refine = 1: exact lists replayed from the stage-1 slabs (0, 4, 8, ...:
// `count` of them), kept only where tighter than the current threshold.
extern "C" __global__ void __launch_bounds__(256) keops_knn_thresholds(const KnnParams P, int refine, int count) {
  const i64 q = (i64)blockIdx.x * 256 + threadIdx.x;
  if (q == 0 && !refine) *P.overflow = 0;  // reset before the filter passes (a fill kernel would be one more launch)
  if (q >= P.nq) return;
  float bv[KNN_K];
  int bi[KNN_K];
  if (refine) knn_merge_lists(P, q, bv, bi, 0, 4, count);
  else knn_merge_lists(P, q, bv, bi, 0, 1, P.nslabs);
  const float tau = bv[KNN_K - 1];
  const float tau_up = tau + tau * (refine ? KNN_DELTA : 3.0f * KNN_DELTA);
  float t = __builtin_fminf(tau_up - P.xkey[q], KNN_FLT_MAX);
  if (refine) t = __builtin_fminf(t, P.thr[q]);
  P.thr[q] = t;
#if KNN_I8
  if (P.scal != nullptr) {
    int ti = knn_i8_threshold(P, q, tau_up);
    if (refine) ti = min(ti, P.thr_i[q]);
    P.thr_i[q] = ti;
    // first estimate: is the slack of the byte filter small against the search radius of this query?
    if (!refine && !(knn_i8_slack(P, q) <= KNN_I8_ETA * __builtin_sqrtf(__builtin_fmaxf(tau_up, 0.f)))) atomicAdd(P.scal + 1, 1u);
  }
#endif
}

// ---- replay of the candidate logs ---------------------------------------------------------------

// One wavefront per log (= per filter wavefront and slab): exact distances for its candidates, 64 at a time,
// and the K best of each of its 32*KNN_FQSETS queries under the key (distance, index).  Lane l owns the sorted
// list of query l in registers; a candidate is first compared with the current K-th entry of its query (kept
// in LDS: most candidates of a fixed-threshold filter lose there), the others are dealt to small per-query
// bins (one LDS atomic each) that the owners fold into their lists.
extern "C" __global__ void __launch_bounds__(64) keops_knn_rerank(const KnnParams P, int fgrid_x) {
  constexpr int QW = 32 * KNN_FQSETS;
  constexpr int QPL = (QW + 63) / 64;  // queries owned by a lane: l, l + 64, ...
  __shared__ int bin_n[QW];
  __shared__ float bin_d[QW * KNN_BIN];
  __shared__ int bin_j[QW * KNN_BIN];
  __shared__ float kth_d[QW];  // current K-th entry of every query
  __shared__ int kth_j[QW];
  const int lane = threadIdx.x;
  const int wave = (int)(blockIdx.x % KNN_FWAVES);
  const i64 rest = blockIdx.x / KNN_FWAVES;
  const i64 bx = rest % fgrid_x, slab = knn_stage_slab(P.stage, (int)(rest / fgrid_x));
  const i64 logid = (slab * fgrid_x + bx) * KNN_FWAVES + wave;
  const i64 qw0 = bx * (KNN_FWAVES * QW) + (i64)wave * QW;
  const float inf = __builtin_huge_valf();
  float ld[QPL][KNN_K];
  int lj[QPL][KNN_K];
#pragma unroll
  for (int o = 0; o < QPL; o++)
#pragma unroll
    for (int k = 0; k < KNN_K; k++) {
      ld[o][k] = inf;
      lj[o][k] = 0;
    }
  volatile int* bn = bin_n;
  volatile float* bd = bin_d;
  volatile int* bj = bin_j;
  volatile float* kd = kth_d;
  volatile int* kj = kth_j;
#pragma unroll
  for (int o = 0; o < QPL; o++)
    if (lane + 64 * o < QW) {
      bn[lane + 64 * o] = 0;
      kd[lane + 64 * o] = inf;
      kj[lane + 64 * o] = 0x7fffffff;
    }
  __threadfence_block();
  const int count = P.logcount[logid];
  const int2* mylog = P.log + logid * P.logcap;
  for (int base = 0; base < count; base += 64) {
    const bool act = base + lane < count;
    int ql = 0, j = 0;
    float d = inf;
    if (act) {
      const int2 e = mylog[base + lane];
      ql = e.x;
      j = e.y;
      d = knn_exact_sqdist(P.xq + (qw0 + ql) * KNN_D, P.yr + (i64)j * KNN_D);
    }
    bool pending = act && knn_better(d, j, kd[ql], kj[ql]);
    while (keops_any(pending)) {
      if (pending) {
        const int pos = atomicAdd(&bin_n[ql], 1);
        if (pos < KNN_BIN) {
          bd[ql * KNN_BIN + pos] = d;
          bj[ql * KNN_BIN + pos] = j;
          pending = false;
        }
      }
      __threadfence_block();
#pragma unroll
      for (int o = 0; o < QPL; o++) {
        const int qo = lane + 64 * o;
        if (qo < QW) {
          const int n = min(bn[qo], KNN_BIN);
          if (n > 0) {
            bn[qo] = 0;
            for (int i = 0; i < n; i++) {
              const float cd = bd[qo * KNN_BIN + i];
              const int cj = bj[qo * KNN_BIN + i];
              // sorted insertion in registers: entry k becomes old[k-1] when the candidate goes before old[k-1],
              // the candidate when it goes before old[k] only, and stays otherwise
              bool before_cur = knn_better(cd, cj, ld[o][KNN_K - 1], lj[o][KNN_K - 1]);
#pragma unroll
              for (int k = KNN_K - 1; k > 0; k--) {
                const bool before_prev = knn_better(cd, cj, ld[o][k - 1], lj[o][k - 1]);
                ld[o][k] = before_prev ? ld[o][k - 1] : (before_cur ? cd : ld[o][k]);
                lj[o][k] = before_prev ? lj[o][k - 1] : (before_cur ? cj : lj[o][k]);
                before_cur = before_prev;
              }
              ld[o][0] = before_cur ? cd : ld[o][0];
              lj[o][0] = before_cur ? cj : lj[o][0];
            }
            kd[qo] = ld[o][KNN_K - 1];
            kj[qo] = lj[o][KNN_K - 1];
          }
        }
      }
      __threadfence_block();
      // candidates that found their bin full try again unless the list has moved past them
      pending = pending && knn_better(d, j, kd[ql], kj[ql]);
    }
  }
#pragma unroll
  for (int o = 0; o < QPL; o++) {
    const i64 q = qw0 + lane + 64 * o;
    if (lane + 64 * o < QW && q < P.nq) {
#pragma unroll
      for (int l = 0; l < KNN_K; l++) {
        const i64 e = (slab * P.nq + q) * KNN_K + l;
        P.plist_d[e] = ld[o][l];
        P.plist_i[e] = lj[o][l];
      }
    }
  }
}
#endif  // !KNN_RANGES
