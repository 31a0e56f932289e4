// K-nearest-neighbour search (KMin / ArgKMin / KMin_ArgKMin of SqDist(x_i, y_j)) for D >= 32:
// matrix-core filter + exact re-rank.
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
//
// The plug-in defines: T (float), KEOPS_NARGS, KNN_D, KNN_DPAD (D rounded up to 16), KNN_K,
// KEOPS_RED_KEEP, KEOPS_DIMOUT, KNN_QSETS, KNN_WAVES (wavefronts per workgroup), KNN_TJ.
#pragma once
#include "keops_common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 knn_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 knn_bf16x4;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float knn_f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float knn_f32x4;

#define KNN_BLOCK (64 * KNN_WAVES)
#define KNN_QW (32 * KNN_QSETS)        // queries per wavefront
#define KNN_QB (KNN_WAVES * KNN_QW)    // queries per workgroup
#define KNN_KB (KNN_DPAD / 16)         // 16-wide k blocks
#define KNN_STRIDE (KNN_DPAD * 2 + 16) // bytes per staged reference row (16 B pad: conflict-free b128 reads)
// filter slack: 4u(1+3u) + 2(D+1) 2^-24 with u = 2^-9, rounded up (see header comment)
#define KNN_C 0.0082f
#define KNN_DELTA 2e-5f
#define KNN_FLT_MAX 3.402823466e38f

struct KnnParams {
  i64 nq, nr;            // queries (output rows), references (reduced rows)
  const float* xq;       // [nq][KNN_D] original queries
  const float* yr;       // [nr][KNN_D] original references
  __bf16* xh;            // [nq][KNN_DPAD] centred bf16 queries
  __bf16* yh;            // [nr][KNN_DPAD]
  float* xkey;           // [nq]  (1-c)|x^|^2
  float* ykey;           // [nr]
  float* colsum;         // [KNN_DPAD] column sums of the references
  float* colpart;        // [nparts][KNN_DPAD] partial column sums
  float* plist_d;        // [nslabs][nq][K] partial lists: distances
  int* plist_i;          //                                indices
  i64 slab_len;
  int nslabs;
  int pad_;
  T* out;                // [nq][KEOPS_DIMOUT]
};

// ---- pre-pass ---------------------------------------------------------------------------------

// Column sums of the references in two deterministic stages (per-workgroup partials, then a
// fixed-order final sum): no atomics.
extern "C" __global__ void __launch_bounds__(256) keops_knn_colsum(const KnnParams P) {
  const i64 rows_per_block = (P.nr + gridDim.x - 1) / gridDim.x;
  const i64 r0 = (i64)blockIdx.x * rows_per_block, r1 = keops_min(P.nr, r0 + rows_per_block);
  for (int c = threadIdx.x; c < KNN_DPAD; c += 256) {
    float s = 0.f;
    if (c < KNN_D)
      for (i64 r = r0; r < r1; r++) s += P.yr[r * KNN_D + c];
    P.colpart[(i64)blockIdx.x * KNN_DPAD + c] = s;
  }
}

extern "C" __global__ void __launch_bounds__(256) keops_knn_colsum_final(const KnnParams P, int nparts) {
  for (int c = threadIdx.x; c < KNN_DPAD; c += 256) {
    float s = 0.f;
    for (int b = 0; b < nparts; b++) s += P.colpart[(i64)b * KNN_DPAD + c];
    P.colsum[c] = s;
  }
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
  float nrm = 0.f;
  const bool live = row < n && sub * 4 < KNN_DPAD;
  if (live) {
    knn_bf16x4 h;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int c = sub * 4 + e;
      float v = 0.f;
      if (c < KNN_D) v = src[row * KNN_D + c] - P.colsum[c] * inv;
      h[e] = (__bf16)v;
      const float r = (float)h[e];
      nrm += r * r;
      // queries are stored as -2 x^ (exact in bf16) so that the MFMA accumulator, initialised with
      // the reference keys, directly holds (1-c)|y^|^2 - 2 <y^, x^>
      if (!which) h[e] = (__bf16)(-2.0f * r);
    }
    *reinterpret_cast<knn_bf16x4*>(dst + row * KNN_DPAD + sub * 4) = h;
  }
#pragma unroll
  for (int o = KNN_LPR / 2; o > 0; o >>= 1) nrm += __shfl_xor(nrm, o, KNN_LPR);
  if (live && sub == 0) key[row] = (1.0f - KNN_C) * nrm;
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

// ---- main kernel ------------------------------------------------------------------------------

extern "C" __global__ void __launch_bounds__(KNN_BLOCK) keops_knn_main(const KnnParams P) {
  __shared__ __attribute__((aligned(16))) unsigned char ys[KNN_TJ * KNN_STRIDE];
  __shared__ __attribute__((aligned(16))) float ykey_s[KNN_TJ];
  __shared__ float lv[KNN_QB][KNN_K];
  __shared__ int li[KNN_QB][KNN_K];
  __shared__ int owner[KNN_QB];
  __shared__ int qq[KNN_WAVES][64];  // queued candidates: local query
  __shared__ int qj[KNN_WAVES][64];  //                    reference index

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, col = lane & 31;
  const i64 qw0 = (i64)blockIdx.x * KNN_QB + (i64)wave * KNN_QW;  // first query of this wavefront
  const float inf = __builtin_huge_valf();

  // queries of this wavefront as MFMA B operands
  knn_bf16x8 bq[KNN_QSETS][KNN_KB];
  float xk[KNN_QSETS], t[KNN_QSETS];
  bool valid[KNN_QSETS];
#pragma unroll
  for (int h = 0; h < KNN_QSETS; h++) {
    i64 q = qw0 + h * 32 + col;
    valid[h] = q < P.nq;
    if (!valid[h]) q = P.nq - 1;
#pragma unroll
    for (int kb = 0; kb < KNN_KB; kb++)
      bq[h][kb] = *reinterpret_cast<const knn_bf16x8*>(P.xh + q * KNN_DPAD + kb * 16 + 8 * half);
    xk[h] = P.xkey[q];
    t[h] = valid[h] ? KNN_FLT_MAX : -inf;  // finite: padded rows carry an infinite key and never pass
  }
  for (int e = tid; e < KNN_QB * KNN_K; e += KNN_BLOCK) {
    (&lv[0][0])[e] = inf;
    (&li[0][0])[e] = 0;
  }
  int qcount = 0;  // wave-uniform number of queued candidates

  // re-examine the queued candidates (one per lane) and refresh the thresholds
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
    const int slot = wave * KNN_QW + ql;
    volatile int* ow = owner;
    bool done = !act;
    while (__any(!done)) {
      if (!done) ow[slot] = lane;
      __threadfence_block();
      if (!done && ow[slot] == lane) {
        knn_insert(lv[slot], li[slot], d, j);
        done = true;
      }
      __threadfence_block();
    }
#pragma unroll
    for (int h = 0; h < KNN_QSETS; h++) {
      const float tau = lv[wave * KNN_QW + h * 32 + col][KNN_K - 1];
      t[h] = valid[h] ? __builtin_fminf((tau + tau * KNN_DELTA) - xk[h], KNN_FLT_MAX) : -inf;
    }
  };

  const i64 jbeg = (i64)blockIdx.y * P.slab_len;
  const i64 jend = keops_min(P.nr, jbeg + P.slab_len);
  // software pipeline: the rows of tile t+1 travel from HBM/L2 to registers while tile t is consumed
  constexpr int CH = KNN_DPAD / 8;                              // 16-byte chunks per staged row
  constexpr int NPF = (KNN_TJ * CH + KNN_BLOCK - 1) / KNN_BLOCK; // chunks per thread and tile
  uint4 pf[NPF];
  float pfkey = inf;
  auto prefetch = [&](i64 j0) {
    const int n = (int)keops_min((i64)KNN_TJ, jend - j0);
    const uint4* src = reinterpret_cast<const uint4*>(P.yh + j0 * KNN_DPAD);
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * KNN_BLOCK;
      pf[u] = (e < n * CH) ? src[e] : make_uint4(0u, 0u, 0u, 0u);
    }
    pfkey = (tid < n) ? P.ykey[j0 + tid] : inf;
  };
  static_assert(KNN_TJ <= KNN_BLOCK, "one key per thread");
  if (jbeg < jend) prefetch(jbeg);
  for (i64 j0 = jbeg; j0 < jend; j0 += KNN_TJ) {
    const int n = (int)keops_min((i64)KNN_TJ, jend - j0);
    __syncthreads();  // every wavefront is done with the previous tile
#pragma unroll
    for (int u = 0; u < NPF; u++) {
      const int e = tid + u * KNN_BLOCK;
      if (e < KNN_TJ * CH) {
        const int row = e / CH, c = e - row * CH;
        *reinterpret_cast<uint4*>(ys + row * KNN_STRIDE + c * 16) = pf[u];
      }
    }
    if (tid < KNN_TJ) ykey_s[tid] = pfkey;
    __syncthreads();
    if (j0 + KNN_TJ < jend) prefetch(j0 + KNN_TJ);
    const int nsub = (n + 31) / 32;
    for (int sub = 0; sub < nsub; sub++) {
      // accumulator register v of this lane is reference row 8*(v/4) + 4*half + v%4 of the sub-tile:
      // start from the keys of those rows
      knn_f32x4 kk[4];
#pragma unroll
      for (int b = 0; b < 4; b++) kk[b] = *reinterpret_cast<const knn_f32x4*>(ykey_s + sub * 32 + 8 * b + 4 * half);
      knn_f32x16 acc[KNN_QSETS];
#pragma unroll
      for (int h = 0; h < KNN_QSETS; h++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[h][v] = kk[v >> 2][v & 3];
      const unsigned char* arow = ys + (sub * 32 + col) * KNN_STRIDE + 16 * half;
#pragma unroll
      for (int kb = 0; kb < KNN_KB; kb++) {
        const knn_bf16x8 a = *reinterpret_cast<const knn_bf16x8*>(arow + kb * 32);
#pragma unroll
        for (int h = 0; h < KNN_QSETS; h++) acc[h] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bq[h][kb], acc[h], 0, 0, 0);
      }
      unsigned mask = 0u;
      bool hit = false;
#pragma unroll
      for (int h = 0; h < KNN_QSETS; h++)
#pragma unroll
        for (int v = 0; v < 16; v++) hit |= acc[h][v] <= t[h];  // one v_cmp each, OR-ed on the scalar unit
      if (__any(hit)) {
#pragma unroll
        for (int h = 0; h < KNN_QSETS; h++)
#pragma unroll
          for (int v = 0; v < 16; v++)
            if (acc[h][v] <= t[h]) mask |= 1u << (h * 16 + v);
        // KNN_QSETS <= 2 keeps the mask in 32 bits
        while (true) {
          const bool has = mask != 0u;
          const unsigned long long bal = __ballot(has);
          if (bal == 0ull) break;
          const int slot = qcount + __popcll(bal & ((1ull << lane) - 1ull));
          if (has && slot < 64) {
            const int bit = __ffs(mask) - 1;
            mask &= mask - 1u;
            const int h = bit >> 4, v = bit & 15;
            qq[wave][slot] = h * 32 + col;
            qj[wave][slot] = (int)(j0 + sub * 32 + 8 * (v >> 2) + 4 * half + (v & 3));
          }
          qcount += __popcll(bal);
          if (qcount >= 64) {
            process(64);
            qcount = 0;
            // candidates that found the queue full retry; drop those the new thresholds exclude
#pragma unroll
            for (int h = 0; h < KNN_QSETS; h++)
#pragma unroll
              for (int v = 0; v < 16; v++)
                if (!(acc[h][v] <= t[h])) mask &= ~(1u << (h * 16 + v));
          }
        }
      }
    }
  }
  if (qcount > 0) process(qcount);
  __syncthreads();
  // partial lists of this slab
  for (int e = tid; e < KNN_QB * KNN_K; e += KNN_BLOCK) {
    const int ql = e / KNN_K, l = e - ql * KNN_K;
    const i64 q = (i64)blockIdx.x * KNN_QB + ql;
    if (q < P.nq) {
      const i64 o = ((i64)blockIdx.y * P.nq + q) * KNN_K + l;
      P.plist_d[o] = lv[ql][l];
      P.plist_i[o] = li[ql][l];
    }
  }
}

// ---- merge of the per-slab lists and output ---------------------------------------------------

extern "C" __global__ void __launch_bounds__(256) keops_knn_merge(const KnnParams P) {
  const i64 q = (i64)blockIdx.x * 256 + threadIdx.x;
  if (q >= P.nq) return;
  float bv[KNN_K];
  int bi[KNN_K];
#pragma unroll
  for (int l = 0; l < KNN_K; l++) {
    bv[l] = P.plist_d[q * KNN_K + l];
    bi[l] = P.plist_i[q * KNN_K + l];
  }
  for (int s = 1; s < P.nslabs; s++) {
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
  T* out = P.out + q * KEOPS_DIMOUT;
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
