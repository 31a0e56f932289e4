// Device code that is compiled into libkeops_hip.so itself (everything else is JIT-compiled per formula):
//   * the static scratch buffer of the entry point that allocates nothing (keops_hip_launch_noalloc),
//   * half <-> float conversion kernels (use_half launches compute in float32),
//   * a fill kernel (zero formulas: a kernel instead of hipMemsetAsync, which must stay out of captured graphs),
//   * the kernels that build the lookup table of a block-sparse launch from the caller's ranges on the device,
//   * loop-only calibration kernels for the vector ALU and the matrix cores (keops_hip_calibrate): they measure
//     what an instruction stream without memory traffic sustains, the ceiling the map-reduce kernels are held to.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <mutex>
#include <type_traits>

#include "keops_static.h"

// ---- static scratch ---------------------------------------------------------------------------------------------

static __device__ __align__(256) unsigned char scratch[KEOPS_STATIC_SCRATCH_BYTES];

namespace {
std::mutex g_scratch_mutex;
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
}  // namespace

// Address of this device's copy of the scratch array (every GPU holds its own copy at its own address); looked up
// once per device with that device current.  Returns a hipError_t.
int keops_static_scratch(int device, void** ptr, size_t* bytes) {
  if (device < 0 || device >= kMaxDevices) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[device]) {
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) return (int)e;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[device] = p;
  }
  *ptr = g_scratch_ptr[device];
  *bytes = (size_t)KEOPS_STATIC_SCRATCH_BYTES;
  return 0;
}

// ---- fill -----------------------------------------------------------------------------------------------------------

static __global__ void __launch_bounds__(256) keops_fill_zero_u32(uint32_t* dst, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = 0u;
}

// zero `bytes` bytes (a multiple of 4) at dst on `stream`
int keops_static_fill_zero(void* dst, size_t bytes, void* stream) {
  const long long n = (long long)(bytes / 4);
  if (n == 0) return 0;
  hipLaunchKernelGGL(keops_fill_zero_u32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, (uint32_t*)dst, n);
  return (int)hipGetLastError();
}

// ---- half precision <-> float -------------------------------------------------------------------------------------

static __global__ void __launch_bounds__(256) keops_half_to_float(float* dst, const _Float16* src, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = (float)src[i];
}
static __global__ void __launch_bounds__(256) keops_float_to_half(_Float16* dst, const float* src, long long n) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = (_Float16)src[i];
}

int keops_static_convert_half(void* dst, const void* src, long long n, int to_float, void* stream) {
  if (n <= 0) return 0;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (to_float)
    hipLaunchKernelGGL(keops_half_to_float, grid, dim3(256), 0, (hipStream_t)stream, (float*)dst, (const _Float16*)src, n);
  else
    hipLaunchKernelGGL(keops_float_to_half, grid, dim3(256), 0, (hipStream_t)stream, (_Float16*)dst, (const float*)src, n);
  return (int)hipGetLastError();
}

// ---- lookup table of block-sparse launches, built on the device --------------------------------------------------
//
// Counterpart of range_preprocess_from_device (keopscore/keopscore/binders/nvrtc/keops_nvrtc.cpp:152-248), which
// copies the row ranges to the host at every call, builds the table there and copies it back.  Here the table is
// built by a few small kernels on the launch stream: no read-back, no synchronisation, and the launch can be
// recorded in a HIP graph.  The number of workgroups is not known on the host, so the grid has nblocks_max =
// nranges + rows_total / rows_per_block workgroups (enough for disjoint row ranges) and the surplus ones find an
// empty entry and return.  Every index is clamped to its axis (the map-reduce kernels sweep the ranges unchecked);
// status records that something had to be clamped.  Row ranges are ordered by the reduced rows they sweep, longest
// first, as the host path does (stable: ties keep their order), up to 16384 ranges; beyond, in table order.

static __global__ void __launch_bounds__(256) keops_ranges_clean_y(const KeopsRangeBuild B) {
  const long long k = (long long)blockIdx.x * 256 + threadIdx.x;
  if (k >= B.nred) return;
  const long long a = B.ry[2 * k], b = B.ry[2 * k + 1];
  const long long a2 = a < 0 ? 0 : (a > B.cols_total ? B.cols_total : a);
  const long long b2 = b < a2 ? a2 : (b > B.cols_total ? B.cols_total : b);
  B.ry_clean[2 * k] = a2;
  B.ry_clean[2 * k + 1] = b2;
  if (a2 != a || b2 != b) atomicOr(B.status, 1u);
}

static __global__ void __launch_bounds__(256) keops_ranges_rows(const KeopsRangeBuild B) {
  const long long r = (long long)blockIdx.x * 256 + threadIdx.x;
  if (r >= B.nranges) return;
  const long long s = B.rx[2 * r], e = B.rx[2 * r + 1];
  const long long s2 = s < 0 ? 0 : (s > B.rows_total ? B.rows_total : s);
  const long long e2 = e < s2 ? s2 : (e > B.rows_total ? B.rows_total : e);
  auto clamp_slice = [&](long long v) { return v < 0 ? 0 : (v > B.nred ? B.nred : v); };
  const long long a = r == 0 ? 0 : clamp_slice(B.sl[r - 1]), b = clamp_slice(B.sl[r]);
  if (s2 != s || e2 != e || b != B.sl[r]) atomicOr(B.status, 1u);
  B.sl_clean[r] = b;
  B.nb[r] = (e2 - s2 + B.rows_per_block - 1) / B.rows_per_block;
  long long w = 0;
  for (long long k = a; k < b; k++) w += B.ry_clean[2 * k + 1] - B.ry_clean[2 * k];
  B.work[r] = w;
}

// order[rank] = r with rank = number of ranges that come before r in a stable sort by decreasing work
static __global__ void __launch_bounds__(256) keops_ranges_rank(const KeopsRangeBuild B, int sorted) {
  __shared__ long long ws[256];
  const long long r = (long long)blockIdx.x * 256 + threadIdx.x;
  if (!sorted) {
    if (r < B.nranges) B.order[r] = r;
    return;
  }
  const long long w = r < B.nranges ? B.work[r] : 0;
  long long rank = 0;
  for (long long q0 = 0; q0 < B.nranges; q0 += 256) {
    __syncthreads();
    ws[threadIdx.x] = q0 + threadIdx.x < B.nranges ? B.work[q0 + threadIdx.x] : -1;
    __syncthreads();
    const int n = (int)(B.nranges - q0 < 256 ? B.nranges - q0 : 256);
    for (int t = 0; t < n; t++) {
      const long long wq = ws[t];
      rank += (wq > w || (wq == w && q0 + t < r)) ? 1 : 0;
    }
  }
  if (r < B.nranges) B.order[rank] = r;
}

// offs[i] = first workgroup of the i-th range in issue order (one workgroup of 1024 threads scans everything)
static __global__ void __launch_bounds__(1024) keops_ranges_scan(const KeopsRangeBuild B) {
  __shared__ long long part[1024];
  const int t = threadIdx.x;
  const long long per = (B.nranges + 1023) / 1024, lo = t * per, hi = lo + per < B.nranges ? lo + per : B.nranges;
  long long s = 0;
  for (long long i = lo; i < hi; i++) s += B.nb[B.order[i]];
  part[t] = s;
  __syncthreads();
  for (int o = 1; o < 1024; o <<= 1) {
    const long long v = t >= o ? part[t - o] : 0;
    __syncthreads();
    part[t] += v;
    __syncthreads();
  }
  long long run = part[t] - s;  // exclusive
  for (long long i = lo; i < hi; i++) {
    B.offs[i] = run;
    run += B.nb[B.order[i]];
  }
  if (t == 1023 && part[1023] > B.nblocks_max) atomicOr(B.status, 2u);
}

// every entry starts empty (range 0, no rows)
static __global__ void __launch_bounds__(256) keops_ranges_clear(const KeopsRangeBuild B) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  if (e < 3 * B.nblocks_max) B.lookup[e] = 0;
}

static __global__ void __launch_bounds__(256) keops_ranges_fill(const KeopsRangeBuild B) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= B.nranges) return;
  const long long r = B.order[i];
  const long long s = B.rx[2 * r], e = B.rx[2 * r + 1];
  const long long s2 = s < 0 ? 0 : (s > B.rows_total ? B.rows_total : s);
  const long long e2 = e < s2 ? s2 : (e > B.rows_total ? B.rows_total : e);
  long long idx = B.offs[i];
  for (long long j = s2; j < e2 && idx < B.nblocks_max; j += B.rows_per_block, idx++) {
    B.lookup[3 * idx] = r;
    B.lookup[3 * idx + 1] = j;
    B.lookup[3 * idx + 2] = j + B.rows_per_block < e2 ? j + B.rows_per_block : e2;
  }
}

size_t keops_static_range_build_words(long long nranges, long long nred, long long nblocks_max) {
  return (size_t)(3 * nblocks_max + nranges + 2 * nred + 4 * nranges + 2);
}

int keops_static_build_ranges(const KeopsRangeBuild* b, void* stream) {
  const KeopsRangeBuild B = *b;
  hipStream_t st = (hipStream_t)stream;
  auto grid = [](long long n) { return dim3((unsigned)((n + 255) / 256 > 0 ? (n + 255) / 256 : 1)); };
  hipLaunchKernelGGL(keops_fill_zero_u32, dim3(1), dim3(256), 0, st, (uint32_t*)B.status, 1LL);
  hipLaunchKernelGGL(keops_ranges_clear, grid(3 * B.nblocks_max), dim3(256), 0, st, B);
  if (B.nred > 0) hipLaunchKernelGGL(keops_ranges_clean_y, grid(B.nred), dim3(256), 0, st, B);
  if (B.nranges > 0) {
    hipLaunchKernelGGL(keops_ranges_rows, grid(B.nranges), dim3(256), 0, st, B);
    hipLaunchKernelGGL(keops_ranges_rank, grid(B.nranges), dim3(256), 0, st, B, B.nranges <= 16384 ? 1 : 0);
    hipLaunchKernelGGL(keops_ranges_scan, dim3(1), dim3(1024), 0, st, B);
    hipLaunchKernelGGL(keops_ranges_fill, grid(B.nranges), dim3(256), 0, st, B);
  }
  return (int)hipGetLastError();
}

// ---- calibration loops ----------------------------------------------------------------------------------------------

// Every lane runs `iters` rounds of CHAINS independent dependency chains.  MIX 0: v_fmac_f32 only; MIX 1: the
// instruction mix of a Gaussian pair (3 subtractions, 1 multiplication, 2 fused multiply-adds, 1 multiplication,
// v_exp_f32, 1 fused multiply-add = 9 instructions per chain and round); MIX 2: the same mix without v_exp_f32
// (8 instructions).  The asm statements are empty: they only keep the compiler from hoisting or folding the rounds.
template <int CHAINS, int MIX>
static __global__ void __launch_bounds__(256) keops_valu_loop(float* out, int iters, float c0, float c1) {
  float a[CHAINS], acc[CHAINS];
#pragma unroll
  for (int k = 0; k < CHAINS; k++) {
    a[k] = 1.0f + 1e-3f * (float)(threadIdx.x + k);
    acc[k] = 0.f;
  }
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int k = 0; k < CHAINS; k++) {
      if (MIX == 0) {
#pragma unroll
        for (int u = 0; u < 8; u++) a[k] = __builtin_fmaf(a[k], c0, c1);
      } else {
        const float d0 = a[k] - c0, d1 = a[k] - c1, d2 = c0 - a[k];
        float s = d0 * d0;
        s = __builtin_fmaf(d1, d1, s);
        s = __builtin_fmaf(d2, d2, s);
        float t = s * c1;
        if (MIX == 1) t = __builtin_amdgcn_exp2f(-t);
        acc[k] = __builtin_fmaf(t, c0, acc[k]);
      }
      asm volatile("" : "+v"(a[k]), "+v"(acc[k]));
    }
  }
  float r = 0.f;
#pragma unroll
  for (int k = 0; k < CHAINS; k++) r += a[k] + acc[k];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = r;
}

typedef float keops_f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 keops_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 keops_f16x8 __attribute__((ext_vector_type(8)));

// `iters` rounds of CHAINS independent v_mfma_f32_32x32x16_bf16 (HALF = 0) or _f16 (HALF = 1) accumulation chains per
// wavefront; the operands carry full-width random significands (the power drawn, hence the sustained clock,
// depends on the data)
template <int CHAINS, int HALF>
static __global__ void __launch_bounds__(256) keops_mfma_loop(float* out, int iters) {
  keops_f32x16 acc[CHAINS];
  typedef typename std::conditional<HALF == 1, keops_f16x8, keops_bf16x8>::type vec8;
  typedef typename std::conditional<HALF == 1, _Float16, __bf16>::type elem;
  vec8 a, b;
  unsigned h = 0x9e3779b9u * (threadIdx.x + 1u);
#pragma unroll
  for (int e = 0; e < 8; e++) {
    h = h * 1664525u + 1013904223u;
    a[e] = (elem)(1.0f + (float)(h >> 8) * (1.0f / 16777216.0f));
    h = h * 1664525u + 1013904223u;
    b[e] = (elem)(((h & 1u) ? -1.0f : 1.0f) * (0.5f + (float)(h >> 8) * (0.5f / 16777216.0f)));
  }
#pragma unroll
  for (int k = 0; k < CHAINS; k++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[k][e] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
      for (int k = 0; k < CHAINS; k++) {
        if constexpr (HALF == 1) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[k], 0, 0, 0);
        else acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[k], 0, 0, 0);
      }
  }
  float r = 0.f;
#pragma unroll
  for (int k = 0; k < CHAINS; k++)
#pragma unroll
    for (int e = 0; e < 16; e++) r += acc[k][e];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = r;
}


typedef int keops_i32x16 __attribute__((ext_vector_type(16)));
typedef int keops_i32x4 __attribute__((ext_vector_type(4)));

// `iters` rounds of CHAINS independent v_mfma_i32_32x32x32_i8 accumulation chains per wavefront (4 instructions per
// chain and round) on random signed bytes
template <int CHAINS>
static __global__ void __launch_bounds__(256) keops_mfma_i8_loop(float* out, int iters) {
  keops_i32x16 acc[CHAINS];
  keops_i32x4 a, b;
  unsigned h = 0x9e3779b9u * (threadIdx.x + 1u);
#pragma unroll
  for (int e = 0; e < 4; e++) {
    h = h * 1664525u + 1013904223u;
    a[e] = (int)h;
    h = h * 1664525u + 1013904223u;
    b[e] = (int)h;
  }
#pragma unroll
  for (int k = 0; k < CHAINS; k++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[k][e] = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 4; u++)
#pragma unroll
      for (int k = 0; k < CHAINS; k++) acc[k] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[k], 0, 0, 0);
  }
  int r = 0;
#pragma unroll
  for (int k = 0; k < CHAINS; k++)
#pragma unroll
    for (int e = 0; e < 16; e++) r += acc[k][e];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = (float)r;
}

// `iters` rounds of 32 matrix instructions (two chains) whose operands change with every instruction, as in a kernel
// that streams tiles: 16 A and 16 B register sets of random data per lane, instruction k of chain c multiplies
// A[k] by B[(k + c) % 16].  TYPE 0: v_mfma_f32_32x32x16_bf16, 1: ..._f16, 2: v_mfma_i32_32x32x32_i8.  The loops above
// feed the same two registers to every instruction, which keeps the operand buses quiet; here they toggle as they do
// on real data, the multipliers draw more power and the sustained clock is lower.
template <int TYPE>
static __global__ void __launch_bounds__(256) keops_mfma_stream_loop(float* out, int iters) {
  typedef typename std::conditional<TYPE == 2, keops_i32x16, keops_f32x16>::type accT;
  keops_i32x4 a[16], b[16];
  unsigned h = 0x9e3779b9u * (threadIdx.x + 1u);
#pragma unroll
  for (int k = 0; k < 16; k++)
#pragma unroll
    for (int e = 0; e < 4; e++) {
      // two 16-bit floats of magnitude 2^-3 .. 2 (sign and significand random), or four random bytes
      h = h * 1664525u + 1013904223u;
      a[k][e] = TYPE == 2 ? (int)h : (int)((h & (TYPE == 1 ? 0x8fff8fffu : 0x81ff81ffu)) | (TYPE == 1 ? 0x30003000u : 0x3e003e00u));
      h = h * 1664525u + 1013904223u;
      b[k][e] = TYPE == 2 ? (int)h : (int)((h & (TYPE == 1 ? 0x8fff8fffu : 0x81ff81ffu)) | (TYPE == 1 ? 0x30003000u : 0x3e003e00u));
    }
  accT acc[2];
#pragma unroll
  for (int c = 0; c < 2; c++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[c][e] = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int k = 0; k < 16; k++)
#pragma unroll
      for (int c = 0; c < 2; c++) {
        const keops_i32x4 av = a[k], bv = b[(k + c) & 15];
        if constexpr (TYPE == 2) acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bv, acc[c], 0, 0, 0);
        else if constexpr (TYPE == 1)
          acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(keops_f16x8, av), __builtin_bit_cast(keops_f16x8, bv), acc[c], 0, 0, 0);
        else
          acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(keops_bf16x8, av), __builtin_bit_cast(keops_bf16x8, bv), acc[c], 0, 0, 0);
      }
    if (TYPE != 2) {  // keep the float sums bounded
#pragma unroll
      for (int c = 0; c < 2; c++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[c][e] *= 0.0009765625f;
    }
  }
  float r = 0.f;
#pragma unroll
  for (int c = 0; c < 2; c++)
#pragma unroll
    for (int e = 0; e < 16; e++) r += (float)acc[c][e];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = r;
}

// The contraction loop of the high-dimensional chunked kernel on its own: 8 wavefronts per workgroup, each with 32
// rows of 256 components in registers as hi and lo half-precision operands, a 32-row tile (hi | lo, 1024 bytes per
// row) brought straight from memory to LDS one round ahead (two buffers, one barrier per round), per k block two LDS
// reads and three v_mfma_f32_32x32x16_f16 (lo*hi, hi*lo, hi*hi).  No vector work, no weighted sum.  RANDOM = 0: every
// operand is the same constant; 1: random signs and significands, hi parts near 2^11, lo parts near 1, like the split
// operands of real data.  `tiles`: KEOPS_STREAM_TILES tiles of 32 x 512 half-precision numbers, swept cyclically.
#define KEOPS_STREAM_TILES 64
template <int RANDOM>
static __global__ void __launch_bounds__(256) keops_stream_fill(_Float16* tiles) {
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;   // one half-precision number each
  unsigned h = 0x9e3779b9u * (unsigned)(e + 1u);
  h = h * 1664525u + 1013904223u;
  const float u = (float)((h >> 8) & 0xffff) * (1.0f / 32768.0f) - 1.0f;
  tiles[e] = RANDOM ? (_Float16)(((e & 511) < 256 ? 4000.f : 2.f) * u) : (_Float16)1.0586f;
}

template <int RANDOM>
static __global__ void __launch_bounds__(512) keops_stream_loop(float* out, const _Float16* tiles, int iters) {
  constexpr int STRIDE = 1024 + 16;
  __shared__ __attribute__((aligned(16))) unsigned char as[2][32 * STRIDE];
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, col = lane & 31;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  keops_f16x8 bh[16], bl[16];
  unsigned h = 0x9e3779b9u * (unsigned)(blockIdx.x * 512 + tid + 1u);
#pragma unroll
  for (int kb = 0; kb < 16; kb++)
#pragma unroll
    for (int e = 0; e < 8; e++) {
      h = h * 1664525u + 1013904223u;
      const float u = (float)((h >> 8) & 0xffff) * (1.0f / 32768.0f) - 1.0f;
      bh[kb][e] = RANDOM ? (_Float16)(4000.f * u) : (_Float16)1.0586f;
      h = h * 1664525u + 1013904223u;
      const float w = (float)((h >> 8) & 0xffff) * (1.0f / 32768.0f) - 1.0f;
      bl[kb][e] = RANDOM ? (_Float16)(2.f * w) : (_Float16)1.0586f;
    }
  if (tid < 2) as[tid][0] = 0;  // (an array the compiler sees no store to would count as uninitialised)
  __syncthreads();
  auto stage = [&](int t) {
    const _Float16* src = tiles + (size_t)(t % KEOPS_STREAM_TILES) * 32 * 512;
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int row = wave + 8 * r;
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const uint4*>(src + row * 512) + lane,
                                       &as[0][0] + __builtin_amdgcn_readfirstlane((t & 1) * 32 * STRIDE + row * STRIDE), 16, 0, 0);
    }
  };
  keops_f32x16 tot;
#pragma unroll
  for (int v = 0; v < 16; v++) tot[v] = 0.f;
  stage(0);
  for (int t = 0; t < iters; t++) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's rows of tile t have landed
    __syncthreads();                     // everybody's have, and tile t - 1 has been consumed
    if (t + 1 < iters) stage(t + 1);
    const unsigned char* arow = as[t & 1] + col * STRIDE + 16 * half;
    keops_f32x16 s;
#pragma unroll
    for (int v = 0; v < 16; v++) s[v] = 0.f;
#pragma unroll
    for (int kb = 0; kb < 16; kb++) {
      const keops_f16x8 ah = *reinterpret_cast<const keops_f16x8*>(arow + kb * 32);
      const keops_f16x8 al = *reinterpret_cast<const keops_f16x8*>(arow + 512 + kb * 32);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bh[kb], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bl[kb], s, 0, 0, 0);
      s = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh[kb], s, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 16; v++) tot[v] += s[v] * 1e-12f;
  }
  float r = 0.f;
#pragma unroll
  for (int v = 0; v < 16; v++) r += tot[v];
  // (blocks * 256 floats of output for workgroups of 512 lanes: the two halves of a workgroup add up)
  __syncthreads();  // every wavefront is done with the last tile
  if (tid >= 256) reinterpret_cast<float*>(as[0])[tid - 256] = r;
  __syncthreads();
  if (tid < 256) out[(size_t)blockIdx.x * 256 + tid] = r + reinterpret_cast<float*>(as[0])[tid];
}

// The inner loop of the signed-byte nearest-neighbour filter without its memory traffic: per round two query sets,
// each two dependent v_mfma_i32_32x32x32_i8 from a constant accumulator, and the minimum over the 16 results of a
// set (v_min3_i32 chain, one compare) taken while the other set's instructions are in the pipe.  MODE 0: as
// described; 1: the minima read registers that no matrix instruction writes (same instruction count, no dependence
// on the matrix results); 2: no vector work.
template <int MODE>
static __global__ void __launch_bounds__(256) keops_mfma_screen_loop(float* out, int iters) {
  keops_i32x4 a[2], b[2];
  unsigned h = 0x9e3779b9u * (threadIdx.x + 1u);
#pragma unroll
  for (int k = 0; k < 2; k++)
#pragma unroll
    for (int e = 0; e < 4; e++) {
      h = h * 1664525u + 1013904223u;
      a[k][e] = (int)h;
      h = h * 1664525u + 1013904223u;
      b[k][e] = (int)h;
    }
  keops_i32x16 c0, acc[2], other;
#pragma unroll
  for (int e = 0; e < 16; e++) {
    c0[e] = (int)(h >> 20) + e;
    other[e] = (int)(h >> 12) - e;
    acc[0][e] = acc[1][e] = 0;
  }
  int hits = 0;
  int thr = -(1 << 30);
  asm volatile("" : "+v"(thr));
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int c = 0; c < 2; c++) {
      acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[0], b[c], c0, 0, 0, 0);
      acc[c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[1], b[1 - c], acc[c], 0, 0, 0);
      if (MODE != 2) {
        keops_i32x16 src = MODE == 0 ? acc[1 - c] : other;
        if (MODE == 1) asm volatile("" : "+v"(src));
        int m = src[0] < src[1] ? src[0] : src[1];
#pragma unroll
        for (int e = 2; e < 16; e += 2) {
          const int t = m < src[e] ? m : src[e];
          m = t < src[e + 1] ? t : src[e + 1];
        }
        hits += m <= thr ? 1 : 0;
      }
    }
  }
  int r = hits;
#pragma unroll
  for (int c = 0; c < 2; c++)
#pragma unroll
    for (int e = 0; e < 16; e++) r += acc[c][e];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = (float)r;
}

// `iters` rounds of 8 v_mfma_f32_32x32x16_bf16 (two dependent chains of 4, the shape of the K-nearest-neighbour
// filter) with NV independent v_fmac_f32 between them: how much vector work fits beside a saturated matrix pipe
template <int NV>
static __global__ void __launch_bounds__(256) keops_mix_loop(float* out, int iters, float c0, float c1) {
  keops_f32x16 acc[2];
  keops_bf16x8 a, b;
  unsigned h = 0x9e3779b9u * (threadIdx.x + 1u);
#pragma unroll
  for (int e = 0; e < 8; e++) {
    h = h * 1664525u + 1013904223u;
    a[e] = (__bf16)(1.0f + (float)(h >> 8) * (1.0f / 16777216.0f));
    h = h * 1664525u + 1013904223u;
    b[e] = (__bf16)(((h & 1u) ? -1.0f : 1.0f) * (0.5f + (float)(h >> 8) * (0.5f / 16777216.0f)));
  }
#pragma unroll
  for (int k = 0; k < 2; k++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[k][e] = 0.f;
  float v[8];
#pragma unroll
  for (int k = 0; k < 8; k++) v[k] = 1.0f + 1e-3f * (float)(threadIdx.x + k);
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int u = 0; u < 4; u++) {
#pragma unroll
      for (int k = 0; k < 2; k++) {
        acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[k], 0, 0, 0);
#pragma unroll
        for (int w = 0; w < NV / 8; w++) {
          const int c = (u * 2 + k + w) & 7;
          v[c] = __builtin_fmaf(v[c], c0, c1);
          asm volatile("" : "+v"(v[c]));
        }
      }
    }
  }
  float r = 0.f;
#pragma unroll
  for (int k = 0; k < 2; k++)
#pragma unroll
    for (int e = 0; e < 16; e++) r += acc[k][e];
#pragma unroll
  for (int k = 0; k < 8; k++) r += v[k];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = r;
}

// Runs one calibration loop on `stream`: grid of `blocks` workgroups of 256 lanes (4 wavefronts), `iters` rounds.
// kind 0/1/2: vector loop with MIX = kind; kind 3 / 4: matrix loop on bf16 / f16 operands; kind 6: on signed bytes
// (v_mfma_i32_32x32x32_i8); kind 5: 8 bf16 matrix
// instructions per round with `chains` v_fmac_f32 after each of them (0, 1, 2, 4, 8); kind 7: 32 matrix instructions
// per round whose operands change with every instruction, `chains` = 0 bf16, 1 f16, 2 signed bytes; kind 8: the loop of
// the signed-byte nearest-neighbour filter without memory traffic, `chains` = 0, 1, 2 (see keops_mfma_screen_loop);
// kind 9: the contraction loop of the high-dimensional chunked kernel on its own (keops_stream_loop; workgroups of 8
// wavefronts, `chains` = 0 constant / 1 random operands; out needs KEOPS_STATIC_STREAM_BYTES more bytes).
// chains: 1, 2, 4 or 8 (vector), 1, 2 or 4 (matrix).
// instr_per_lane receives the number of counted instructions one wavefront issues (vector: per lane = per wavefront
// instruction count; matrix: v_mfma instructions).  out must hold blocks * 256 floats.
int keops_static_calibrate(int kind, int chains, int blocks, int iters, float* out, void* stream, double* instr_per_wave) {
  hipStream_t s = (hipStream_t)stream;
  const dim3 g((unsigned)blocks), b(256);
#define VALU_CASE(C, M) hipLaunchKernelGGL((keops_valu_loop<C, M>), g, b, 0, s, out, iters, 1.0009765625f, 0.99951171875f)
  if (kind >= 0 && kind <= 2) {
    const double per_round = kind == 0 ? 8.0 : (kind == 1 ? 9.0 : 8.0);
    *instr_per_wave = per_round * chains * (double)iters;
    if (kind == 0) {
      if (chains == 1) VALU_CASE(1, 0); else if (chains == 2) VALU_CASE(2, 0); else if (chains == 4) VALU_CASE(4, 0);
      else if (chains == 8) VALU_CASE(8, 0); else return (int)hipErrorInvalidValue;
    } else if (kind == 1) {
      if (chains == 1) VALU_CASE(1, 1); else if (chains == 2) VALU_CASE(2, 1); else if (chains == 4) VALU_CASE(4, 1);
      else if (chains == 8) VALU_CASE(8, 1); else return (int)hipErrorInvalidValue;
    } else {
      if (chains == 1) VALU_CASE(1, 2); else if (chains == 2) VALU_CASE(2, 2); else if (chains == 4) VALU_CASE(4, 2);
      else if (chains == 8) VALU_CASE(8, 2); else return (int)hipErrorInvalidValue;
    }
  } else if (kind == 3 || kind == 4) {
    *instr_per_wave = 4.0 * chains * (double)iters;
#define MFMA_CASE(C) do { if (kind == 3) hipLaunchKernelGGL((keops_mfma_loop<C, 0>), g, b, 0, s, out, iters); \
                          else hipLaunchKernelGGL((keops_mfma_loop<C, 1>), g, b, 0, s, out, iters); } while (0)
    if (chains == 1) MFMA_CASE(1);
    else if (chains == 2) MFMA_CASE(2);
    else if (chains == 4) MFMA_CASE(4);
    else return (int)hipErrorInvalidValue;
#undef MFMA_CASE
  } else if (kind == 6) {
    *instr_per_wave = 4.0 * chains * (double)iters;
    if (chains == 1) hipLaunchKernelGGL((keops_mfma_i8_loop<1>), g, b, 0, s, out, iters);
    else if (chains == 2) hipLaunchKernelGGL((keops_mfma_i8_loop<2>), g, b, 0, s, out, iters);
    else if (chains == 4) hipLaunchKernelGGL((keops_mfma_i8_loop<4>), g, b, 0, s, out, iters);
    else return (int)hipErrorInvalidValue;
  } else if (kind == 7) {
    // chains = operand type: 0 bf16, 1 f16, 2 signed bytes
    *instr_per_wave = 32.0 * (double)iters;
    if (chains == 0) hipLaunchKernelGGL((keops_mfma_stream_loop<0>), g, b, 0, s, out, iters);
    else if (chains == 1) hipLaunchKernelGGL((keops_mfma_stream_loop<1>), g, b, 0, s, out, iters);
    else if (chains == 2) hipLaunchKernelGGL((keops_mfma_stream_loop<2>), g, b, 0, s, out, iters);
    else return (int)hipErrorInvalidValue;
  } else if (kind == 9) {
    // workgroups of 8 wavefronts; chains = 0: constant operands, 1: random ones; 48 matrix instructions per round.
    // out: blocks * 256 floats followed by KEOPS_STREAM_TILES * 32 * 512 half-precision numbers of tile data
    *instr_per_wave = 48.0 * (double)iters;
    _Float16* tiles = reinterpret_cast<_Float16*>(out + (size_t)blocks * 256);
    const dim3 gf(KEOPS_STREAM_TILES * 32 * 512 / 256), b8(512);
    if (chains == 0) {
      hipLaunchKernelGGL((keops_stream_fill<0>), gf, b, 0, s, tiles);
      hipLaunchKernelGGL((keops_stream_loop<0>), g, b8, 0, s, out, tiles, iters);
    } else if (chains == 1) {
      hipLaunchKernelGGL((keops_stream_fill<1>), gf, b, 0, s, tiles);
      hipLaunchKernelGGL((keops_stream_loop<1>), g, b8, 0, s, out, tiles, iters);
    } else {
      return (int)hipErrorInvalidValue;
    }
  } else if (kind == 8) {
    // chains = 0: minima over the other set's results, 1: over registers no matrix instruction writes, 2: none
    *instr_per_wave = 4.0 * (double)iters;
    if (chains == 0) hipLaunchKernelGGL((keops_mfma_screen_loop<0>), g, b, 0, s, out, iters);
    else if (chains == 1) hipLaunchKernelGGL((keops_mfma_screen_loop<1>), g, b, 0, s, out, iters);
    else if (chains == 2) hipLaunchKernelGGL((keops_mfma_screen_loop<2>), g, b, 0, s, out, iters);
    else return (int)hipErrorInvalidValue;
  } else if (kind == 5) {
    // chains = vector instructions per matrix instruction: 0, 1, 2, 4, 8
    *instr_per_wave = 8.0 * (double)iters;
#define MIX_CASE(N) hipLaunchKernelGGL((keops_mix_loop<N>), g, b, 0, s, out, iters, 1.0009765625f, 0.99951171875f)
    if (chains == 0) MIX_CASE(0); else if (chains == 1) MIX_CASE(8); else if (chains == 2) MIX_CASE(16);
    else if (chains == 4) MIX_CASE(32); else if (chains == 8) MIX_CASE(64); else return (int)hipErrorInvalidValue;
#undef MIX_CASE
  } else {
    return (int)hipErrorInvalidValue;
  }
#undef VALU_CASE
  return (int)hipGetLastError();
}
